// A feed-forward of many small experts of which every token uses a few.
//
// An *entry* is one (token, choice) pair, numbered token * top + choice.  The entries are put in the order of
// their experts (entries of one expert side by side, in ascending entry number), the experts' products then run
// over tiles of rows of that order, and the outputs are added up per token in the order of its choices.
// Nothing is decided on the host and every grid is sized by the step's shape alone (tiles that turn out empty
// leave at once), so a captured step replays; no sum depends on what else the step holds.
//
//   pa_moe_choices_by_table   which experts: a row of an integer table per token id (no router)
//   pa_moe_route              which experts: a router's scores, a correction added for the choice alone, the
//                             chosen scores normed over their sum; beside them a gate for the shared expert
//   pa_moe_order              entries by expert: offsets [E + 1], order [entries] (position -> entry),
//                             place [entries] (entry -> position)
//   pa_moe_linear             y[p, :] = act(W[expert of p] x[row of p, :]) over the ordered positions p
//   pa_moe_combine            out[t] = base_scale[t] * base[t] + sum_j weight[t, j] * y[place[t * top + j]]
#include "common.h"
#include "api.h"

namespace pa {

__global__ void moe_choices_by_table_kernel(const int* __restrict__ ids, const int* __restrict__ table,
                                            int* __restrict__ choice, int entries, int top, int vocab, int experts) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= entries) return;
  int id = ids[e / top];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  int x = table[(size_t)id * top + e % top];
  choice[e] = x < 0 ? 0 : (x >= experts ? experts - 1 : x);   // a table out of range must not index outside the weights
}

// One wavefront a token.  logits [tokens, ld] 32-bit: the first `experts` columns are the router's, column `gate_col`
// (>= 0) is a gate of its own.  s = softmax(logits) over the experts; the `top` experts with the largest
// s + correction are chosen (the lowest index among equals), in descending order of that sum; their weights are
// s / (sum of the chosen s + 1e-20) * scale; gate_out[t] = sigmoid(logits[t, gate_col]).  A lane holds the experts
// lane, lane + 64, ..: up to kRouteMax of them.
constexpr int kRoutePerLane = 8;
constexpr int kRouteMax = kRoutePerLane * kWave;

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ correction,
                                                       int* __restrict__ choice, float* __restrict__ weights,
                                                       float* __restrict__ gate_out, int tokens, int experts, int top,
                                                       float scale, int gate_col, const float* __restrict__ bias, int by_logit) {
  const int lane = threadIdx.x % kWave;
  const int t = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (t >= tokens) return;
  const float* z = logits + (size_t)t * ld;
  float s[kRoutePerLane], c[kRoutePerLane];
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < kRoutePerLane; ++j) {
    const int e = lane + j * kWave;
    s[j] = e < experts ? z[e] + (bias ? bias[e] : 0.f) : -INFINITY;
    c[j] = s[j];   // by_logit: the choice goes by the logit itself
    m = fmaxf(m, s[j]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < kRoutePerLane; ++j) {
    const int e = lane + j * kWave;
    s[j] = e < experts ? expf(s[j] - m) : 0.f;
    sum += s[j];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int j = 0; j < kRoutePerLane; ++j) {
    const int e = lane + j * kWave;
    if (by_logit) continue;   // s stays exp(logit - max): over the chosen ones' sum it is the softmax over them alone
    s[j] = s[j] / sum;
    c[j] = e < experts ? s[j] + (correction ? correction[e] : 0.f) : -INFINITY;
  }
  float chosen_sum = 0.f;
  float mine = 0.f;      // lane i < top: the score of the i-th chosen expert
  int mine_e = 0;
  for (int i = 0; i < top; ++i) {
    float best = -INFINITY, best_s = 0.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < kRoutePerLane; ++j) {
      const int e = lane + j * kWave;
      if (c[j] > best) best = c[j], best_e = e, best_s = s[j];   // ascending e within a lane: the lowest index among equals
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, kWave), os = __shfl_xor(best_s, off, kWave);
      const int oe = __shfl_xor(best_e, off, kWave);
      if (ob > best || (ob == best && oe < best_e)) best = ob, best_e = oe, best_s = os;
    }
#pragma unroll
    for (int j = 0; j < kRoutePerLane; ++j)
      if (lane + j * kWave == best_e) c[j] = -INFINITY;
    chosen_sum += best_s;
    if (lane == i % kWave && i < kWave) mine = best_s, mine_e = best_e;
    if (i >= kWave && lane == 0) {   // more than 64 chosen: written one by one, weights in a second pass below
      choice[(size_t)t * top + i] = best_e;
      weights[(size_t)t * top + i] = best_s;
    }
  }
  const float norm = scale / (chosen_sum + 1e-20f);
  if (lane < top) {
    choice[(size_t)t * top + lane] = mine_e;
    weights[(size_t)t * top + lane] = mine * norm;
  }
  if (top > kWave && lane == 0)
    for (int i = kWave; i < top; ++i) weights[(size_t)t * top + i] *= norm;
  if (gate_out && lane == 0) gate_out[t] = gate_col >= 0 ? 1.0f / (1.0f + expf(-z[gate_col])) : 1.0f;
}

// One workgroup an expert.  Pass 0 (counts == out): counts[e] = entries of e.  Pass 1: the expert's start is the
// sum of the counts before it; its entries are written in ascending entry number.
__global__ __launch_bounds__(256) void moe_order_kernel(const int* __restrict__ choice, int entries, int experts,
                                                       int* __restrict__ counts, int* __restrict__ offsets,
                                                       int* __restrict__ order, int* __restrict__ place, int pass) {
  __shared__ int wave_count[4];
  __shared__ int base_s;
  const int e = blockIdx.x;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  int base = 0;
  if (pass == 1) {
    if (threadIdx.x == 0) {
      int s = 0;
      for (int i = 0; i < e; ++i) s += counts[i];
      base_s = s;
      offsets[e] = s;
      if (e == experts - 1) offsets[experts] = s + counts[e];
    }
    __syncthreads();
    base = base_s;
  }
  int running = 0;
  for (int i0 = 0; i0 < entries; i0 += 256) {
    const int i = i0 + threadIdx.x;
    const bool mine = i < entries && choice[i] == e;
    const unsigned long long ballot = __ballot(mine);
    const int before = __popcll(ballot & ((1ull << lane) - 1ull));
    __syncthreads();
    if (lane == 0) wave_count[wave] = __popcll(ballot);
    __syncthreads();
    int prior = 0;
    for (int w = 0; w < wave; ++w) prior += wave_count[w];
    if (pass == 1 && mine) {
      const int p = base + running + prior + before;
      order[p] = i;
      place[i] = p;
    }
    running += wave_count[0] + wave_count[1] + wave_count[2] + wave_count[3];
  }
  if (pass == 0 && threadIdx.x == 0) counts[e] = running;
}

// Tiles of kMoeRows positions of one expert x 256 outputs.  blockIdx.x walks the tiles of all experts in order
// (an expert with c entries has ceil(c / kMoeRows) tiles); a block beyond the last tile leaves.  The weight lies
// [expert, k, n] with n fastest.  `from_tokens`: position p reads row order[p] / top of x (the token's
// hidden state), else row p (what the product before left).  act 1: the square of relu.
constexpr int kMoeRows = 16;
constexpr int kMoeChunk = 128;

template <typename TX, typename TW, typename TY>
__global__ __launch_bounds__(256) void moe_linear_kernel(const TX* __restrict__ x, const TW* __restrict__ wt,
                                                        TY* __restrict__ y, const int* __restrict__ offsets,
                                                        const int* __restrict__ order, int experts, int top, int K, int N,
                                                        int from_tokens, int act) {
  __shared__ float xs[kMoeRows][kMoeChunk];
  __shared__ int rows[kMoeRows];
  int tile = blockIdx.x, e = 0, p0 = 0, p1 = 0;
  for (; e < experts; ++e) {
    const int a = offsets[e], b = offsets[e + 1];
    const int tiles = (b - a + kMoeRows - 1) / kMoeRows;
    if (tile < tiles) {
      p0 = a + tile * kMoeRows;
      p1 = p0 + kMoeRows < b ? p0 + kMoeRows : b;
      break;
    }
    tile -= tiles;
  }
  if (e >= experts) return;
  const int n = blockIdx.y * 256 + threadIdx.x;
  if (threadIdx.x < kMoeRows) {
    const int p = p0 + threadIdx.x;
    rows[threadIdx.x] = p < p1 ? (from_tokens ? order[p] / top : p) : -1;
  }
  const TW* w = wt + (size_t)e * K * N;
  float acc[kMoeRows];
#pragma unroll
  for (int m = 0; m < kMoeRows; ++m) acc[m] = 0.f;
  for (int k0 = 0; k0 < K; k0 += kMoeChunk) {
    __syncthreads();
    for (int i = threadIdx.x; i < kMoeRows * kMoeChunk; i += 256) {
      const int m = i / kMoeChunk, k = i % kMoeChunk;
      const int r = rows[m];
      xs[m][k] = (r >= 0 && k0 + k < K) ? to_f32(x[(size_t)r * K + k0 + k]) : 0.f;
    }
    __syncthreads();
    if (n < N) {
      const int kn = K - k0 < kMoeChunk ? K - k0 : kMoeChunk;
      for (int k = 0; k < kn; ++k) {
        const float wv = to_f32(w[(size_t)(k0 + k) * N + n]);
#pragma unroll
        for (int m = 0; m < kMoeRows; ++m) acc[m] = fmaf(xs[m][k], wv, acc[m]);
      }
    }
  }
  if (n < N) {
#pragma unroll
    for (int m = 0; m < kMoeRows; ++m) {
      if (p0 + m < p1) {
        float v = acc[m];
        if (act == 1) {
          v = fmaxf(v, 0.f);
          v = v * v;
        }
        y[(size_t)(p0 + m) * N + n] = from_f32<TY>(v);
      }
    }
  }
}

// out[t, i] = base[t, i] + sum_j weight * y[place[t * top + j], i], in ascending j; `weights` per entry, or the
// same `weight` for all when it is null.
constexpr int kCombineTop = 64;   // choices a token whose places and weights are staged in LDS

// grid (tokens, slices of 1,024 columns): a thread adds up four columns 256 apart.  A token's places and weights are
// read once into LDS (up to kCombineTop choices; beyond that every thread reads them as it goes).
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ place,
                                                         const float* __restrict__ weights, float weight,
                                                         const T* __restrict__ base, const float* __restrict__ base_scale,
                                                         T* __restrict__ out, int top, int width, float* __restrict__ into,
                                                         const T* __restrict__ other) {
  __shared__ int place_s[kCombineTop];
  __shared__ float weight_s[kCombineTop];
  const int t = blockIdx.x;
  const bool staged = top <= kCombineTop;
  if (staged && (int)threadIdx.x < top) {
    place_s[threadIdx.x] = place[t * top + threadIdx.x];
    weight_s[threadIdx.x] = weights ? weights[t * top + threadIdx.x] : weight;
  }
  __syncthreads();
  const float bs = base_scale ? base_scale[t] : 1.0f;
  const int i0 = blockIdx.y * 1024 + threadIdx.x;
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < top; ++j) {
    const size_t row = (size_t)(staged ? place_s[j] : place[t * top + j]) * width;
    const float w = staged ? weight_s[j] : (weights ? weights[t * top + j] : weight);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int i = i0 + 256 * c;
      s[c] += w * y[row + (i < width ? i : width - 1)];
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int i = i0 + 256 * c;
    if (i >= width) continue;
    float v = s[c];
    if (base) v += base_scale ? bs * to_f32(base[(size_t)t * width + i]) : to_f32(base[(size_t)t * width + i]);
    if (into) {   // the branches' sum first, then the stream: x + (other + this)
      if (other) v += to_f32(other[(size_t)t * width + i]);
      into[(size_t)t * width + i] += v;
      continue;
    }
    out[(size_t)t * width + i] = from_f32<T>(v);
  }
}

}  // namespace pa

using namespace pa;

extern "C" int pa_moe_choices_by_table(void* stream, const int* ids, const int* table, int* choice, int tokens, int top,
                                       int vocab, int experts) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && top > 0 && vocab > 0 && experts > 0, "moe_choices_by_table: bad sizes tokens=%d top=%d vocab=%d experts=%d",
             tokens, top, vocab, experts);
  const int entries = tokens * top;
  hipLaunchKernelGGL(moe_choices_by_table_kernel, dim3((entries + 255) / 256), dim3(256), 0, (hipStream_t)stream, ids, table,
                     choice, entries, top, vocab, experts);
  return check_launch("moe_choices_by_table");
}

// counts [experts], offsets [experts + 1], order / place [entries]
extern "C" int pa_moe_order(void* stream, const int* choice, int entries, int experts, int* counts, int* offsets, int* order,
                            int* place) {
  if (entries == 0) return 0;
  PA_REQUIRE(entries > 0 && experts > 0, "moe_order: bad sizes entries=%d experts=%d", entries, experts);
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(moe_order_kernel, dim3(experts), dim3(256), 0, st, choice, entries, experts, counts, offsets, order, place, 0);
  hipLaunchKernelGGL(moe_order_kernel, dim3(experts), dim3(256), 0, st, choice, entries, experts, counts, offsets, order, place, 1);
  return check_launch("moe_order");
}

extern "C" int pa_moe_linear(void* stream, int x_dtype, int w_dtype, int y_dtype, const void* x, const void* wt, void* y,
                             const int* offsets, const int* order, int entries, int experts, int top, int K, int N,
                             int from_tokens, int act) {
  if (entries == 0) return 0;
  PA_REQUIRE(entries > 0 && experts > 0 && top > 0 && K > 0 && N > 0, "moe_linear: bad sizes entries=%d experts=%d k=%d n=%d",
             entries, experts, K, N);
  PA_REQUIRE(act == 0 || act == 1, "moe_linear: unknown activation code %d", act);
  dim3 grid((entries + kMoeRows - 1) / kMoeRows + experts, (N + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
#define PA_MOE(TX, TW, TY)                                                                                              \
  hipLaunchKernelGGL((moe_linear_kernel<TX, TW, TY>), grid, dim3(256), 0, st, (const TX*)x, (const TW*)wt, (TY*)y, offsets, \
                     order, experts, top, K, N, from_tokens, act)
  if (x_dtype == kF32 && w_dtype == kF32 && y_dtype == kF32) PA_MOE(float, float, float);
  else if (x_dtype == kBF16 && w_dtype == kBF16 && y_dtype == kBF16) PA_MOE(bf16, bf16, bf16);
  else if (x_dtype == kBF16 && w_dtype == kBF16 && y_dtype == kF32) PA_MOE(bf16, bf16, float);
  else return pa::fail("moe_linear: element types %d / %d / %d are not a combination it has", x_dtype, w_dtype, y_dtype);
#undef PA_MOE
  return check_launch("moe_linear");
}

extern "C" int pa_moe_route(void* stream, const float* logits, int ld, const float* correction, int* choice, float* weights,
                            float* gate_out, int tokens, int experts, int top, float scale, int gate_col, const float* bias,
                            int by_logit) {
  if (tokens == 0) return 0;
  PA_REQUIRE(!(by_logit && correction), "moe_route: a choice by the logits takes no correction");
  PA_REQUIRE(tokens > 0 && experts > 0 && top > 0 && top <= experts && ld >= experts, "moe_route: bad sizes tokens=%d experts=%d top=%d ld=%d",
             tokens, experts, top, ld);
  PA_REQUIRE(experts <= kRouteMax, "moe_route: %d experts are more than the %d the kernel takes", experts, kRouteMax);
  PA_REQUIRE(gate_col < ld, "moe_route: gate column %d is outside rows of %d", gate_col, ld);
  hipLaunchKernelGGL(moe_route_kernel, dim3((tokens + 3) / 4), dim3(256), 0, (hipStream_t)stream, logits, ld, correction, choice,
                     weights, gate_out, tokens, experts, top, scale, gate_col, bias, by_logit ? 1 : 0);
  return check_launch("moe_route");
}

extern "C" int pa_moe_combine(void* stream, int dtype, const float* y, const int* place, const float* weights, float weight,
                              const void* base, const float* base_scale, void* out, int tokens, int top, int width, float* into,
                              const void* other) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && top > 0 && width > 0, "moe_combine: bad sizes tokens=%d top=%d width=%d", tokens, top, width);
  PA_REQUIRE(into || out, "moe_combine: nowhere to write");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32)
    hipLaunchKernelGGL(moe_combine_kernel<float>, dim3(tokens, (width + 1023) / 1024), dim3(256), 0, st, y, place, weights, weight, (const float*)base,
                       base_scale, (float*)out, top, width, into, (const float*)other);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(moe_combine_kernel<bf16>, dim3(tokens, (width + 1023) / 1024), dim3(256), 0, st, y, place, weights, weight, (const bf16*)base,
                       base_scale, (bf16*)out, top, width, into, (const bf16*)other);
  else
    return pa::fail("moe_combine: unknown element type code %d", dtype);
  return check_launch("moe_combine");
}
