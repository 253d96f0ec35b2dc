// Small parts around a 32-bit residual stream and in front of and behind attention:
//
//   pa_pair_embed          out[t] = table[id] * scale + pair[(prev * mul_prev + id * mul_cur) mod buckets], 32-bit; the
//                          previous token of a portion's first token comes from a per-request slot, which then takes
//                          the portion's last token; a sequence's first token reads row `buckets`
//   pa_time_conv_add       out = h + conv(h): a causal convolution over time on each channel (weights [taps, channels]),
//                          the last taps - 1 inputs carried per request
//   pa_stream_add_row      x[t] += row, in place
//   pa_stream_add_branches x += a + b, in place (b may be absent)
//   pa_qkv_rope_prepare    queries, keys and values out of a merged projection: the first `rot` dimensions of every
//                          query and key head turned by position (in halves or in pairs), queries times a number per
//                          head, keys and values into the paged cache; keys and values have widths and head counts
//                          of their own
//   pa_diff_combine        out[t, h] = u / sqrt(mean(u^2) + eps) * scale with u = a[t, h] - lambda a[t, heads + h]
//   pa_sigmoid_gate        out = o * sigmoid(gate)
//   pa_cap_logits          x <- cap * tanh(x / cap), in place
//
// All arithmetic is 32-bit; storage is 32-bit or bfloat16.
#include "common.h"
#include "api.h"

namespace pa {

template <typename T>
__global__ __launch_bounds__(256) void pair_embed_kernel(const int* __restrict__ ids, const int* __restrict__ positions,
                                                         const int* __restrict__ seq_of_token, const int* __restrict__ cu_q,
                                                         const int* __restrict__ state_slots, int* __restrict__ prev_state,
                                                         const T* __restrict__ table, const T* __restrict__ pair,
                                                         float* __restrict__ out, int H, int vocab, int buckets,
                                                         long long mul_prev, long long mul_cur, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const int seq = seq_of_token[t];
  const int begin = cu_q[seq];
  const int slot = state_slots[seq];
  int prev = 0;
  if (t > begin) prev = ids[t - 1];
  else if (slot >= 0) prev = prev_state[slot];
  long long row = buckets;   // a sequence's first token
  if (positions[t] > 0) {
    row = ((long long)prev * mul_prev + (long long)id * mul_cur) % buckets;
    if (row < 0) row += buckets;
  }
  const T* e = table + (size_t)id * H;
  const T* b = pair + (size_t)row * H;
  float* o = out + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_f32(e[i]) * scale + to_f32(b[i]);
  // the workgroup of a portion's first token is the only one that reads the slot; it leaves the portion's last token
  if (t == begin && slot >= 0) {
    __syncthreads();
    if (threadIdx.x == 0) prev_state[slot] = ids[cu_q[seq + 1] - 1];
  }
}

// state [slots, taps - 1, C] 32-bit: the inputs at the taps - 1 positions before the portion's start, oldest first (zeros
// before the sequence's start).  A thread owns V consecutive channels of a token (V = 8: 16-byte pieces of bfloat16).  A
// sequence that brings one token is the only reader of its slot, so its thread moves the carried inputs on itself;
// portions leave that to time_conv_carry_kernel, which runs behind this one.
constexpr int kConvMaxTaps = 17;

template <typename T, int V>
__global__ __launch_bounds__(256) void time_conv_add_kernel(const T* __restrict__ h, const float* __restrict__ w,
                                                            float* __restrict__ state, const int* __restrict__ seq_of_token,
                                                            const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                                                            T* __restrict__ out, int C, int taps) {
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int t = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * V;
  if (c >= C) return;
  const int seq = seq_of_token[t];
  const int begin = cu_q[seq];
  const int rel = t - begin;
  const bool single = cu_q[seq + 1] - begin == 1;
  const int keep = taps - 1;
  float* st = keep > 0 ? state + (size_t)state_slots[seq] * keep * C : nullptr;
  const vec_t xv = *reinterpret_cast<const vec_t*>(h + (size_t)t * C + c);
  float x[V], acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) x[e] = to_f32(xv[e]), acc[e] = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = keep - j;   // the input `back` positions before this token
    float v[V];
    if (back == 0) {
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = x[e];
    } else if (rel - back >= 0) {
      const vec_t pv = *reinterpret_cast<const vec_t*>(h + (size_t)(t - back) * C + c);
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = to_f32(pv[e]);
    } else {
      const float* sp = st + (size_t)(rel - back + keep) * C + c;
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = sp[e];
      if (single && j > 0) {     // one token: the place before this one takes what this place held
        float* dp = st + (size_t)(j - 1) * C + c;
#pragma unroll
        for (int e = 0; e < V; ++e) dp[e] = v[e];
      }
    }
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = fmaf(w[(size_t)j * C + c + e], v[e], acc[e]);   // w [taps, C]: a tap's weights side by side
  }
  if (single && keep > 0) {
    float* dp = st + (size_t)(keep - 1) * C + c;
#pragma unroll
    for (int e = 0; e < V; ++e) dp[e] = x[e];
  }
  vec_t ov;
#pragma unroll
  for (int e = 0; e < V; ++e) ov[e] = from_f32<T>(x[e] + acc[e]);
  *reinterpret_cast<vec_t*>(out + (size_t)t * C + c) = ov;
}

// A thread a (sequence, channel) of the sequences that bring more than one token: it reads all it needs before it writes.
template <typename T>
__global__ __launch_bounds__(256) void time_conv_carry_kernel(const T* __restrict__ h, float* __restrict__ state,
                                                              const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                                                              int C, int taps) {
  const int seq = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int begin = cu_q[seq], n = cu_q[seq + 1] - begin;
  if (n <= 1) return;
  const int keep = taps - 1;
  float* st = state + (size_t)state_slots[seq] * keep * C;
  float fresh[kConvMaxTaps - 1];
  for (int i = 0; i < keep; ++i) {
    const int rel = n - keep + i;   // the step's token this place now holds, or an older input when negative
    fresh[i] = rel >= 0 ? to_f32(h[(size_t)(begin + rel) * C + c]) : st[(size_t)(i + n) * C + c];
  }
  for (int i = 0; i < keep; ++i) st[(size_t)i * C + c] = fresh[i];
}

__global__ void stream_add_row_kernel(float* __restrict__ x, const float* __restrict__ row, size_t total, int H) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) x[i] += row[i % H];
}

// Four elements a thread where the size allows (V = 4), else one.
template <typename T, int V>
__global__ void stream_add_branches_kernel(float* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b, size_t total) {
  typedef T vec_t __attribute__((ext_vector_type(V)));
  typedef float fvec_t __attribute__((ext_vector_type(V)));
  const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (i >= total) return;
  const vec_t av = *reinterpret_cast<const vec_t*>(a + i);
  fvec_t xv = *reinterpret_cast<fvec_t*>(x + i);
  if (b) {
    const vec_t bv = *reinterpret_cast<const vec_t*>(b + i);
#pragma unroll
    for (int e = 0; e < V; ++e) xv[e] += to_f32(av[e]) + to_f32(bv[e]);
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) xv[e] += to_f32(av[e]);
  }
  *reinterpret_cast<fvec_t*>(x + i) = xv;
}

constexpr int kPrepWaves = 4;
constexpr int kPrepMaxDim = 256;

// One wavefront a (token, head) over nq query, nk key and nv value heads.
template <typename T>
__global__ __launch_bounds__(kPrepWaves* kWave) void qkv_rope_prepare_kernel(
    const T* __restrict__ p, size_t stride, int q_off, int k_off, int v_off, const float* __restrict__ inv_freq,
    const int* __restrict__ positions, const int* __restrict__ slots, const float* __restrict__ q_scale, T* __restrict__ q_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int tokens, int nq, int nk, int nv, int hd, int vd, int rot, int pairs,
    int page_size) {
  __shared__ float xs[kPrepWaves][kPrepMaxDim];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int heads = nq + nk + nv;
  const long long unit = (long long)blockIdx.x * kPrepWaves + wave;
  const bool active = unit < (long long)tokens * heads;
  const int t = active ? (int)(unit / heads) : 0;
  const int h = active ? (int)(unit % heads) : 0;
  const T* row = p + (size_t)t * stride;
  const long long slot = (active && slots) ? (long long)slots[t] : -1;
  const long long page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  if (active && h >= nq + nk) {   // a value head: copied into its transposed page
    if (slot >= 0) {
      const int vh = h - nq - nk;
      const T* src = row + v_off + (size_t)vh * vd;
      T* dst = v_cache + ((size_t)page * nv + vh) * vd * page_size + off;
      for (int i = lane; i < vd; i += kWave) dst[(size_t)i * page_size] = src[i];
    }
  }
  const bool is_q = h < nq;
  const bool turns = active && h < nq + nk;
  const T* src = is_q ? row + q_off + (size_t)h * hd : row + k_off + (size_t)(h - nq) * hd;
  if (turns)
    for (int i = lane; i < hd; i += kWave) xs[wave][i] = to_f32(src[i]);
  __syncthreads();
  if (!turns || (!is_q && slot < 0)) return;
  T* dst = is_q ? q_out + ((size_t)t * nq + h) * hd : k_cache + (((size_t)page * nk + (h - nq)) * page_size + off) * hd;
  const float mul = (is_q && q_scale) ? q_scale[h] : 1.0f;
  const int half = rot / 2;
  const int pos = rot > 0 ? positions[t] : 0;
  for (int i = lane; i < hd; i += kWave) {
    float r = xs[wave][i];
    if (i < rot) {
      // the pair (u, v) = (x[a], x[b]) becomes (u cos - v sin, v cos + u sin); frequency j
      int j, other;
      bool first;
      if (pairs) j = i / 2, other = i ^ 1, first = (i & 1) == 0;
      else j = i < half ? i : i - half, other = i < half ? i + half : i - half, first = i < half;
      float sj, cj;
      sincosf((float)pos * inv_freq[j], &sj, &cj);
      const float o = xs[wave][other];
      r = first ? r * cj - o * sj : r * cj + o * sj;
    }
    dst[i] = from_f32<T>(r * mul);
  }
}

// One wavefront a (token, head).  a [T, 2 * heads, vd]: the first `heads` are the first maps' outputs.
template <typename T>
__global__ __launch_bounds__(256) void diff_combine_kernel(const T* __restrict__ a, T* __restrict__ out, long long units, int heads,
                                                           int vd, float lambda, float eps, float scale) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const long long unit = (long long)blockIdx.x * 4 + wave;
  if (unit >= units) return;
  const long long t = unit / heads;
  const int h = (int)(unit % heads);
  const T* a1 = a + ((size_t)t * 2 * heads + h) * vd;
  const T* a2 = a + ((size_t)t * 2 * heads + heads + h) * vd;
  float u[kPrepMaxDim / kWave];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < kPrepMaxDim / kWave; ++e) {
    const int i = lane + e * kWave;
    u[e] = i < vd ? to_f32(a1[i]) - lambda * to_f32(a2[i]) : 0.f;
    ss += u[e] * u[e];
  }
  ss = wave_sum(ss);
  const float inv = rsqrtf(ss / (float)vd + eps) * scale;
  T* o = out + ((size_t)t * heads + h) * vd;
#pragma unroll
  for (int e = 0; e < kPrepMaxDim / kWave; ++e) {
    const int i = lane + e * kWave;
    if (i < vd) o[i] = from_f32<T>(u[e] * inv);
  }
}

template <typename T>
__global__ void sigmoid_gate_kernel(const T* __restrict__ o, size_t o_stride, const T* __restrict__ gate, size_t gate_stride,
                                    T* __restrict__ out, int rows, int width) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)rows * width) return;
  const size_t r = i / width, c = i % width;
  const float g = to_f32(gate[r * gate_stride + c]);
  out[i] = from_f32<T>(to_f32(o[r * o_stride + c]) / (1.0f + expf(-g)));
}

__global__ void cap_logits_kernel(float* __restrict__ x, size_t total, float cap) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) x[i] = cap * tanhf(x[i] / cap);
}

}  // namespace pa

using namespace pa;

extern "C" int pa_pair_embed(void* stream, int dtype, const int* ids, const int* positions, const int* seq_of_token,
                             const int* cu_q, const int* state_slots, int* prev_state, const void* table, const void* pair,
                             float* out, int tokens, int hidden, int vocab, int buckets, long mul_prev, long mul_cur, float scale) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && hidden > 0 && vocab > 0 && buckets > 0, "pair_embed: bad sizes tokens=%d hidden=%d vocab=%d buckets=%d",
             tokens, hidden, vocab, buckets);
  PA_REQUIRE(ids && positions && seq_of_token && cu_q && state_slots && prev_state, "pair_embed: an index array is missing");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32)
    hipLaunchKernelGGL(pair_embed_kernel<float>, dim3(tokens), dim3(256), 0, st, ids, positions, seq_of_token, cu_q, state_slots,
                       prev_state, (const float*)table, (const float*)pair, out, hidden, vocab, buckets, (long long)mul_prev,
                       (long long)mul_cur, scale);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(pair_embed_kernel<bf16>, dim3(tokens), dim3(256), 0, st, ids, positions, seq_of_token, cu_q, state_slots,
                       prev_state, (const bf16*)table, (const bf16*)pair, out, hidden, vocab, buckets, (long long)mul_prev,
                       (long long)mul_cur, scale);
  else
    return pa::fail("pair_embed: unknown element type code %d", dtype);
  return check_launch("pair_embed");
}

extern "C" int pa_time_conv_add(void* stream, int dtype, const void* h, const float* w, float* state, const int* seq_of_token,
                                const int* cu_q, const int* state_slots, void* out, int tokens, int nseq, int channels, int taps,
                                int all_single) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && nseq > 0 && channels > 0 && taps >= 1 && taps <= kConvMaxTaps, "time_conv_add: bad sizes tokens=%d "
             "sequences=%d channels=%d taps=%d", tokens, nseq, channels, taps);
  PA_REQUIRE(taps == 1 || state, "time_conv_add: %d taps need the carried inputs", taps);
  PA_REQUIRE((channels + 255) / 256 <= 65535, "time_conv_add: %d channels exceed the grid", channels);
  hipStream_t st = (hipStream_t)stream;
  const bool wide = channels % 8 == 0 && (reinterpret_cast<uintptr_t>(h) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  const int per = wide ? 8 : 1;
  dim3 grid(tokens, (channels / per + 255) / 256), cgrid(nseq, (channels + 255) / 256);
  const int threads = channels / per >= 256 ? 256 : 64 * ((channels / per + 63) / 64);
#define PA_CONV(T)                                                                                                              \
  do {                                                                                                                          \
    if (wide)                                                                                                                   \
      hipLaunchKernelGGL((time_conv_add_kernel<T, 8>), grid, dim3(threads), 0, st, (const T*)h, w, state, seq_of_token, cu_q,    \
                         state_slots, (T*)out, channels, taps);                                                                 \
    else                                                                                                                        \
      hipLaunchKernelGGL((time_conv_add_kernel<T, 1>), grid, dim3(threads), 0, st, (const T*)h, w, state, seq_of_token, cu_q,    \
                         state_slots, (T*)out, channels, taps);                                                                 \
    if (taps > 1 && !all_single)                                                                                                \
      hipLaunchKernelGGL(time_conv_carry_kernel<T>, cgrid, dim3(256), 0, st, (const T*)h, state, cu_q, state_slots, channels,   \
                         taps);                                                                                                 \
  } while (0)
  if (dtype == kF32) PA_CONV(float);
  else if (dtype == kBF16) PA_CONV(bf16);
  else return pa::fail("time_conv_add: unknown element type code %d", dtype);
#undef PA_CONV
  return check_launch("time_conv_add");
}

extern "C" int pa_stream_add_row(void* stream, float* x, const float* row, int tokens, int hidden) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && hidden > 0, "stream_add_row: bad sizes tokens=%d hidden=%d", tokens, hidden);
  const size_t total = (size_t)tokens * hidden;
  hipLaunchKernelGGL(stream_add_row_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, row,
                     total, hidden);
  return check_launch("stream_add_row");
}

extern "C" int pa_stream_add_branches(void* stream, int dtype, float* x, const void* a, const void* b, long total) {
  if (total == 0) return 0;
  PA_REQUIRE(total > 0 && x && a, "stream_add_branches: bad size %ld", total);
  hipStream_t st = (hipStream_t)stream;
  const bool wide = total % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0;
  const long per = wide ? 4 : 1;
  dim3 grid((unsigned)((total / per + 255) / 256));
  if (dtype == kF32 && wide)
    hipLaunchKernelGGL((stream_add_branches_kernel<float, 4>), grid, dim3(256), 0, st, x, (const float*)a, (const float*)b, (size_t)total);
  else if (dtype == kF32)
    hipLaunchKernelGGL((stream_add_branches_kernel<float, 1>), grid, dim3(256), 0, st, x, (const float*)a, (const float*)b, (size_t)total);
  else if (dtype == kBF16 && wide)
    hipLaunchKernelGGL((stream_add_branches_kernel<bf16, 4>), grid, dim3(256), 0, st, x, (const bf16*)a, (const bf16*)b, (size_t)total);
  else if (dtype == kBF16)
    hipLaunchKernelGGL((stream_add_branches_kernel<bf16, 1>), grid, dim3(256), 0, st, x, (const bf16*)a, (const bf16*)b, (size_t)total);
  else
    return pa::fail("stream_add_branches: unknown element type code %d", dtype);
  return check_launch("stream_add_branches");
}

extern "C" int pa_qkv_rope_prepare(void* stream, int dtype, const void* p, long stride, int q_off, int k_off, int v_off,
                                   const float* inv_freq, const int* positions, const int* slots, const float* q_scale,
                                   void* q_out, void* k_cache, void* v_cache, int tokens, int nq, int nk, int nv, int hd, int vd,
                                   int rot, int pairs, int page_size) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && nq >= 0 && hd > 0 && hd <= kPrepMaxDim && p && (q_out || nq == 0) && (nq > 0 || slots),
             "qkv_rope_prepare: bad sizes tokens=%d nq=%d hd=%d", tokens, nq, hd);
  PA_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0 && (rot == 0 || (inv_freq && positions)),
             "qkv_rope_prepare: %d rotated dimensions of %d, or frequencies or positions missing", rot, hd);
  PA_REQUIRE(q_off >= 0 && q_off + (long)nq * hd <= stride, "qkv_rope_prepare: the queries do not fit the row of %ld", stride);
  if (slots) {
    PA_REQUIRE(nk > 0 && nv > 0 && vd > 0 && vd <= kPrepMaxDim && page_size > 0 && k_cache && v_cache,
               "qkv_rope_prepare: bad sizes nk=%d nv=%d vd=%d page=%d", nk, nv, vd, page_size);
    PA_REQUIRE(k_off >= 0 && k_off + (long)nk * hd <= stride && v_off >= 0 && v_off + (long)nv * vd <= stride,
               "qkv_rope_prepare: keys or values do not fit the row of %ld", stride);
  } else {
    nk = nv = 0;
  }
  hipStream_t st = (hipStream_t)stream;
  const long long units = (long long)tokens * (nq + nk + nv);
  dim3 grid((unsigned)((units + kPrepWaves - 1) / kPrepWaves));
  if (dtype == kF32)
    hipLaunchKernelGGL(qkv_rope_prepare_kernel<float>, grid, dim3(kPrepWaves * kWave), 0, st, (const float*)p, (size_t)stride, q_off,
                       k_off, v_off, inv_freq, positions, slots, q_scale, (float*)q_out, (float*)k_cache, (float*)v_cache, tokens,
                       nq, nk, nv, hd, vd, rot, pairs ? 1 : 0, page_size);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(qkv_rope_prepare_kernel<bf16>, grid, dim3(kPrepWaves * kWave), 0, st, (const bf16*)p, (size_t)stride, q_off,
                       k_off, v_off, inv_freq, positions, slots, q_scale, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, tokens, nq,
                       nk, nv, hd, vd, rot, pairs ? 1 : 0, page_size);
  else
    return pa::fail("qkv_rope_prepare: unknown element type code %d", dtype);
  return check_launch("qkv_rope_prepare");
}

extern "C" int pa_diff_combine(void* stream, int dtype, const void* a, void* out, int tokens, int heads, int vd, float lambda,
                               float eps, float scale) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && heads > 0 && vd > 0 && vd <= kPrepMaxDim, "diff_combine: bad sizes tokens=%d heads=%d vd=%d", tokens,
             heads, vd);
  hipStream_t st = (hipStream_t)stream;
  const long long units = (long long)tokens * heads;
  dim3 grid((unsigned)((units + 3) / 4));
  if (dtype == kF32)
    hipLaunchKernelGGL(diff_combine_kernel<float>, grid, dim3(256), 0, st, (const float*)a, (float*)out, units, heads, vd, lambda,
                       eps, scale);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(diff_combine_kernel<bf16>, grid, dim3(256), 0, st, (const bf16*)a, (bf16*)out, units, heads, vd, lambda, eps,
                       scale);
  else
    return pa::fail("diff_combine: unknown element type code %d", dtype);
  return check_launch("diff_combine");
}

extern "C" int pa_sigmoid_gate(void* stream, int dtype, const void* o, long o_stride, const void* gate, long gate_stride, void* out,
                               int rows, int width) {
  if (rows == 0) return 0;
  PA_REQUIRE(rows > 0 && width > 0 && o_stride >= width && gate_stride >= width, "sigmoid_gate: bad sizes rows=%d width=%d", rows,
             width);
  hipStream_t st = (hipStream_t)stream;
  const size_t total = (size_t)rows * width;
  dim3 grid((unsigned)((total + 255) / 256));
  if (dtype == kF32)
    hipLaunchKernelGGL(sigmoid_gate_kernel<float>, grid, dim3(256), 0, st, (const float*)o, (size_t)o_stride, (const float*)gate,
                       (size_t)gate_stride, (float*)out, rows, width);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(sigmoid_gate_kernel<bf16>, grid, dim3(256), 0, st, (const bf16*)o, (size_t)o_stride, (const bf16*)gate,
                       (size_t)gate_stride, (bf16*)out, rows, width);
  else
    return pa::fail("sigmoid_gate: unknown element type code %d", dtype);
  return check_launch("sigmoid_gate");
}

extern "C" int pa_cap_logits(void* stream, float* x, long total, float cap) {
  if (total == 0) return 0;
  PA_REQUIRE(total > 0 && cap > 0.f, "cap_logits: bad size %ld or cap %g", total, (double)cap);
  hipLaunchKernelGGL(cap_logits_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, (size_t)total, cap);
  return check_launch("cap_logits");
}
