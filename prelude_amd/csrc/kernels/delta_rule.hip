// The gated delta rule, a recurrent mixer with a state of fixed size per request, and what stands in front of a
// recurrence: a short causal convolution per channel with its own carried inputs, unit vectors per head, decays from
// a softplus, and (for linear attention with rotary positions) the rotation of queries and keys in 32-bit.
//
// Per head, with unit vectors q, k [d] (q also times d^(-1/2)), values v [e], a gate beta and a decay g [d] per key
// channel, the state S [d, e] (32-bit, zero at a request's start) moves token by token:
//
//     S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
//
// so the read-out sees the token's own write.  Everything here is 32-bit; the order of every sum follows the token's
// place alone, so outputs and state are the same bits however a prompt is cut into steps.
#include "common.h"
#include "api.h"

namespace pa {

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// A workgroup of two wavefronts a (token, unit).  p [T, stride] holds, from column `off`, the channels [qk | qk | vv]
// (queries and keys of `kvh` heads of d, values of `heads` heads of e).  Every channel c:
// y_t = silu(sum_s w[c, s] x_(t - (taps - 1 - s))), inputs before the step's first token of the sequence from
// conv_state [slots, C, taps - 1] (oldest first; zero for a request that starts).  The units, blockIdx.y: a query or
// key head (2 kvh of them), whose d channels then become a unit vector (x / sqrt(sum x^2 + 1e-6)), a query also times
// d^(-1/2); a value head's e channels; a head's d decays, decay [T, heads * d] = exp(-exp(a_log[h]) *
// softplus(a[t, h * d + j] + dt_bias[h * d + j])) from a [T, a_stride] at column a_off, the first of them also
// beta [T, heads] = sigmoid(b[t, h]) from p at column b_off.  out [T, C] 32-bit.
constexpr int kPrepareThreads = 128;
constexpr int kPrepareMost = 256;   // most channels of a query or key head

template <typename T>
__global__ __launch_bounds__(kPrepareThreads) void delta_prepare_kernel(
    const T* __restrict__ p, size_t stride, int off, int b_off, const float* __restrict__ w, int taps,
    const float* __restrict__ conv_state, const int* __restrict__ seq_of_token, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, const T* __restrict__ a, size_t a_stride, int a_off,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, float* __restrict__ out,
    float* __restrict__ decay, float* __restrict__ beta, int heads, int kvh, int d, int e) {
  __shared__ float sums[kPrepareThreads / kWave];
  const int t = blockIdx.x, u = blockIdx.y;
  const int qk = kvh * d, C = 2 * qk + heads * e;
  if (u >= 2 * kvh + heads) {                 // a head's decays
    const int h = u - 2 * kvh - heads;
    const float rate = expf(a_log[h]);
    for (int j = threadIdx.x; j < d; j += kPrepareThreads) {
      const int i = h * d + j;
      decay[(size_t)t * heads * d + i] = expf(-rate * softplus_f(to_f32(a[(size_t)t * a_stride + a_off + i]) + dt_bias[i]));
    }
    if (h == 0)
      for (int g = threadIdx.x; g < heads; g += kPrepareThreads)
        beta[(size_t)t * heads + g] = 1.0f / (1.0f + expf(-to_f32(p[(size_t)t * stride + b_off + g])));
    return;
  }
  const int seq = seq_of_token[t];
  const int local = t - cu_q[seq];          // tokens of this sequence in the step before this one
  const float* st = conv_state + (size_t)state_slots[seq] * C * (taps - 1);
  auto conv = [&](int c) {
    float acc = 0.f;
    for (int s = 0; s < taps; ++s) {
      const int back = taps - 1 - s;          // how many tokens back this tap reaches
      float x;
      if (back <= local) x = to_f32(p[(size_t)(t - back) * stride + off + c]);
      else x = st[(size_t)c * (taps - 1) + (taps - 1) - (back - local)];
      acc = fmaf(w[(size_t)c * taps + s], x, acc);
    }
    return silu_f(acc);
  };
  if (u >= 2 * kvh) {                         // a value head
    const int c0 = 2 * qk + (u - 2 * kvh) * e;
    for (int j = threadIdx.x; j < e; j += kPrepareThreads) out[(size_t)t * C + c0 + j] = conv(c0 + j);
    return;
  }
  const int c0 = u * d;                       // a query or key head: a unit vector
  float y[kPrepareMost / kPrepareThreads];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kPrepareMost / kPrepareThreads; ++i) {
    const int j = i * kPrepareThreads + threadIdx.x;
    y[i] = j < d ? conv(c0 + j) : 0.f;
    ss += y[i] * y[i];
  }
  ss = wave_sum(ss);
  if (threadIdx.x % kWave == 0) sums[threadIdx.x / kWave] = ss;
  __syncthreads();
  ss = sums[0] + sums[1];
  float f = 1.0f / sqrtf(ss + 1e-6f);
  if (u < kvh) f *= 1.0f / sqrtf((float)d);
#pragma unroll
  for (int i = 0; i < kPrepareMost / kPrepareThreads; ++i) {
    const int j = i * kPrepareThreads + threadIdx.x;
    if (j < d) out[(size_t)t * C + c0 + j] = y[i] * f;
  }
}

// After the step's convolutions: a sequence's carried inputs become the last taps - 1 inputs it has seen.  A thread a
// (sequence, channel); it reads all it needs before it writes.
template <typename T>
__global__ void conv_state_update_kernel(const T* __restrict__ p, size_t stride, int off, int C, int taps,
                                         float* __restrict__ conv_state, const int* __restrict__ cu_q,
                                         const int* __restrict__ state_slots, int nseq) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C || seq >= nseq) return;
  const int begin = cu_q[seq], n = cu_q[seq + 1] - begin;
  if (n <= 0) return;
  const int keep = taps - 1;
  float* st = conv_state + ((size_t)state_slots[seq] * C + c) * keep;
  float fresh[8];
  for (int i = 0; i < keep; ++i) {
    const int rel = n - keep + i;     // the step's token this place now holds, or an older one when negative
    fresh[i] = rel >= 0 ? to_f32(p[(size_t)(begin + rel) * stride + off + c]) : st[i + n];
  }
  for (int i = 0; i < keep; ++i) st[i] = fresh[i];
}

// The recurrence.  x [T, C] 32-bit as delta_prepare left it ([q | k | v]), decay [T, heads, d], beta [T, heads];
// state [slots, heads, d, e]; out [T, heads, e].  The columns of S do not depend on each other.  A column is spread over
// R neighbouring lanes, each keeping D / R rows in registers (four consecutive rows of every R-th group of four, so
// that the R lanes of a column read one contiguous stretch of LDS), and the two dot products are summed across the R
// lanes inside the wavefront's rows of 16 lanes: a sequence of one head is 256 / R columns a workgroup, and the
// dependent chain a token D / R multiply-adds.  The order of every sum follows the token's place alone, so outputs
// and state are the same bits however a prompt is cut into steps.
template <int R>
__device__ __forceinline__ float sum_over_lanes(float v) {
  static_assert(R == 8 || R == 16, "a column's lanes lie inside a row of 16");
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));    // lane ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));    // lane ^ 2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));   // 7 - lane within eight
  if (R == 16) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // 15 - lane
  return v;
}

// Tokens go through LDS NT at a time, in two buffers: the next NT are asked for (16-byte pieces where the key width
// and the row allow, VEC) before the current ones are worked through and put into the other buffer afterwards, one
// barrier a block of tokens.  Places past a sequence's end or past the key width hold k = q = 0, g = 1, beta = 0,
// which leave the state as it is: the walk over a block's tokens has no branch, so the reads of the next token's
// rows can run ahead of the sums of this one.
template <int D, int R, bool VEC>
__global__ __launch_bounds__(256) void gated_delta_rows_kernel(const float* __restrict__ x, const float* __restrict__ decay,
                                                               const float* __restrict__ beta, float* __restrict__ state,
                                                               const int* __restrict__ state_slots, const int* __restrict__ cu_q,
                                                               float* __restrict__ out, int heads, int kvh, int d, int e) {
  constexpr int NT = D <= 128 ? 16 : 8;   // tokens staged at a time
  constexpr int NV = D / R / 4;           // groups of four rows a lane keeps
  constexpr int COLS = 256 / R;
  constexpr int PER = (NT * (D / 4) + 255) / 256;   // 16-byte pieces of each staged array a thread moves
  static_assert(D % (4 * R) == 0, "a lane keeps whole groups of four rows");
  __shared__ float4 ks[2][NT][D / 4], qs[2][NT][D / 4], gs[2][NT][D / 4];
  __shared__ float bs[2][NT];
  const int seq = blockIdx.x, h = blockIdx.y;
  const int rho = threadIdx.x % R;
  const int col = blockIdx.z * COLS + threadIdx.x / R;
  const bool live = col < e;
  const int begin = cu_q[seq], end = cu_q[seq + 1];
  if (end <= begin) return;
  const int kh = h / (heads / kvh);
  const int qk = kvh * d, C = 2 * qk + heads * e;
  float* S = state + (((size_t)state_slots[seq] * heads + h) * d) * e;
  float s[NV][4];
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int j = 4 * (i * R + rho) + c;
      s[i][c] = (live && j < d) ? S[(size_t)j * e + col] : 0.f;
    }
  float4 rq[PER], rk[PER], rg[PER];
  float rb = 0.f;
  float v[NT], v_next[NT];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int p = 0; p < PER; ++p) {
      const int piece = p * 256 + threadIdx.x;
      const int tk = piece / (D / 4), j = 4 * (piece % (D / 4));
      const size_t t = (size_t)t0 + tk;
      rq[p] = rk[p] = float4{0.f, 0.f, 0.f, 0.f};
      rg[p] = float4{1.f, 1.f, 1.f, 1.f};
      if (tk < NT && t < (size_t)end) {
        const float* qp = x + t * C + kh * d + j;
        const float* kp = qp + qk;
        const float* gp = decay + (t * heads + h) * d + j;
        if (VEC) {
          if (j < d) {
            rq[p] = *reinterpret_cast<const float4*>(qp);
            rk[p] = *reinterpret_cast<const float4*>(kp);
            rg[p] = *reinterpret_cast<const float4*>(gp);
          }
        } else {
          float* fq = reinterpret_cast<float*>(&rq[p]);
          float* fk = reinterpret_cast<float*>(&rk[p]);
          float* fg = reinterpret_cast<float*>(&rg[p]);
#pragma unroll
          for (int c = 0; c < 4; ++c)
            if (j + c < d) {
              fq[c] = qp[c];
              fk[c] = kp[c];
              fg[c] = gp[c];
            }
        }
      }
    }
    rb = (threadIdx.x < NT && t0 + (int)threadIdx.x < end) ? beta[(size_t)(t0 + threadIdx.x) * heads + h] : 0.f;
#pragma unroll
    for (int tk = 0; tk < NT; ++tk) v_next[tk] = (live && t0 + tk < end) ? x[(size_t)(t0 + tk) * C + 2 * qk + h * e + col] : 0.f;
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int p = 0; p < PER; ++p) {
      const int piece = p * 256 + threadIdx.x;
      if (piece < NT * (D / 4)) {
        (&qs[buf][0][0])[piece] = rq[p];
        (&ks[buf][0][0])[piece] = rk[p];
        (&gs[buf][0][0])[piece] = rg[p];
      }
    }
    if (threadIdx.x < NT) bs[buf][threadIdx.x] = rb;
  };
  fetch(begin);
  put(0);
#pragma unroll
  for (int tk = 0; tk < NT; ++tk) v[tk] = v_next[tk];
  __syncthreads();
  int buf = 0;
  for (int t0 = begin; t0 < end; t0 += NT, buf ^= 1) {
    const bool more = t0 + NT < end;
    if (more) fetch(t0 + NT);
    float ob[NT];
#pragma unroll
    for (int tk = 0; tk < NT; ++tk) {
      float4 kk[NV];
      float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const float4 gg = gs[buf][tk][i * R + rho];
        kk[i] = ks[buf][tk][i * R + rho];
        s[i][0] *= gg.x; s[i][1] *= gg.y; s[i][2] *= gg.z; s[i][3] *= gg.w;
        part[0] = fmaf(s[i][0], kk[i].x, part[0]);
        part[1] = fmaf(s[i][1], kk[i].y, part[1]);
        part[2] = fmaf(s[i][2], kk[i].z, part[2]);
        part[3] = fmaf(s[i][3], kk[i].w, part[3]);
      }
      const float kv = sum_over_lanes<R>((part[0] + part[1]) + (part[2] + part[3]));
      const float u = bs[buf][tk] * (v[tk] - kv);
      float po[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const float4 qq = qs[buf][tk][i * R + rho];
        s[i][0] = fmaf(kk[i].x, u, s[i][0]); s[i][1] = fmaf(kk[i].y, u, s[i][1]);
        s[i][2] = fmaf(kk[i].z, u, s[i][2]); s[i][3] = fmaf(kk[i].w, u, s[i][3]);
        po[0] = fmaf(s[i][0], qq.x, po[0]);
        po[1] = fmaf(s[i][1], qq.y, po[1]);
        po[2] = fmaf(s[i][2], qq.z, po[2]);
        po[3] = fmaf(s[i][3], qq.w, po[3]);
      }
      ob[tk] = sum_over_lanes<R>((po[0] + po[1]) + (po[2] + po[3]));
    }
    // the block's outputs leave together: a store a token would end a basic block a token, and the reads of the next
    // token's rows could not be moved ahead of this token's sums
    if (live && rho == 0) {
#pragma unroll
      for (int tk = 0; tk < NT; ++tk)
        if (t0 + tk < end) out[((size_t)(t0 + tk) * heads + h) * e + col] = ob[tk];
    }
    if (more) {
      put(buf ^ 1);
#pragma unroll
      for (int tk = 0; tk < NT; ++tk) v[tk] = v_next[tk];
    }
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int j = 4 * (i * R + rho) + c;
        if (j < d) S[(size_t)j * e + col] = s[i][c];
      }
  }
}

// p [T, stride] -> out [T, 2 * heads * d + heads * e] 32-bit: queries (from q_off) and keys (from k_off) with the
// first `rot` dimensions of every head turned, dimension i with i + rot / 2, by positions[t] * inv_freq[i]; the keys
// then times k_scale; values (from v_off) as they are.  A thread an element (a pair's two ends are two threads).
template <typename T>
__global__ void rotate_halves_f32_kernel(const T* __restrict__ p, size_t stride, int q_off, int k_off, int v_off,
                                         const float* __restrict__ inv_freq, const int* __restrict__ positions,
                                         float* __restrict__ out, int tokens, int heads, int d, int e, int rot, float k_scale) {
  const int qk = heads * d, width = 2 * qk + heads * e;
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)tokens * width) return;
  const size_t t = i / width;
  const int c = (int)(i % width);
  const T* row = p + t * stride;
  if (c >= 2 * qk) {
    out[i] = to_f32(row[v_off + c - 2 * qk]);
    return;
  }
  const bool key = c >= qk;
  const int base = key ? k_off : q_off;
  const int cc = key ? c - qk : c;
  const int j = cc % d;
  float val = to_f32(row[base + cc]);
  if (j < rot) {
    const int half = rot / 2;
    const int f = j < half ? j : j - half;
    const float ang = (float)positions[t] * inv_freq[f];
    const float cs = cosf(ang), sn = sinf(ang);
    const float other = to_f32(row[base + cc + (j < half ? half : -half)]);
    val = j < half ? val * cs - other * sn : val * cs + other * sn;
  }
  out[i] = key ? val * k_scale : val;
}

}  // namespace pa

using namespace pa;

extern "C" int pa_delta_prepare(void* stream, int dtype, const void* p, long stride, int off, int b_off, const float* w,
                                int taps, float* conv_state, const int* seq_of_token, const int* cu_q, const int* state_slots,
                                const void* a, long a_stride, int a_off, const float* a_log, const float* dt_bias, float* out,
                                float* decay, float* beta, int tokens, int nseq, int heads, int kvh, int d, int e) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && nseq > 0 && heads > 0 && kvh > 0 && d > 0 && e > 0 && heads % kvh == 0,
             "delta_prepare: bad sizes tokens=%d sequences=%d heads=%d key heads=%d d=%d e=%d", tokens, nseq, heads, kvh, d, e);
  PA_REQUIRE(taps >= 1 && taps <= 9, "delta_prepare: a convolution of %d taps is outside 1..9", taps);
  const long C = 2L * kvh * d + (long)heads * e;
  PA_REQUIRE(off >= 0 && off + C <= stride && b_off >= 0 && b_off + heads <= stride && a_off >= 0 &&
             a_off + (long)heads * d <= a_stride, "delta_prepare: the columns do not fit their rows");
  hipStream_t st = (hipStream_t)stream;
  PA_REQUIRE(d <= kPrepareMost, "delta_prepare: a key width of %d is more than the %d the kernel takes", d, kPrepareMost);
  const dim3 pgrid(tokens, 2 * kvh + 2 * heads);
  if (dtype == kF32) {
    hipLaunchKernelGGL(delta_prepare_kernel<float>, pgrid, dim3(kPrepareThreads), 0, st, (const float*)p, (size_t)stride, off,
                       b_off, w, taps, conv_state, seq_of_token, cu_q, state_slots, (const float*)a, (size_t)a_stride, a_off,
                       a_log, dt_bias, out, decay, beta, heads, kvh, d, e);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<float>, dim3((unsigned)((C + 255) / 256), nseq), dim3(256), 0, st,
                         (const float*)p, (size_t)stride, off, (int)C, taps, conv_state, cu_q, state_slots, nseq);
  } else if (dtype == kBF16) {
    hipLaunchKernelGGL(delta_prepare_kernel<bf16>, pgrid, dim3(kPrepareThreads), 0, st, (const bf16*)p, (size_t)stride, off, b_off,
                       w, taps, conv_state, seq_of_token, cu_q, state_slots, (const bf16*)a, (size_t)a_stride, a_off, a_log,
                       dt_bias, out, decay, beta, heads, kvh, d, e);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<bf16>, dim3((unsigned)((C + 255) / 256), nseq), dim3(256), 0, st,
                         (const bf16*)p, (size_t)stride, off, (int)C, taps, conv_state, cu_q, state_slots, nseq);
  } else {
    return pa::fail("delta_prepare: unknown element type code %d", dtype);
  }
  return check_launch("delta_prepare");
}

extern "C" int pa_gated_delta(void* stream, const float* x, const float* decay, const float* beta, float* state,
                              const int* state_slots, const int* cu_q, float* out, int nseq, int heads, int kvh, int d, int e) {
  if (nseq == 0) return 0;
  PA_REQUIRE(nseq > 0 && heads > 0 && kvh > 0 && heads % kvh == 0 && d > 0 && e > 0,
             "gated_delta: bad sizes sequences=%d heads=%d key heads=%d d=%d e=%d", nseq, heads, kvh, d, e);
  PA_REQUIRE(d <= 256, "gated_delta: a key width of %d is more than the 256 the kernel takes", d);
  hipStream_t st = (hipStream_t)stream;
  // 16-byte loads of queries, keys and decays where every row of them starts at a multiple of four floats
  const bool vec = d % 4 == 0 && (2 * kvh * d + heads * e) % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(decay) & 15) == 0;
#define PA_DELTA_ROWS(D, R)                                                                                                       \
  do {                                                                                                                            \
    dim3 rgrid(nseq, heads, (e + 256 / R - 1) / (256 / R));                                                                       \
    if (vec)                                                                                                                      \
      hipLaunchKernelGGL((gated_delta_rows_kernel<D, R, true>), rgrid, dim3(256), 0, st, x, decay, beta, state, state_slots, cu_q, \
                         out, heads, kvh, d, e);                                                                                  \
    else                                                                                                                          \
      hipLaunchKernelGGL((gated_delta_rows_kernel<D, R, false>), rgrid, dim3(256), 0, st, x, decay, beta, state, state_slots,      \
                         cu_q, out, heads, kvh, d, e);                                                                            \
  } while (0)
  if (d <= 32) PA_DELTA_ROWS(32, 8);
  else if (d <= 64) PA_DELTA_ROWS(64, 16);
  else if (d <= 128) PA_DELTA_ROWS(128, 16);
  else PA_DELTA_ROWS(256, 16);
#undef PA_DELTA_ROWS
  return check_launch("gated_delta");
}

extern "C" int pa_rotate_halves_f32(void* stream, int dtype, const void* p, long stride, int q_off, int k_off, int v_off,
                                    const float* inv_freq, const int* positions, float* out, int tokens, int heads, int d,
                                    int e, int rot, float k_scale) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && heads > 0 && d > 0 && e > 0, "rotate_halves: bad sizes tokens=%d heads=%d d=%d e=%d", tokens, heads, d, e);
  PA_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= d && (rot == 0 || inv_freq),
             "rotate_halves: %d turned dimensions must be even, at most %d, and come with frequencies", rot, d);
  PA_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + (long)heads * d <= stride && k_off + (long)heads * d <= stride &&
             v_off + (long)heads * e <= stride, "rotate_halves: the columns do not fit the row of %ld", stride);
  const long total = (long)tokens * (2L * heads * d + (long)heads * e);
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32)
    hipLaunchKernelGGL(rotate_halves_f32_kernel<float>, dim3(blocks), dim3(256), 0, st, (const float*)p, (size_t)stride, q_off,
                       k_off, v_off, inv_freq, positions, out, tokens, heads, d, e, rot, k_scale);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(rotate_halves_f32_kernel<bf16>, dim3(blocks), dim3(256), 0, st, (const bf16*)p, (size_t)stride, q_off,
                       k_off, v_off, inv_freq, positions, out, tokens, heads, d, e, rot, k_scale);
  else
    return pa::fail("rotate_halves: unknown element type code %d", dtype);
  return check_launch("rotate_halves");
}
