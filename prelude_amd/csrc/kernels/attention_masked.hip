// Paged causal attention with the masks and score terms the plain kernels do not have, for any mix of prompt
// portions and single tokens, in 32-bit or bfloat16 storage, all arithmetic 32-bit on the vector ALU:
//
//   * a window that keeps the first tokens: the query at i sees the key at j <= i when i - j < window (0: no window)
//     or j < keep_first;
//   * a bias by distance: slope_h * (i - j) is taken off the (scaled, capped) score;
//   * values of a width of their own (vdim);
//   * a sink per head in the softmax's denominator;
//   * a gate per (token, head): the head's output times sigmoid(gate), and a constant `out_scale`, before it is
//     rounded; the output may lie inside a wider row (`out_stride`).
//
// And the kernel in front of it: a token's queries, keys and values taken from the merged projection, queries and
// keys optionally brought to unit RMS over the whole projection (all heads at once) and multiplied by a weight of
// that size, keys and values written to the paged cache.
//
// One wavefront per (query token, query head).  Keys are walked in chunks of 64 anchored at multiples of 64: first
// the chunks that hold kept first tokens outside the window, then the window's.  The order of every sum depends on
// the query's position and the mask alone, so a token's result is the same bits in a whole prompt, in a portion or
// alone, whatever pages hold its keys.  Pages between the kept ones and the window may have been given back: no key
// outside the mask is ever touched.
//
// K pages are [page, kv_head, offset, dim], V pages [page, kv_head, vdim, offset].
#include "common.h"
#include "api.h"

namespace pa {

constexpr int kMaskedWaves = 4;
constexpr int kMaskedMaxDim = 256;

template <typename T>
__global__ __launch_bounds__(kMaskedWaves* kWave) void attn_masked_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ seq_of_token,
    const int* __restrict__ positions, T* __restrict__ out, size_t out_stride, int nh, int nkv, int hd, int vd,
    int page_size, int window, int keep_first, float scale, float softcap, const float* __restrict__ slopes,
    const float* __restrict__ sink, const T* __restrict__ gate, size_t gate_stride, float out_scale) {
  __shared__ float qs[kMaskedWaves][kMaskedMaxDim];
  __shared__ float ps[kMaskedWaves][kWave];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int t = blockIdx.x;
  const int h = blockIdx.y * kMaskedWaves + wave;
  const bool active = h < nh;  // every wave of the block shares the token, hence the trip counts below
  const int pos = positions[t];
  const int seq = seq_of_token[t];
  const int hi = pos;
  int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  int kept = keep_first < lo ? keep_first : lo;   // keys [0, kept) are seen beside [lo, hi]
  if (kept < 0) kept = 0;
  if (kept >= lo) { lo = 0; kept = 0; }           // the two ranges meet: one range from the start
  const int kept_chunks = (kept + kWave - 1) / kWave;
  const int first_window_chunk = lo / kWave > kept_chunks ? lo / kWave : kept_chunks;
  const int last_chunk = hi / kWave;
  const int kvh = active ? h / (nh / nkv) : 0;
  const int* table = block_table + (size_t)seq * table_stride;
  const float slope = (slopes && active) ? slopes[h] : 0.f;

  if (active) {
    const T* qr = q + ((size_t)t * nh + h) * hd;
    for (int d = lane; d < hd; d += kWave) qs[wave][d] = to_f32(qr[d]);
  }
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float o[kMaskedMaxDim / kWave] = {};
  for (int chunk = 0; chunk <= last_chunk; ++chunk) {
    if (chunk == kept_chunks && chunk < first_window_chunk) chunk = first_window_chunk;
    const int c0 = chunk * kWave;
    const int c = c0 + lane;
    const bool valid = active && c <= hi && (c >= lo || c < kept);
    float s = -INFINITY;
    if (valid) {
      const int page = table[c / page_size];
      const T* kr = k_cache + (((size_t)page * nkv + kvh) * page_size + (c % page_size)) * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(qs[wave][d], to_f32(kr[d]), dot);
      s = dot * scale;
      if (softcap != 0.f) s = softcap * tanhf(s / softcap);
      s -= slope * (float)(pos - c);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = (active && m > -INFINITY) ? expf(m - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    ps[wave][lane] = p;
    __syncthreads();
#pragma unroll
    for (int e = 0; e < kMaskedMaxDim / kWave; ++e) o[e] *= alpha;
    if (active) {
      for (int j = 0; j < kWave; ++j) {
        const int cj = c0 + j;
        if (cj > hi) break;
        if (!(cj >= lo || cj < kept)) continue;
        const int page = table[cj / page_size];
        const T* vr = v_cache + ((size_t)page * nkv + kvh) * vd * page_size + (cj % page_size);
        const float pj = ps[wave][j];
#pragma unroll
        for (int e = 0; e < kMaskedMaxDim / kWave; ++e) {
          const int d = lane + e * kWave;
          if (d < vd) o[e] = fmaf(pj, to_f32(vr[(size_t)d * page_size]), o[e]);
        }
      }
    }
    __syncthreads();
    m = m_new;
  }
  if (active) {
    T* orow = out + (size_t)t * out_stride + (size_t)h * vd;
    float inv = 1.0f / l;
    if (sink) {   // one more term exp(sink) of the denominator that brings no value
      const float m_fin = fmaxf(m, sink[h]);
      const float alpha = expf(m - m_fin);
      inv = alpha / (l * alpha + expf(sink[h] - m_fin));
    }
    if (gate) inv *= 1.0f / (1.0f + expf(-to_f32(gate[(size_t)t * gate_stride + h])));
    inv *= out_scale;
#pragma unroll
    for (int e = 0; e < kMaskedMaxDim / kWave; ++e) {
      const int d = lane + e * kWave;
      if (d < vd) orow[d] = from_f32<T>(o[e] * inv);
    }
  }
}

// A workgroup a token.  p [T, stride]: queries [nh * hd] at q_off, keys [nkv * hd] at k_off, values [nkv * vd] at
// v_off.  With qw / kw: the whole query (key) projection over sqrt(mean^2 + eps) times the weight.  q_out [T, nh * hd];
// keys and values to the caches at slots[t] (slots null: queries only).
template <typename T>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(const T* __restrict__ p, size_t stride, int q_off, int k_off,
                                                         int v_off, const float* __restrict__ qw,
                                                         const float* __restrict__ kw, const int* __restrict__ slots,
                                                         T* __restrict__ q_out, T* __restrict__ k_cache,
                                                         T* __restrict__ v_cache, int nh, int nkv, int hd, int vd,
                                                         int page_size, float eps) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  const T* row = p + t * stride;
  const int nq = nh * hd, nk = nkv * hd, nv = nkv * vd;
  float q_inv = 1.f, k_inv = 1.f;
  if (qw) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nq; i += blockDim.x) {
      const float v = to_f32(row[q_off + i]);
      ss += v * v;
    }
    q_inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)nq + eps);
  }
  for (int i = threadIdx.x; i < nq; i += blockDim.x) {
    const float v = to_f32(row[q_off + i]);
    q_out[t * nq + i] = qw ? from_f32<T>(v * q_inv * qw[i]) : row[q_off + i];
  }
  if (!slots) return;
  if (kw) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nk; i += blockDim.x) {
      const float v = to_f32(row[k_off + i]);
      ss += v * v;
    }
    k_inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)nk + eps);
  }
  const int slot = slots[t];
  const size_t page = slot / page_size, off = slot % page_size;
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const int g = i / hd, d = i % hd;
    const float v = to_f32(row[k_off + i]);
    k_cache[((page * nkv + g) * page_size + off) * hd + d] = kw ? from_f32<T>(v * k_inv * kw[i]) : row[k_off + i];
  }
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const int g = i / vd, d = i % vd;
    v_cache[((page * nkv + g) * vd + d) * page_size + off] = row[v_off + i];
  }
}

}  // namespace pa

using namespace pa;

extern "C" int pa_attn_masked(void* stream, int dtype, const void* q, const void* k_cache, const void* v_cache,
                              const int* block_table, int table_stride, const int* seq_of_token, const int* positions,
                              void* out, long out_stride, int tokens, int nh, int nkv, int hd, int vd, int page_size,
                              int window, int keep_first, float scale, float softcap, const float* slopes,
                              const float* sink, const void* gate, long gate_stride, float out_scale) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && nh > 0 && nkv > 0 && page_size > 0 && table_stride > 0,
             "attn_masked: bad sizes tokens=%d nh=%d nkv=%d page=%d table_stride=%d", tokens, nh, nkv, page_size, table_stride);
  PA_REQUIRE(nh % nkv == 0, "attn_masked: %d query heads are not a multiple of %d KV heads", nh, nkv);
  PA_REQUIRE(hd > 0 && hd <= kMaskedMaxDim && vd > 0 && vd <= kMaskedMaxDim,
             "attn_masked: key width %d or value width %d is outside 1..%d", hd, vd, kMaskedMaxDim);
  PA_REQUIRE(window >= 0 && keep_first >= 0, "attn_masked: window %d or kept first tokens %d negative", window, keep_first);
  PA_REQUIRE(softcap >= 0.f, "attn_masked: a score cap of %g is negative (0 means none)", (double)softcap);
  PA_REQUIRE(out_stride >= (long)nh * vd && (!gate || gate_stride >= nh), "attn_masked: output stride %ld or gate stride %ld "
             "too small for %d heads of %d", out_stride, gate_stride, nh, vd);
  dim3 grid(tokens, (nh + kMaskedWaves - 1) / kMaskedWaves);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32) {
    hipLaunchKernelGGL(attn_masked_kernel<float>, grid, dim3(kMaskedWaves * kWave), 0, st, (const float*)q,
                       (const float*)k_cache, (const float*)v_cache, block_table, table_stride, seq_of_token, positions,
                       (float*)out, (size_t)out_stride, nh, nkv, hd, vd, page_size, window, keep_first, scale, softcap, slopes,
                       sink, (const float*)gate, (size_t)gate_stride, out_scale);
  } else if (dtype == kBF16) {
    hipLaunchKernelGGL(attn_masked_kernel<bf16>, grid, dim3(kMaskedWaves * kWave), 0, st, (const bf16*)q,
                       (const bf16*)k_cache, (const bf16*)v_cache, block_table, table_stride, seq_of_token, positions,
                       (bf16*)out, (size_t)out_stride, nh, nkv, hd, vd, page_size, window, keep_first, scale, softcap, slopes,
                       sink, (const bf16*)gate, (size_t)gate_stride, out_scale);
  } else {
    return pa::fail("attn_masked: unknown element type code %d", dtype);
  }
  return check_launch("attn_masked");
}

extern "C" int pa_qkv_prepare(void* stream, int dtype, const void* p, long stride, int q_off, int k_off, int v_off,
                              const float* qw, const float* kw, const int* slots, void* q_out, void* k_cache, void* v_cache,
                              int tokens, int nh, int nkv, int hd, int vd, int page_size, float eps) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && nh > 0 && hd > 0 && p && q_out, "qkv_prepare: bad sizes tokens=%d nh=%d hd=%d", tokens, nh, hd);
  PA_REQUIRE(q_off >= 0 && q_off + (long)nh * hd <= stride, "qkv_prepare: the queries do not fit the row of %ld", stride);
  if (slots) {
    PA_REQUIRE(nkv > 0 && vd > 0 && page_size > 0 && k_cache && v_cache, "qkv_prepare: bad sizes nkv=%d vd=%d page=%d", nkv, vd,
               page_size);
    PA_REQUIRE(k_off >= 0 && k_off + (long)nkv * hd <= stride && v_off >= 0 && v_off + (long)nkv * vd <= stride,
               "qkv_prepare: keys or values do not fit the row of %ld", stride);
  }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32)
    hipLaunchKernelGGL(qkv_prepare_kernel<float>, dim3(tokens), dim3(256), 0, st, (const float*)p, (size_t)stride, q_off, k_off,
                       v_off, qw, kw, slots, (float*)q_out, (float*)k_cache, (float*)v_cache, nh, nkv, hd, vd, page_size, eps);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(qkv_prepare_kernel<bf16>, dim3(tokens), dim3(256), 0, st, (const bf16*)p, (size_t)stride, q_off, k_off,
                       v_off, qw, kw, slots, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, nh, nkv, hd, vd, page_size, eps);
  else
    return pa::fail("qkv_prepare: unknown element type code %d", dtype);
  return check_launch("qkv_prepare");
}
