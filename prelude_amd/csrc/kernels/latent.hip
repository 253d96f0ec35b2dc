// Attention through a latent: what a token leaves in the cache is one vector, the normed latent c of `rank`
// elements followed by `rot` elements of a rotated key part that all heads share.  A head's unrotated key is a
// linear map of c and so is its value, so the maps are moved to the query side: the query's unrotated part is
// taken through the key map's transpose (rank elements a head), scores are dot products with the cached vector
// itself, the weighted sum of cached latents (rank elements a head) is taken through the value map afterwards.
// All heads read the same keys: one "KV head" of width rank + rot whose value is its own first `rank` elements.
//
//   pa_latent_prep    the merged down projection's row [q_rank | rank | rot]: RMS norm of the query latent (out),
//                     RMS norm of c and rotation of the shared key part (into the paged cache; c a second time
//                     transposed, where the cache keeps that copy for the matrix-core kernel)
//   pa_rotate_pairs   rotation of a part of every head's vector by position, pairs (2i, 2i+1)
//   pa_head_linear    y[t, h, :] = W[h] x[t, h, :], a product per head
//   pa_latent_attn    causal softmax attention over the latent cache with a learned sink per head in the
//                     denominator; 32-bit arithmetic on the vector ALU, any sizes: the true 32-bit path and
//                     the sizes the matrix-core kernel does not take
//
// Rotation: the pair (u, v) = (x[2i], x[2i+1]) at position p becomes (u cos a - v sin a, v cos a + u sin a),
// a = float(p) * inv_freq[i] in 32-bit; the angles are computed here from the frequencies, so there is no table
// and no longest position.
#include "common.h"
#include "api.h"

namespace pa {

constexpr int kLatMaxDk = 1024;   // rank + rot
constexpr int kLatWaves = 4;

template <typename T>
__global__ __launch_bounds__(256) void latent_gather_kernel(const T* __restrict__ cache, const int* __restrict__ block_table,
                                                            int table_stride, const int* __restrict__ seq, const int* __restrict__ pos,
                                                            T* __restrict__ out, int rows, int rank, int width, int page_size) {
  const int i = blockIdx.x * 4 + threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (i >= rows) return;
  const int p = pos[i];
  const int page = block_table[(size_t)seq[i] * table_stride + p / page_size];
  const T* src = cache + ((size_t)page * page_size + p % page_size) * width;
  T* dst = out + (size_t)i * rank;
  if (sizeof(T) == 2 && rank % 8 == 0 && width % 8 == 0) {   // 16-byte pieces
    typedef T vec_t __attribute__((ext_vector_type(8)));
    for (int e = lane * 8; e < rank; e += kWave * 8) *reinterpret_cast<vec_t*>(dst + e) = *reinterpret_cast<const vec_t*>(src + e);
  } else {
    for (int e = lane; e < rank; e += kWave) dst[e] = src[e];
  }
}

// ---- prep ------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(const T* __restrict__ in, const float* __restrict__ wq,
                                                         const float* __restrict__ wc, const float* __restrict__ inv_freq,
                                                         const int* __restrict__ positions, const int* __restrict__ slots,
                                                         T* __restrict__ cq_out, T* __restrict__ cache,
                                                         T* __restrict__ cache_t, int page_size, int q_rank,
                                                         int rank, int rot, int rot_dims, float eps, size_t in_stride) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int width = q_rank + rank + rot;
  const T* row = in + (size_t)t * in_stride;   // the row may lie inside a wider one
  float sq = 0.f, sc = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
    const float v = to_f32(row[i]);
    sq += v * v;
  }
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float v = to_f32(row[q_rank + i]);
    sc += v * v;
  }
  sq = block_sum(sq, scratch);
  sc = block_sum(sc, scratch);
  if (cq_out) {
    const float inv = rsqrtf(sq / (float)q_rank + eps);
    T* o = cq_out + (size_t)t * q_rank;
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) o[i] = from_f32<T>(to_f32(row[i]) * inv * wq[i]);
  }
  if (!slots) return;
  const int slot = slots[t];
  if (slot < 0) return;
  T* dst = cache + (size_t)slot * (rank + rot);
  const float inv = rsqrtf(sc / (float)rank + eps);
  // the latent a second time, transposed ([page, element, offset]): the weighted sum's operand for the matrix cores
  T* dst_t = cache_t ? cache_t + (size_t)(slot / page_size) * rank * page_size + slot % page_size : nullptr;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const T v = from_f32<T>(to_f32(row[q_rank + i]) * inv * wc[i]);
    dst[i] = v;
    if (dst_t) dst_t[(size_t)i * page_size] = v;
  }
  const float p = (float)positions[t];
  const T* kr = row + q_rank + rank;
  for (int i = threadIdx.x; i < rot_dims / 2; i += blockDim.x) {
    float s, c;
    sincosf(p * inv_freq[i], &s, &c);
    const float u = to_f32(kr[2 * i]), v = to_f32(kr[2 * i + 1]);
    dst[rank + 2 * i] = from_f32<T>(u * c - v * s);
    dst[rank + 2 * i + 1] = from_f32<T>(v * c + u * s);
  }
  for (int i = rot_dims + threadIdx.x; i < rot; i += blockDim.x) dst[rank + i] = kr[i];
}

// ---- rotation of a part of every head ---------------------------------------
// in [T, heads, in_stride] -> out [T, heads, out_stride]: elements in_off .. in_off + width of a head go to
// out_off .., the first rot_dims of them rotated in pairs.
template <typename T>
__global__ void rotate_pairs_kernel(const T* __restrict__ in, T* __restrict__ out, const float* __restrict__ inv_freq,
                                    const int* __restrict__ positions, int heads, int in_stride, int in_off,
                                    int out_stride, int out_off, int width, int rot_dims) {
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  const int half = rot_dims / 2;
  const int per_head = half + (width - rot_dims);
  for (int e = threadIdx.x; e < heads * per_head; e += blockDim.x) {
    const int h = e / per_head, i = e % per_head;
    const T* src = in + ((size_t)t * heads + h) * in_stride + in_off;
    T* dst = out + ((size_t)t * heads + h) * out_stride + out_off;
    if (i < half) {
      float s, c;
      sincosf(p * inv_freq[i], &s, &c);
      const float u = to_f32(src[2 * i]), v = to_f32(src[2 * i + 1]);
      dst[2 * i] = from_f32<T>(u * c - v * s);
      dst[2 * i + 1] = from_f32<T>(v * c + u * s);
    } else {
      const int d = rot_dims + (i - half);
      dst[d] = src[d];
    }
  }
}

// ---- a product per head -------------------------------------------------------
// y[t, h, n] = sum_k x[t, h, k] * wt[h, k, n]; x rows x_stride_t / x_stride_h apart, y likewise.  The weight lies
// with n running fastest, so a thread's loads of its column join those of its neighbours.  32-bit sums in
// ascending k whatever the batch: a row's result does not depend on the other rows.
constexpr int kHlRows = 16;
constexpr int kHlChunk = 128;

template <typename T>
__global__ __launch_bounds__(256) void head_linear_kernel(const T* __restrict__ x, const T* __restrict__ wt,
                                                         T* __restrict__ y, int tokens, int K, int N, long xs_t, long xs_h,
                                                         long ys_t, long ys_h) {
  __shared__ float xs[kHlRows][kHlChunk];
  const int t0 = blockIdx.x * kHlRows, h = blockIdx.y;
  const int n = blockIdx.z * 256 + threadIdx.x;
  const T* w = wt + (size_t)h * K * N;
  float acc[kHlRows];
#pragma unroll
  for (int m = 0; m < kHlRows; ++m) acc[m] = 0.f;
  for (int k0 = 0; k0 < K; k0 += kHlChunk) {
    __syncthreads();
    for (int e = threadIdx.x; e < kHlRows * kHlChunk; e += 256) {
      const int m = e / kHlChunk, k = e % kHlChunk;
      const int t = t0 + m;
      xs[m][k] = (t < tokens && k0 + k < K) ? to_f32(x[(size_t)t * xs_t + (size_t)h * xs_h + k0 + k]) : 0.f;
    }
    __syncthreads();
    if (n < N) {
      const int kn = K - k0 < kHlChunk ? K - k0 : kHlChunk;
      for (int k = 0; k < kn; ++k) {
        const float wv = to_f32(w[(size_t)(k0 + k) * N + n]);
#pragma unroll
        for (int m = 0; m < kHlRows; ++m) acc[m] = fmaf(xs[m][k], wv, acc[m]);
      }
    }
  }
  if (n < N) {
#pragma unroll
    for (int m = 0; m < kHlRows; ++m) {
      const int t = t0 + m;
      if (t < tokens) y[(size_t)t * ys_t + (size_t)h * ys_h + n] = from_f32<T>(acc[m]);
    }
  }
}

// ---- attention over the latent cache, vector ALU ---------------------------------
// One wavefront per (query token, head).  Keys are walked in chunks of 64 anchored at absolute positions that
// are multiples of 64: the order of every sum follows from the query's position alone, so a token's result is
// the same bits in a whole prompt, in a portion and as a single decoded token, whatever pages hold its keys.
// The sink joins at the end as one more term of the denominator, exp(sink_h), that brings no value.
template <typename T>
__global__ __launch_bounds__(kLatWaves* kWave) void latent_attn_kernel(
    const T* __restrict__ q, const T* __restrict__ cache, const float* __restrict__ sink,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ seq_of_token,
    const int* __restrict__ positions, T* __restrict__ out, int nh, int rank, int rot, int page_size, int window,
    float scale) {
  __shared__ float qs[kLatWaves][kLatMaxDk];
  __shared__ float ps[kLatWaves][kWave];
  constexpr int kOut = kLatMaxDk / kWave;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int t = blockIdx.x;
  const int h = blockIdx.y * kLatWaves + wave;
  const bool active = h < nh;
  const int dk = rank + rot;
  const int pos = positions[t];
  const int seq = seq_of_token[t];
  const int hi = pos;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* table = block_table + (size_t)seq * table_stride;

  if (active) {
    const T* qr = q + ((size_t)t * nh + h) * dk;
    for (int d = lane; d < dk; d += kWave) qs[wave][d] = to_f32(qr[d]);
  }
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float o[kOut] = {};
  for (int c0 = (lo / kWave) * kWave; c0 <= hi; c0 += kWave) {
    const int c = c0 + lane;
    const bool valid = active && c >= lo && c <= hi;
    float s = -INFINITY;
    if (valid) {
      const int page = table[c / page_size];
      const T* kr = cache + ((size_t)page * page_size + (c % page_size)) * dk;
      float dot = 0.f;
      for (int d = 0; d < dk; ++d) dot = fmaf(qs[wave][d], to_f32(kr[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = active ? expf(m - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    ps[wave][lane] = p;
    __syncthreads();
#pragma unroll
    for (int e = 0; e < kOut; ++e) o[e] *= alpha;
    if (active) {
      const int j_lo = lo > c0 ? lo - c0 : 0;
      const int j_hi = hi - c0 < kWave - 1 ? hi - c0 : kWave - 1;
      for (int j = j_lo; j <= j_hi; ++j) {
        const int cj = c0 + j;
        const int page = table[cj / page_size];
        const T* vr = cache + ((size_t)page * page_size + (cj % page_size)) * dk;
        const float pj = ps[wave][j];
#pragma unroll
        for (int e = 0; e < kOut; ++e) {
          const int d = lane + e * kWave;
          if (d < rank) o[e] = fmaf(pj, to_f32(vr[d]), o[e]);
        }
      }
    }
    __syncthreads();
    m = m_new;
  }
  if (active) {
    if (sink) {
      const float sk = sink[h];
      const float m_new = fmaxf(m, sk);
      const float alpha = expf(m - m_new);
      l = l * alpha + expf(sk - m_new);
#pragma unroll
      for (int e = 0; e < kOut; ++e) o[e] *= alpha;
    }
    T* orow = out + ((size_t)t * nh + h) * rank;
    const float inv = 1.0f / l;
#pragma unroll
    for (int e = 0; e < kOut; ++e) {
      const int d = lane + e * kWave;
      if (d < rank) orow[d] = from_f32<T>(o[e] * inv);
    }
  }
}

}  // namespace pa

using namespace pa;

#define PA_BY_TYPE(dtype, what, ...)                                   \
  do {                                                                 \
    if ((dtype) == kF32) {                                             \
      typedef float T;                                                 \
      __VA_ARGS__;                                                     \
    } else if ((dtype) == kBF16) {                                     \
      typedef bf16 T;                                                  \
      __VA_ARGS__;                                                     \
    } else {                                                           \
      return pa::fail(what ": unknown element type code %d", (dtype)); \
    }                                                                  \
  } while (0)

extern "C" int pa_latent_prep(void* stream, int dtype, const void* in, const float* wq, const float* wc,
                              const float* inv_freq, const int* positions, const int* slots, void* cq_out, void* cache,
                              void* cache_t, int page_size, int tokens, int q_rank, int rank, int rot, int rot_dims, float eps,
                              long in_stride) {
  if (tokens == 0) return 0;
  if (in_stride <= 0) in_stride = q_rank + rank + rot;
  PA_REQUIRE(in_stride >= q_rank + rank + rot, "latent_prep: a row stride of %ld is less than the row", in_stride);
  PA_REQUIRE(tokens > 0 && q_rank > 0 && rank > 0 && rot >= 0, "latent_prep: bad sizes tokens=%d q_rank=%d rank=%d rot=%d",
             tokens, q_rank, rank, rot);
  PA_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, "latent_prep: %d rotated of %d is not an even part", rot_dims, rot);
  PA_REQUIRE(!slots || cache, "latent_prep: slots without a cache");
  PA_REQUIRE(!cache_t || page_size > 0, "latent_prep: a transposed copy needs the page size");
  PA_BY_TYPE(dtype, "latent_prep",
             hipLaunchKernelGGL(latent_prep_kernel<T>, dim3(tokens), dim3(256), 0, (hipStream_t)stream, (const T*)in, wq, wc,
                                inv_freq, positions, slots, (T*)cq_out, (T*)cache, (T*)cache_t, page_size, q_rank, rank, rot,
                                rot_dims, eps, (size_t)in_stride));
  return check_launch("latent_prep");
}

// out[i, :] = the first `rank` elements of the cached vector of (seq[i], pos[i]); a wavefront a row.
extern "C" int pa_latent_gather(void* stream, int dtype, const void* cache, const int* block_table, int table_stride, const int* seq,
                                const int* pos, void* out, int rows, int rank, int width, int page_size) {
  if (rows == 0) return 0;
  PA_REQUIRE(rows > 0 && rank > 0 && rank <= width && page_size > 0 && table_stride > 0, "latent_gather: bad sizes rows=%d rank=%d "
             "width=%d page=%d", rows, rank, width, page_size);
  PA_BY_TYPE(dtype, "latent_gather",
             hipLaunchKernelGGL(latent_gather_kernel<T>, dim3((rows + 3) / 4), dim3(256), 0, (hipStream_t)stream, (const T*)cache,
                                block_table, table_stride, seq, pos, (T*)out, rows, rank, width, page_size));
  return check_launch("latent_gather");
}

extern "C" int pa_rotate_pairs(void* stream, int dtype, const void* in, void* out, const float* inv_freq,
                               const int* positions, int tokens, int heads, int in_stride, int in_off, int out_stride,
                               int out_off, int width, int rot_dims) {
  if (tokens == 0 || width == 0) return 0;
  PA_REQUIRE(tokens > 0 && heads > 0 && width > 0 && rot_dims >= 0 && rot_dims <= width && rot_dims % 2 == 0,
             "rotate_pairs: bad sizes tokens=%d heads=%d width=%d rotated=%d", tokens, heads, width, rot_dims);
  PA_REQUIRE(in_off >= 0 && out_off >= 0 && in_off + width <= in_stride && out_off + width <= out_stride,
             "rotate_pairs: a part of %d at %d / %d does not fit heads of %d / %d", width, in_off, out_off, in_stride, out_stride);
  PA_BY_TYPE(dtype, "rotate_pairs",
             hipLaunchKernelGGL(rotate_pairs_kernel<T>, dim3(tokens), dim3(256), 0, (hipStream_t)stream, (const T*)in, (T*)out,
                                inv_freq, positions, heads, in_stride, in_off, out_stride, out_off, width, rot_dims));
  return check_launch("rotate_pairs");
}

extern "C" int pa_head_linear(void* stream, int dtype, const void* x, const void* wt, void* y, int tokens, int heads, int K,
                              int N, long xs_t, long xs_h, long ys_t, long ys_h) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && heads > 0 && K > 0 && N > 0, "head_linear: bad sizes tokens=%d heads=%d k=%d n=%d", tokens, heads, K, N);
  PA_REQUIRE(heads <= 65535 && (N + 255) / 256 <= 65535, "head_linear: %d heads or %d outputs exceed the grid", heads, N);
  dim3 grid((tokens + kHlRows - 1) / kHlRows, heads, (N + 255) / 256);
  PA_BY_TYPE(dtype, "head_linear",
             hipLaunchKernelGGL(head_linear_kernel<T>, grid, dim3(256), 0, (hipStream_t)stream, (const T*)x, (const T*)wt,
                                (T*)y, tokens, K, N, xs_t, xs_h, ys_t, ys_h));
  return check_launch("head_linear");
}

extern "C" int pa_latent_attn(void* stream, int dtype, const void* q, const void* cache, const float* sink,
                              const int* block_table, int table_stride, const int* seq_of_token, const int* positions,
                              void* out, int tokens, int nh, int rank, int rot, int page_size, int window, float scale) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && nh > 0 && page_size > 0 && table_stride > 0, "latent_attn: bad sizes tokens=%d heads=%d page=%d stride=%d",
             tokens, nh, page_size, table_stride);
  PA_REQUIRE(rank > 0 && rot >= 0 && rank + rot <= kLatMaxDk, "latent_attn: a latent of %d + %d is outside 1..%d", rank, rot, kLatMaxDk);
  PA_REQUIRE(window >= 0, "latent_attn: window %d is negative (0 means none)", window);
  dim3 grid(tokens, (nh + kLatWaves - 1) / kLatWaves);
  PA_BY_TYPE(dtype, "latent_attn",
             hipLaunchKernelGGL(latent_attn_kernel<T>, grid, dim3(kLatWaves * kWave), 0, (hipStream_t)stream, (const T*)q,
                                (const T*)cache, sink, block_table, table_stride, seq_of_token, positions, (T*)out, nh, rank,
                                rot, page_size, window, scale));
  return check_launch("latent_attn");
}
