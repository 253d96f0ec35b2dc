// Row-wise kernels whose statistics are taken over parts of a row: the RMS norm in groups around a 32-bit stream,
// the polynomial activation whose three powers are each brought to unit RMS, and the per-head norm with a gate that
// follows a recurrent mixer.  All arithmetic is 32-bit; the order of every sum follows the thread layout alone, so a
// row's result never depends on what else the launch holds.
#include "common.h"
#include "api.h"

namespace pa {

constexpr int kRowThreads = 256;

// Sum of squares of part `g` (elements [g * len, (g + 1) * len)) of a row held in LDS.
__device__ __forceinline__ float part_square_sum(const float* row, int g, int len, float* scratch) {
  float ss = 0.f;
  for (int i = threadIdx.x; i < len; i += blockDim.x) {
    const float v = row[g * len + i];
    ss += v * v;
  }
  return block_sum(ss, scratch);
}

// One step around a stream kept in 32-bit, a workgroup a row:
//   with y:      residual[r] += norm_g(y[r]) * w_add        (a branch's output normed in groups and added)
//   with out:    out[r] = norm_g(residual[row]) * w_out     (the next branch's input, in the engine's type)
// norm_g: the row in `groups` equal consecutive parts, each over its own sqrt(mean(part^2) + eps).
// `rows` (only without y): output row r is the norm of residual row rows[r].
template <typename T>
__global__ __launch_bounds__(kRowThreads) void group_norm_step_kernel(
    const T* __restrict__ y, const float* __restrict__ w_add, float* __restrict__ residual,
    const float* __restrict__ w_out, T* __restrict__ out, const int* __restrict__ rows, int hidden, int groups, float eps) {
  extern __shared__ float row[];
  __shared__ float scratch[16];
  __shared__ float inv[64];
  const size_t r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : r;
  const int len = hidden / groups;
  float* res = residual + src * hidden;
  if (y) {
    const T* yr = y + r * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) row[i] = to_f32(yr[i]);
    __syncthreads();
    for (int g0 = 0; g0 < groups; g0 += 64) {
      const int n = groups - g0 < 64 ? groups - g0 : 64;
      for (int g = 0; g < n; ++g) {
        const float ss = part_square_sum(row, g0 + g, len, scratch);
        if (threadIdx.x == 0) inv[g] = 1.0f / sqrtf(ss / (float)len + eps);
      }
      __syncthreads();
      for (int i = g0 * len + threadIdx.x; i < (g0 + n) * len; i += blockDim.x) {
        const float v = res[i] + row[i] * inv[i / len - g0] * w_add[i];
        res[i] = v;
        row[i] = v;
      }
      __syncthreads();
    }
  } else if (out) {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) row[i] = res[i];
    __syncthreads();
  }
  if (!out) return;
  T* dst = out + r * hidden;
  for (int g0 = 0; g0 < groups; g0 += 64) {
    const int n = groups - g0 < 64 ? groups - g0 : 64;
    for (int g = 0; g < n; ++g) {
      const float ss = part_square_sum(row, g0 + g, len, scratch);
      if (threadIdx.x == 0) inv[g] = 1.0f / sqrtf(ss / (float)len + eps);
    }
    __syncthreads();
    for (int i = g0 * len + threadIdx.x; i < (g0 + n) * len; i += blockDim.x)
      dst[i] = from_f32<T>(row[i] * inv[i / len - g0] * w_out[i]);
    __syncthreads();
  }
}

// Eight consecutive elements of a row as 32-bit values, in 16-byte loads and stores.
__device__ __forceinline__ void load8(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16* p, float* v) {
  const bf16x8 a = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (float)a[i];
}
__device__ __forceinline__ void store8(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
  *reinterpret_cast<float4*>(p + 4) = float4{v[4], v[5], v[6], v[7]};
}
__device__ __forceinline__ void store8(bf16* p, const float* v) {
  bf16x8 a;
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = (bf16)v[i];
  *reinterpret_cast<bf16x8*>(p) = a;
}

// The same step for rows of up to 8 * 256 * VPT elements whose groups are whole pieces of eight: a thread keeps VPT
// pieces of the row in registers, and everything it will need (the branch, the stream, both weights) is asked for
// at once.  A wavefront's 64 pieces of one round are 512 consecutive elements; it sums the squares of each group
// that has pieces among them, and a group's sum is its wavefronts' sums added in their order: one barrier a norm.
template <typename T, int VPT>
__global__ __launch_bounds__(256) void group_norm_step_vec_kernel(
    const T* __restrict__ y, const float* __restrict__ w_add, float* __restrict__ residual,
    const float* __restrict__ w_out, T* __restrict__ out, const int* __restrict__ rows, int hidden, int groups, float eps) {
  __shared__ float partial[2][4 * VPT][64];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const size_t r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : r;
  const int len = hidden / groups;
  const int pieces = hidden / 8;
  float cur[VPT][8], yv[VPT][8], wa[VPT][8], wo[VPT][8];
  float* res = residual + src * hidden;
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int piece = v * 256 + threadIdx.x;
    if (piece < pieces) {
      load8(res + 8 * piece, cur[v]);
      if (y) {
        load8(y + r * hidden + 8 * piece, yv[v]);
        load8(w_add + 8 * piece, wa[v]);
      }
      if (out) load8(w_out + 8 * piece, wo[v]);
    }
  }
  // 1 / sqrt(mean^2 + eps) of the group of each of the thread's pieces of `vals`
  auto group_inv = [&](float (*vals)[8], float* inv, int buf) {
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
      const int piece = v * 256 + threadIdx.x;
      const bool on = piece < pieces;
      float ss = 0.f;
      if (on) {
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += vals[v][i] * vals[v][i];
      }
      const int e0 = (v * 4 + wave) * 512;          // the wavefront's first element of this round
      if (e0 < hidden) {
        const int e1 = (e0 + 512 < hidden ? e0 + 512 : hidden) - 1;
        const int glo = e0 / len, ghi = e1 / len;
        const int mine = on ? (8 * piece) / len : -1;
        for (int g = glo; g <= ghi; ++g) {
          const float s = wave_sum(mine == g ? ss : 0.f);
          if (lane == 0) partial[buf][v * 4 + wave][g - glo] = s;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
      const int piece = v * 256 + threadIdx.x;
      inv[v] = 0.f;
      if (piece < pieces) {
        const int g = (8 * piece) / len;
        float total = 0.f;
        for (int vw = (g * len) / 512; vw <= ((g + 1) * len - 1) / 512; ++vw) total += partial[buf][vw][g - (vw * 512) / len];
        inv[v] = 1.0f / sqrtf(total / (float)len + eps);
      }
    }
  };
  float inv[VPT];
  if (y) {
    group_inv(yv, inv, 0);
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
      const int piece = v * 256 + threadIdx.x;
      if (piece < pieces) {
#pragma unroll
        for (int i = 0; i < 8; ++i) cur[v][i] += yv[v][i] * inv[v] * wa[v][i];
        store8(res + 8 * piece, cur[v]);
      }
    }
  }
  if (!out) return;
  group_inv(cur, inv, 1);
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int piece = v * 256 + threadIdx.x;
    if (piece < pieces) {
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = cur[v][i] * inv[v] * wo[v][i];
      store8(out + r * hidden + 8 * piece, o);
    }
  }
}

// out = a N(z) + b N(z^2) + c N(z^3) + e over a row, z = x (+ bias), powers element by element, N(u) = u over
// sqrt(mean(u^2) + eps); coeff = (a, b, c, e) on the device.  A workgroup a row; the row is read twice.
template <typename T>
__global__ __launch_bounds__(kRowThreads) void poly_norm_kernel(const T* __restrict__ x, const float* __restrict__ bias,
                                                               const float* __restrict__ coeff, T* __restrict__ out,
                                                               int width, float eps) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  const T* xr = x + r * width;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float z = to_f32(xr[i]) + (bias ? bias[i] : 0.f);
    const float z2 = z * z;
    s2 += z2;
    s4 += z2 * z2;
    s6 += z2 * z2 * z2;
  }
  s2 = block_sum(s2, scratch);
  s4 = block_sum(s4, scratch);
  s6 = block_sum(s6, scratch);
  const float n = (float)width;
  const float a = coeff[0] / sqrtf(s2 / n + eps), b = coeff[1] / sqrtf(s4 / n + eps), c = coeff[2] / sqrtf(s6 / n + eps);
  const float e = coeff[3];
  T* dst = out + r * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float z = to_f32(xr[i]) + (bias ? bias[i] : 0.f);
    dst[i] = from_f32<T>(a * z + b * (z * z) + c * (z * z * z) + e);
  }
}

// The same for bfloat16 rows of a multiple of 8 up to 8 * 256 * VPT elements: a thread keeps its pieces of 8 elements
// (with the bias added, in 32-bit) in registers, so the row is read once, in 16-byte loads.
template <int VPT>
__global__ __launch_bounds__(256) void poly_norm_vec_kernel(const bf16* __restrict__ x, const float* __restrict__ bias,
                                                            const float* __restrict__ coeff, bf16* __restrict__ out, int width,
                                                            float eps) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  const bf16* xr = x + r * width;
  const int pieces = width / 8;
  float z[VPT][8];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int piece = v * 256 + threadIdx.x;
    if (piece < pieces) {
      const bf16x8 raw = *reinterpret_cast<const bf16x8*>(xr + 8 * piece);
      float4 b0{0.f, 0.f, 0.f, 0.f}, b1{0.f, 0.f, 0.f, 0.f};
      if (bias) {
        b0 = *reinterpret_cast<const float4*>(bias + 8 * piece);
        b1 = *reinterpret_cast<const float4*>(bias + 8 * piece + 4);
      }
      const float bb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        z[v][i] = (float)raw[i] + bb[i];
        const float z2 = z[v][i] * z[v][i];
        s2 += z2;
        s4 += z2 * z2;
        s6 += z2 * z2 * z2;
      }
    }
  }
  s2 = block_sum(s2, scratch);
  s4 = block_sum(s4, scratch);
  s6 = block_sum(s6, scratch);
  const float n = (float)width;
  const float a = coeff[0] / sqrtf(s2 / n + eps), b = coeff[1] / sqrtf(s4 / n + eps), c = coeff[2] / sqrtf(s6 / n + eps);
  const float e = coeff[3];
  bf16* dst = out + r * width;
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int piece = v * 256 + threadIdx.x;
    if (piece < pieces) {
      bf16x8 o;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float zz = z[v][i];
        o[i] = (bf16)(a * zz + b * (zz * zz) + c * (zz * zz * zz) + e);
      }
      *reinterpret_cast<bf16x8*>(dst + 8 * piece) = o;
    }
  }
}

// A wavefront a (row, head): out[r, h, :] = o[r, h, :] / sqrt(mean(o[r, h, :]^2) + eps) * w * act(gate[r, h, :]) * scale.
// w (or null: no weight) has `vdim` elements shared by the heads; gate act: 0 sigmoid(g), 1 g * sigmoid(g).
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                            size_t gate_stride, const float* __restrict__ w,
                                                            T* __restrict__ out, size_t out_stride, int nrows, int heads,
                                                            int vdim, float eps, int act, float scale) {
  const int lane = threadIdx.x % kWave;
  const size_t item = (size_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= (size_t)nrows * heads) return;
  const size_t r = item / heads;
  const int h = (int)(item % heads);
  const float* src = o + (r * heads + h) * vdim;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += kWave) ss += src[i] * src[i];
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
  const T* g = gate + r * gate_stride + (size_t)h * vdim;
  T* dst = out + r * out_stride + (size_t)h * vdim;
  for (int i = lane; i < vdim; i += kWave) {
    const float gv = to_f32(g[i]);
    const float sg = 1.0f / (1.0f + expf(-gv));
    dst[i] = from_f32<T>(src[i] * inv * (w ? w[i] : 1.0f) * (act == 1 ? gv * sg : sg) * scale);
  }
}

}  // namespace pa

using namespace pa;

extern "C" int pa_group_norm_step(void* stream, int dtype, const void* y, const float* w_add, float* residual,
                                  const float* w_out, void* out, const int* rows, int nrows, int hidden, int groups,
                                  float eps) {
  if (nrows == 0) return 0;
  PA_REQUIRE(nrows > 0 && hidden > 0 && groups > 0 && hidden % groups == 0,
             "group_norm_step: bad sizes rows=%d hidden=%d groups=%d (the groups must divide the row)", nrows, hidden, groups);
  PA_REQUIRE(hidden <= 16384, "group_norm_step: rows of %d elements are more than the 16384 the kernel takes", hidden);
  PA_REQUIRE(residual && (y || out), "group_norm_step: needs the stream and a branch to add or an output to write");
  PA_REQUIRE(!y || w_add, "group_norm_step: a branch to add needs its norm's weight");
  PA_REQUIRE(!out || w_out, "group_norm_step: an output needs its norm's weight");
  PA_REQUIRE(!(y && rows), "group_norm_step: rows are chosen only where nothing is added");
  hipStream_t st = (hipStream_t)stream;
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if ((dtype == kF32 || dtype == kBF16) && hidden % 8 == 0 && (hidden / groups) % 8 == 0 && hidden <= 8 * 256 * 4 && aligned(y) &&
      aligned(w_add) && aligned(residual) && aligned(w_out) && aligned(out)) {
    const int vpt = (hidden / 8 + 255) / 256;
#define PA_GNORM(T, V) hipLaunchKernelGGL((group_norm_step_vec_kernel<T, V>), dim3(nrows), dim3(256), 0, st, (const T*)y, w_add, \
                                          residual, w_out, (T*)out, rows, hidden, groups, eps)
    if (dtype == kF32) {
      if (vpt <= 1) PA_GNORM(float, 1);
      else if (vpt <= 2) PA_GNORM(float, 2);
      else PA_GNORM(float, 4);
    } else {
      if (vpt <= 1) PA_GNORM(bf16, 1);
      else if (vpt <= 2) PA_GNORM(bf16, 2);
      else PA_GNORM(bf16, 4);
    }
#undef PA_GNORM
    return check_launch("group_norm_step");
  }
  const size_t lds = (size_t)hidden * sizeof(float);
  if (dtype == kF32)
    hipLaunchKernelGGL(group_norm_step_kernel<float>, dim3(nrows), dim3(kRowThreads), lds, st, (const float*)y, w_add, residual,
                       w_out, (float*)out, rows, hidden, groups, eps);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(group_norm_step_kernel<bf16>, dim3(nrows), dim3(kRowThreads), lds, st, (const bf16*)y, w_add, residual,
                       w_out, (bf16*)out, rows, hidden, groups, eps);
  else
    return pa::fail("group_norm_step: unknown element type code %d", dtype);
  return check_launch("group_norm_step");
}

extern "C" int pa_poly_norm(void* stream, int dtype, const void* x, const float* bias, const float* coeff, void* out,
                            int nrows, int width, float eps) {
  if (nrows == 0) return 0;
  PA_REQUIRE(nrows > 0 && width > 0 && x && coeff && out, "poly_norm: bad sizes rows=%d width=%d or a null operand", nrows, width);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32)
    hipLaunchKernelGGL(poly_norm_kernel<float>, dim3(nrows), dim3(kRowThreads), 0, st, (const float*)x, bias, coeff,
                       (float*)out, width, eps);
  else if (dtype == kBF16 && width % 8 == 0 && width <= 8 * 256 * 8 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
           (reinterpret_cast<uintptr_t>(out) & 15) == 0 && (reinterpret_cast<uintptr_t>(bias) & 15) == 0) {
    const int vpt = (width / 8 + 255) / 256;
#define PA_POLY(V) hipLaunchKernelGGL(poly_norm_vec_kernel<V>, dim3(nrows), dim3(256), 0, st, (const bf16*)x, bias, coeff, (bf16*)out, width, eps)
    if (vpt <= 1) PA_POLY(1);
    else if (vpt <= 2) PA_POLY(2);
    else if (vpt <= 4) PA_POLY(4);
    else PA_POLY(8);
#undef PA_POLY
  } else if (dtype == kBF16)
    hipLaunchKernelGGL(poly_norm_kernel<bf16>, dim3(nrows), dim3(kRowThreads), 0, st, (const bf16*)x, bias, coeff, (bf16*)out,
                       width, eps);
  else
    return pa::fail("poly_norm: unknown element type code %d", dtype);
  return check_launch("poly_norm");
}

extern "C" int pa_head_norm_gate(void* stream, int dtype, const float* o, const void* gate, long gate_stride, const float* w,
                                 void* out, long out_stride, int nrows, int heads, int vdim, float eps, int act, float scale) {
  if (nrows == 0) return 0;
  PA_REQUIRE(nrows > 0 && heads > 0 && vdim > 0 && gate_stride >= (long)heads * vdim && out_stride >= (long)heads * vdim,
             "head_norm_gate: bad sizes rows=%d heads=%d vdim=%d gate stride=%ld out stride=%ld", nrows, heads, vdim,
             gate_stride, out_stride);
  PA_REQUIRE(act == 0 || act == 1, "head_norm_gate: gate activation code %d is not 0 (sigmoid) or 1 (silu)", act);
  hipStream_t st = (hipStream_t)stream;
  const long items = (long)nrows * heads;
  const int blocks = (int)((items + 3) / 4);
  if (dtype == kF32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, dim3(blocks), dim3(256), 0, st, o, (const float*)gate, (size_t)gate_stride,
                       w, (float*)out, (size_t)out_stride, nrows, heads, vdim, eps, act, scale);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16>, dim3(blocks), dim3(256), 0, st, o, (const bf16*)gate, (size_t)gate_stride, w,
                       (bf16*)out, (size_t)out_stride, nrows, heads, vdim, eps, act, scale);
  else
    return pa::fail("head_norm_gate: unknown element type code %d", dtype);
  return check_launch("head_norm_gate");
}
