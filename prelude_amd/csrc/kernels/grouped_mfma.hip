// Products with a weight per group of rows, on the matrix cores (bfloat16, 32-bit sums): the experts' products
// (group = expert, rows = the step's entries in expert order) and the per-head maps of attention through a latent
// (group = head, rows = tokens).
//
// y[row, n] = sum_k x[row, k] * w[group, n, k], the weight as stored ([out, in], in fastest).  A workgroup of four
// wavefronts owns up to 64 rows of one group and 256 (or 128) outputs: each wavefront four (two) tiles of 16 outputs against the
// four tiles of 16 rows, W^T tile as A (row = output), X^T as B (column = row of x), both straight from memory in
// 16-byte pieces (v_mfma_f32_16x16x32_bf16: A row r, columns 8g..8g+7; B column r, rows 8g..8g+7; C column r,
// rows 4g..4g+3).  A weight element is read once per 64 rows, and sums run over k in ascending steps of 32
// whatever else the launch holds.
#include "common.h"
#include "api.h"

namespace pa {

constexpr int kGmRows = 64;
// tiles of 16 outputs a wavefront: four where there are rows enough to reuse them (a workgroup then owns 256 outputs),
// two for the few rows of a step of single tokens, where what counts is how many workgroups stream the weights (128)

// xrow(m) / yrow(m): element offsets of row m's input and output, < 0 for a row that does not exist.
template <typename TY, int NT, typename RowX, typename RowY>
__device__ __forceinline__ void grouped_tile(const bf16* __restrict__ x, const bf16* __restrict__ w, TY* __restrict__ y,
                                             int K, int N, int n_rows, int n0, int act, float limit, float alpha, RowX xrow, RowY yrow) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  const int row_tiles = (n_rows + 15) / 16;
  // Every load is unconditional (rows, outputs and the last step of k that do not exist are clamped to ones that do:
  // loads under branches are waited for one by one); what a clamped row or output brings is never stored, and the
  // one thing that must not count, a step past the end of k, is zeroed on the x side by a select.
  const bf16* xr[4];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) xr[mt] = x + xrow(mt * 16 + r < n_rows ? mt * 16 + r : 0) + 8 * g;
  const int nb = n0 + wave * 16 * NT;
  if (nb >= N) return;
  const bf16* wr[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n = nb + 16 * j + r;
    wr[j] = w + (size_t)(n < N ? n : N - 1) * K + 8 * g;
  }
  f32x4 acc[NT][4];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) acc[j][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  // The operands of the three steps after this one are on their way while this step is multiplied, in four sets of
  // registers named by constants (the loop takes four steps a turn): with few rows a workgroup is one chain of steps
  // through its slice of the weight, a step's loads take some ten times as long as its products, and what streams
  // the weight at the memory's rate is how much of it is in flight.
  bf16x8 wf[4][NT], xf[4][4];
  const int last_k0 = ((K - 1) / 32) * 32;
  auto load_step = [&](int k0, int b) {
    k0 = k0 <= last_k0 ? k0 : last_k0;                           // (past the end: the last step once more, not multiplied)
    const bool kok = k0 + 8 * g + 8 <= K;
    const int kc = kok ? k0 : K - 8 - 8 * g;                    // (K is a multiple of 8: the clamped piece lies inside the row)
#pragma unroll
    for (int j = 0; j < NT; ++j) wf[b][j] = *reinterpret_cast<const bf16x8*>(wr[j] + kc);
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      if (mt < row_tiles) {                                      // (the same in every lane of the workgroup)
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(xr[mt] + kc);
        xf[b][mt] = kok ? v : bf16x8{};
      }
    }
  };
  auto multiply = [&](int k0, int b) {
    if (k0 >= K) return;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      if (mt < row_tiles) {
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[j][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[b][j], xf[b][mt], acc[j][mt], 0, 0, 0);
      }
    }
  };
  load_step(0, 0);
  load_step(32, 1);
  load_step(64, 2);
  for (int k0 = 0; k0 < K; k0 += 128) {
    load_step(k0 + 96, 3);
    multiply(k0, 0);
    load_step(k0 + 128, 0);
    multiply(k0 + 32, 1);
    load_step(k0 + 160, 1);
    multiply(k0 + 64, 2);
    load_step(k0 + 192, 2);
    multiply(k0 + 96, 3);
  }
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    if (mt * 16 + r >= n_rows) continue;
    const long yo = yrow(mt * 16 + r);
    if (yo < 0) continue;
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = nb + 16 * j + 4 * g + i;
        if (n < N) {
          float v = acc[j][mt][i];
          if (act >= 2) {   // a lane's four outputs are two (gate, up) pairs: one output a pair, rows of N / 2
            if ((i & 1) == 0)
              y[yo + n / 2] = from_f32<TY>(act == 2 ? clamped_gate(v, acc[j][mt][i | 1], limit, alpha)
                                                    : gate_activation(v, kActSilu) * acc[j][mt][i | 1]);
            continue;
          }
          if (act == 1) {
            v = fmaxf(v, 0.f);
            v = v * v;
          }
          y[yo + n] = from_f32<TY>(v);
        }
      }
  }
}

// Which expert a tile belongs to: an expert with c entries has ceil(c / rows) tiles, the tiles of all experts are
// numbered in order.  Every lane takes an expert (64 at a time), the tiles are summed across the wavefront, and the
// first expert whose running total passes `tile` is the one: no chain of dependent loads over the experts.
// Returns false for a tile beyond the last.  All lanes of a wavefront call it with the same arguments.
__device__ __forceinline__ bool find_tile(const int* __restrict__ offsets, int experts, int rows, int tile, int& e_out,
                                          int& p0, int& p1) {
  const int lane = threadIdx.x % kWave;
  int before = 0;                                              // tiles of the experts of earlier rounds
  for (int base = 0; base < experts; base += kWave) {
    const int e = base + lane;
    int a = 0, b = 0;
    if (e < experts) {
      a = offsets[e];
      b = offsets[e + 1];
    }
    const int mine = (b - a + rows - 1) / rows;
    int incl = mine;                                           // inclusive running total over the lanes
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int up = __shfl_up(incl, d, kWave);
      if (lane >= d) incl += up;
    }
    const unsigned long long hit = __ballot(before + incl > tile);
    if (hit) {
      const int src = __ffsll((long long)hit) - 1;
      const int first = tile - (before + __shfl(incl, src, kWave) - __shfl(mine, src, kWave));   // tile within its expert
      const int ea = __shfl(a, src, kWave), eb = __shfl(b, src, kWave);
      e_out = base + src;
      p0 = ea + first * rows;
      p1 = p0 + rows < eb ? p0 + rows : eb;
      return true;
    }
    before += __shfl(incl, kWave - 1, kWave);
  }
  return false;
}

// Experts: blockIdx.x walks the tiles of 64 positions of all experts in order (an expert with c entries has
// ceil(c / 64) tiles; blocks beyond the last leave).  `from_tokens`: position p reads row order[p] / top of x.
template <typename TY, int NT>
__global__ __launch_bounds__(256) void moe_linear_mfma_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                             TY* __restrict__ y, const int* __restrict__ offsets,
                                                             const int* __restrict__ order, int entries, int experts,
                                                             int top, int K, int N, int col_chunks, int from_tokens, int act,
                                                             float limit, float alpha) {
  // The launch is a line of workgroups that the hardware deals out to the eight XCDs in turn (each with an L2 of
  // its own); work item w = (chunk of outputs, tile of positions), tiles fastest, and every XCD is given one stretch
  // of the items: the tiles of one expert against one chunk of its weight then run on one XCD one after the other,
  // and the chunk comes from memory once instead of once a tile.
  const int tiles_max = (entries + kGmRows - 1) / kGmRows + experts;
  const int total = tiles_max * col_chunks;
  const int per_xcd = (total + 7) / 8;
  const int item = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
  if (blockIdx.x / 8 >= (unsigned)per_xcd || item >= total) return;
  int e = 0, p0 = 0, p1 = 0;
  const int col_chunk = item / tiles_max;
  if (!find_tile(offsets, experts, kGmRows, item % tiles_max, e, p0, p1)) return;
  grouped_tile<TY, NT>(x, w + (size_t)e * N * K, y, K, N, p1 - p0, col_chunk * 64 * NT, act, limit, alpha,
                   [&](int m) { return (long)(from_tokens ? order[p0 + m] / top : p0 + m) * K; },
                   [&](int m) { return (long)(p0 + m) * (act >= 2 ? N / 2 : N); });
}

// The experts' product for many rows: a workgroup owns 128 positions of one expert and 128 outputs.  What limits
// the kernel above at many rows is the bytes that travel from the L2 to the compute units (every wavefront loads
// the rows of x for itself): here the 128 rows of x go through LDS once per workgroup (16-byte pieces, held in
// registers while the step before is multiplied, two buffers, rows padded to 80 bytes), the weight still straight
// from memory, a step ahead: 16 KB a step of k for the same products as the 32 KB above.
constexpr int kGbRows = 128;
constexpr int kGbStride = 40;   // elements of an LDS row: 32 of a step and 8 of padding

template <typename TY>
__global__ __launch_bounds__(256) void moe_linear_mfma_big_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                                 TY* __restrict__ y, const int* __restrict__ offsets,
                                                                 const int* __restrict__ order, int entries, int experts,
                                                                 int top, int K, int N, int col_chunks, int from_tokens,
                                                                 int act, float limit, float alpha) {
  __shared__ __attribute__((aligned(16))) bf16 xs[2][kGbRows * kGbStride];
  const int tiles_max = (entries + kGbRows - 1) / kGbRows + experts;
  const int total = tiles_max * col_chunks;
  const int per_xcd = (total + 7) / 8;
  const int item = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
  if (blockIdx.x / 8 >= (unsigned)per_xcd || item >= total) return;
  int e = 0, p0 = 0, p1 = 0;
  const int col_chunk = item / tiles_max;
  if (!find_tile(offsets, experts, kGbRows, item % tiles_max, e, p0, p1)) return;
  const int n_rows = p1 - p0;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  const int row_tiles = (n_rows + 15) / 16;
  const bf16* we = w + (size_t)e * N * K;
  constexpr int NT = 2;                                        // 32 outputs a wavefront: registers for three workgroups a compute unit
  const int nb = col_chunk * 64 * NT + wave * 16 * NT;                  // (a wavefront whose outputs do not exist still stages x)
  const bool cols_ok = nb < N;
  const bf16* wr[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n = nb + 16 * j + r;
    wr[j] = we + (size_t)(n < N ? n : N - 1) * K + 8 * g;
  }
  // this thread's two pieces of a step's x tile: piece c = thread + 256 i is row c / 4, elements 8 (c % 4)...
  const bf16* xsrc[2];
  int xdst[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = threadIdx.x + 256 * i;
    const int m = c / 4 < n_rows ? c / 4 : 0;
    const long row = from_tokens ? order[p0 + m] / top : p0 + m;
    xsrc[i] = x + row * K + 8 * (c % 4);
    xdst[i] = (c / 4) * kGbStride + 8 * (c % 4);
  }
  f32x4 acc[NT][8];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) acc[j][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  bf16x8 wf[2][NT], xreg[2];
  auto load_step = [&](int k0, int b) {                        // unconditional, clamped; a piece past the end of k is zeroed in x
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int kc = k0 + 8 * g + 8 <= K ? k0 : K - 8 - 8 * g;
      wf[b][j] = *reinterpret_cast<const bf16x8*>(wr[j] + kc);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int piece = (threadIdx.x + 256 * i) % 4;
      const bool kok = k0 + 8 * piece + 8 <= K;
      const bf16x8 v = *reinterpret_cast<const bf16x8*>(xsrc[i] + (kok ? k0 : K - 8 - 8 * piece));
      xreg[i] = kok ? v : bf16x8{};
    }
  };
  auto stage = [&](int b) {
#pragma unroll
    for (int i = 0; i < 2; ++i) *reinterpret_cast<bf16x8*>(&xs[b][xdst[i]]) = xreg[i];
  };
  // (the two sets of registers and the two buffers are named by constants, the loop taking two steps a turn: an
  // index that is only known at run time would send the register arrays to memory)
  auto multiply = [&](int b) {
    if (!cols_ok) return;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      bf16x8 xf[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) xf[q] = *reinterpret_cast<const bf16x8*>(&xs[b][((4 * half + q) * 16 + r) * kGbStride + 8 * g]);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (4 * half + q < row_tiles) {
#pragma unroll
          for (int j = 0; j < NT; ++j)
            acc[j][4 * half + q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[b][j], xf[q], acc[j][4 * half + q], 0, 0, 0);
        }
      }
    }
  };
  load_step(0, 0);
  stage(0);
  __syncthreads();
  for (int k0 = 0; k0 < K; k0 += 64) {
    // step k0 from set 0 while step k0 + 32 arrives in set 1, then the other way round
    const bool more1 = k0 + 32 < K;
    if (more1) load_step(k0 + 32, 1);
    multiply(0);
    if (more1) stage(1);                                       // (everyone left that buffer at the barrier before this step)
    __syncthreads();
    if (!more1) break;
    const bool more0 = k0 + 64 < K;
    if (more0) load_step(k0 + 64, 0);
    multiply(1);
    if (more0) stage(0);
    __syncthreads();
  }
  if (!cols_ok) return;
#pragma unroll
  for (int mt = 0; mt < 8; ++mt) {
    if (mt * 16 + r >= n_rows) continue;
    TY* yr = y + (size_t)(p0 + mt * 16 + r) * (act >= 2 ? N / 2 : N);
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = nb + 16 * j + 4 * g + i;
        if (n < N) {
          float v = acc[j][mt][i];
          if (act >= 2) {
            if ((i & 1) == 0)
              yr[n / 2] = from_f32<TY>(act == 2 ? clamped_gate(v, acc[j][mt][i | 1], limit, alpha)
                                                : gate_activation(v, kActSilu) * acc[j][mt][i | 1]);
            continue;
          }
          if (act == 1) {
            v = fmaxf(v, 0.f);
            v = v * v;
          }
          yr[n] = from_f32<TY>(v);
        }
      }
  }
}

// Heads: grid (tiles of 64 tokens, heads, chunks of 64 NT outputs).
template <int NT>
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                              bf16* __restrict__ y, int tokens, int K, int N, long xs_t,
                                                              long xs_h, long ys_t, long ys_h) {
  const int t0 = blockIdx.x * kGmRows, h = blockIdx.y;
  const int n_rows = tokens - t0 < kGmRows ? tokens - t0 : kGmRows;
  grouped_tile<bf16, NT>(x, w + (size_t)h * N * K, y, K, N, n_rows, blockIdx.z * 64 * NT, 0, 0.f, 0.f,
                     [&](int m) { return (long)(t0 + m) * xs_t + (long)h * xs_h; },
                     [&](int m) { return (long)(t0 + m) * ys_t + (long)h * ys_h; });
}

}  // namespace pa

using namespace pa;

// x [rows, K] bfloat16 (a row per token when from_tokens, else per position), w [experts, N, K] bfloat16,
// y [entries, N] of y_dtype; K a multiple of 8.
extern "C" int pa_moe_linear_mfma(void* stream, int y_dtype, const void* x, const void* w, void* y, const int* offsets,
                                  const int* order, int entries, int experts, int top, int K, int N, int from_tokens, int act,
                                  float limit, float alpha) {
  if (entries == 0) return 0;
  PA_REQUIRE(entries > 0 && experts > 0 && top > 0 && K > 0 && N > 0 && K % 8 == 0, "moe_linear_mfma: bad sizes entries=%d experts=%d k=%d n=%d",
             entries, experts, K, N);
  PA_REQUIRE(act >= 0 && act <= 3, "moe_linear_mfma: unknown activation code %d", act);
  PA_REQUIRE(act < 2 || N % 2 == 0, "moe_linear_mfma: gated pairs need an even number of outputs");
  PA_REQUIRE(act != 2 || limit > 0.f, "moe_linear_mfma: clamped gated pairs need a clamp > 0");
  const bool few = entries <= 4 * kGmRows;
  const int cols = 128;
  const int col_chunks = (N + cols - 1) / cols;
  hipStream_t st = (hipStream_t)stream;
  if (!few) {
    // many rows: tiles of 128 positions with the rows of x through LDS
    const long items = (long)((entries + kGbRows - 1) / kGbRows + experts) * col_chunks;
    PA_REQUIRE(items <= 0x7fffff00L, "moe_linear_mfma: %ld work items exceed the grid", items);
    dim3 grid((unsigned)(((items + 7) / 8) * 8));
    if (y_dtype == kBF16)
      hipLaunchKernelGGL(moe_linear_mfma_big_kernel<bf16>, grid, dim3(256), 0, st, (const bf16*)x, (const bf16*)w, (bf16*)y, offsets,
                         order, entries, experts, top, K, N, col_chunks, from_tokens, act, limit, alpha);
    else if (y_dtype == kF32)
      hipLaunchKernelGGL(moe_linear_mfma_big_kernel<float>, grid, dim3(256), 0, st, (const bf16*)x, (const bf16*)w, (float*)y, offsets,
                         order, entries, experts, top, K, N, col_chunks, from_tokens, act, limit, alpha);
    else
      return pa::fail("moe_linear_mfma: unknown output type code %d", y_dtype);
    return check_launch("moe_linear_mfma");
  }
  const long items = (long)((entries + kGmRows - 1) / kGmRows + experts) * col_chunks;
  PA_REQUIRE(items <= 0x7fffff00L, "moe_linear_mfma: %ld work items exceed the grid", items);
  dim3 grid((unsigned)(((items + 7) / 8) * 8));
#define PA_GM(TY, NT)                                                                                                       \
  hipLaunchKernelGGL((moe_linear_mfma_kernel<TY, NT>), grid, dim3(256), 0, st, (const bf16*)x, (const bf16*)w, (TY*)y, offsets, \
                     order, entries, experts, top, K, N, col_chunks, from_tokens, act, limit, alpha)
  if (y_dtype == kBF16) {
    PA_GM(bf16, 2);
  } else if (y_dtype == kF32) {
    PA_GM(float, 2);
  } else {
    return pa::fail("moe_linear_mfma: unknown output type code %d", y_dtype);
  }
#undef PA_GM
  return check_launch("moe_linear_mfma");
}

// y[t, h, n] = sum_k x[t, h, k] w[h, n, k]; strides in elements, multiples of 8 (16-byte pieces), K a multiple of 8.
extern "C" int pa_head_linear_mfma(void* stream, const void* x, const void* w, void* y, int tokens, int heads, int K, int N,
                                   long xs_t, long xs_h, long ys_t, long ys_h) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && heads > 0 && K > 0 && N > 0 && K % 8 == 0 && xs_t % 8 == 0 && xs_h % 8 == 0,
             "head_linear_mfma: bad sizes tokens=%d heads=%d k=%d n=%d strides %ld %ld", tokens, heads, K, N, xs_t, xs_h);
  PA_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0, "head_linear_mfma: operands are not 16-byte aligned");
  const bool few = tokens <= kGmRows;
  const int cols = few ? 128 : 256;
  PA_REQUIRE(heads <= 65535 && (N + cols - 1) / cols <= 65535, "head_linear_mfma: %d heads or %d outputs exceed the grid", heads, N);
  dim3 grid((tokens + kGmRows - 1) / kGmRows, heads, (N + cols - 1) / cols);
  if (few)
    hipLaunchKernelGGL(head_linear_mfma_kernel<2>, grid, dim3(256), 0, (hipStream_t)stream, (const bf16*)x, (const bf16*)w, (bf16*)y,
                       tokens, K, N, xs_t, xs_h, ys_t, ys_h);
  else
    hipLaunchKernelGGL(head_linear_mfma_kernel<4>, grid, dim3(256), 0, (hipStream_t)stream, (const bf16*)x, (const bf16*)w, (bf16*)y,
                       tokens, K, N, xs_t, xs_h, ys_t, ys_h);
  return check_launch("head_linear_mfma");
}
