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
//
// In bfloat16, with keys and values of 32, 64, 96 or 128 and pages of a power of two, the same attention runs on the
// matrix cores (`attn_masked_mfma_kernel` below), with the inner step of the plain matrix-core kernels: a wavefront
// owns 16 tokens of two heads that share a KV head (one when the group is odd) and walks, 32 keys a step, first the steps that hold kept
// first tokens and then the window's; a sequence that brings one token has its steps dealt out to the workgroup's
// wavefronts (eight where the whole step is single tokens), whose sums are merged through LDS.
#include "common.h"
#include "api.h"
#include "attention_mfma_core.h"

namespace pa {

constexpr int kMaskedWaves = 4;
constexpr int kMaskedMaxDim = 256;

template <typename T>
__global__ __launch_bounds__(kMaskedWaves* kWave) void attn_masked_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ seq_of_token,
    const int* __restrict__ positions, T* __restrict__ out, size_t out_stride, int nh, int nkv, int hd, int vd,
    int page_size, int window, int keep_first, float scale, float softcap, const float* __restrict__ slopes,
    const float* __restrict__ sink, const T* __restrict__ gate, size_t gate_stride, float out_scale, int nv) {
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
  const int vh = kvh % nv;   // fewer value heads than key heads: key head k goes with value head k mod nv
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
        const T* vr = v_cache + ((size_t)page * nv + vh) * vd * page_size + (cj % page_size);
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

// ---- on the matrix cores -------------------------------------------------------------------------------------------
// Keys [kept, lo) lie between the kept first tokens and the window and may have lost their pages: a K row or a chunk
// of V^T there is read from the last kept key's place (or from lo when nothing is kept), one past the end from the
// last key; the caller masks their scores.
template <int KD>
__device__ __forceinline__ void load_k_gap(const KeyWalk& w, int kept, int key0, int g, int r, KFrag<KD>& f) {
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    int key = key0 + 8 * (r / 4) + 4 * t + (r % 4);
    if (key >= w.hi) key = w.hi - 1;
    else if (key < w.lo && key >= kept) key = kept > 0 ? kept - 1 : w.lo;
    const int page = w.table[key >> w.page_shift];
    const bf16* row = w.kc + ((((size_t)page * w.nkv + w.kvh) << w.page_shift) + (key & w.page_mask)) * KD + 8 * g;
#pragma unroll
    for (int s = 0; s < KFrag<KD>::KS; ++s) f.k[t][s] = *reinterpret_cast<const bf16x8*>(row + 32 * s);
  }
}

// nv value heads in a page, of which this walk reads head vh (key head k goes with value head k mod nv).
template <int VD>
__device__ __forceinline__ VChunks v_chunks_gap(const KeyWalk& w, int kept, int key0, int g, int nv, int vh) {
  VChunks v;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    int c = key0 + 8 * g + 4 * t;  // first key of the chunk; a chunk that holds a visible key lies in a live page
    if (c >= w.hi) c = (w.hi - 1) & ~3;
    else if (c + 3 < w.lo && c >= kept) c = kept > 0 ? (kept - 1) & ~3 : w.lo & ~3;
    const int page = w.table[c >> w.page_shift];
    v.p[t] = w.vc + ((((size_t)page * nv + vh) * VD) << w.page_shift) + (c & w.page_mask);
  }
  v.joined = w.page_shift >= 3 && __all(v.p[1] == v.p[0] + 4);
  return v;
}

// One step over 32 keys for GT heads that share them, as attend32 of the plain kernels, with keys of KD and values of
// VD, and per head a bias `bias[j]` per key of distance (in the units of the raw scores) taken off the (capped) score.
template <int KD, int VD, int GT, typename Visible>
__device__ __forceinline__ void attend32_masked(const KeyWalk& w, int kept, int key0, int g, int r, const KFrag<KD>& kf,
                                                const bf16x8 (*qf)[KD / 32], const ScoreMap& sm, const float* bias, int my_pos,
                                                bool masked, HeadState<VD>* st, Visible vis, int nv, int vh) {
  constexpr int OT = VD / 16;
  const VChunks vch = v_chunks_gap<VD>(w, kept, key0, g, nv, vh);
  bf16x8 va[OT];
#pragma unroll
  for (int t = 0; t < OT; ++t) va[t] = load_v(vch, 16 * t + r, w.page_shift);
  bf16x8 pb[GT];
  const float c = sm.c;
  const float over = kLazyLog2 / c;
#pragma unroll
  for (int j = 0; j < GT; ++j) {
    float s[8];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      f32x4 acc{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KD / 32; ++ks) acc = mfma16(kf.k[t][ks], qf[j][ks], acc);
#pragma unroll
      for (int i = 0; i < 4; ++i) s[4 * t + i] = acc[i];
    }
    if (sm.cap != 0.f) {   // tanh(x) = 1 - 2 / (1 + e^(2x)), with the hardware's exponential and reciprocal
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float e2 = __builtin_amdgcn_exp2f(s[i] * sm.cap_in * (2.0f * kLog2e));
        s[i] = sm.cap - 2.0f * sm.cap * __builtin_amdgcn_rcpf(1.0f + e2);
      }
    }
    if (bias[j] != 0.f) {
      const float d0 = (float)(my_pos - (key0 + 8 * g));
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) s[4 * t + i] -= bias[j] * (d0 - (float)(4 * t + i));
    }
    if (masked) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (!vis(key0 + 8 * g + 4 * t + i)) s[4 * t + i] = -INFINITY;
    }
    float mx = s[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) mx = fmaxf(mx, s[i]);
    if (__any(mx > st[j].lim)) {
      asm volatile("" ::: "memory");
      move_reference<VD>(st[j], mx, c, over);
    }
    pb[j] = probabilities(s, c, st[j].shift);
  }
  const bf16x8 ones = ones8();
#pragma unroll
  for (int j = 0; j < GT; ++j) st[j].l = mfma16(ones, pb[j], st[j].l);
#pragma unroll
  for (int t = 0; t < OT; ++t)
#pragma unroll
    for (int j = 0; j < GT; ++j) st[j].o[t] = mfma16(va[t], pb[j], st[j].o[t]);
}

struct MaskedArgs {
  const bf16* q;
  const bf16* kc;
  const bf16* vc;
  const int* block_table;
  int table_stride;
  const int* cu_q;
  const int* context_lens;
  bf16* out;
  size_t out_stride;
  int nh, nkv, page_shift, window, keep_first;
  ScoreMap sm;
  float bias_unit;          // what a slope is multiplied by to be in the units of the raw scores
  const float* slopes;      // per head, or null
  const bf16* gate;         // [T, gate_stride], or null
  size_t gate_stride;
  float out_scale;
  int nv;                   // value heads in a page: key head k goes with value head k mod nv
};

// Grid (tiles of 64 tokens, nkv * head groups, sequences); WAVES wavefronts: four, or eight for steps in which every
// sequence brings one token (half the steps a wavefront, which is what such a step's time is made of).
template <int KD, int VD, int GT, int WAVES>
__global__ __launch_bounds__(WAVES* kWave, WAVES == 8 ? 1 : 2) void attn_masked_mfma_kernel(MaskedArgs a) {
  constexpr int OT = VD / 16;
  constexpr int KS = KD / 32;
  __shared__ float lds_o[WAVES][GT][VD];
  __shared__ float lds_ml[WAVES][GT][2];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  const int group = a.nh / a.nkv;
  const int hgroups = group / GT;
  const int kvh = blockIdx.y / hgroups, hg = blockIdx.y % hgroups;
  const int head0 = kvh * group + hg * GT;
  const int seq = blockIdx.z;
  const int row0 = a.cu_q[seq];
  const int q_len = a.cu_q[seq + 1] - row0;
  if (q_len <= 0) return;
  const int ctx = a.context_lens[seq];
  const bool single = q_len == 1;            // one token: its steps are dealt out to the wavefronts
  if (WAVES != 4 && !single) return;         // (the launch with more wavefronts is for steps of single tokens alone)
  const int tiles = (q_len + 63) / 64;
  const int tile = tiles - 1 - (int)blockIdx.x;   // late tiles first
  if (tile < 0) return;
  const int t0 = single ? 0 : tile * 64 + wave * 16;
  if (t0 >= q_len) return;                   // (never a single token's workgroup: no barrier is missed)
  const int window = a.window, keep = a.keep_first;
  const int start = ctx - q_len;
  const bool qvalid = t0 + r < q_len;
  const int my_pos = start + t0 + r;
  const int last_valid = t0 + 15 < q_len ? t0 + 15 : q_len - 1;
  const int last_pos = start + last_valid, first_pos = start + t0;
  int lo = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
  const int hi = last_pos + 1;
  const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
  const int all_lo = (window > 0 && last_pos - window + 1 > 0) ? last_pos - window + 1 : 0;
  const int all_hi = first_pos + 1;
  int kept = keep < lo ? keep : 0;           // keys [0, kept) are walked apart from [lo, hi)
  if (keep >= lo) lo = 0;                    // the two ranges meet: one range from the start
  const int kept_end = (kept + 31) & ~31;    // the kept keys' steps end here
  int win0 = (lo / 32) * 32;
  if (win0 < kept_end) win0 = kept_end;
  const int n_kept = kept_end / 32;
  const int n_steps = n_kept + (hi - win0 + 31) / 32;

  KeyWalk w{a.kc, a.vc, a.block_table + (size_t)seq * a.table_stride, a.nkv, kvh, a.page_shift, (1 << a.page_shift) - 1, lo, hi};
  bf16x8 qf[GT][KS];
  HeadState<VD> st[GT];
  float bias[GT];
#pragma unroll
  for (int j = 0; j < GT; ++j) {
    load_q<KD>(a.q + ((size_t)(row0 + (qvalid ? t0 + r : 0)) * a.nh + head0 + j) * KD, qvalid, g, qf[j]);
    bias[j] = a.slopes ? a.slopes[head0 + j] * a.bias_unit : 0.f;
  }
  auto vis = [&](int key) { return key <= my_pos && (key >= my_lo || key < keep); };
  auto key_of = [&](int i) { return i < n_kept ? 32 * i : win0 + 32 * (i - n_kept); };
  // every query of the wavefront sees every key of a step that lies at or before the first query and inside the last
  // query's window or among the kept keys
  auto masked_at = [&](int key0) { return !(key0 + 32 <= all_hi && (key0 >= all_lo || key0 + 32 <= keep)); };
  if (!single) {
    KFrag<KD> kf_next;
    load_k_gap<KD>(w, kept, key_of(0), g, r, kf_next);
    for (int i = 0; i < n_steps; ++i) {
      const KFrag<KD> kf = kf_next;
      const int key0 = key_of(i);
      if (i + 1 < n_steps) load_k_gap<KD>(w, kept, key_of(i + 1), g, r, kf_next);   // the next step's K rows, a step ahead
      attend32_masked<KD, VD, GT>(w, kept, key0, g, r, kf, qf, a.sm, bias, my_pos, masked_at(key0), st, vis, a.nv, kvh % a.nv);
    }
    if (!qvalid) return;
    const size_t t = (size_t)(row0 + t0 + r);
#pragma unroll
    for (int j = 0; j < GT; ++j) {
      const int h = head0 + j;
      float inv = a.out_scale / (st[j].l[0] + a.sm.sink_term(h, st[j].reference()));
      if (a.gate) inv *= 1.0f / (1.0f + __expf(-(float)a.gate[t * a.gate_stride + h]));
      bf16* orow = a.out + t * a.out_stride + (size_t)h * VD;
#pragma unroll
      for (int tt = 0; tt < OT; ++tt) {
        bf16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (bf16)(st[j].o[tt][i] * inv);
        *reinterpret_cast<bf16x4*>(orow + 16 * tt + 4 * g) = v;
      }
    }
    return;
  }
  for (int i = wave; i < n_steps; i += WAVES) {
    const int key0 = key_of(i);
    KFrag<KD> kf;
    load_k_gap<KD>(w, kept, key0, g, r, kf);
    attend32_masked<KD, VD, GT>(w, kept, key0, g, r, kf, qf, a.sm, bias, my_pos, true, st, vis, a.nv, kvh % a.nv);
  }
  if (r == 0) {
#pragma unroll
    for (int j = 0; j < GT; ++j) {
      if (g == 0) {
        lds_ml[wave][j][0] = st[j].reference();
        lds_ml[wave][j][1] = st[j].l[0];
      }
#pragma unroll
      for (int tt = 0; tt < OT; ++tt)
#pragma unroll
        for (int i = 0; i < 4; ++i) lds_o[wave][j][16 * tt + 4 * g + i] = st[j].o[tt][i];
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < GT * VD; e += blockDim.x) {
    const int j = e / VD, d = e % VD;
    float mm = lds_ml[0][j][0];
#pragma unroll
    for (int v = 1; v < WAVES; ++v) mm = fmaxf(mm, lds_ml[v][j][0]);
    float o = 0.f, l = 0.f;
#pragma unroll
    for (int v = 0; v < WAVES; ++v) {   // in the order of the wavefronts
      const float f = lds_ml[v][j][0] == -INFINITY ? 0.f : exp2f(lds_ml[v][j][0] - mm);
      o += lds_o[v][j][d] * f;
      l += lds_ml[v][j][1] * f;
    }
    const int h = head0 + j;
    float inv = a.out_scale / (l + a.sm.sink_term(h, mm));
    if (a.gate) inv *= 1.0f / (1.0f + __expf(-(float)a.gate[(size_t)row0 * a.gate_stride + h]));
    a.out[(size_t)row0 * a.out_stride + (size_t)h * VD + d] = (bf16)(o * inv);
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

// Whether the matrix-core kernel takes bfloat16 keys of `hd`, values of `vd` and pages of `page_size`.
extern "C" int pa_attn_masked_mfma_supports(int hd, int vd, int page_size) {
  const bool same = hd == vd && (hd == 32 || hd == 64 || hd == 96 || hd == 128);
  const bool twice = vd == 2 * hd && (hd == 32 || hd == 64);   // values twice as wide as the keys (two maps a head over one value)
  return (same || twice) && page_size >= 4 && (page_size & (page_size - 1)) == 0;
}

extern "C" int pa_attn_masked(void* stream, int dtype, const void* q, const void* k_cache, const void* v_cache,
                              const int* block_table, int table_stride, const int* seq_of_token, const int* positions,
                              void* out, long out_stride, int tokens, int nh, int nkv, int hd, int vd, int page_size,
                              int window, int keep_first, float scale, float softcap, const float* slopes,
                              const float* sink, const void* gate, long gate_stride, float out_scale, const int* cu_q,
                              const int* context_lens, int nseq, int max_q_len, int nv) {
  if (tokens == 0) return 0;
  if (nv <= 0) nv = nkv;
  PA_REQUIRE(nkv % nv == 0, "attn_masked: %d key heads are not a multiple of %d value heads", nkv, nv);
  PA_REQUIRE(tokens > 0 && nh > 0 && nkv > 0 && page_size > 0 && table_stride > 0,
             "attn_masked: bad sizes tokens=%d nh=%d nkv=%d page=%d table_stride=%d", tokens, nh, nkv, page_size, table_stride);
  PA_REQUIRE(nh % nkv == 0, "attn_masked: %d query heads are not a multiple of %d KV heads", nh, nkv);
  PA_REQUIRE(hd > 0 && hd <= kMaskedMaxDim && vd > 0 && vd <= kMaskedMaxDim,
             "attn_masked: key width %d or value width %d is outside 1..%d", hd, vd, kMaskedMaxDim);
  PA_REQUIRE(window >= 0 && keep_first >= 0, "attn_masked: window %d or kept first tokens %d negative", window, keep_first);
  PA_REQUIRE(softcap >= 0.f, "attn_masked: a score cap of %g is negative (0 means none)", (double)softcap);
  PA_REQUIRE(out_stride >= (long)nh * vd && (!gate || gate_stride >= nh), "attn_masked: output stride %ld or gate stride %ld "
             "too small for %d heads of %d", out_stride, gate_stride, nh, vd);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kBF16 && pa_attn_masked_mfma_supports(hd, vd, page_size) && cu_q && context_lens && nseq > 0 && max_q_len > 0) {
    const int group = nh / nkv;
    // two heads a wavefront where the group is even: four leave a head of 128 no registers and measured slower
    const int gt = group % 2 == 0 ? 2 : 1;
    MaskedArgs a{(const bf16*)q, (const bf16*)k_cache, (const bf16*)v_cache, block_table, table_stride, cu_q, context_lens,
                 (bf16*)out, (size_t)out_stride, nh, nkv, __builtin_ctz(page_size), window, window > 0 ? keep_first : 0,
                 score_map(scale, softcap, sink), softcap > 0.f ? 1.0f : 1.0f / scale, slopes, (const bf16*)gate,
                 (size_t)gate_stride, out_scale, nv};
    dim3 mgrid((max_q_len + 63) / 64, nkv * (group / gt), nseq);
    const bool singles = max_q_len == 1;
#define PA_MASKED(D, V, GT)                                                                                   \
  do {                                                                                                        \
    if (singles) hipLaunchKernelGGL((attn_masked_mfma_kernel<D, V, GT, 8>), mgrid, dim3(512), 0, st, a);       \
    else hipLaunchKernelGGL((attn_masked_mfma_kernel<D, V, GT, 4>), mgrid, dim3(256), 0, st, a);               \
  } while (0)
#define PA_MASKED_GT(D, V)              \
  do {                                  \
    if (gt == 2) PA_MASKED(D, V, 2);    \
    else PA_MASKED(D, V, 1);            \
  } while (0)
    if (hd == 32 && vd == 32) PA_MASKED_GT(32, 32);
    else if (hd == 32) PA_MASKED_GT(32, 64);
    else if (hd == 64 && vd == 64) PA_MASKED_GT(64, 64);
    else if (hd == 64) PA_MASKED_GT(64, 128);
    else if (hd == 96) PA_MASKED_GT(96, 96);
    else PA_MASKED_GT(128, 128);
#undef PA_MASKED_GT
#undef PA_MASKED
    return check_launch("attn_masked (matrix cores)");
  }
  dim3 grid(tokens, (nh + kMaskedWaves - 1) / kMaskedWaves);
  if (dtype == kF32) {
    hipLaunchKernelGGL(attn_masked_kernel<float>, grid, dim3(kMaskedWaves * kWave), 0, st, (const float*)q,
                       (const float*)k_cache, (const float*)v_cache, block_table, table_stride, seq_of_token, positions,
                       (float*)out, (size_t)out_stride, nh, nkv, hd, vd, page_size, window, keep_first, scale, softcap, slopes,
                       sink, (const float*)gate, (size_t)gate_stride, out_scale, nv);
  } else if (dtype == kBF16) {
    hipLaunchKernelGGL(attn_masked_kernel<bf16>, grid, dim3(kMaskedWaves * kWave), 0, st, (const bf16*)q,
                       (const bf16*)k_cache, (const bf16*)v_cache, block_table, table_stride, seq_of_token, positions,
                       (bf16*)out, (size_t)out_stride, nh, nkv, hd, vd, page_size, window, keep_first, scale, softcap, slopes,
                       sink, (const bf16*)gate, (size_t)gate_stride, out_scale, nv);
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
