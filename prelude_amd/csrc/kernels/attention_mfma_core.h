// The inner step of paged attention on the matrix cores, shared by the kernels that walk keys with it: how raw
// scores become exponents, a head's running sums with a lazily moving reference maximum, K rows and V^T tiles loaded
// from paged caches straight into the operand layout of v_mfma_f32_16x16x32_bf16, and one step over 32 keys for the
// heads that share them.  The layout and the reasons are described at the head of attention_mfma.hip.
#pragma once
#include "common.h"

namespace pa {

typedef short short4_t __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;

// How raw scores become exponents: 2^(s c - m c) with c = scale log2(e).  With a cap on the scores (cap > 0) a raw
// score is first bent to cap tanh(s scale / cap) and c is log2(e) alone.  Off (cap == 0) nothing is touched: the
// same instructions on the same numbers as without the parameter.
struct ScoreMap {
  float c;        // exponent per unit of (bent) score
  float cap;      // 0: none
  float cap_in;   // scale / cap
  // a sink per head (or null): one more term exp(sink[h]) of the softmax's denominator that brings no value, in the
  // units of the scaled scores.  It joins when a row's sums are finished: against the reference exponent `ref` (the
  // row's maximum times c, log2 domain) the term is 2^(sink log2(e) - ref).
  const float* sink;
  __device__ __forceinline__ float sink_term(int h, float ref) const {
    return sink ? exp2f(sink[h] * kLog2e - ref) : 0.f;
  }
};
__host__ inline ScoreMap score_map(float scale, float softcap, const float* sink = nullptr) {
  return softcap > 0.f ? ScoreMap{kLog2e, softcap, scale / softcap, sink} : ScoreMap{scale * kLog2e, 0.f, 0.f, sink};
}

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Reductions over the four lanes r, r + 16, r + 32, r + 48 (one query column), the result in all four.
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its second,
// v_permlane32_swap the upper half of the first with the lower half of the second: given the same value
// twice, the two results hold a lane's own value and its partner's.
__device__ __forceinline__ float xor_max16_32(float v) {
  const unsigned u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const unsigned w = __float_as_uint(v);
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float xor_sum16_32(float v) {
  const unsigned u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const unsigned w = __float_as_uint(v);
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// What a wavefront keeps per head while it walks keys: per lane, query column r.
//
// The exponentials are taken against a reference maximum `m` that follows the true running maximum lazily: it
// moves only when a score exceeds it by more than kLazyLog2 in the exponent (then every term so far is rescaled);
// until then a probability may be as large as 2^kLazyLog2 instead of at most 1, which costs 32-bit sums and bfloat16
// probabilities nothing (the quotient O / l is the same), and spares the rescaling of the whole output in most steps.
// Whether it must move is asked of every lane's own eight scores against `lim` = m + kLazyLog2 / c, one compare;
// only when some lane of the wavefront says yes is the column's maximum formed across its four lanes (the same
// compare on it then decides per column, so a column's sums do not depend on what its neighbours hold).
// The sum `l` is formed by the matrix cores too, as one more row of V^T that holds ones: it adds up the same
// rounded probabilities the output is made of, all 32 keys of a step at once, and every lane of a column has it.
constexpr float kLazyLog2 = 8.0f;

template <int HD>
struct HeadState {
  static constexpr int OT = HD / 16;
  // The reference maximum m of the raw scores, equal in the four lanes of a column, is kept as what is made of it:
  float lim = -INFINITY;  // a score above this moves m: m + kLazyLog2 / c (-inf while the column has seen no key)
  float shift = 0.f;      // -m c (0 while the column has seen no key): the exponent is s c + shift
  // m c, the exponent's reference, as the merge of splits wants it
  __device__ __forceinline__ float reference() const { return lim == -INFINITY ? -INFINITY : -shift; }
  f32x4 l;              // running sum of the column's probabilities (every element the same)
  f32x4 o[OT];          // O^T tiles: head_dim rows 16 t + 4g + i, column r
  __device__ HeadState() {
    l = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < OT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
};

template <int HD>
struct KFrag {
  static constexpr int KS = (HD + 31) / 32;
  bf16x8 k[2][KS];
};

// Where a sequence's keys are.  Page sizes are powers of two here, so a key's page and offset are a shift and a mask.
struct KeyWalk {
  const bf16* kc;
  const bf16* vc;
  const int* table;
  int nkv, kvh, page_shift, page_mask;
  int lo, hi;  // keys [lo, hi) exist and may be read
};

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
}

// K rows of keys key0 .. key0+31 as A operands: row r of tile t is key 8 (r / 4) + 4 t + r % 4.  Keys outside
// [lo, hi) are read from the nearest key inside (their scores are masked by the caller).
template <int HD>
__device__ __forceinline__ void load_k(const KeyWalk& w, int key0, int g, int r, KFrag<HD>& f) {
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    int key = key0 + 8 * (r / 4) + 4 * t + (r % 4);
    key = key < w.lo ? w.lo : (key >= w.hi ? w.hi - 1 : key);
    const int page = w.table[key >> w.page_shift];
    const bf16* row =
        w.kc + ((((size_t)page * w.nkv + w.kvh) << w.page_shift) + (key & w.page_mask)) * HD + 8 * g;
#pragma unroll
    for (int s = 0; s < KFrag<HD>::KS; ++s) {
      if (HD % 32 == 0 || 32 * s + 8 * g < HD) {
        f.k[t][s] = *reinterpret_cast<const bf16x8*>(row + 32 * s);
      } else {
        f.k[t][s] = zero8();
      }
    }
  }
}

// Where lane group g finds its eight keys key0 + 8g .. + 7 of a 32-key step in V^T: two chunks of four keys,
// each inside one page (pages hold a multiple of four keys), side by side when a page holds eight or more.
// p[t] points at head_dim row 0; row d is d pages further.
struct VChunks {
  const bf16* p[2];
  bool joined;  // p[1] == p[0] + 4: one 16-byte load
};

template <int HD>
__device__ __forceinline__ VChunks v_chunks(const KeyWalk& w, int key0, int g) {
  VChunks v;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    int c = key0 + 8 * g + 4 * t;  // first key of the chunk
    // a chunk wholly outside [lo, hi) is read from the chunk that holds the nearest key inside
    if (c + 3 < w.lo) c = w.lo & ~3;
    if (c >= w.hi) c = (w.hi - 1) & ~3;
    const int page = w.table[c >> w.page_shift];
    v.p[t] = w.vc + ((((size_t)page * w.nkv + w.kvh) * HD) << w.page_shift) + (c & w.page_mask);
  }
  v.joined = w.page_shift >= 3 && __all(v.p[1] == v.p[0] + 4);
  return v;
}

__device__ __forceinline__ bf16x8 load_v(const VChunks& v, int d, int page_shift) {
  if (v.joined) return *reinterpret_cast<const bf16x8*>(v.p[0] + ((size_t)d << page_shift));
  union {
    bf16x8 v8;
    short4_t h[2];
  } u;
  u.h[0] = *reinterpret_cast<const short4_t*>(v.p[0] + ((size_t)d << page_shift));
  u.h[1] = *reinterpret_cast<const short4_t*>(v.p[1] + ((size_t)d << page_shift));
  return u.v8;
}

__device__ __forceinline__ bf16x8 ones8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)1.f;
  return z;
}

// Scores of 32 keys against one head's 16 queries, s[8] per lane (keys key0 + 8g + 0..7 of query r), and the
// largest of the lane's eight.
// `masked` false: every key of the step is visible to every query (no comparisons).
// `vis(key)` says whether this lane's query may see the key (and the key exists).
template <int HD, typename Visible>
__device__ __forceinline__ float scores32(int key0, int g, const KFrag<HD>& kf, const bf16x8* qf, bool masked,
                                          const ScoreMap& sm, float* s, Visible vis) {
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    f32x4 acc{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KFrag<HD>::KS; ++ks) acc = mfma16(kf.k[t][ks], qf[ks], acc);
#pragma unroll
    for (int i = 0; i < 4; ++i) s[4 * t + i] = acc[i];
  }
  if (sm.cap != 0.f) {   // before the mask: a masked score must stay -inf
#pragma unroll
    for (int i = 0; i < 8; ++i) s[i] = sm.cap * tanhf(s[i] * sm.cap_in);
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
  return mx;
}

// The reference maximum of a head's columns moves where the step's largest score (`mx_lane`: the lane's own) lies
// above the column's limit; the sums so far are rescaled by 2^((m_before - m) c) there.  Called only when some
// lane of the wavefront is above its limit.
template <int HD>
__device__ __forceinline__ void move_reference(HeadState<HD>& st, float mx_lane, float c, float over) {
  constexpr int OT = HeadState<HD>::OT;
  const float mx = xor_max16_32(mx_lane);
  const bool moved = mx > st.lim;   // from -inf any finite score; -inf against -inf is false
  // 2^((m_before - mx) c).  A column's first keys rescale nothing (its sums are zero): the factor is 1 there and
  // not 2^(-mx c), which for a first score far below zero is +inf and would turn the zero sums into NaN
  const float alpha = moved && st.lim != -INFINITY ? __builtin_amdgcn_exp2f(-st.shift - mx * c) : 1.0f;
  if (moved) {
    st.lim = mx + over;
    st.shift = -mx * c;
  }
#pragma unroll
  for (int t = 0; t < OT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) st.o[t][i] *= alpha;
#pragma unroll
  for (int i = 0; i < 4; ++i) st.l[i] *= alpha;
}

// The probabilities 2^((s - m) c), c = scale * log2(e), packed as the B operand of O^T = V^T P^T.
__device__ __forceinline__ bf16x8 probabilities(const float* s, float c, float shift) {
  bf16x8 pb;
#pragma unroll
  for (int i = 0; i < 8; ++i) pb[i] = (bf16)__builtin_amdgcn_exp2f(fmaf(s[i], c, shift));
  return pb;
}

// Q^T of 16 queries of one head as B operands: lane (g, r) holds query r, head_dim 32 ks + 8g .. +7.
template <int HD>
__device__ __forceinline__ void load_q(const bf16* qrow, bool valid, int g, bf16x8* qf) {
#pragma unroll
  for (int ks = 0; ks < (HD + 31) / 32; ++ks) {
    if (valid && (HD % 32 == 0 || 32 * ks + 8 * g < HD)) {
      qf[ks] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks + 8 * g);
    } else {
      qf[ks] = zero8();
    }
  }
}

// The arithmetic of one step over 32 keys for GT heads that share the keys: the scores and softmax of every
// head first, then each V^T tile is used by all heads.  A head's sums are rescaled only in steps in which the
// reference maximum of one of its columns moved.
template <int HD, int GT, typename Visible>
__device__ __forceinline__ void attend32_core(int key0, int g, const KFrag<HD>& kf, const bf16x8* va,
                                              const bf16x8 (*qf)[(HD + 31) / 32], const ScoreMap& sm, bool masked,
                                              HeadState<HD>* st, Visible vis) {
  constexpr int OT = HeadState<HD>::OT;
  bf16x8 pb[GT];
  const float c = sm.c;
  const float over = kLazyLog2 / c;
#pragma unroll
  for (int j = 0; j < GT; ++j) {
    float s[8];
    const float mx = scores32<HD>(key0, g, kf, qf[j], masked, sm, s, vis);
    if (__any(mx > st[j].lim)) {
      asm volatile("" ::: "memory");  // keep this a branch: as selects it would cost a multiply per output every step
      move_reference<HD>(st[j], mx, c, over);
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

// One step over 32 keys read from the cache: the V^T tiles are asked for at the start of the step, so they
// arrive under the scores.  `kf` holds the step's K rows, loaded a step ahead.
template <int HD, int GT, typename Visible>
__device__ __forceinline__ void attend32(const KeyWalk& w, int key0, int g, int r, const KFrag<HD>& kf,
                                         const bf16x8 (*qf)[(HD + 31) / 32], const ScoreMap& c, bool masked,
                                         HeadState<HD>* st, Visible vis) {
  constexpr int OT = HeadState<HD>::OT;
  const VChunks vch = v_chunks<HD>(w, key0, g);
  bf16x8 va[OT];
#pragma unroll
  for (int t = 0; t < OT; ++t) va[t] = load_v(vch, 16 * t + r, w.page_shift);
  attend32_core<HD, GT>(key0, g, kf, va, qf, c, masked, st, vis);
}

}  // namespace pa
