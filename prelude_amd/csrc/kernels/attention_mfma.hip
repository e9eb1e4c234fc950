// Paged causal attention on the matrix cores (bfloat16 in, 32-bit softmax and
// accumulation), in two kernels that share their inner step:
//
//   attn_decode  -- one query token per sequence; the keys of a sequence are
//                   cut into splits of a fixed number of keys, each workgroup
//                   reduces one split, a second kernel merges the splits.
//   attn_prefill -- portions of several tokens; a wavefront owns 16 tokens of
//                   up to four query heads that share a KV head and walks the
//                   keys they may see.
//
// Both compute S^T = K Q^T and O^T = V^T P^T with v_mfma_f32_16x16x32_bf16, so
// that a query is a column (lane % 16) in the scores and in the output alike:
// the running maximum, the sum and the rescaling stay in the lane, and the
// probabilities leave the first product in exactly the register layout the
// second one wants.  K pages are [page, kv_head, offset, head_dim] and V pages
// [page, kv_head, head_dim, offset]: in both, the contraction index of the
// product they feed is contiguous, so every operand is loaded from memory
// straight into registers, with no staging in LDS and no barrier in the loop.
// Heads that share a KV head share every K and V register: a step computes
// all their scores first, then walks V once.  Comparisons with the mask are
// made only in steps that touch the diagonal, a window's edge or the end, and
// an output is rescaled only in steps where a running maximum moved.
//
// Operand layout of v_mfma_f32_16x16x32_bf16 (lane l, g = l / 16, r = l % 16):
//   A[16 x 32]: row r,    columns 8g .. 8g+7        B[32 x 16]: column r, rows 8g .. 8g+7
//   C[16 x 16]: column r, rows 4g .. 4g+3
// A step takes 32 keys as two score tiles.  Which key a tile's row stands for is
// free, and is chosen so that lane group g ends up with the scores of the eight
// consecutive keys 8g .. 8g+7: row 4a + i of tile t is key 8a + 4t + i.  Packed
// in that order they are the B operand of O^T = V^T P^T, whose A operand is then
// eight consecutive keys of one head_dim row of V^T: one 16-byte load.
//
// Reference counterparts: the FA4 / FlashInfer paged kernels the reference
// calls (crates/prelude-cuda/src/attn/flash_v4.rs:125-277,
// crates/prelude-cuda/src/attn/flashinfer.rs:737-797); formula as in
// crates/prelude-core/src/ops/traits/attention.rs:10-99.
#include "common.h"
#include "api.h"

#include <stdlib.h>

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
};
__host__ inline ScoreMap score_map(float scale, float softcap) {
  return softcap > 0.f ? ScoreMap{kLog2e, softcap, scale / softcap} : ScoreMap{scale * kLog2e, 0.f, 0.f};
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

// ---------------------------------------------------------------------------
// decode: grid (nkv * qtiles, splits, sequences), WAVES wavefronts (4, or 2 for small grids), each taking every
// WAVES-th step of 32 keys
// ---------------------------------------------------------------------------

// What the decode kernel needs to take the merged QKV projection as it leaves the product instead of queries
// that have been through the QK-norm + RoPE kernel: it norms and rotates its own queries, and the workgroup
// whose split holds the token's own position first norms, rotates and writes the token's key and copies its
// value into the cache (the kernel of qknorm_rope.hip, for one token and KV head).
struct FusedQkv {
  const bf16* qkv;          // [tokens, (nh + 2 nkv) * head_dim]
  const float* q_weight;    // may be null: no norm
  const float* k_weight;
  const float* cos_table;   // [positions, head_dim / 2]
  const float* sin_table;
  const int* slots;
  float eps;
};

template <int HD>
__device__ __forceinline__ void fused_write_kv(const FusedQkv& f, bf16* kc, bf16* vc, size_t token, int pos, int heads,
                                               int nh, int nkv, int kvh, int page_shift, int lane) {
  constexpr int EPL = HD / kWave;   // 64 -> 1, 128 -> 2: a lane's elements; its rotation partner is lane ^ 32
  typedef bf16 vec_t __attribute__((ext_vector_type(EPL)));
  const int slot = f.slots[token];
  if (slot < 0) return;
  const int page = slot >> page_shift, off = slot & ((1 << page_shift) - 1);
  const bf16* krow = f.qkv + (token * heads + nh + kvh) * HD;
  const bf16* vrow = f.qkv + (token * heads + nh + nkv + kvh) * HD;
  const vec_t kv = *reinterpret_cast<const vec_t*>(krow + lane * EPL);
  const vec_t vv = *reinterpret_cast<const vec_t*>(vrow + lane * EPL);
  // the scale and the angles of the lane's elements, asked for with the rows (not one by one after the sum)
  typedef float fvec_t __attribute__((ext_vector_type(EPL)));
  const int j0 = (lane % 32) * EPL;
  fvec_t kw;
  if (f.k_weight) kw = *reinterpret_cast<const fvec_t*>(f.k_weight + lane * EPL);
  const fvec_t csv = *reinterpret_cast<const fvec_t*>(f.cos_table + (size_t)pos * (HD / 2) + j0);
  const fvec_t snv = *reinterpret_cast<const fvec_t*>(f.sin_table + (size_t)pos * (HD / 2) + j0);
  bf16* vdst = vc + ((((size_t)page * nkv + kvh) * HD) << page_shift) + off;
#pragma unroll
  for (int e = 0; e < EPL; ++e) vdst[(size_t)(lane * EPL + e) << page_shift] = vv[e];
  float x[EPL], ss = 0.f;
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    x[e] = (float)kv[e];
    ss += x[e] * x[e];
  }
  ss = wave_sum(ss);
  const float inv = rsqrtf(ss / (float)HD + f.eps);
  vec_t ov;
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    if (f.k_weight) x[e] = x[e] * inv * kw[e];
    const float partner = __shfl_xor(x[e], 32, kWave);
    const float cs = csv[e], sn = snv[e];
    ov[e] = (bf16)(lane < 32 ? x[e] * cs - partner * sn : partner * sn + x[e] * cs);
  }
  bf16* kdst = kc + ((((size_t)page * nkv + kvh) << page_shift) + off) * HD;
  *reinterpret_cast<vec_t*>(kdst + lane * EPL) = ov;
}

// Element i of a float4 (i known when the loops around it are unrolled).
__device__ __forceinline__ float f4(const float4& v, int i) { return i == 0 ? v.x : (i == 1 ? v.y : (i == 2 ? v.z : v.w)); }

// Q^T of one head as B operands from the raw projection: normed and rotated in the lane.  Lane (g, r) holds
// head_dim 32 ks + 8g .. + 7 of its head; the element head_dim / 2 further on, its rotation partner, is in
// the same lane (ks + KS / 2), and the sum of squares runs over the lane's elements and the four lane groups.
template <int HD>
__device__ __forceinline__ void fused_load_q(const FusedQkv& f, const bf16* qrow, bool valid, int pos, int g, bf16x8* qf) {
  constexpr int KS = HD / 32;
  static_assert(HD == 64 || HD == 128, "the rotation partner must sit in the same lane");
  // Everything the lane needs is asked for at once, in 16-byte pieces: its elements of the row, and for each of
  // its KS / 2 first-half stretches of eight elements the two stretches of the norm's scale and the angles' cosines
  // and sines.  (Element by element, under the test for a scale, the loads had been issued and waited for one
  // pair at a time: sixteen trips to the cache in a row.)
  bf16x8 raw[KS];
  float4 wa[KS / 2][2], wb[KS / 2][2], cs4[KS / 2][2], sn4[KS / 2][2];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    raw[ks] = zero8();
    if (valid) raw[ks] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks + 8 * g);
  }
#pragma unroll
  for (int ks = 0; ks < KS / 2; ++ks) {
    const int d = 32 * ks + 8 * g;   // the first-half element; its partner is d + HD / 2
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if (f.q_weight) {
        wa[ks][h] = *reinterpret_cast<const float4*>(f.q_weight + d + 4 * h);
        wb[ks][h] = *reinterpret_cast<const float4*>(f.q_weight + d + HD / 2 + 4 * h);
      }
      cs4[ks][h] = *reinterpret_cast<const float4*>(f.cos_table + (size_t)pos * (HD / 2) + d + 4 * h);
      sn4[ks][h] = *reinterpret_cast<const float4*>(f.sin_table + (size_t)pos * (HD / 2) + d + 4 * h);
    }
  }
  float x[KS][8];
  float ss = 0.f;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      x[ks][j] = (float)raw[ks][j];
      ss += x[ks][j] * x[ks][j];
    }
  }
  ss = xor_sum16_32(ss);
  const float inv = rsqrtf(ss / (float)HD + f.eps);
#pragma unroll
  for (int ks = 0; ks < KS / 2; ++ks) {
    bf16x8 lo, hi;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float a = x[ks][j], b = x[ks + KS / 2][j];
      if (f.q_weight) {
        a = a * inv * f4(wa[ks][j / 4], j % 4);
        b = b * inv * f4(wb[ks][j / 4], j % 4);
      }
      const float cs = f4(cs4[ks][j / 4], j % 4), sn = f4(sn4[ks][j / 4], j % 4);
      lo[j] = (bf16)(a * cs - b * sn);
      hi[j] = (bf16)(a * sn + b * cs);
    }
    qf[ks] = lo;
    qf[ks + KS / 2] = hi;
  }
}

template <int HD, bool FUSED, int WAVES>
__global__ __launch_bounds__(WAVES* kWave, WAVES == 8 ? 1 : 3) void attn_decode_kernel(
    const bf16* __restrict__ q, const bf16* kc, const bf16* vc,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ seq_ids,
    const int* __restrict__ cu_q, const int* __restrict__ context_lens, bf16* __restrict__ out,
    float* __restrict__ part_o, float* __restrict__ part_ml, int nh, int nkv, int page_shift, int window, ScoreMap c,
    int split_keys, int max_splits, FusedQkv fq, int contiguous) {
  constexpr int OT = HD / 16;
  constexpr int KS = (HD + 31) / 32;
  // eight wavefronts (grids of at most a workgroup a compute unit, groups of up to eight heads) keep eight query rows
  constexpr int QR = WAVES == 8 ? 8 : 16;
  __shared__ float lds_o[WAVES][QR][HD + 1];
  __shared__ float lds_ml[WAVES][QR][2];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  const int group = nh / nkv;
  const int qtiles = (group + 15) / 16;
  // The KV heads run fastest over the grid: the workgroups in flight at any time then read all heads of the same
  // pages, whole stretches of memory, instead of one head's 4 KB out of every page's nkv * 4 KB (with the splits
  // fastest, long contexts of few sequences left memory channels idle: 8 x 32,768 keys took 207 us where 64 x 4,096,
  // the same bytes, took 187; now 170 and 176).  Small grids (contiguous == 1) are dealt out so that every XCD, which
  // gets every eighth workgroup, works through one contiguous stretch of that order.
  int split_idx, head_idx, seq_idx;
  if (!contiguous) {
    split_idx = blockIdx.y, head_idx = blockIdx.x, seq_idx = blockIdx.z;
  } else {
    const unsigned hq = nkv * qtiles;
    const unsigned total = gridDim.x;
    const unsigned id = blockIdx.x;
    const unsigned per = total / 8, rem = total % 8, x = id % 8;
    const unsigned v = x * per + (x < rem ? x : rem) + id / 8;
    head_idx = v % hq;
    split_idx = (v / hq) % max_splits;
    seq_idx = v / (hq * max_splits);
  }
  const int kvh = head_idx / qtiles, qt = head_idx % qtiles;
  const int seq = seq_ids ? seq_ids[seq_idx] : seq_idx;   // no list: every sequence of the step
  const int ctx = context_lens[seq];
  const int pos = ctx - 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int first_split = lo / split_keys;
  const int nsplit = (ctx + split_keys - 1) / split_keys - first_split;
  if (split_idx >= nsplit) return;
  const int sp = first_split + split_idx;
  const int k_begin = sp * split_keys > lo ? sp * split_keys : lo;
  const int k_end = (sp + 1) * split_keys < ctx ? (sp + 1) * split_keys : ctx;

  KeyWalk w{kc, vc, block_table + (size_t)seq * table_stride, nkv, kvh, page_shift, (1 << page_shift) - 1, lo, ctx};
  const int head = kvh * group + qt * 16 + r;  // this lane's query head
  const bool qvalid = qt * 16 + r < group;
  const size_t token = cu_q[seq];
  bf16x8 qf[1][KS];
  if constexpr (FUSED) {
    const int heads = nh + 2 * nkv;
    // a sequence that feeds one token feeds the one at its last position: no need to wait for positions[token]
    fused_load_q<HD>(fq, fq.qkv + (token * heads + (qvalid ? head : 0)) * HD, qvalid, pos, g, qf[0]);
    if (split_idx == nsplit - 1) {   // the split that holds the token's own position: its key and value first
      if (wave == 0)
        fused_write_kv<HD>(fq, const_cast<bf16*>(kc), const_cast<bf16*>(vc), token, pos, heads, nh, nkv, kvh, page_shift,
                           lane);
      __syncthreads();   // the other wavefronts read them from the cache below
    }
  } else {
    load_q<HD>(q + (token * nh + (qvalid ? head : 0)) * HD, qvalid, g, qf[0]);
  }

  HeadState<HD> st[1];
  const int step0 = (sp * split_keys) / 32;  // splits start at multiples of 32 keys
  const int steps = split_keys / 32;
  // a wavefront has two steps here (four with two wavefronts): many wavefronts per SIMD hide the latency, not a prefetch
  for (int i = wave; i < steps; i += WAVES) {
    const int key0 = (step0 + i) * 32;
    if (key0 + 32 <= k_begin || key0 >= k_end) continue;
    KFrag<HD> kf;
    load_k<HD>(w, key0, g, r, kf);
    const bool masked = key0 < k_begin || key0 + 32 > k_end;
    attend32<HD, 1>(w, key0, g, r, kf, qf, c, masked, st, [&](int key) { return key >= k_begin && key < k_end; });
  }
  // merge the wavefronts through LDS; maxima leave in the log2 domain (raw maximum times c)
  const float l_wave = st[0].l[0];
  if (g == 0 && r < QR) {
    lds_ml[wave][r][0] = st[0].reference();
    lds_ml[wave][r][1] = l_wave;
  }
  if (r < QR) {
#pragma unroll
    for (int t = 0; t < OT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) lds_o[wave][r][16 * t + 4 * g + i] = st[0].o[t][i];
  }
  __syncthreads();
  const int nq = group - qt * 16 < 16 ? group - qt * 16 : 16;
  for (int e = threadIdx.x; e < nq * HD; e += blockDim.x) {
    const int qi = e / HD, d = e % HD;
    float mm = lds_ml[0][qi][0];
#pragma unroll
    for (int v = 1; v < WAVES; ++v) mm = fmaxf(mm, lds_ml[v][qi][0]);
    float o = 0.f, l = 0.f;
#pragma unroll
    for (int v = 0; v < WAVES; ++v) {
      const float f = lds_ml[v][qi][0] == -INFINITY ? 0.f : exp2f(lds_ml[v][qi][0] - mm);
      o += lds_o[v][qi][d] * f;
      l += lds_ml[v][qi][1] * f;
    }
    const int h = kvh * group + qt * 16 + qi;
    if (nsplit == 1) {
      out[(token * nh + h) * HD + d] = (bf16)(o / l);
    } else {
      const size_t slot = ((size_t)seq_idx * nh + h) * max_splits + split_idx;
      part_o[slot * HD + d] = o;
      if (d == 0) {
        part_ml[slot * 2] = mm;
        part_ml[slot * 2 + 1] = l;
      }
    }
  }
}

// Merges the splits of one (sequence, head): grid (nh, sequences), groups of a thread per head_dim column.
// Every wavefront keeps a split per lane (maximum, weight), sixteen splits' outputs are asked for before the
// weights are known, and the sums run over the splits in order.  The splits go to the groups in runs of 64
// (run c to group c mod merge_groups_of(HD)), and the groups' sums are added in group order: a request's result
// depends on its own number of splits alone, and up to 64 splits (16,384 keys) it is one group's sum as it
// stands.  The launch brings as many groups as the longest context has runs (eight at most): a merge of 512
// splits by one group waits 32 times for memory, one after the other.
constexpr int kMergeGroups = 8;
// ... as far as a workgroup's 1,024 threads go: heads wider than 128 get fewer groups
constexpr int merge_groups_of(int hd) {
  const int threads = (hd + kWave - 1) / kWave * kWave;
  return kMergeGroups * threads <= 1024 ? kMergeGroups : 1024 / threads;
}

template <int HD>
__global__ __launch_bounds__(merge_groups_of(HD) * ((HD + kWave - 1) / kWave * kWave)) void attn_decode_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ seq_ids,
    const int* __restrict__ cu_q, const int* __restrict__ context_lens, bf16* __restrict__ out, int nh, int window,
    int split_keys, int max_splits) {
  constexpr int kBatch = 16;
  constexpr int TPG = (HD + kWave - 1) / kWave * kWave;   // threads a group
  __shared__ float group_acc[kMergeGroups][TPG];
  __shared__ float group_l[kMergeGroups];
  const int h = blockIdx.x;
  const int seq = seq_ids ? seq_ids[blockIdx.y] : (int)blockIdx.y;
  const int ctx = context_lens[seq];
  const size_t token = cu_q[seq];
  const int pos = ctx - 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int nsplit = (ctx + split_keys - 1) / split_keys - lo / split_keys;
  if (nsplit == 1) return;  // written by the first kernel
  const int groups = blockDim.x / TPG;                     // the launch's: all runs of the longest context, or eight
  const int grp = threadIdx.x / TPG, d = threadIdx.x % TPG, lane = threadIdx.x % kWave;
  const bool col = d < HD;
  const size_t base = ((size_t)blockIdx.y * nh + h) * max_splits;
  const float* po = part_o + base * HD + (col ? d : 0);
  const int first = grp * kWave;                           // this group's first run
  // the first batch of outputs, on its way while the weights are worked out
  float o[kBatch];
#pragma unroll
  for (int i = 0; i < kBatch; ++i) o[i] = (col && first + i < nsplit) ? po[(size_t)(first + i) * HD] : 0.f;
  float mm = -INFINITY;
  for (int s = lane; s < nsplit; s += kWave) mm = fmaxf(mm, part_ml[(base + s) * 2]);
  mm = wave_max(mm);
  float acc = 0.f, l = 0.f;
  for (int s0 = first; s0 < nsplit; s0 += merge_groups_of(HD) * kWave) {   // a split per lane; in order of the splits
    const int s = s0 + lane;
    float f = 0.f, ls = 0.f;
    if (s < nsplit) {
      f = exp2f(part_ml[(base + s) * 2] - mm);
      ls = part_ml[(base + s) * 2 + 1] * f;
    }
    l += wave_sum(ls);
    const int count = nsplit - s0 < kWave ? nsplit - s0 : kWave;
    for (int b0 = 0; b0 < count; b0 += kBatch) {
      if (s0 + b0 > first) {
#pragma unroll
        for (int i = 0; i < kBatch; ++i) o[i] = (col && b0 + i < count) ? po[(size_t)(s0 + b0 + i) * HD] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        // the index is the same in every lane: a read of one lane's register, no exchange
        const float fi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(f), b0 + i < kWave ? b0 + i : 0));
        if (b0 + i < count) acc += o[i] * fi;
      }
    }
  }
  if (groups == 1) {
    if (col) out[(token * nh + h) * HD + d] = (bf16)(acc / l);
    return;
  }
  group_acc[grp][d] = acc;
  if (d == 0) group_l[grp] = l;
  __syncthreads();
  if (grp == 0 && col) {
    float a = group_acc[0][d], ll = group_l[0];
    for (int g = 1; g < groups; ++g) {
      a += group_acc[g][d];
      ll += group_l[g];
    }
    out[(token * nh + h) * HD + d] = (bf16)(a / ll);
  }
}

// ---------------------------------------------------------------------------
// prefill: grid (pairs of 64-token tiles, nkv * head groups, sequences); a wavefront owns 16 tokens x GT heads
// ---------------------------------------------------------------------------
// One wavefront's share of a 64-token tile: 16 tokens from t0, all keys they may see.
template <int HD, int GT>
__device__ __forceinline__ void prefill_tile(const bf16* __restrict__ q, bf16* __restrict__ out, const bf16* kc,
                                             const bf16* vc, const int* table, int row0, int q_len, int ctx, int t0,
                                             int nh, int nkv, int kvh, int head0, int page_shift, int window,
                                             const ScoreMap& c, int g, int r) {
  constexpr int OT = HD / 16;
  constexpr int KS = (HD + 31) / 32;
  const int start = ctx - q_len;                // position of the portion's first token
  const bool qvalid = t0 + r < q_len;
  const int my_pos = start + t0 + r;            // this lane's query position
  const int last_valid = t0 + 15 < q_len ? t0 + 15 : q_len - 1;
  const int last_pos = start + last_valid;
  const int first_pos = start + t0;
  const int lo = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
  const int hi = last_pos + 1;
  const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
  // keys every valid query of the tile sees: from the last token's window start up to the first token's position
  const int all_lo = (window > 0 && last_pos - window + 1 > 0) ? last_pos - window + 1 : 0;
  const int all_hi = first_pos + 1;

  KeyWalk w{kc, vc, table, nkv, kvh, page_shift, (1 << page_shift) - 1, lo, hi};
  bf16x8 qf[GT][KS];
  HeadState<HD> st[GT];
#pragma unroll
  for (int j = 0; j < GT; ++j)
    load_q<HD>(q + ((size_t)(row0 + (qvalid ? t0 + r : 0)) * nh + head0 + j) * HD, qvalid, g, qf[j]);

  int key0 = (lo / 32) * 32;
  KFrag<HD> kf_next;
  load_k<HD>(w, key0, g, r, kf_next);
  for (; key0 < hi; key0 += 32) {
    const KFrag<HD> kf = kf_next;
    if (key0 + 32 < hi) load_k<HD>(w, key0 + 32, g, r, kf_next);   // the next step's K rows, a step ahead
    const bool masked = key0 < all_lo || key0 + 32 > all_hi;
    attend32<HD, GT>(w, key0, g, r, kf, qf, c, masked, st, [&](int key) { return key >= my_lo && key <= my_pos; });
  }
  if (!qvalid) return;
#pragma unroll
  for (int j = 0; j < GT; ++j) {
    const float inv = 1.0f / st[j].l[0];
    bf16* orow = out + ((size_t)(row0 + t0 + r) * nh + head0 + j) * HD;
#pragma unroll
    for (int t = 0; t < OT; ++t) {
      bf16x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = (bf16)(st[j].o[t][i] * inv);
      *reinterpret_cast<bf16x4*>(orow + 16 * t + 4 * g) = v;
    }
  }
}

// A workgroup takes the tiles p and (last - p) of its sequence: under the causal mask a late tile sees many
// keys and an early one few, and a pair always sees about the same number, so workgroups finish together.
template <int HD, int GT>
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ seq_ids,
    const int* __restrict__ cu_q, const int* __restrict__ context_lens, bf16* __restrict__ out, int nh, int nkv,
    int page_shift, int window, ScoreMap c, int paired) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  const int group = nh / nkv;
  const int hgroups = group / GT;
  const int kvh = blockIdx.x / hgroups, hg = blockIdx.x % hgroups;   // head groups fastest over the grid
  const int seq = seq_ids[blockIdx.z];
  const int row0 = cu_q[seq];
  const int q_len = cu_q[seq + 1] - row0;
  const int ctx = context_lens[seq];
  const int tiles = (q_len + 63) / 64;
  // unpaired: one tile per workgroup, late (long) tiles first
  const int first = paired ? (int)blockIdx.y : tiles - 1 - (int)blockIdx.y;
  const int second = paired ? tiles - 1 - (int)blockIdx.y : first;
  if (first > second || first < 0) return;
  const int* table = block_table + (size_t)seq * table_stride;
  const int head0 = kvh * group + hg * GT;
  {
    const int t0 = second * 64 + wave * 16;   // the long one first
    if (t0 < q_len)
      prefill_tile<HD, GT>(q, out, kc, vc, table, row0, q_len, ctx, t0, nh, nkv, kvh, head0, page_shift, window, c, g, r);
  }
  if (first != second) {
    const int t0 = first * 64 + wave * 16;
    if (t0 < q_len)
      prefill_tile<HD, GT>(q, out, kc, vc, table, row0, q_len, ctx, t0, nh, nkv, kvh, head0, page_shift, window, c, g, r);
  }
}

// ---------------------------------------------------------------------------
// prefill with the keys staged in LDS: grid as above; the four wavefronts of a workgroup own 16 tokens each
// of one 64-token tile and see almost the same keys, so the workgroup reads every block of 64 keys from the
// cache once (each thread a few 16-byte pieces, a block ahead, into registers), puts it into one of two LDS
// buffers, and all four take their MFMA operands from there.  One barrier a block.
//
// LDS layout: K rows [key][head_dim], the keys of each 32 in the order the score tiles want them (key
// 8a + 4t + i in row 16t + 4a + i); V^T rows [head_dim][64 keys], keys in their own order.  Rows are padded
// to 32 bytes past a multiple of 64: measured on gfx950, 16-byte reads of sixteen rows at such a stride run
// at the full 256 bytes a cycle, and at half that with 16 bytes of padding.
// ---------------------------------------------------------------------------
constexpr int kStageKeys = 64;

template <int HD>
struct StageLds {
  static constexpr int KROW = (2 * HD + 63) / 64 * 32 + 16;   // elements
  static constexpr int VROW = kStageKeys + 16;
  bf16 k[2][kStageKeys][KROW];
  bf16 v[2][HD][VROW];
};

// A thread's share of the staging, for workgroups of WAVES = 4 or 8 wavefronts.  Wavefront w takes the
// KW = 64 / WAVES keys KW w .. of a block of 64: of K, lane (r = lane / QL, q = lane % QL; QL = 64 / KW) takes the
// 16-byte pieces q, q + QL, .. of key KW w + r, so that the lanes of a load cover whole 64-byte stretches of a row
// (a lane per row would ask the memory pipeline for four times as many of them); of V^T, lane (d = lane / HL, h = lane % HL; HL = KW / 8 halves)
// takes the eight keys KW w + 8h .. + 7 of the rows d, d + 64 / HL, ...  Pages hold 8 keys or more here, a power of
// two: a block of 64 starts at a page's first key or lies inside one page, so a thread reads one page of each cache
// per block, `base` keys into it (always 0 for pages of up to 64 keys).  A page outside the pages [lo_page, hi_page]
// that hold the tile's keys is replaced by the nearest of those; the scores of its keys are masked.
template <int HD, int WAVES>
struct Stage {
  static_assert(WAVES == 4 || WAVES == 8, "four or eight wavefronts stage a block");
  static constexpr int KW = kStageKeys / WAVES;   // keys a wavefront stages
  static constexpr int QL = kWave / KW;           // lane groups along a K row
  static constexpr int HL = KW / 8;               // 8-key halves of a wavefront's keys
  static constexpr int DL = kWave / HL;           // V^T rows a wavefront covers at once
  static constexpr int CPK = HD / 8;              // 16-byte pieces per K row
  static constexpr int NK = (CPK + QL - 1) / QL;
  static constexpr int NV = (HD + DL - 1) / DL;
  bf16x8 k[NK];
  bf16x8 v[NV];
  int kpage, vpage, base;

  __device__ __forceinline__ void load_pages(const KeyWalk& w, int key0, int wave, int lane, int lo_page, int hi_page) {
    base = key0 & w.page_mask;
    int kp = (key0 + KW * wave + lane / QL) >> w.page_shift;
    int vp = (key0 + KW * wave + 8 * (lane % HL)) >> w.page_shift;
    kp = kp < lo_page ? lo_page : (kp > hi_page ? hi_page : kp);
    vp = vp < lo_page ? lo_page : (vp > hi_page ? hi_page : vp);
    kpage = w.table[kp];
    vpage = w.table[vp];
  }

  __device__ __forceinline__ void load(const KeyWalk& w, int wave, int lane) {
    const unsigned page_elems = ((unsigned)w.nkv * HD) << w.page_shift;   // elements per page, all KV heads
    const unsigned head_off = ((unsigned)w.kvh * HD) << w.page_shift;
    const int r = lane / QL, q = lane % QL;
    const bf16* kp = w.kc + ((unsigned long long)(unsigned)kpage * page_elems + head_off +
                             (unsigned)((base + KW * wave + r) & w.page_mask) * HD + 8 * q);
#pragma unroll
    for (int j = 0; j < NK; ++j)
      if (CPK % QL == 0 || QL * j + q < CPK) k[j] = *reinterpret_cast<const bf16x8*>(kp + 8 * QL * j);
    const int d = lane / HL, h = lane % HL;
    const bf16* vp = w.vc + ((unsigned long long)(unsigned)vpage * page_elems + head_off + ((unsigned)d << w.page_shift) +
                             (unsigned)((base + KW * wave + 8 * h) & w.page_mask));
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (HD % DL == 0 || d + DL * j < HD) v[j] = *reinterpret_cast<const bf16x8*>(vp + ((size_t)(DL * j) << w.page_shift));
  }

  __device__ __forceinline__ void store(StageLds<HD>& lds, int buf, int wave, int lane) const {
    const int r = lane / QL, q = lane % QL;
    const int key = KW * wave + r;   // 32 s + 8 a + 4 t + i  ->  row 32 s + 16 t + 4 a + i
    const int row = (key & 32) | ((key & 4) << 2) | ((key & 24) >> 1) | (key & 3);
#pragma unroll
    for (int j = 0; j < NK; ++j)
      if (CPK % QL == 0 || QL * j + q < CPK) *reinterpret_cast<bf16x8*>(&lds.k[buf][row][8 * (QL * j + q)]) = k[j];
    const int d = lane / HL, h = lane % HL;
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (HD % DL == 0 || d + DL * j < HD) *reinterpret_cast<bf16x8*>(&lds.v[buf][d + DL * j][KW * wave + 8 * h]) = v[j];
  }
};

// One step over the 32 keys `sub` of the staged block.
template <int HD, int GT, typename Visible>
__device__ __forceinline__ void attend32_lds(const StageLds<HD>& lds, int buf, int sub, int key0, int g, int r,
                                             const bf16x8 (*qf)[(HD + 31) / 32], const ScoreMap& c, bool masked,
                                             HeadState<HD>* st, Visible vis) {
  constexpr int OT = HeadState<HD>::OT;
  KFrag<HD> kf;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int ks = 0; ks < KFrag<HD>::KS; ++ks) {
      if (HD % 32 == 0 || 32 * ks + 8 * g < HD) {
        kf.k[t][ks] = *reinterpret_cast<const bf16x8*>(&lds.k[buf][32 * sub + 16 * t + r][32 * ks + 8 * g]);
      } else {
        kf.k[t][ks] = zero8();
      }
    }
  bf16x8 va[OT];
#pragma unroll
  for (int t = 0; t < OT; ++t) va[t] = *reinterpret_cast<const bf16x8*>(&lds.v[buf][16 * t + r][32 * sub + 8 * g]);
  attend32_core<HD, GT>(key0, g, kf, va, qf, c, masked, st, vis);
}

// A 64-token tile from tile0 for GT * HW heads from head0: wavefront `wave` owns the tokens 16 (wave % 4) .. + 15 of
// the GT heads from head0 + GT (wave / 4).  Every wavefront takes part in the staging and the barriers, also one
// whose tokens lie beyond the portion's end.
template <int HD, int GT, int HW>
__device__ __forceinline__ void prefill_tile_lds(StageLds<HD>& lds, const bf16* __restrict__ q, bf16* __restrict__ out,
                                                 const bf16* kc, const bf16* vc, const int* table, int row0, int q_len,
                                                 int ctx, int tile0, int nh, int nkv, int kvh, int head0, int page_shift,
                                                 int window, const ScoreMap& c, int wave, int g, int r) {
  constexpr int OT = HD / 16;
  constexpr int KS = (HD + 31) / 32;
  const int lane = 16 * g + r;
  const int start = ctx - q_len;                // position of the portion's first token
  const int t0 = tile0 + 16 * (wave % 4);
  head0 += GT * (wave / 4);
  const bool wave_on = t0 < q_len;
  const bool qvalid = t0 + r < q_len;
  const int my_pos = start + t0 + r;            // this lane's query position
  const int last_valid = t0 + 15 < q_len ? t0 + 15 : q_len - 1;
  const int last_pos = start + last_valid;
  const int first_pos = start + t0;
  const int lo = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
  const int hi = last_pos + 1;
  const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
  const int all_lo = (window > 0 && last_pos - window + 1 > 0) ? last_pos - window + 1 : 0;
  const int all_hi = first_pos + 1;
  // what the workgroup stages: from the first token's window start to the last valid token of the tile
  const int wg_first = start + tile0;
  const int wg_last = start + (tile0 + 63 < q_len ? tile0 + 63 : q_len - 1);
  const int wg_lo = (window > 0 && wg_first - window + 1 > 0) ? wg_first - window + 1 : 0;
  const int wg_hi = wg_last + 1;

  KeyWalk w{kc, vc, table, nkv, kvh, page_shift, (1 << page_shift) - 1, wg_lo, wg_hi};
  bf16x8 qf[GT][KS];
  HeadState<HD> st[GT];
#pragma unroll
  for (int j = 0; j < GT; ++j)
    load_q<HD>(q + ((size_t)(row0 + (qvalid ? t0 + r : 0)) * nh + head0 + j) * HD, qvalid, g, qf[j]);

  Stage<HD, 4 * HW> stage;
  const int lo_page = wg_lo >> page_shift, hi_page = (wg_hi - 1) >> page_shift;
  // A block is put into LDS a whole block before it is used: while the wavefronts work on block b out of one
  // buffer, each first writes its share of block b + 1 (asked for from memory a block ago) into the other and asks
  // for block b + 2; the barrier at the block's end then says both that block b + 1 is complete and that nobody
  // reads block b any more.  (Written right before its use, the LDS writes and the barrier stood between every
  // block's arrival and its first product.)
  int key0 = (wg_lo / kStageKeys) * kStageKeys;
  stage.load_pages(w, key0, wave, lane, lo_page, hi_page);
  stage.load(w, wave, lane);
  if (key0 + kStageKeys < wg_hi) stage.load_pages(w, key0 + kStageKeys, wave, lane, lo_page, hi_page);
  stage.store(lds, 0, wave, lane);
  if (key0 + kStageKeys < wg_hi) {
    stage.load(w, wave, lane);
    if (key0 + 2 * kStageKeys < wg_hi) stage.load_pages(w, key0 + 2 * kStageKeys, wave, lane, lo_page, hi_page);
  }
  __syncthreads();
  int buf = 0;
  for (; key0 < wg_hi; key0 += kStageKeys, buf ^= 1) {
    if (key0 + kStageKeys < wg_hi) {
      stage.store(lds, buf ^ 1, wave, lane);   // the next block, asked for a block ago
      if (key0 + 2 * kStageKeys < wg_hi) {
        stage.load(w, wave, lane);             // the one after it, from the pages looked up a block ago
        if (key0 + 3 * kStageKeys < wg_hi)
          stage.load_pages(w, key0 + 3 * kStageKeys, wave, lane, lo_page, hi_page);
      }
    }
    if (wave_on) {
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        const int k32 = key0 + 32 * sub;
        if (k32 + 32 <= lo || k32 >= hi) continue;
        const bool masked = k32 < all_lo || k32 + 32 > all_hi;
        attend32_lds<HD, GT>(lds, buf, sub, k32, g, r, qf, c, masked, st,
                             [&](int key) { return key >= my_lo && key <= my_pos; });
      }
    }
    __syncthreads();
  }
  // (the loop's last barrier leaves the buffers free for the next tile)
  if (!qvalid) return;
#pragma unroll
  for (int j = 0; j < GT; ++j) {
    const float inv = 1.0f / st[j].l[0];
    bf16* orow = out + ((size_t)(row0 + t0 + r) * nh + head0 + j) * HD;
#pragma unroll
    for (int t = 0; t < OT; ++t) {
      bf16x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = (bf16)(st[j].o[t][i] * inv);
      *reinterpret_cast<bf16x4*>(orow + 16 * t + 4 * g) = v;
    }
  }
}

template <int HD, int GT, int HW>
__global__ __launch_bounds__(256 * HW, 2) void attn_prefill_lds_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ seq_ids,
    const int* __restrict__ cu_q, const int* __restrict__ context_lens, bf16* __restrict__ out, int nh, int nkv,
    int page_shift, int window, ScoreMap c, int paired) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  StageLds<HD>& lds = *reinterpret_cast<StageLds<HD>*>(lds_raw);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  const int group = nh / nkv;
  const int hgroups = group / (GT * HW);
  const int kvh = blockIdx.x / hgroups, hg = blockIdx.x % hgroups;   // head groups fastest over the grid
  // paired 2: unpaired, and the tiles (not the sequences) slowest over the grid, so that the long tiles of every
  // sequence are handed out before any short one
  const bool tile_slowest = paired == 2;
  const int seq = seq_ids[tile_slowest ? blockIdx.y : blockIdx.z];
  const int at = tile_slowest ? (int)blockIdx.z : (int)blockIdx.y;
  const int row0 = cu_q[seq];
  const int q_len = cu_q[seq + 1] - row0;
  const int ctx = context_lens[seq];
  const int tiles = (q_len + 63) / 64;
  const int first = paired == 1 ? at : tiles - 1 - at;
  const int second = paired == 1 ? tiles - 1 - at : first;
  if (first > second || first < 0) return;   // the same for the whole workgroup
  const int* table = block_table + (size_t)seq * table_stride;
  const int head0 = kvh * group + hg * GT * HW;
  prefill_tile_lds<HD, GT, HW>(lds, q, out, kc, vc, table, row0, q_len, ctx, second * 64, nh, nkv, kvh, head0,
                               page_shift, window, c, wave, g, r);   // the long one first
  if (first != second)
    prefill_tile_lds<HD, GT, HW>(lds, q, out, kc, vc, table, row0, q_len, ctx, first * 64, nh, nkv, kvh, head0,
                                 page_shift, window, c, wave, g, r);
}

// ---------------------------------------------------------------------------
template <int HD, bool FUSED>
int launch_decode(hipStream_t st, const void* q, const void* kc, const void* vc, const int* block_table,
                  int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                  float* part_o, float* part_ml, int nseq, int nh, int nkv, int page_shift, int window, float scale,
                  float softcap, int split_keys, int max_splits, const FusedQkv& fq) {
  const int qtiles = (nh / nkv + 15) / 16;
  // Grids of 513 to 4,096 workgroups are dealt out so that each XCD gets a contiguous stretch of them; measured in
  // the decode step of a 4B model: batch 8 at 4,096 keys +0.9 %, batch 9 to 12 +0.8 to 1.2 %, and the kernel alone
  // (32 heads over 8, in a graph, us contiguous / plain): 768 workgroups 25.8 / 26.1, 1,536 42.7 / 44.5, 2,048
  // 54.5 / 56.5, 4,096 99.8 / 101.7; larger and smaller grids do better dealt out plainly (8,192: 194.1 / 191.9,
  // 16,384: 372.6 / 359.8; 512: 21.3 / 20.4, 256: 13.9 / 13.4, 128: 11.5 / 11.2)
  const long total = (long)nkv * qtiles * max_splits * nseq;
  const int contiguous = total > 512 && total <= 4096;
  dim3 grid(nkv * qtiles, max_splits, nseq);
  if (contiguous) grid = dim3((unsigned)total, 1, 1);
  // Twelve wavefronts fit a compute unit (three a SIMD by their registers): three workgroups of four, 768 on the
  // chip.  A grid just above that would run a second, nearly empty round; with two wavefronts a workgroup six fit,
  // 1,536 on the chip, and the whole grid is there at once: batch 7 to 12 at 4,096 keys +0.3 to 2.3 % of the decode
  // step.  Smaller grids want the four wavefronts for their parallelism (batch 1: -3.7 % with two), larger ones
  // measured 1 to 2 % slower with two.  With two wavefronts a split's steps are added in another order (wavefront w
  // takes the steps w, w + 2, .. instead of w, w + 4, ..), so a token's sums can differ in their last bits between
  // steps whose grids fall on either side of these limits; what else is in the batch changes nothing beyond that.
  // A grid of less than one workgroup a compute unit (one sequence of 4,096 keys: 128) runs with eight, a step of
  // 32 keys each: batch 1 of a 4B model 2.518 -> 2.499 ms a step; 256 workgroups are level or better off with four
  // (13.4 against 13.7 us), and with eight up to 512 workgroups batch 3 and 4 lose 4 %.
  const bool two_wavefronts = total > 768 && total <= 1536;
  const bool eight_wavefronts = total <= 192 && nh / nkv <= 8 && split_keys == 256;
  if (eight_wavefronts) {
    hipLaunchKernelGGL((attn_decode_kernel<HD, FUSED, 8>), grid, dim3(8 * kWave), 0, st, (const bf16*)q, (const bf16*)kc,
                       (const bf16*)vc, block_table, table_stride, seq_ids, cu_q, context_lens, (bf16*)out, part_o,
                       part_ml, nh, nkv, page_shift, window, score_map(scale, softcap), split_keys, max_splits, fq, contiguous);
  } else if (two_wavefronts) {
    hipLaunchKernelGGL((attn_decode_kernel<HD, FUSED, 2>), grid, dim3(2 * kWave), 0, st, (const bf16*)q, (const bf16*)kc,
                       (const bf16*)vc, block_table, table_stride, seq_ids, cu_q, context_lens, (bf16*)out, part_o,
                       part_ml, nh, nkv, page_shift, window, score_map(scale, softcap), split_keys, max_splits, fq, contiguous);
  } else {
    hipLaunchKernelGGL((attn_decode_kernel<HD, FUSED, 4>), grid, dim3(4 * kWave), 0, st, (const bf16*)q, (const bf16*)kc,
                       (const bf16*)vc, block_table, table_stride, seq_ids, cu_q, context_lens, (bf16*)out, part_o,
                       part_ml, nh, nkv, page_shift, window, score_map(scale, softcap), split_keys, max_splits, fq, contiguous);
  }
  if (int rc = check_launch("attn_decode")) return rc;
  if (max_splits > 1) {
    // a group for every run of 64 splits the longest context can have, eight at most
    const int runs = (max_splits + kWave - 1) / kWave;
    const int groups = runs < merge_groups_of(HD) ? runs : merge_groups_of(HD);
    hipLaunchKernelGGL(attn_decode_merge_kernel<HD>, dim3(nh, nseq), dim3(groups * ((HD + kWave - 1) / kWave * kWave)),
                       0, st, part_o, part_ml, seq_ids, cu_q, context_lens, (bf16*)out, nh, window, split_keys,
                       max_splits);
    return check_launch("attn_decode_merge");
  }
  return 0;
}

template <int HD, int GT, int HW>
int launch_prefill_staged(hipStream_t st, const void* q, const void* kc, const void* vc, const int* block_table,
                          int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                          int nseq, int max_q_len, int nh, int nkv, int page_shift, int window, float scale,
                          float softcap, int paired) {
  const int tiles = (max_q_len + 63) / 64;
  dim3 grid(nkv * (nh / nkv / (GT * HW)), paired == 1 ? (tiles + 1) / 2 : tiles, nseq);
  if (paired == 2) grid = dim3(grid.x, nseq, tiles);
  // the two buffers are more than the 64 KB a kernel may declare: asked for at launch, allowed once per kernel
  static const hipError_t allowed =
      hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_prefill_lds_kernel<HD, GT, HW>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(StageLds<HD>));
  if (allowed != hipSuccess)
    return pa::fail("attn_prefill: %zu bytes of LDS refused: %s", sizeof(StageLds<HD>), hipGetErrorString(allowed));
  hipLaunchKernelGGL((attn_prefill_lds_kernel<HD, GT, HW>), grid, dim3(256 * HW), sizeof(StageLds<HD>), st,
                     (const bf16*)q, (const bf16*)kc, (const bf16*)vc, block_table, table_stride, seq_ids, cu_q,
                     context_lens, (bf16*)out, nh, nkv, page_shift, window, score_map(scale, softcap), paired);
  return check_launch("attn_prefill");
}

template <int HD, int GT>
int launch_prefill_gt(hipStream_t st, const void* q, const void* kc, const void* vc, const int* block_table,
                      int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                      int nseq, int max_q_len, int nh, int nkv, int page_shift, int window, float scale, float softcap,
                      int paired, int hw, bool staged) {
  const int tiles = (max_q_len + 63) / 64;
  if (!staged && paired == 2) paired = 0;   // the kernel that reads the cache itself has the one order
  dim3 grid(nkv * (nh / nkv / GT), paired == 1 ? (tiles + 1) / 2 : tiles, nseq);
  if (staged) {
    if (hw == 2)
      return launch_prefill_staged<HD, GT, 2>(st, q, kc, vc, block_table, table_stride, seq_ids, cu_q, context_lens, out,
                                              nseq, max_q_len, nh, nkv, page_shift, window, scale, softcap, paired);
    return launch_prefill_staged<HD, GT, 1>(st, q, kc, vc, block_table, table_stride, seq_ids, cu_q, context_lens, out,
                                            nseq, max_q_len, nh, nkv, page_shift, window, scale, softcap, paired);
  }
  hipLaunchKernelGGL((attn_prefill_kernel<HD, GT>), grid, dim3(256), 0, st, (const bf16*)q, (const bf16*)kc,
                     (const bf16*)vc, block_table, table_stride, seq_ids, cu_q, context_lens, (bf16*)out, nh, nkv,
                     page_shift, window, score_map(scale, softcap), paired);
  return check_launch("attn_prefill");
}

// How a prefill launch is cut, -1 where the launcher chooses: tiles in pairs, heads a wavefront (1, 2, 4), head
// groups a workgroup (1, 2), keys staged in LDS.
struct PrefillCut {
  int paired = -1, heads = -1, groups = -1, staged = -1;
};

template <int HD>
int launch_prefill(hipStream_t st, const void* q, const void* kc, const void* vc, const int* block_table,
                   int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out, int nseq,
                   int max_q_len, int min_prefix, int nh, int nkv, int page_shift, int window, float scale,
                   float softcap, const PrefillCut& want) {
  const int group = nh / nkv;
  // How the work is cut: tiles in pairs (an early and a late tile of the causal triangle, so workgroups finish
  // together) and as many heads per wavefront as share the keys and fit the registers (wider heads would not fit
  // four heads' state in 256) -- unless that leaves compute units without a workgroup: a short prompt is better
  // off unpaired and with a head per wavefront.  Measured at head_dim 128: one prompt of 512 tokens takes 16 us
  // as 256 workgroups and 26 us as 64.
  // (four heads a wavefront, which heads of up to 64 wide have registers for, measured slower than two at every
  // size but 8,192 tokens, where it is level: 32 heads over 8 of 64 at 2,048 tokens 66 us against 45 and 36 with
  // two and one; the kernel stays for callers that ask for it)
  const int gt_best = group % 2 == 0 ? 2 : 1;
  const int gt_most = (HD <= 64 && group % 4 == 0) ? 4 : gt_best;   // what a caller's own cut may ask for
  const long tiles = (max_q_len + 63) / 64;
  const bool can_stage = page_shift >= 3;
  auto workgroups = [&](int p, int g_, int h_ = 1) {
    return (p ? (tiles + 1) / 2 : tiles) * nkv * (group / (g_ * h_)) * nseq;
  };
  const long enough = 256;
  int paired = tiles >= 2, gt = gt_best, hw = 1;
  // every portion has at least as many keys before it as tokens in it: its tiles see about the same number of keys
  // and need no pairing, which doubles the workgroups there are to hand out
  const bool level = min_prefix >= max_q_len;
  const bool wide_ok = can_stage && group % (gt_best * 2) == 0;   // eight wavefronts: two groups of gt_best heads
  const int gt_half = gt_best >= 2 ? gt_best / 2 : 1;
  const bool half_ok = can_stage && gt_best >= 2 && group % (gt_half * 2) == 0;
  // Pairs are workgroups of one length, so they come in rounds, and a last round that is half empty costs as much
  // as a full one: pairs pay where the rounds are full (or many).  Unpaired, the tiles are of every length from one
  // block to the whole context, the longest are handed out first, and from one and a half workgroups a compute
  // unit on they balance out by themselves.  Measured, 32 heads over 8 of 128: 1,536 tokens as 384 pairs of a head
  // a wavefront 47.2 us, unpaired with eight wavefronts 36.5; 3,072 tokens as 384 pairs 134.3, unpaired with two
  // heads a wavefront 105.0; 2,048 and 4,096 tokens, whose pairs are one full round, 53.0 and 144.5 paired against
  // 55.0 and 150.1.
  // (7,168 tokens, 448 pairs: 466 against 437 us unpaired; three prompts of 1,024, 192 pairs: 50.4 against 57.2 --
  // short tiles carry a workgroup's fixed cost less well, so one round that is three quarters full still counts)
  auto full_rounds = [&](long w, long slots) {
    return (w >= slots && (w % slots == 0 || w >= 4 * slots)) || (tiles <= 16 && 4 * w >= 3 * slots && w <= slots);
  };
  const long spread = enough * 3 / 2;
  // Two to six prompts: within a launch the workgroups are handed out sequence by sequence, so unpaired the last
  // prompt's long tiles start late; with the tiles slowest over the grid (paired 2) every prompt's long tiles
  // come first, and unpaired is ahead of pairs wherever the pairs are not exactly whole rounds (32 heads over 8 of
  // 128, us: three prompts of 512 tokens 20.0 against 22.1 in pairs and 23.2 sequence by sequence, six of 512 32.1
  // against 35.0, three of 1,024 44.6 against 49.9, three of 2,048 131.6 against 147.1; 40 heads over 8, two of 512
  // 17.7 against 23.8).  With many prompts the interleaving costs more in the L2 than the order gains (sixteen of
  // 512: 80.9 against 70.5).
  const bool few = can_stage && !level && nseq >= 2 && nseq <= 6 && tiles >= 2;
  auto whole = [&](long w, long slots) { return w >= slots && w % slots == 0; };
  if (few) {
    // the kinds of workgroup from the most heads down; of each, pairs if they are whole rounds, else unpaired if
    // there are workgroups enough to balance out
    if (wide_ok && whole(workgroups(1, gt_best, 2), enough)) {
      hw = 2;
    } else if (wide_ok && workgroups(0, gt_best, 2) >= spread) {
      paired = 2, hw = 2;
    } else if (whole(workgroups(1, gt_best, 1), 2 * enough)) {
      hw = 1;
    } else if (gt_best >= 2 && workgroups(0, gt_best, 1) >= 2 * spread) {
      paired = 2, hw = 1;
    } else if (half_ok && whole(workgroups(1, gt_half, 2), enough)) {
      gt = gt_half, hw = 2;
    } else if (half_ok && workgroups(0, gt_half, 2) >= spread) {
      paired = 2, gt = gt_half, hw = 2;
    } else {
      paired = 2, gt = gt_half, hw = 1;
    }
  } else if (wide_ok && tiles > 8 && full_rounds(workgroups(1, gt_best, 2), enough)) {
    // the most work per staged key that still gives every compute unit a workgroup (measured at head_dim 128,
    // 32 heads over 8: 4,096 tokens 171 against 186 us, 8,192 tokens 624 against 648); not for many short prompts,
    // whose workgroups are over after a few blocks (16 prompts of 512 tokens: 66 against 70 us with four
    // wavefronts a workgroup, 32 of 256: 51 against 60)
    hw = 2;
  } else if (wide_ok && tiles > 8 && !level && workgroups(0, gt_best, 2) >= spread) {
    paired = 0, hw = 2;
  } else if (level && workgroups(0, gt_best, wide_ok ? 2 : 1) >= (wide_ok ? enough : 2 * enough)) {
    // (workgroups of four wavefronts want two on a compute unit: 16 heads over 8, 2,048 tokens behind 6,144, as 256
    // of them 274 us, as 256 of eight wavefronts with a head each 166)
    paired = 0;   // 2,048 tokens behind 6,144: 297 against 342 us
    hw = wide_ok ? 2 : 1;
  } else if (level && can_stage && group % 2 == 0 && workgroups(0, 1, 2) >= enough) {
    paired = 0, gt = 1, hw = 2;   // 1,024 tokens behind 7,168: 205 against 293 us
  } else if (!wide_ok && gt_best >= 2 && tiles > 8 && full_rounds(workgroups(1, gt_best, 1), 2 * enough)) {
    // whole rounds of pairs of four wavefronts, two heads each (16 heads over 8 at 8,192 tokens: 307 against 332 us)
  } else if (half_ok && tiles > 8 && full_rounds(workgroups(1, gt_half, 2), enough)) {
    gt = gt_half, hw = 2;         // 2,048 tokens: 256 pairs of eight wavefronts, a head each
  } else if (half_ok && tiles > 8 && workgroups(0, gt_half, 2) >= spread) {
    paired = 0, gt = gt_half, hw = 2;
  } else if (half_ok && workgroups(0, gt_half, 2) == enough) {
    // exactly one workgroup of eight wavefronts a compute unit, two wavefronts a SIMD and one round (two prompts
    // of 512 tokens: 16.0 us against 17.7 as pairs of four wavefronts)
    paired = 0, gt = gt_half, hw = 2;
  } else {
    if (workgroups(paired, gt) < enough) {
      if (gt > 1 && workgroups(paired, 1) >= enough) {
        gt = 1;
      } else if (workgroups(0, gt) >= enough) {
        paired = 0;
      } else {
        paired = 0;
        gt = 1;
      }
    }
    // one workgroup per compute unit is one wavefront per SIMD, which waits for every one of its own steps: then
    // rather eight wavefronts a workgroup, half of them on the other heads (measured at 2,048 tokens: 69 against 77 us)
    // (up to one and a quarter: six prompts of 512 tokens, 384 pairs, 35.6 us as they are and 40.7 with eight wavefronts)
    if (can_stage && workgroups(paired, gt) >= enough && workgroups(paired, gt) <= enough * 5 / 4 && gt >= 2 && gt == gt_best) {
      gt /= 2;
      hw = 2;
    }
    // pairs in rounds that are not full: unpaired, if that gives workgroups enough to balance out
    // (prompts of up to 512 tokens are over too soon for rounds to form: twelve of 512 tokens 60.3 us in pairs, 64.7 without)
    if (paired && tiles > 8 && !full_rounds(workgroups(1, gt, hw), hw == 2 ? enough : 2 * enough) && workgroups(0, gt, hw) >= spread)
      paired = 0;
  }
  // keys staged in LDS for pages of 8 keys or more; pages of 4 go to the kernel that reads them itself
  bool staged = can_stage;
  // a caller's own cut (tests and measurements), where it is one the kernels have
  if (want.paired >= 0) paired = want.paired == 2 ? 2 : (want.paired != 0 && tiles >= 2);
  if (want.heads >= 0) {
    PA_REQUIRE((want.heads == 1 || want.heads == 2 || want.heads == 4) && want.heads <= gt_most,
               "attn_prefill: %d heads a wavefront, this shape takes up to %d (1, 2 or 4)", want.heads, gt_most);
    gt = want.heads;
    if (want.groups < 0) hw = 1;
  }
  if (want.groups >= 0) {
    PA_REQUIRE(want.groups == 1 || (want.groups == 2 && group % (gt * 2) == 0),
               "attn_prefill: %d head groups a workgroup with %d heads a wavefront and %d heads a KV head", want.groups,
               gt, group);
    hw = want.groups;
  }
  if (want.staged >= 0) {
    PA_REQUIRE(want.staged == 0 || staged, "attn_prefill: pages of %d keys are not staged", 1 << page_shift);
    staged = want.staged != 0;
  }
  PA_REQUIRE(staged || hw == 1, "attn_prefill: two head groups a workgroup only with staged keys");
  PA_REQUIRE(gt <= gt_most, "attn_prefill: %d heads a wavefront, head_dim %d takes up to %d", gt, HD, gt_most);
#define PA_GT(GT)                                                                                                   \
  return launch_prefill_gt<HD, GT>(st, q, kc, vc, block_table, table_stride, seq_ids, cu_q, context_lens, out, nseq, \
                                   max_q_len, nh, nkv, page_shift, window, scale, softcap, paired, hw, staged)
  if constexpr (HD <= 64) {   // four heads' state of a wider head does not fit 256 registers: not built, never chosen
    if (gt == 4) PA_GT(4);
  }
  if (gt == 2) PA_GT(2);
  PA_GT(1);
#undef PA_GT
}

}  // namespace pa

using namespace pa;

#define PA_HD_SWITCH(hd, CALL)                                                                              \
  switch (hd) {                                                                                             \
    case 16: CALL(16);                                                                                      \
    case 32: CALL(32);                                                                                      \
    case 48: CALL(48);                                                                                      \
    case 64: CALL(64);                                                                                      \
    case 96: CALL(96);                                                                                      \
    case 128: CALL(128);                                                                                    \
    default: return pa::fail("MFMA attention: head_dim %d is not one of 16, 32, 48, 64, 96, 128", hd);      \
  }

static int check_common(const char* what, int nseq, int nh, int nkv, int page_size, int table_stride, int window) {
  PA_REQUIRE(nseq > 0 && nh > 0 && nkv > 0 && table_stride > 0, "%s: bad sizes sequences=%d nh=%d nkv=%d table_stride=%d",
             what, nseq, nh, nkv, table_stride);
  PA_REQUIRE(nh % nkv == 0, "%s: %d query heads are not a multiple of %d KV heads", what, nh, nkv);
  PA_REQUIRE(page_size >= 4 && (page_size & (page_size - 1)) == 0, "%s: page size %d is not a power of two >= 4", what,
             page_size);
  PA_REQUIRE(window >= 0, "%s: window %d is negative (0 means none)", what, window);
  PA_REQUIRE(nseq <= 65535, "%s: %d sequences exceed the grid", what, nseq);
  return 0;
}

// 1 if the MFMA kernels take this head_dim and page size, else 0 (the caller then uses the generic kernel).
extern "C" int pa_attn_mfma_supports(int hd, int page_size) {
  const bool hd_ok = hd == 16 || hd == 32 || hd == 48 || hd == 64 || hd == 96 || hd == 128;
  return hd_ok && page_size >= 4 && (page_size & (page_size - 1)) == 0;
}

// Workspace the decode kernel needs, in floats, for `nseq` sequences cut into at most `max_splits` splits.
extern "C" long pa_attn_decode_workspace(int nseq, int nh, int hd, int max_splits) {
  return max_splits <= 1 ? 0 : (long)nseq * nh * max_splits * (hd + 2);
}

extern "C" int pa_attn_decode(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                              int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens,
                              void* out, float* workspace, int nseq, int nh, int nkv, int hd, int page_size,
                              int window, float scale, float softcap, int split_keys, int max_splits) {
  if (nseq == 0) return 0;
  PA_REQUIRE(softcap >= 0.f, "attn_decode: a score cap of %g is negative (0 means none)", (double)softcap);
  if (int rc = check_common("attn_decode", nseq, nh, nkv, page_size, table_stride, window)) return rc;
  PA_REQUIRE(split_keys >= 32 && split_keys % 32 == 0, "attn_decode: split of %d keys is not a multiple of 32", split_keys);
  PA_REQUIRE(max_splits >= 1 && max_splits <= 65535, "attn_decode: %d splits", max_splits);
  PA_REQUIRE(max_splits == 1 || workspace, "attn_decode: no workspace for %d splits", max_splits);
  float* part_o = workspace;
  float* part_ml = workspace ? workspace + (size_t)nseq * nh * max_splits * hd : nullptr;
#define PA_CALL(HD)                                                                                                  \
  return launch_decode<HD, false>((hipStream_t)stream, q, kc, vc, block_table, table_stride, seq_ids, cu_q,         \
                                  context_lens, out, part_o, part_ml, nseq, nh, nkv, __builtin_ctz(page_size), window, \
                                  scale, softcap, split_keys, max_splits, FusedQkv{})
  PA_HD_SWITCH(hd, PA_CALL)
#undef PA_CALL
}

// 1 if pa_attn_decode_fused takes these sizes: whole-width rotation of a head_dim whose half is a multiple of
// 32, and all query heads of a KV head in one tile (two workgroups must not wait for one another's key).
extern "C" int pa_attn_decode_fused_supports(int nh, int nkv, int hd, int rot, int page_size) {
  return (hd == 64 || hd == 128) && rot == hd && nkv > 0 && nh % nkv == 0 && nh / nkv <= 16 &&
         pa_attn_mfma_supports(hd, page_size);
}

// pa_qknorm_rope_kv and pa_attn_decode in one: `qkv` is the merged projection [tokens, (nh + 2 nkv) * hd] of a
// step in which the sequences `seq_ids` feed one token each; their keys and values are written to the caches
// at `slots` and their outputs to `out`; a token's position is its sequence's context length less one.  Tokens
// of other sequences are not touched.
extern "C" int pa_attn_decode_fused(void* stream, const void* qkv, const float* q_weight, const float* k_weight,
                                    const float* cos_table, const float* sin_table, const int* slots, float eps, void* kc, void* vc, const int* block_table,
                                    int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens,
                                    void* out, float* workspace, int nseq, int nh, int nkv, int hd, int page_size,
                                    int window, float scale, float softcap, int split_keys, int max_splits) {
  if (nseq == 0) return 0;
  PA_REQUIRE(softcap >= 0.f, "attn_decode_fused: a score cap of %g is negative (0 means none)", (double)softcap);
  if (int rc = check_common("attn_decode_fused", nseq, nh, nkv, page_size, table_stride, window)) return rc;
  PA_REQUIRE(pa_attn_decode_fused_supports(nh, nkv, hd, hd, page_size), "attn_decode_fused: nh=%d nkv=%d head_dim=%d page=%d are not taken",
             nh, nkv, hd, page_size);
  PA_REQUIRE(qkv && cos_table && sin_table && slots && kc && vc, "attn_decode_fused: a null operand");
  PA_REQUIRE(split_keys >= 32 && split_keys % 32 == 0, "attn_decode_fused: split of %d keys is not a multiple of 32", split_keys);
  PA_REQUIRE(max_splits >= 1 && max_splits <= 65535, "attn_decode_fused: %d splits", max_splits);
  PA_REQUIRE(max_splits == 1 || workspace, "attn_decode_fused: no workspace for %d splits", max_splits);
  float* part_o = workspace;
  float* part_ml = workspace ? workspace + (size_t)nseq * nh * max_splits * hd : nullptr;
  const FusedQkv fq{(const bf16*)qkv, q_weight, k_weight, cos_table, sin_table, slots, eps};
  const int shift = __builtin_ctz(page_size);
  if (hd == 64)
    return launch_decode<64, true>((hipStream_t)stream, nullptr, kc, vc, block_table, table_stride, seq_ids, cu_q,
                                   context_lens, out, part_o, part_ml, nseq, nh, nkv, shift, window, scale, softcap,
                                   split_keys, max_splits, fq);
  return launch_decode<128, true>((hipStream_t)stream, nullptr, kc, vc, block_table, table_stride, seq_ids, cu_q,
                                  context_lens, out, part_o, part_ml, nseq, nh, nkv, shift, window, scale, softcap,
                                  split_keys, max_splits, fq);
}

// min_prefix: the fewest keys any of the sequences has before its portion (0 if unknown): only a hint for how
// the work is cut.
// pa_attn_prefill with the cut given: paired (tiles in pairs), heads a wavefront (1, 2, 4), head groups a
// workgroup (1, 2), staged (keys through LDS); -1 leaves one to the launcher.  A cut the shape does not take is
// refused.  Every cut gives the same result up to rounding.
extern "C" int pa_attn_prefill_cut(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                                   int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens,
                                   void* out, int nseq, int max_q_len, int min_prefix, int nh, int nkv, int hd,
                                   int page_size, int window, float scale, float softcap, int paired, int heads,
                                   int groups, int staged) {
  if (nseq == 0) return 0;
  if (int rc = check_common("attn_prefill", nseq, nh, nkv, page_size, table_stride, window)) return rc;
  PA_REQUIRE(max_q_len >= 1 && min_prefix >= 0, "attn_prefill: longest portion %d, shortest prefix %d", max_q_len, min_prefix);
  PA_REQUIRE(softcap >= 0.f, "attn_prefill: a score cap of %g is negative (0 means none)", (double)softcap);
  PrefillCut cut;
  cut.paired = paired, cut.heads = heads, cut.groups = groups, cut.staged = staged;
#define PA_CALL(HD)                                                                                                   \
  return launch_prefill<HD>((hipStream_t)stream, q, kc, vc, block_table, table_stride, seq_ids, cu_q, context_lens, \
                            out, nseq, max_q_len, min_prefix, nh, nkv, __builtin_ctz(page_size), window, scale, softcap, cut)
  PA_HD_SWITCH(hd, PA_CALL)
#undef PA_CALL
}

extern "C" int pa_attn_prefill(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                               int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens,
                               void* out, int nseq, int max_q_len, int min_prefix, int nh, int nkv, int hd,
                               int page_size, int window, float scale, float softcap) {
  if (nseq == 0) return 0;
  if (int rc = check_common("attn_prefill", nseq, nh, nkv, page_size, table_stride, window)) return rc;
  PA_REQUIRE(max_q_len >= 1 && min_prefix >= 0, "attn_prefill: longest portion %d, shortest prefix %d", max_q_len, min_prefix);
  PA_REQUIRE(softcap >= 0.f, "attn_prefill: a score cap of %g is negative (0 means none)", (double)softcap);
#define PA_CALL(HD)                                                                                                   \
  return launch_prefill<HD>((hipStream_t)stream, q, kc, vc, block_table, table_stride, seq_ids, cu_q, context_lens, \
                            out, nseq, max_q_len, min_prefix, nh, nkv, __builtin_ctz(page_size), window, scale, softcap,  \
                            PrefillCut{})
  PA_HD_SWITCH(hd, PA_CALL)
#undef PA_CALL
}
