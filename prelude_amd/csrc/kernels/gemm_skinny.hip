// C[M,N] = X[M,K] * W[N,K]^T (+ bias) for few rows (M <= 64) in bfloat16 with
// 32-bit accumulation: the matrix product of decode steps, where every weight
// is read once and the time is the time to stream W from HBM.
//
// A workgroup owns 16 rows of W (16 outputs per token) and all of K; its
// wavefronts take the 64-wide k-steps in turn and are summed through LDS in
// wavefront order.  Both operands go from memory straight into
// v_mfma_f32_16x16x32_bf16 registers: W^T tile as A (row = output n), X^T as B
// (column = token m), so a lane ends up with four consecutive n of one token.
// Within a k-step a lane reads 32 contiguous bytes of its row (k0 + 16g .. +15):
// the first half feeds one MFMA, the second half the next, and X is read with
// the same pattern, so the order of k inside the step is the same on both
// sides; a wavefront's loads cover whole 128-byte lines of 16 rows.
//
// What keeps HBM busy is bytes in flight, not the number of compute units at
// work: a narrow weight (N = 2560 gives 160 tiles for 256 units) gets 16
// wavefronts per workgroup, a wide one 4, so that some thousands of wavefronts
// each have two k-steps of loads outstanding.  Nothing is split across
// workgroups, so there is no workspace, no counter and no fence, and the
// result of a row depends on the weight's shape alone.
//
// Epilogues: plain (bfloat16 or float32 out, optional bias), and SiLU(gate)*up
// for a weight whose rows alternate gate_j, up_j: a lane's four outputs are two
// (gate, up) pairs, and [M, N/2] is written with no [M, N] intermediate.
//
// Reference counterpart: the GEMM dispatch of crates/prelude-cuda/src/ops/gemm.rs:35-137
// (library kernels there; 32-bit accumulation as there, :151, :365) and the
// activation of crates/prelude-cuda/src/kernels/kernels_src/elementwise/silu_mul.cu:26-33.
#include "common.h"
#include "api.h"


namespace pa {

constexpr int kSkinnyMaxM = 64;
constexpr int kDepth = 2;  // k-steps of loads a wavefront keeps in flight from a row-major weight

struct Frag {
  bf16x8 lo, hi;
};

__device__ __forceinline__ Frag load_frag(const bf16* row, int k0, int k, bool ok) {
  Frag f;
  const bool lo_ok = ok && k0 + 8 <= k, hi_ok = ok && k0 + 16 <= k;
  if (lo_ok) {
    f.lo = *reinterpret_cast<const bf16x8*>(row + k0);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) f.lo[i] = (bf16)0.f;
  }
  if (hi_ok) {
    f.hi = *reinterpret_cast<const bf16x8*>(row + k0 + 8);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) f.hi[i] = (bf16)0.f;
  }
  return f;
}

enum Epilogue : int { kPlain = 0, kSiluMul = 1 };

// NT tiles of 16 rows of W per workgroup: with two, every X fragment serves two products, which halves the
// share of the loads that X makes up (X comes from L2, but the loads cost the same as any).
// A fragment of a weight stored in tiles (see pa_pack_tiles): the wavefront's 64 lanes read 1 KB side by side.
// No load of the tiled kernel stands under a condition: a step past the end reads the last step again (its
// product is left out), a row past m reads row 0 (its column of the result is never stored), and columns past K
// read the row's first ones (the tiles hold zeros there, and a row is only ever mixed with itself).  Straight
// code is a microsecond a product faster at 8 and 16 rows than loads behind lane masks, and it is what lets the
// compiler count the loads in flight at all: after a load that may or may not have been issued it waits for all
// of them.  (With the count right, more than one step in flight per wavefront was measured again, 2 to 4 steps
// at the shapes of a 4B model: still slower than one, by 5 to 50 %.)
__device__ __forceinline__ Frag load_tiled(const bf16* tile, int step, int lane) {
  Frag f;
  const bf16* p = tile + (size_t)step * 1024 + lane * 8;
  f.lo = *reinterpret_cast<const bf16x8*>(p);
  f.hi = *reinterpret_cast<const bf16x8*>(p + 512);
  return f;
}

// X for a tiled product: columns at, at + 8 .. of a row of k columns, both halves.  A half that would pass the
// row's end reads the row's first eight columns instead (k is a multiple of 8 and at least 8): memory of the same
// row, always there, and finite where the row is; the tile holds zeros at those places.
__device__ __forceinline__ Frag load_x_always(const bf16* row, int at, int k) {
  Frag f;
  f.lo = *reinterpret_cast<const bf16x8*>(row + (at + 8 <= k ? at : 0));
  f.hi = *reinterpret_cast<const bf16x8*>(row + (at + 16 <= k ? at + 8 : 0));
  return f;
}

template <int MT, int NT, int WAVES, typename TC, int EPI, bool TILED, int DEPTH>
__global__ __launch_bounds__(WAVES* kWave) void gemm_skinny_kernel(const bf16* __restrict__ x,
                                                                   const bf16* __restrict__ w,
                                                                   const float* __restrict__ bias,
                                                                   TC* __restrict__ c, int m, int n, int k, long ldx,
                                                                   long ldc, int act, int steps_per_slice) {
  __shared__ float red[WAVES][NT * MT][kWave][4];
  // the wavefront's number as a scalar: what depends on it (the steps it takes, the loop's end) is then uniform
  // for the compiler too, and a branch on it is a branch, not a mask
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  const int n0 = blockIdx.x * 16 * NT;
  // grid.y cuts K into slices of steps_per_slice k-steps, each with an output of its own (32-bit, m * ldc apart) for
  // a reader that adds them; one slice: all of K
  const int steps_lo = blockIdx.y * steps_per_slice;
  const int steps_all = (k + 63) / 64;
  const int steps = steps_lo + steps_per_slice < steps_all ? steps_lo + steps_per_slice : steps_all;
  if (gridDim.y > 1) {
    c += (size_t)blockIdx.y * m * ldc;
    if (blockIdx.y) bias = nullptr;
  }

  bool n_ok[NT];
  const bf16* wrow[NT];
#pragma unroll
  for (int u = 0; u < NT; ++u) {
    n_ok[u] = TILED ? n0 + 16 * u < n : n0 + 16 * u + r < n;
    wrow[u] = TILED ? w + (size_t)(n_ok[u] ? n0 / 16 + u : 0) * steps_all * 1024
                    : w + (size_t)(n_ok[u] ? n0 + 16 * u + r : 0) * k + 16 * g;
  }
  const bf16* xrow[MT];
  bool m_ok[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    m_ok[t] = 16 * t + r < m;
    // a tiled product addresses X from the row's start (its loads stand under no condition and must stay inside the row)
    xrow[t] = x + (size_t)(m_ok[t] ? 16 * t + r : 0) * ldx + (TILED ? 0 : 16 * g);
  }
  f32x4 acc[NT][MT];
#pragma unroll
  for (int u = 0; u < NT; ++u)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // DEPTH k-steps in flight per wavefront: a ring of fragments, refilled as soon as a slot has been used.
  // Steps past the end load zeros (rows) or the last step again, left out of the sums (tiles): no tail handling.
  const int kk = k - 16 * g;
  const int last = steps - 1;
  Frag wbuf[DEPTH][NT], xbuf[DEPTH][MT];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    const int s = steps_lo + wave + d * WAVES;
    const int sc = s < steps ? s : last;
#pragma unroll
    for (int u = 0; u < NT; ++u)
      wbuf[d][u] = TILED ? load_tiled(wrow[u], sc, lane) : load_frag(wrow[u], s * 64, kk, n_ok[u] && s < steps);
#pragma unroll
    for (int t = 0; t < MT; ++t)
      xbuf[d][t] = TILED ? load_x_always(xrow[t], sc * 64 + 16 * g, k) : load_frag(xrow[t], s * 64, kk, m_ok[t] && s < steps);
  }
  for (int s0 = steps_lo + wave; s0 < steps; s0 += WAVES * DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      Frag wc[NT], xc[MT];
#pragma unroll
      for (int u = 0; u < NT; ++u) wc[u] = wbuf[d][u];
#pragma unroll
      for (int t = 0; t < MT; ++t) xc[t] = xbuf[d][t];
      const int next = s0 + (d + DEPTH) * WAVES;
      const int nc = next < steps ? next : last;
#pragma unroll
      for (int u = 0; u < NT; ++u)
        wbuf[d][u] = TILED ? load_tiled(wrow[u], nc, lane) : load_frag(wrow[u], next * 64, kk, n_ok[u] && next < steps);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        xbuf[d][t] = TILED ? load_x_always(xrow[t], nc * 64 + 16 * g, k)
                           : load_frag(xrow[t], next * 64, kk, m_ok[t] && next < steps);
      // with two tiles or more, every load of the next step is on its way before this step's products: left to
      // itself the compiler moves the loads of a second tile behind the products of the first (fewer registers, and
      // half the bytes in flight: [5120, 25600] at 8 rows took 69 us so, 49 with the loads held together); with one
      // tile its own order is the faster one by half a microsecond
      if (TILED && NT > 1) __builtin_amdgcn_sched_barrier(0);
      if (TILED && s0 + d * WAVES >= steps) continue;   // a step past the end: read again, not counted (no load inside)
#pragma unroll
      for (int u = 0; u < NT; ++u)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[u].lo, xc[t].lo, acc[u][t], 0, 0, 0);
          acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[u].hi, xc[t].hi, acc[u][t], 0, 0, 0);
        }
    }
  }
  // the wavefronts' shares, added in wavefront order; wavefront u finishes tile u (NT <= WAVES)
#pragma unroll
  for (int u = 0; u < NT; ++u)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][u * MT + t][lane][i] = acc[u][t][i];
  __syncthreads();
  if (wave >= NT) return;
  const int u = wave;
  f32x4 fin[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = red[0][u * MT + t][lane][i];
#pragma unroll
      for (int q = 1; q < WAVES; ++q) v += red[q][u * MT + t][lane][i];
      fin[t][i] = v;
    }
  // epilogue: lane (g, r) writes four consecutive n of token 16t + r
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int mi = 16 * t + r;
    if (mi >= m) continue;
    const int nb = n0 + 16 * u + 4 * g;
    if (EPI == kSiluMul) {
      // rows alternate gate_j, up_j: outputs nb/2 and nb/2 + 1
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int nn = nb + 2 * j;
        if (nn + 1 < n) {
          const float gate = fin[t][2 * j], up = fin[t][2 * j + 1];
          c[(size_t)mi * ldc + nn / 2] = from_f32<TC>(gate_activation(gate, act) * up);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (nb + i < n) {
          float v = fin[t][i];
          if (bias) v += bias[nb + i];
          c[(size_t)mi * ldc + nb + i] = from_f32<TC>(v);
        }
      }
    }
  }
}

// Shape of the launch for an [n, k] weight: tiles of 16 rows per workgroup, wavefronts per workgroup, k-steps
// of loads a wavefront keeps in flight.  Row-major: wide weights take two tiles; then about 3000 wavefronts on
// the chip, each with at least two k-steps.  Depends on the weight's shape and layout only, never on the batch.
static void skinny_shape(int m, int n, int k, int mt, bool tiled, int* nt, int* waves, int* depth) {
  const int tiles = (n + 15) / 16, steps = (k + 63) / 64;
  if (tiled) {
    // measured over (tiles per workgroup, wavefronts, depth) at the shapes of a 4B model: one step in flight per
    // wavefront streams a tiled weight best; long rows want 16 wavefronts, the widest weights two tiles
    // (how K is split over wavefronts fixes the order of the sums and follows the weight alone; the tiles per
    // workgroup do not touch it, and more than 8 rows read X often enough that sharing it over two tiles pays)
    *nt = tiles >= 4096 ? 2 : 1;
    if (m > 8 && tiles >= 320) *nt *= 2;   // [5120, 5120] at 16 rows: 14 against 19 us
    if (mt > 1 && *nt > 2) *nt = 2;
    *waves = steps >= 128 ? 16 : 8;
    if (steps >= 128 && (mt > 1 || tiles >= 320)) {
      // long rows: 16 wavefronts' sums of more than 16 rows would not fit LDS, and where there are tiles enough,
      // eight wavefronts on two tiles stream better than sixteen on one ([5120, 25600] at 1 / 8 / 16 rows:
      // 52 / 51 / 57 against 55 / 60 / 83 us; [4096, 12288], 256 tiles, is still better off with sixteen on one)
      *waves = 8;
      // ... two tiles except for up to 4 rows of rows shorter than 256 steps ([5120, 8192] at 1 / 4 / 8 rows:
      // 17 / 17 / 20 us on one tile against 19 to 20 on two)
      if (tiles >= 320 && (m > 4 || steps >= 256)) *nt = 2;
    }
    *depth = 1;
    return;
  }
  *nt = mt > 1 ? 1 : (tiles >= 4096 ? 4 : (tiles >= 768 ? 2 : 1));
  const int wgs = (tiles + *nt - 1) / *nt;
  int w = 4;
  while (w < 16 && wgs * w < 3000 && steps / (2 * w) >= 2) w *= 2;
  *waves = w;
  *depth = kDepth;
}

// The kernels that are built: the (tiles per workgroup, wavefronts) that skinny_shape can ask for with this many
// row tiles and this layout.  Sixteen wavefronts leave 128 registers each, enough for 16 rows of one tile: a tiled
// weight never takes them with more rows, a row-major one does (its split of K must not depend on the rows, and
// beyond 16 rows it is not the layout that serving uses) and spills.
template <int MT, bool TILED, int NT, int WV>
constexpr bool skinny_built() {
  if (TILED) return WV == 8 ? (NT <= 2 || MT == 1) : (WV == 16 && MT == 1 && NT == 1);
  if (MT > 1) return NT == 1;
  return NT == 1 || (NT == 2 && WV <= 8) || (NT == 4 && WV == 4);
}

template <int MT, int NT, int WV, typename TC, int EPI, bool TILED, int DEPTH>
int launch_skinny_as(hipStream_t st, const void* x, const void* w, const float* bias, void* c, int m, int n, int k,
                     long ldx, long ldc, int act, int slices = 1) {
  if constexpr (skinny_built<MT, TILED, NT, WV>()) {
    const int steps = (k + 63) / 64, per = (steps + slices - 1) / slices;
    dim3 grid(((n + 15) / 16 + NT - 1) / NT, (steps + per - 1) / per);
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, NT, WV, TC, EPI, TILED, DEPTH>), grid, dim3(WV * kWave), 0, st,
                       (const bf16*)x, (const bf16*)w, bias, (TC*)c, m, n, k, ldx, ldc, act, per);
    return check_launch("gemm_skinny");
  } else {
    return pa::fail("gemm_skinny: no kernel for %d row tiles with %d tiles a workgroup on %d wavefronts (%s weight)", MT,
                    NT, WV, TILED ? "tiled" : "row-major");
  }
}

template <int MT, typename TC, int EPI, bool TILED, int DEPTH>
int launch_skinny_depth(hipStream_t st, const void* x, const void* w, const float* bias, void* c, int m, int n, int k,
                        long ldx, long ldc, int act, int slices = 1, int waves_asked = 0) {
  int nt, waves, depth;
  skinny_shape(m, n, k, MT, TILED, &nt, &waves, &depth);
  if (waves_asked) waves = waves_asked, nt = 1;
#define PA_AS(NT, WV) \
  return launch_skinny_as<MT, NT, WV, TC, EPI, TILED, DEPTH>(st, x, w, bias, c, m, n, k, ldx, ldc, act, slices)
#define PA_WAVES(NT)     \
  switch (waves) {       \
    case 16: PA_AS(NT, 16); \
    case 8: PA_AS(NT, 8);   \
    case 4: PA_AS(NT, 4);   \
  }                      \
  break;
  switch (nt) {
    case 4: PA_WAVES(4)
    case 2: PA_WAVES(2)
    case 1: PA_WAVES(1)
  }
#undef PA_WAVES
#undef PA_AS
  return pa::fail("gemm_skinny: no kernel with %d tiles a workgroup on %d wavefronts", nt, waves);
}

template <int MT, typename TC, int EPI, bool TILED>
int launch_skinny(hipStream_t st, const void* x, const void* w, const float* bias, void* c, int m, int n, int k,
                  long ldx, long ldc, int act) {
  // the depth is part of the kernel's type: one step in flight for tiles, kDepth for rows (see skinny_shape)
  return launch_skinny_depth<MT, TC, EPI, TILED, TILED ? 1 : kDepth>(st, x, w, bias, c, m, n, k, ldx, ldc, act);
}

template <typename TC, int EPI>
int launch_skinny_mt(hipStream_t st, const void* x, const void* w, const float* bias, void* c, int m, int n, int k,
                     long ldx, long ldc, int act, int tiled) {
  if (tiled) {
    switch ((m + 15) / 16) {
      case 1: return launch_skinny<1, TC, EPI, true>(st, x, w, bias, c, m, n, k, ldx, ldc, act);
      case 2: return launch_skinny<2, TC, EPI, true>(st, x, w, bias, c, m, n, k, ldx, ldc, act);
      case 3: return launch_skinny<3, TC, EPI, true>(st, x, w, bias, c, m, n, k, ldx, ldc, act);
      default: return launch_skinny<4, TC, EPI, true>(st, x, w, bias, c, m, n, k, ldx, ldc, act);
    }
  }
  switch ((m + 15) / 16) {
    case 1: return launch_skinny<1, TC, EPI, false>(st, x, w, bias, c, m, n, k, ldx, ldc, act);
    case 2: return launch_skinny<2, TC, EPI, false>(st, x, w, bias, c, m, n, k, ldx, ldc, act);
    case 3: return launch_skinny<3, TC, EPI, false>(st, x, w, bias, c, m, n, k, ldx, ldc, act);
    default: return launch_skinny<4, TC, EPI, false>(st, x, w, bias, c, m, n, k, ldx, ldc, act);
  }
}

__global__ void pack_tiles_kernel(const bf16* __restrict__ w, bf16* __restrict__ out, int n, int k, int steps,
                                  long total) {
  const long p = (long)blockIdx.x * blockDim.x + threadIdx.x;   // piece [tile][step][half][g][r]
  if (p >= total) return;
  const int r = p % 16, g = (p / 16) % 4, half = (p / 64) % 2;
  const long ts = p / 128;
  const int step = ts % steps;
  const long tile = ts / steps;
  const long row = 16 * tile + r;
  const int col = 64 * step + 16 * g + 8 * half;
  bf16x8 v;
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = (row < n && col + j < k) ? w[row * k + col + j] : (bf16)0.f;
  *reinterpret_cast<bf16x8*>(out + p * 8) = v;
}

}  // namespace pa

using namespace pa;

// epilogue 0: C[m, n] (+ bias); 1: C[m, n/2] = silu(gate) * up over a weight whose rows alternate gate_j, up_j.
// out[tile][step][half][g][r][j] = w[16 tile + r][64 step + 16 g + 8 half + j], zero beyond n and k: every
// fragment a wavefront of the product kernel loads is then 1 KB of consecutive memory, and a workgroup's tile
// one run of ceil(k / 64) * 2 KB.  `out` holds ceil(n / 16) * ceil(k / 64) * 1024 elements.
extern "C" int pa_pack_tiles(void* stream, const void* w, void* out, int n, int k) {
  PA_REQUIRE(n > 0 && k > 0, "pack_tiles: bad sizes n=%d k=%d", n, k);
  const long tiles = (n + 15) / 16, steps = (k + 63) / 64;
  const long total = tiles * steps * 128;   // 16-byte pieces
  hipLaunchKernelGGL(pack_tiles_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const bf16*)w, (bf16*)out, n, k, (int)steps, total);
  return check_launch("pack_tiles");
}

// tiled 1: w is the weight in tiles (pa_pack_tiles).  epilogue 0: C (+ bias); 1 + a: C[m, n/2] = act_a(gate) * up
// over rows that alternate gate_j, up_j, a one of the GateActivation codes (1: SiLU, 2: GELU in its tanh form).
extern "C" int pa_gemm_skinny(void* stream, int out_dtype, int epilogue, const void* x, const void* w,
                              const float* bias, void* c, int m, int n, int k, long ldx, long ldc, int tiled) {
  if (m == 0 || n == 0) return 0;
  PA_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_skinny: bad sizes m=%d n=%d k=%d", m, n, k);
  PA_REQUIRE(m <= kSkinnyMaxM, "gemm_skinny: %d rows exceed %d", m, kSkinnyMaxM);
  PA_REQUIRE(k % 8 == 0 && ldx % 8 == 0, "gemm_skinny: k=%d and the row stride %ld must be multiples of 8", k, ldx);
  PA_REQUIRE(ldx >= k, "gemm_skinny: row stride %ld is smaller than k=%d", ldx, k);
  PA_REQUIRE(epilogue >= 0 && epilogue <= kActCount, "gemm_skinny: unknown epilogue %d", epilogue);
  const bool gated = epilogue != kPlain;
  const int act = gated ? epilogue - 1 : 0;
  PA_REQUIRE(!gated || (n % 2 == 0 && !bias), "gemm_skinny: the gated epilogue needs an even n and no bias");
  PA_REQUIRE(ldc >= (gated ? n / 2 : n), "gemm_skinny: output row stride %ld is too small", ldc);

  hipStream_t st = (hipStream_t)stream;
  if (!gated && out_dtype == kBF16)
    return launch_skinny_mt<bf16, kPlain>(st, x, w, bias, c, m, n, k, ldx, ldc, act, tiled);
  if (!gated && out_dtype == kF32)
    return launch_skinny_mt<float, kPlain>(st, x, w, bias, c, m, n, k, ldx, ldc, act, tiled);
  if (gated && out_dtype == kBF16)
    return launch_skinny_mt<bf16, kSiluMul>(st, x, w, bias, c, m, n, k, ldx, ldc, act, tiled);
  return pa::fail("gemm_skinny: unsupported output type %d with epilogue %d", out_dtype, epilogue);
}

// pa_gemm_skinny of up to 16 rows of a tiled weight with K cut into `slices` (the last may be shorter; the launch
// makes ceil(steps / ceil(steps / slices)) of them, which pa_gemm_skinny_slices tells): parts[slice][m][n] in 32-bit,
// the bias in slice 0, for a reader that adds the slices in their order (the residual add + RMSNorm does).  A narrow
// weight has too few tiles to give every compute unit a workgroup; its slices do.  waves: 8 or 16 wavefronts a
// workgroup, 0 for the launcher's choice by the slice's length.
extern "C" int pa_gemm_skinny_slices(int k, int slices) {
  const int steps = (k + 63) / 64;
  if (slices < 1) slices = 1;
  const int per = (steps + slices - 1) / slices;
  return (steps + per - 1) / per;
}
extern "C" int pa_gemm_skinny_sliced(void* stream, const void* x, const void* w, const float* bias, float* parts, int m,
                                     int n, int k, long ldx, int slices, int waves) {
  if (m == 0 || n == 0) return 0;
  PA_REQUIRE(m > 0 && m <= 16 && n > 0 && k > 0, "gemm_skinny_sliced: bad sizes m=%d (up to 16) n=%d k=%d", m, n, k);
  PA_REQUIRE(k % 8 == 0 && ldx % 8 == 0 && ldx >= k, "gemm_skinny_sliced: k=%d and the row stride %ld must be multiples of 8, the stride at least k", k, ldx);
  PA_REQUIRE(slices >= 1 && slices <= (k + 63) / 64, "gemm_skinny_sliced: %d slices of %d steps", slices, (k + 63) / 64);
  PA_REQUIRE(waves == 0 || waves == 8 || waves == 16, "gemm_skinny_sliced: %d wavefronts a workgroup (8, 16 or 0)", waves);
  PA_REQUIRE(x && w && parts, "gemm_skinny_sliced: an operand is missing");
  if (!waves) waves = ((k + 63) / 64 + slices - 1) / slices >= 128 ? 16 : 8;
  return launch_skinny_depth<1, float, kPlain, true, 1>((hipStream_t)stream, x, w, bias, parts, m, n, k, ldx, n, 0, slices, waves);
}
