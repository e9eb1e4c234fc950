// C[M,N] = X[M,K] * W[N,K]^T for many rows (beyond what gemm_mid.hip takes) in bfloat16 with 32-bit accumulation,
// from the weight in tiles (pa_pack_tiles): prompt portions of some hundred to some thousand tokens.
//
// The output is tiled both ways.  A workgroup of four wavefronts owns 16 MT rows of X and 64 NT rows of W; every
// wavefront owns all of the workgroup's rows of X and NT tiles of 16 rows of W, so it holds MT x NT accumulator
// tiles and every fragment it loads feeds NT (an X fragment) or MT (a W fragment) products.  X goes through LDS, a
// step of 64 columns at a time, staged through registers as many steps ahead of its use as the weight (a ring of
// register sets, two LDS buffers, one barrier a step); W goes from memory straight into registers, as in gemm_mid.hip: the
// tiled layout makes every fragment 1 KB of consecutive memory in the lanes' order, so it needs no LDS, and no
// two wavefronts of a workgroup load the same bytes.
//
// Workgroups that share their rows of W (the row tiles of one column group) get consecutive places on one XCD:
// its L2 then sees a weight's bytes asked for by all of them while they are there.  K may be cut into slices
// (grid.y) whose 32-bit partial sums the reader adds (as gemm_mid.hip: the residual add + RMSNorm kernel does it
// as it loads), for narrow weights that would otherwise leave most compute units idle.
//
// Epilogues: bfloat16 out (+ bias), SiLU(gate) * up over rows that alternate gate_j, up_j, or the slices.
//
// Reference counterpart: the GEMM dispatch of crates/prelude-cuda/src/ops/gemm.rs:35-137 (library kernels there).
#include "common.h"
#include "api.h"

namespace pa {

struct TallFrag {
  bf16x8 lo, hi;
};

__device__ __forceinline__ TallFrag tall_load_w(const bf16* tile, int step, int lane) {
  TallFrag f;
  const bf16* p = tile + (size_t)step * 1024 + lane * 8;
  f.lo = *reinterpret_cast<const bf16x8*>(p);
  f.hi = *reinterpret_cast<const bf16x8*>(p + 512);
  return f;
}

enum TallEpilogue : int { kTallPlain = 0, kTallSiluMul = 1, kTallSlices = 2 };

constexpr int kTallWaves = 4;
constexpr int kTallThreads = kTallWaves * kWave;
constexpr int kTallRow = 64 + 16;   // an LDS row: 32 bytes past the step's 64 columns (measured: 16-byte reads of sixteen rows run
                                    // at the full rate at such a stride, at half of it with 16 bytes of padding)

// MT tiles of 16 rows of X a workgroup, NT tiles of 16 rows of W a wavefront, a ring of DEPTH steps of W in registers,
// OCC workgroups a compute unit the registers are budgeted for.
template <int MT, int NT, int DEPTH, int OCC, typename TC, int EPI>
__global__ __launch_bounds__(kTallThreads, OCC) void gemm_tall_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ w, const float* __restrict__ bias, TC* __restrict__ c,
    float* __restrict__ parts, int m, int n, int k, long ldx, long ldc, int steps_per_slice, int row_tiles,
    int col_groups, int act) {
  static_assert(MT % 2 == 0 && DEPTH % 2 == 0, "pieces and buffers are dealt out in twos");
  constexpr int ROWS = 16 * MT;
  constexpr int PIECES = ROWS * 8 / kTallThreads;   // 16-byte pieces of a step a thread stages
  __shared__ __align__(16) bf16 xs[2][ROWS][kTallRow];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  // every eighth workgroup runs on the same XCD: a column group's row tiles side by side there
  const int xcd = blockIdx.x % 8, place = blockIdx.x / 8;
  const int rt = place % row_tiles, cg = (place / row_tiles) * 8 + xcd;
  if (cg >= col_groups) return;
  const int tiles = (n + 15) / 16, steps = (k + 63) / 64;
  const int tile0 = (cg * kTallWaves + wave) * NT;
  const bf16* wt[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) wt[j] = w + (size_t)(tile0 + j < tiles ? tile0 + j : tiles - 1) * steps * 1024;
  const int m0 = rt * ROWS;
  const int s_begin = blockIdx.y * steps_per_slice;
  const int s_end = s_begin + steps_per_slice < steps ? s_begin + steps_per_slice : steps;
  const int last = s_end - 1;

  // piece p = tid + j * threads of a step: columns 8 (p % 8) .. + 7 of row p / 8.  A row past m reads row 0 and
  // columns past k the row's first ones: memory that is there and finite (the columns meet zeros in the tile, the
  // rows are never stored).
  const bf16* src[PIECES];
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int p = threadIdx.x + j * kTallThreads;
    const int row = m0 + p / 8;
    src[j] = x + (size_t)(row < m ? row : 0) * ldx;
  }
  const int col = 8 * (threadIdx.x % 8);
  bf16x8 staged[DEPTH][PIECES];
  auto stage_load = [&](int set, int step) {
    const int at = (step < s_end ? step : last) * 64 + col;
#pragma unroll
    for (int j = 0; j < PIECES; ++j) staged[set][j] = *reinterpret_cast<const bf16x8*>(src[j] + (at + 8 <= k ? at : 0));
  };
  auto stage_store = [&](int set, int buf) {
#pragma unroll
    for (int j = 0; j < PIECES; ++j)
      *reinterpret_cast<bf16x8*>(&xs[buf][(threadIdx.x + j * kTallThreads) / 8][col]) = staged[set][j];
  };

  f32x4 acc[MT][NT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[t][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // No load stands under a condition (a step past the slice's end reads the last one again and counts nothing),
  // so the compiler knows how many loads are in flight at every use and waits for no more than it must.
  TallFrag wb[DEPTH][NT];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
#pragma unroll
    for (int j = 0; j < NT; ++j) wb[d][j] = tall_load_w(wt[j], s_begin + d < s_end ? s_begin + d : last, lane);
  // set d holds step s_begin + d; step 0 goes to LDS at once and its set takes step DEPTH
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) stage_load(d, s_begin + d);
  stage_store(0, 0);
  stage_load(0, s_begin + DEPTH);
  __syncthreads();

  for (int s0 = s_begin; s0 < s_end; s0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const int s = s0 + u;          // past the slice's end (the ring spans several steps): loads again, no products
      const int buf = u & 1;         // s - s_begin and u have the same parity: DEPTH is even
      TallFrag wc[NT];
#pragma unroll
      for (int j = 0; j < NT; ++j) wc[j] = wb[u][j];
      // the next step's X into the other buffer (everyone left it at the last barrier), and in its registers' place
      // the step DEPTH steps on: asked for before the weight, so that waiting for it later waits for nothing newer.
      // Loads come back in the order they were asked for, so everything is asked for the same DEPTH steps ahead:
      // a wait for a load of short lead would wait for every older load of long lead too.
      stage_store((u + 1) % DEPTH, buf ^ 1);
      stage_load((u + 1) % DEPTH, s + 1 + DEPTH);
#pragma unroll
      for (int j = 0; j < NT; ++j) wb[u][j] = tall_load_w(wt[j], s + DEPTH < s_end ? s + DEPTH : last, lane);
      if (s < s_end) {
        bf16x8 xf[2][2];
        {
          const bf16* xr = &xs[buf][r][16 * g];
          xf[0][0] = *reinterpret_cast<const bf16x8*>(xr);
          xf[0][1] = *reinterpret_cast<const bf16x8*>(xr + 8);
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          if (t + 1 < MT) {   // the next row tile's fragments, under this one's products
            const bf16* xr = &xs[buf][16 * (t + 1) + r][16 * g];
            xf[(t + 1) & 1][0] = *reinterpret_cast<const bf16x8*>(xr);
            xf[(t + 1) & 1][1] = *reinterpret_cast<const bf16x8*>(xr + 8);
          }
#pragma unroll
          for (int j = 0; j < NT; ++j) {
            acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[j].lo, xf[t & 1][0], acc[t][j], 0, 0, 0);
            acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[j].hi, xf[t & 1][1], acc[t][j], 0, 0, 0);
          }
        }
      }
      __syncthreads();
    }
  }

  // lane (g, r) holds four consecutive n of row 16 t + r of the row tile
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    if (tile0 + j >= tiles) continue;
    const int nb = 16 * (tile0 + j) + 4 * g;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int mi = m0 + 16 * t + r;
      if (mi >= m) continue;
      if (EPI == kTallSlices) {
        float* dst = parts + ((size_t)blockIdx.y * m + mi) * n + nb;
        if (nb + 3 < n && n % 4 == 0) {
          float4 v{acc[t][j][0], acc[t][j][1], acc[t][j][2], acc[t][j][3]};
          if (bias && blockIdx.y == 0) v.x += bias[nb], v.y += bias[nb + 1], v.z += bias[nb + 2], v.w += bias[nb + 3];
          *reinterpret_cast<float4*>(dst) = v;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (nb + i < n) dst[i] = acc[t][j][i] + (bias && blockIdx.y == 0 ? bias[nb + i] : 0.f);
        }
      } else if (EPI == kTallSiluMul) {
        TC* dst = c + (size_t)mi * ldc + nb / 2;
        if (nb + 3 < n) {
          const float g0 = acc[t][j][0], u0 = acc[t][j][1], g1 = acc[t][j][2], u1 = acc[t][j][3];
          dst[0] = from_f32<TC>(gate_activation(g0, act) * u0);
          dst[1] = from_f32<TC>(gate_activation(g1, act) * u1);
        } else if (nb + 1 < n) {
          const float g0 = acc[t][j][0], u0 = acc[t][j][1];
          dst[0] = from_f32<TC>(gate_activation(g0, act) * u0);
        }
      } else {
        TC* dst = c + (size_t)mi * ldc + nb;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (nb + i < n) {
            float v = acc[t][j][i];
            if (bias) v += bias[nb + i];
            dst[i] = from_f32<TC>(v);
          }
        }
      }
    }
  }
}

template <int MT, int NT, int DEPTH, int OCC, typename TC, int EPI>
int launch_tall(hipStream_t st, const void* x, const void* w, const float* bias, void* c, float* parts, int m, int n, int k,
                long ldx, long ldc, int slices, int act) {
  const int tiles = (n + 15) / 16, steps = (k + 63) / 64;
  const int sps = (steps + slices - 1) / slices;
  const int row_tiles = (m + 16 * MT - 1) / (16 * MT);
  const int col_groups = (tiles + kTallWaves * NT - 1) / (kTallWaves * NT);
  dim3 grid((unsigned)((col_groups + 7) / 8 * 8 * row_tiles), (unsigned)((steps + sps - 1) / sps));
  hipLaunchKernelGGL((gemm_tall_kernel<MT, NT, DEPTH, OCC, TC, EPI>), grid, dim3(kTallThreads), 0, st, (const bf16*)x,
                     (const bf16*)w, bias, (TC*)c, parts, m, n, k, ldx, ldc, sps, row_tiles, col_groups, act);
  return check_launch("gemm_tall");
}

template <typename TC, int EPI>
int launch_tall_shape(hipStream_t st, const void* x, const void* w, const float* bias, void* c, float* parts, int m, int n,
                      int k, long ldx, long ldc, int slices, int mt, int nt, int act = 0) {
#define PA_TALL(MT, NT, D, OCC) \
  if (mt == MT && nt == NT) return launch_tall<MT, NT, D, OCC, TC, EPI>(st, x, w, bias, c, parts, m, n, k, ldx, ldc, slices, act)
  // a ring of two steps: four and six measured the same (the loop is not waiting for the loads' latency)
  PA_TALL(4, 2, 2, 2);
  PA_TALL(4, 3, 2, 2);
  PA_TALL(8, 2, 2, 2);
  PA_TALL(8, 3, 2, 2);
#undef PA_TALL
  return pa::fail("gemm_tall: no kernel of %d row tiles a workgroup and %d tiles a wavefront", mt, nt);
}

}  // namespace pa

using namespace pa;

// The workgroup's shape the launcher takes for a product of m rows by an [n, k] weight in `slices` slices:
// out[0] = tiles of 16 rows of X a workgroup (4 or 8), out[1] = tiles of 16 rows of W a wavefront (2 or 3).
//
// The kernel's time follows the bytes its workgroups pull in (with the loop's products and LDS traffic taken out the
// loads alone take four fifths of it: a [19456, 2560] weight at 256 rows 53 us as 64 x 128 tiles, which move 600 MB,
// 37 us as 128 x 192 tiles, which move 330 MB; the kernel 55 and 47; some 9 to 11 TB/s into all compute units
// together, of which a tenth comes from memory, every byte of W once, and the rest from L2), and a compute unit
// pulls at one rate with one workgroup on it and at 1.4 times that with two (the same product at 512 rows, twice
// the workgroups: 70 us).  So a shape is priced at the bytes a step of one workgroup brings in, times what the
// fullest compute unit has to work off: 1 for one workgroup, 1.43 for two at once, and so on in rounds of two; the
// cheapest shape is taken.  Measured over the four shapes at the widths of 0.6B to 32B models, 129 to 512 rows, the
// shape so chosen is the fastest or within a twentieth of it: small weights keep 64 x 128 at every number of rows
// ([6144, 1024] at 256 rows 11.7 us against 21.5 as 128 x 192), 384 rows of a large one take 128 x 128 ([19456, 2560]
// 54.8 against 68.8, [5120, 17408] in four slices 87.5 against 113.8), 256 and 512 rows 128 x 192.
static double tall_price(int mt, int nt, int m, int tiles, int slices) {
  const long row_tiles = (m + 16 * mt - 1) / (16 * mt), col_groups = (tiles + kTallWaves * nt - 1) / (kTallWaves * nt);
  const long on_the_fullest = (row_tiles * col_groups * slices + 255) / 256;
  const double rounds = 1.43 * (double)(on_the_fullest / 2) + (double)(on_the_fullest % 2);
  return (16.0 * mt * 128.0 + 2048.0 * kTallWaves * nt) * rounds;
}

extern "C" void pa_gemm_tall_shape(int m, int n, int k, int slices, int* out) {
  (void)k;
  const int tiles = (n + 15) / 16;
  static const int shapes[4][2] = {{8, 3}, {8, 2}, {4, 3}, {4, 2}};   // at equal price the larger tile
  double best = 0.0;
  for (int i = 0; i < 4; ++i) {
    const double price = tall_price(shapes[i][0], shapes[i][1], m, tiles, slices < 1 ? 1 : slices);
    if (i == 0 || price < best) best = price, out[0] = shapes[i][0], out[1] = shapes[i][1];
  }
}

// C[m, n] = X[m, k] W^T from the weight in tiles, any m.  slices 1: epilogue 0 writes C (+ bias) in bfloat16,
// epilogue 1 + a C[m, n/2] = act_a(gate) * up (GateActivation codes: 1 SiLU, 2 GELU-tanh).  slices > 1 (epilogue 0 only): nothing is written to C; parts
// [slices, m, n] receives each slice's 32-bit sums (the bias in the first).  mt, nt: the workgroup's shape (tiles
// of 16 rows of X a workgroup, tiles of 16 rows of W a wavefront), or 0, 0 for the launcher's choice; the sums are
// the same bits at every shape.
extern "C" int pa_gemm_tall(void* stream, int epilogue, const void* x, const void* w, const float* bias, void* c,
                            float* parts, int m, int n, int k, long ldx, long ldc, int slices, int mt, int nt) {
  if (m == 0 || n == 0) return 0;
  PA_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_tall: bad sizes m=%d n=%d k=%d", m, n, k);
  PA_REQUIRE(k % 8 == 0 && ldx % 8 == 0 && ldx >= k, "gemm_tall: k=%d and the row stride %ld must be multiples of 8, the stride at least k",
             k, ldx);
  const int steps = (k + 63) / 64;
  PA_REQUIRE(slices >= 1 && slices <= steps && slices <= 64, "gemm_tall: %d slices of %d steps", slices, steps);
  {
    const int sps = (steps + slices - 1) / slices;   // every slice must get a step, or its part would stay unwritten
    PA_REQUIRE((steps + sps - 1) / sps == slices, "gemm_tall: %d steps do not cut into %d slices of %d", steps, slices, sps);
  }
  if (mt == 0 && nt == 0) {
    int shape[2];
    pa_gemm_tall_shape(m, n, k, slices, shape);
    mt = shape[0], nt = shape[1];
  }
  hipStream_t st = (hipStream_t)stream;
  if (slices > 1) {
    PA_REQUIRE(epilogue == kTallPlain && parts, "gemm_tall: a product in slices has no epilogue and needs `parts`");
    return launch_tall_shape<float, kTallSlices>(st, x, w, bias, nullptr, parts, m, n, k, ldx, ldc, slices, mt, nt);
  }
  PA_REQUIRE(c, "gemm_tall: no output");
  PA_REQUIRE(epilogue >= 0 && epilogue <= kActCount, "gemm_tall: unknown epilogue %d", epilogue);
  const bool gated = epilogue != kTallPlain;
  PA_REQUIRE(!gated || (n % 2 == 0 && !bias), "gemm_tall: the gated epilogue needs an even n and no bias");
  PA_REQUIRE(ldc >= (gated ? n / 2 : n), "gemm_tall: output row stride %ld is too small", ldc);
  if (!gated)
    return launch_tall_shape<bf16, kTallPlain>(st, x, w, bias, c, nullptr, m, n, k, ldx, ldc, 1, mt, nt);
  return launch_tall_shape<bf16, kTallSiluMul>(st, x, w, bias, c, nullptr, m, n, k, ldx, ldc, 1, mt, nt, epilogue - 1);
}
