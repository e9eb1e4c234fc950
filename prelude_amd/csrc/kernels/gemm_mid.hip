// C[M,N] = X[M,K] * W[N,K]^T for up to 128 rows in bfloat16 with 32-bit accumulation, from the weight in tiles
// (pa_pack_tiles): the product of decode steps of many requests, and of narrow weights at any number of rows.
//
// With more than a few rows the weight-streaming kernel of gemm_skinny.hip reads X as often as it has
// workgroups: every workgroup owns 16 rows of W and all of K, so a [2560, 9728] weight at 64 rows moves four
// times as many bytes of X through the caches as it streams of W, and a wavefront that holds the sums of 64
// rows has few loads in flight.  Here a workgroup owns 48 to 128 rows of W (three to eight wavefronts, a tile of
// 16 rows each; the number that leaves the fewest compute units idle for the weight's shape) and a slice of K.
// X goes through LDS: the slice's columns are staged once per workgroup, in chunks of KC columns two chunks
// ahead of the products, and every wavefront takes its MFMA operands from there; W goes from memory straight
// into registers, each wavefront streaming its own tile's 2 KB steps with a ring of four of them in flight.
// X is then read once per workgroup whatever the number of slices, and a narrow weight still gives every
// compute unit a workgroup: [2560, 4096] is 32 blocks of rows times 8 slices of K.
//
// A product cut into slices leaves one 32-bit partial sum per slice, [slices, M, N], and no workgroup waits for
// another: whoever reads the result adds the slices in order (the residual add + RMSNorm kernel does, as it
// loads; pa_sum_slices for any other reader).  The order of every sum is fixed by the weight's shape and the
// number of slices alone.
//
// Epilogues of an uncut product as in gemm_skinny.hip: bfloat16 or float32 out, optional bias, or SiLU(gate) * up
// over rows that alternate gate_j, up_j.
//
// Reference counterpart: the GEMM dispatch of crates/prelude-cuda/src/ops/gemm.rs:35-137 (library kernels there).
#include "common.h"
#include "api.h"

namespace pa {

constexpr int kMidMaxM = 128;

struct MidFrag {
  bf16x8 lo, hi;
};

// A step of a tile as pa_pack_tiles lays it out: the wavefront's 64 lanes read 1 KB side by side, twice.
__device__ __forceinline__ MidFrag mid_load_w(const bf16* tile, int step, int lane) {
  MidFrag f;
  const bf16* p = tile + (size_t)step * 1024 + lane * 8;
  f.lo = *reinterpret_cast<const bf16x8*>(p);
  f.hi = *reinterpret_cast<const bf16x8*>(p + 512);
  return f;
}

enum MidEpilogue : int { kMidPlain = 0, kMidSiluMul = 1, kMidSlices = 2 };

// The residual add and RMSNorm in front of the product, done as X is staged (NORM kernels): X is `x` + `res`, summed
// in 32-bit; the sum rounded once is the new residual (`res_out`, another buffer than `res`: every workgroup reads
// `res`, the first one writes `res_out`), the sum times the norm's gain is what goes to LDS, and the row's scale
// rsqrt(mean of squares + eps), which is the same for all its columns, is applied to the finished sums of products.
// Every workgroup sees all of K (no slices), so each forms the rows' sums of squares itself, in a fixed order.
struct MidNorm {
  const bf16* res;
  const float* gain;
  bf16* res_out;
  float eps;
};

// MT tiles of 16 rows of X; KC columns of X a chunk (a multiple of 64): KC / 64 steps between two barriers; WN
// wavefronts a workgroup, a tile of 16 rows of W each.
template <int MT, int KC, int DEPTH, int WN, typename TC, int EPI, bool NORM = false>
__global__ __launch_bounds__(WN* kWave, 2) void gemm_mid_kernel(const bf16* __restrict__ x,
                                                                       const bf16* __restrict__ w,
                                                                       const float* __restrict__ bias,
                                                                       TC* __restrict__ c, float* __restrict__ parts,
                                                                       int m, int n, int k, long ldx, long ldc,
                                                                       int steps_per_slice, int act, MidNorm nm = MidNorm{}) {
  constexpr int SPC = KC / 64;                  // steps a chunk
  constexpr int CPR = DEPTH / SPC;              // chunks the ring of W steps spans
  static_assert(DEPTH % SPC == 0 && CPR >= 1, "the ring holds whole chunks");
  constexpr int ROW = KC + 8;                   // an LDS row: 16 bytes past KC columns, so that the sixteen rows a
                                                // quarter of a wavefront reads together lie in different banks
  constexpr int ROWS = 16 * MT;
  constexpr int PPR = KC / 8;                   // 16-byte pieces a row of a chunk
  constexpr int THREADS = WN * kWave;
  constexpr int PIECES = (ROWS * PPR + THREADS - 1) / THREADS;   // pieces a thread stages
  constexpr bool EVEN = ROWS * PPR % THREADS == 0;               // else the last piece of the later threads is none
  extern __shared__ __align__(16) unsigned char mid_lds[];
  bf16 (*xs)[ROWS][ROW] = reinterpret_cast<bf16 (*)[ROWS][ROW]>(mid_lds);   // two buffers
  // NORM: behind them a row's sums of squares, one per piece of a chunk's row (each from one thread)
  float (*ssl)[PPR] = reinterpret_cast<float (*)[PPR]>(mid_lds + 2 * sizeof(bf16) * ROWS * ROW);

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  const int tiles = (n + 15) / 16, steps = (k + 63) / 64;
  const int tile = blockIdx.x * WN + wave;
  const bool n_ok = tile < tiles;
  const bf16* wtile = w + (size_t)(n_ok ? tile : 0) * steps * 1024;
  const int s_begin = blockIdx.y * steps_per_slice;
  const int s_end = s_begin + steps_per_slice < steps ? s_begin + steps_per_slice : steps;
  const int nchunks = (s_end - s_begin + SPC - 1) / SPC;

  // What a thread stages of a chunk: piece p = tid + j * threads is columns 8 (p % PPR) .. + 7 of row p / PPR.
  // A row past m reads row 0 and columns past k the row's first ones: memory that is there and finite (the
  // columns meet zeros in the tile, the rows are never stored).
  const bf16* src[PIECES];
  int col[PIECES];
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int p = threadIdx.x + j * THREADS;
    const int row = p / PPR;
    col[j] = 8 * (p % PPR);
    src[j] = x + (size_t)(row < m ? row : 0) * ldx;   // a piece past the chunk reads row 0 and is not stored
  }
  // The pieces are dealt out over a chunk's SPC steps (group q: pieces [q * PIECES / SPC, (q + 1) * PIECES / SPC)):
  // at step q of chunk c a thread stores group q, which it loaded a chunk ago and which belongs to chunk c + 1, and
  // loads group q of chunk c + 2 in its place.  A wait for staged pieces then never asks for more of the weight's
  // loads than the step at hand needs anyway (loads come back in the order they were asked for: one wait for a
  // whole chunk's pieces at the chunk's end would drain the ring of weight steps each time).
  bf16x8 staged[PIECES];
  bf16x8 staged_r[NORM ? PIECES : 1];      // NORM: the residual's piece, the gain's eight columns, where they belong
  float4 staged_g[NORM ? PIECES : 1][2];
  int staged_at[NORM ? PIECES : 1];
  float ssp[NORM ? PIECES : 1];            // this thread's share of its rows' sums of squares
  if constexpr (NORM) {
#pragma unroll
    for (int j = 0; j < PIECES; ++j) ssp[j] = 0.f;
  }
  auto stage_load = [&](int chunk, int q0, int q1) {
    const int k0 = (s_begin + chunk * SPC) * 64;
#pragma unroll
    for (int j = 0; j < PIECES; ++j) {
      if (j < q0 * PIECES / SPC || j >= q1 * PIECES / SPC) continue;
      const int at = k0 + col[j];
      const int from = at + 8 <= k ? at : 0;
      staged[j] = *reinterpret_cast<const bf16x8*>(src[j] + from);
      if constexpr (NORM) {
        staged_r[j] = *reinterpret_cast<const bf16x8*>(nm.res + (src[j] - x) + from);
        staged_g[j][0] = *reinterpret_cast<const float4*>(nm.gain + from);
        staged_g[j][1] = *reinterpret_cast<const float4*>(nm.gain + from + 4);
        staged_at[j] = at + 8 <= k ? at : -1;
      }
    }
  };
  // `fresh`: the chunk is stored for the first time (the last chunk is staged again while the ring of W steps runs
  // out: its squares must count once, and the new residual is written once)
  auto stage_store = [&](int buf, int q0, int q1, bool fresh = true) {
#pragma unroll
    for (int j = 0; j < PIECES; ++j) {
      if (j < q0 * PIECES / SPC || j >= q1 * PIECES / SPC) continue;
      const int p = threadIdx.x + j * THREADS;
      if (!(EVEN || j + 1 < PIECES || p < ROWS * PPR)) continue;
      if constexpr (NORM) {
        const int row = p / PPR;
        const float gn[8] = {staged_g[j][0].x, staged_g[j][0].y, staged_g[j][0].z, staged_g[j][0].w,
                             staged_g[j][1].x, staged_g[j][1].y, staged_g[j][1].z, staged_g[j][1].w};
        bf16x8 sum, scaled;
        float sq = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float s = to_f32(staged[j][i]) + to_f32(staged_r[j][i]);
          sq += s * s;
          sum[i] = from_f32<bf16>(s);
          scaled[i] = from_f32<bf16>(s * gn[i]);
        }
        const bool counts = fresh && row < m && staged_at[j] >= 0;
        if (counts) {
          ssp[j] += sq;
          if (blockIdx.x == 0) *reinterpret_cast<bf16x8*>(nm.res_out + (size_t)row * ldx + staged_at[j]) = sum;
        }
        *reinterpret_cast<bf16x8*>(&xs[buf][row][col[j]]) = scaled;
      } else {
        *reinterpret_cast<bf16x8*>(&xs[buf][p / PPR][col[j]]) = staged[j];
      }
    }
  };

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // No load stands under a condition (a chunk or a step past the slice's end reads the last one again and is not
  // used): the compiler then knows how many loads are in flight at every use and waits for no more than it must;
  // behind a load that may or may not have been issued it would wait for all of them, the newest included.
  MidFrag wbuf[DEPTH];
  const int last = s_end - 1;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) wbuf[d] = mid_load_w(wtile, s_begin + d < s_end ? s_begin + d : last, lane);
  stage_load(0, 0, SPC);
  stage_store(0, 0, SPC);
  stage_load(nchunks > 1 ? 1 : 0, 0, SPC);
  __syncthreads();
  // X fragments of a step, all asked for from LDS before the step's first product
  auto load_x = [&](int buf, int ss, bf16x8 (*xf)[2]) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const bf16* xr = &xs[buf][16 * t + r][64 * ss + 16 * g];
      xf[t][0] = *reinterpret_cast<const bf16x8*>(xr);
      xf[t][1] = *reinterpret_cast<const bf16x8*>(xr + 8);
    }
  };
  for (int ch0 = 0; ch0 < nchunks; ch0 += CPR) {
#pragma unroll
    for (int u = 0; u < CPR; ++u) {
      const int ch = ch0 + u;   // past the last chunk (the ring spans several): everything again, nothing counted
      const int buf = ch & 1;
      const int ahead = ch + 2 < nchunks ? ch + 2 : nchunks - 1;
      bf16x8 xf[2][MT][2];
      load_x(buf, 0, xf[0]);
#pragma unroll
      for (int ss = 0; ss < SPC; ++ss) {
        const int s = s_begin + ch * SPC + ss;
        MidFrag wc = wbuf[u * SPC + ss];
        // the step that takes this slot of the ring next; past the slice's end the last step again, never used
        wbuf[u * SPC + ss] = mid_load_w(wtile, s + DEPTH < s_end ? s + DEPTH : last, lane);
        stage_store(buf ^ 1, ss, ss + 1, ch + 1 < nchunks);
        stage_load(ahead, ss, ss + 1);
        if (ss + 1 < SPC) load_x(buf, ss + 1, xf[(ss + 1) & 1]);   // the next step's, under this step's products
        if (s >= s_end) {   // a step past the slice's end counts nothing: zeros for W, and no branch around the products
#pragma unroll
          for (int i = 0; i < 8; ++i) wc.lo[i] = (bf16)0.f, wc.hi[i] = (bf16)0.f;
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc.lo, xf[ss & 1][t][0], acc[t], 0, 0, 0);
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc.hi, xf[ss & 1][t][1], acc[t], 0, 0, 0);
        }
      }
      __syncthreads();
    }
  }
  float inv[NORM ? MT : 1];
  if constexpr (NORM) {
    // a row's squares: one sum per piece of a chunk's row and thread, added in the pieces' order
#pragma unroll
    for (int j = 0; j < PIECES; ++j) {
      const int p = threadIdx.x + j * THREADS;
      if (EVEN || j + 1 < PIECES || p < ROWS * PPR) ssl[p / PPR][p % PPR] = ssp[j];
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      float total = 0.f;
      for (int i = 0; i < PPR; ++i) total += ssl[16 * t + r][i];
      inv[t] = rsqrtf(total / (float)k + nm.eps);
    }
  }
  if (!n_ok) return;
  // lane (g, r) holds four consecutive n of token 16 t + r
  const int nb = 16 * tile + 4 * g;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int mi = 16 * t + r;
    if (mi >= m) continue;
    if constexpr (NORM) {
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[t][i] *= inv[t];
    }
    if (EPI == kMidSlices) {
      float* dst = parts + ((size_t)blockIdx.y * m + mi) * n + nb;
      if (nb + 3 < n && n % 4 == 0) {
        float4 v{acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
        if (bias && blockIdx.y == 0) v.x += bias[nb], v.y += bias[nb + 1], v.z += bias[nb + 2], v.w += bias[nb + 3];
        *reinterpret_cast<float4*>(dst) = v;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nb + i < n) dst[i] = acc[t][i] + (bias && blockIdx.y == 0 ? bias[nb + i] : 0.f);
      }
    } else if (EPI == kMidSiluMul) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int nn = nb + 2 * j;
        if (nn + 1 < n) {
          const float gate = acc[t][2 * j], up = acc[t][2 * j + 1];
          c[(size_t)mi * ldc + nn / 2] = from_f32<TC>(gate_activation(gate, act) * up);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (nb + i < n) {
          float v = acc[t][i];
          if (bias) v += bias[nb + i];
          c[(size_t)mi * ldc + nb + i] = from_f32<TC>(v);
        }
      }
    }
  }
}

// out[row, col] = sum over the slices, in their order, of parts[slice, row, col]
template <typename T>
__global__ void sum_slices_kernel(const float* __restrict__ parts, T* __restrict__ out, int slices, size_t total) {
  const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= total) return;
  if (i + 3 < total) {
    float4 s = *reinterpret_cast<const float4*>(parts + i);
    // up to eight slices are asked for together and then added in their order
    float4 b[7];
#pragma unroll
    for (int p = 1; p < 8; ++p)
      if (p < slices) b[p - 1] = *reinterpret_cast<const float4*>(parts + (size_t)p * total + i);
#pragma unroll
    for (int p = 1; p < 8; ++p)
      if (p < slices) s.x += b[p - 1].x, s.y += b[p - 1].y, s.z += b[p - 1].z, s.w += b[p - 1].w;
    for (int p = 8; p < slices; ++p) {
      const float4 v = *reinterpret_cast<const float4*>(parts + (size_t)p * total + i);
      s.x += v.x, s.y += v.y, s.z += v.z, s.w += v.w;
    }
    out[i] = from_f32<T>(s.x), out[i + 1] = from_f32<T>(s.y), out[i + 2] = from_f32<T>(s.z), out[i + 3] = from_f32<T>(s.w);
  } else {
    for (size_t e = i; e < total; ++e) {
      float s = parts[e];
      for (int p = 1; p < slices; ++p) s += parts[(size_t)p * total + e];
      out[e] = from_f32<T>(s);
    }
  }
}

template <int MT, int KC, int DEPTH, int WN, typename TC, int EPI, bool NORM = false>
int launch_mid(hipStream_t st, const void* x, const void* w, const float* bias, void* c, float* parts, int m, int n, int k,
               long ldx, long ldc, int slices, int act, MidNorm nm = MidNorm{}) {
  const int tiles = (n + 15) / 16, steps = (k + 63) / 64;
  const int sps = (steps + slices - 1) / slices;
  constexpr size_t lds = 2 * (size_t)(16 * MT) * (KC + 8) * sizeof(bf16) + (NORM ? (size_t)(16 * MT) * (KC / 8) * sizeof(float) : 0);
  static const hipError_t allowed = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_mid_kernel<MT, KC, DEPTH, WN, TC, EPI, NORM>),
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (allowed != hipSuccess) return pa::fail("gemm_mid: %zu bytes of LDS refused: %s", lds, hipGetErrorString(allowed));
  dim3 grid((tiles + WN - 1) / WN, (steps + sps - 1) / sps);
  hipLaunchKernelGGL((gemm_mid_kernel<MT, KC, DEPTH, WN, TC, EPI, NORM>), grid, dim3(WN * kWave), lds, st, (const bf16*)x,
                     (const bf16*)w, bias, (TC*)c, parts, m, n, k, ldx, ldc, sps, act, nm);
  return check_launch("gemm_mid");
}

// How many wavefronts (tiles of 16 rows of W) a workgroup takes: the number from 3 to 8 that leaves the compute
// units the least idle when every unit works through its workgroups one after the other -- 1,216 tiles are 304
// workgroups of four (a quarter of the units get two, the others wait: 59 % busy) or 244 of five (95 %).
// Equal numbers go to four, then to the larger.  (The model is one of few rounds; see below for many.)
inline int mid_waves(int n, int slices) {
  const int tiles = (n + 15) / 16;
  // a grid of many rounds whatever the number: the most wavefronts, which stage X the fewest times (the head of
  // 151,936 rows at 64 rows of X: 166 us with eight, 179 with four, 185 with three)
  if ((long)((tiles + 7) / 8) * slices >= 4 * 256) return 8;
  const int order[] = {4, 5, 6, 8, 3};
  int best = 4;
  double best_busy = 0.0;
  for (int wn : order) {
    // three wavefronts are for small weights: every workgroup stages all of X, and a wide weight has many
    // ([34816, 5120] with the gated epilogue at 64 rows: 86.5 us with three, 75.2 with five)
    if (wn == 3 && tiles >= 1024) continue;
    const long groups = (long)((tiles + wn - 1) / wn) * slices;
    const long rounds = (groups + 255) / 256;
    const double busy = (double)tiles * slices / (double)(rounds * 256 * wn);
    if (busy > best_busy + 0.02) best = wn, best_busy = busy;
  }
  return best;
}

template <int WN, typename TC, int EPI>
int launch_mid_mt(hipStream_t st, const void* x, const void* w, const float* bias, void* c, float* parts, int m, int n,
                  int k, long ldx, long ldc, int slices, int act) {
#define PA_MID(MT, KC, D) return launch_mid<MT, KC, D, WN, TC, EPI>(st, x, w, bias, c, parts, m, n, k, ldx, ldc, slices, act)
  // chunks of 256 columns and a ring of four steps up to 64 rows; 128 columns beyond (LDS holds two chunks);
  // measured over chunk sizes and ring depths at the shapes of a 4B model: within a microsecond of one another
  switch ((m + 15) / 16) {
    case 1: PA_MID(1, 256, 4);
    case 2: PA_MID(2, 256, 4);
    case 3: PA_MID(3, 256, 4);
    case 4: PA_MID(4, 256, 4);
    case 5:
    case 6: PA_MID(6, 128, 4);
    default: PA_MID(8, 128, 4);
  }
#undef PA_MID
}

template <typename TC, int EPI>
int launch_mid_wn(hipStream_t st, const void* x, const void* w, const float* bias, void* c, float* parts, int m, int n,
                  int k, long ldx, long ldc, int slices, int waves, int act = 0) {
  switch (waves ? waves : mid_waves(n, slices)) {
    case 3: return launch_mid_mt<3, TC, EPI>(st, x, w, bias, c, parts, m, n, k, ldx, ldc, slices, act);
    case 5: return launch_mid_mt<5, TC, EPI>(st, x, w, bias, c, parts, m, n, k, ldx, ldc, slices, act);
    case 6: return launch_mid_mt<6, TC, EPI>(st, x, w, bias, c, parts, m, n, k, ldx, ldc, slices, act);
    case 8: return launch_mid_mt<8, TC, EPI>(st, x, w, bias, c, parts, m, n, k, ldx, ldc, slices, act);
    default: return launch_mid_mt<4, TC, EPI>(st, x, w, bias, c, parts, m, n, k, ldx, ldc, slices, act);
  }
}

}  // namespace pa

using namespace pa;

// How many slices of K pa_gemm_mid cuts a product into when its reader takes slices: as many as give every
// compute unit a workgroup or two, each slice at least eight steps of 64 columns; four at most, eight for long rows
// of a narrow weight.  Every slice is another 32-bit copy of the output that the product writes and the norm behind it
// reads, with few workgroups: with the norm behind it, [2560, 4096] at 16 / 32 / 64 / 128 rows takes 10.7 / 11.6 /
// 13.0 / 17.8 us in four slices and 12.0 / 13.4 / 15.7 / 19.3 in eight, [4096, 4096] 14.6 / 15.0 / 18.4 / 22.5 and
// 16.7 / 17.4 / 20.3 / 26.2, [4096, 12288] 24.9 / 25.5 / 29.8 / 41.8 and 27.7 / 27.9 / 33.2 / 43.1; [2560, 9728] is
// level or better in eight (18.2 / 18.8 / 21.0 / 27.5 against 17.8 / 19.6 / 21.3 / 30.0).  In the decode step
// (context 2,048, same box, eight slices at most against this): 4B shape batch 32 / 64 4.61 / 6.64 against 4.58 /
// 6.59 ms, 8B shape batch 32 / 64 / 128 6.05 / 7.95 / 12.54 against 5.89 / 7.90 / 12.39.  Follows the weight's
// shape alone.
extern "C" int pa_gemm_mid_slices(int n, int k) {
  if (n <= 0 || k <= 0) return 1;
  const int blocks = ((n + 15) / 16 + 4) / 5, steps = (k + 63) / 64;
  const int most = (blocks * 4 < 160 && steps >= 128) ? 8 : 4;
  int s = 1;
  while (s < most && blocks * s < 256 && steps / (2 * s) >= 8) s *= 2;
  return s;
}

// The gated product of up to 16 rows with the residual add and RMSNorm in front of it (see MidNorm):
// res_out[m, k] = x + res (rounded once), c[m, n/2] = act(gate) * up of rmsnorm(x + res; gain, eps) W^T.  x, res and
// res_out have the row stride ldx; res_out must be another buffer than res and x.  epilogue 1 + a as in pa_gemm_mid.
extern "C" int pa_gemm_mid_normed(void* stream, int epilogue, const void* x, const void* res, const float* gain, float eps,
                                  void* res_out, const void* w, void* c, int m, int n, int k, long ldx, long ldc,
                                  int waves) {
  if (m == 0 || n == 0) return 0;
  PA_REQUIRE(m > 0 && m <= 16 && n > 0 && k > 0, "gemm_mid_normed: bad sizes m=%d (up to 16) n=%d k=%d", m, n, k);
  PA_REQUIRE(k % 8 == 0 && ldx % 8 == 0 && ldx >= k, "gemm_mid_normed: k=%d and the row stride %ld must be multiples of 8, the stride at least k",
             k, ldx);
  PA_REQUIRE(x && res && gain && res_out && w && c, "gemm_mid_normed: an operand is missing");
  PA_REQUIRE(res_out != res && res_out != x, "gemm_mid_normed: the new residual needs a buffer of its own");
  PA_REQUIRE(epilogue >= 1 && epilogue <= kActCount && n % 2 == 0, "gemm_mid_normed: a gated epilogue (1 + activation) and an even n");
  PA_REQUIRE(ldc >= n / 2, "gemm_mid_normed: output row stride %ld is too small", ldc);
  PA_REQUIRE(waves == 0 || waves == 3 || waves == 4 || waves == 5 || waves == 6 || waves == 8,
             "gemm_mid_normed: %d wavefronts a workgroup (3, 4, 5, 6, 8, or 0 to let the launcher choose)", waves);
  hipStream_t st = (hipStream_t)stream;
  const MidNorm nm{(const bf16*)res, gain, (bf16*)res_out, eps};
  const int act = epilogue - 1;
#define PA_NORMED(WN) \
  return launch_mid<1, 256, 4, WN, bf16, kMidSiluMul, true>(st, x, w, nullptr, c, nullptr, m, n, k, ldx, ldc, 1, act, nm)
  switch (waves ? waves : mid_waves(n, 1)) {
    case 3: PA_NORMED(3);
    case 5: PA_NORMED(5);
    case 6: PA_NORMED(6);
    case 8: PA_NORMED(8);
    default: PA_NORMED(4);
  }
#undef PA_NORMED
}

// Floats of `parts` a product of m rows cut into `slices` needs.
extern "C" long pa_gemm_mid_parts(int m, int n, int slices) { return slices <= 1 ? 0 : (long)slices * m * n; }

// C[m, n] = X[m, k] W^T for m <= 128 from the weight in tiles.  slices 1: epilogue 0 writes C (+ bias) as
// out_dtype (0 float32, 1 bfloat16), epilogue 1 + a C[m, n/2] = act_a(gate) * up (GateActivation codes: 1 SiLU, 2 GELU-tanh).  slices > 1 (epilogue 0 only):
// nothing is written to C; parts [slices, m, n] receives each slice's 32-bit sums (the bias in the first).
// waves: wavefronts (tiles of 16 rows of W) a workgroup, 3, 4, 5, 6 or 8, or 0 for the launcher's choice; the sums
// are the same bits at every number.
extern "C" int pa_gemm_mid(void* stream, int out_dtype, int epilogue, const void* x, const void* w, const float* bias,
                           void* c, float* parts, int m, int n, int k, long ldx, long ldc, int slices, int waves) {
  if (m == 0 || n == 0) return 0;
  PA_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_mid: bad sizes m=%d n=%d k=%d", m, n, k);
  PA_REQUIRE(m <= kMidMaxM, "gemm_mid: %d rows exceed %d", m, kMidMaxM);
  PA_REQUIRE(k % 8 == 0 && ldx % 8 == 0 && ldx >= k, "gemm_mid: k=%d and the row stride %ld must be multiples of 8, the stride at least k",
             k, ldx);
  const int steps = (k + 63) / 64;
  PA_REQUIRE(slices >= 1 && slices <= steps && slices <= 64, "gemm_mid: %d slices of %d steps", slices, steps);
  PA_REQUIRE(waves == 0 || waves == 3 || waves == 4 || waves == 5 || waves == 6 || waves == 8,
             "gemm_mid: %d wavefronts a workgroup (3, 4, 5, 6, 8, or 0 to let the launcher choose)", waves);
  {
    const int sps = (steps + slices - 1) / slices;   // every slice must get a step, or its part would stay unwritten
    PA_REQUIRE((steps + sps - 1) / sps == slices, "gemm_mid: %d steps do not cut into %d slices of %d", steps, slices, sps);
  }
  hipStream_t st = (hipStream_t)stream;
  if (slices > 1) {
    PA_REQUIRE(epilogue == kMidPlain && parts, "gemm_mid: a product in slices has no epilogue and needs `parts`");
    return launch_mid_wn<float, kMidSlices>(st, x, w, bias, nullptr, parts, m, n, k, ldx, ldc, slices, waves);
  }
  PA_REQUIRE(c, "gemm_mid: no output");
  PA_REQUIRE(epilogue >= 0 && epilogue <= kActCount, "gemm_mid: unknown epilogue %d", epilogue);
  const bool gated = epilogue != kMidPlain;
  PA_REQUIRE(!gated || (n % 2 == 0 && !bias), "gemm_mid: the gated epilogue needs an even n and no bias");
  PA_REQUIRE(ldc >= (gated ? n / 2 : n), "gemm_mid: output row stride %ld is too small", ldc);
  if (!gated && out_dtype == kBF16)
    return launch_mid_wn<bf16, kMidPlain>(st, x, w, bias, c, nullptr, m, n, k, ldx, ldc, 1, waves);
  if (!gated && out_dtype == kF32)
    return launch_mid_wn<float, kMidPlain>(st, x, w, bias, c, nullptr, m, n, k, ldx, ldc, 1, waves);
  if (gated && out_dtype == kBF16)
    return launch_mid_wn<bf16, kMidSiluMul>(st, x, w, bias, c, nullptr, m, n, k, ldx, ldc, 1, waves, epilogue - 1);
  return pa::fail("gemm_mid: unsupported output type %d with epilogue %d", out_dtype, epilogue);
}

// out[i] = sum of parts[p, i] over p in order; out_dtype 0 float32, 1 bfloat16; total = rows * columns.
extern "C" int pa_sum_slices(void* stream, int out_dtype, const float* parts, void* out, int slices, long total) {
  if (total == 0) return 0;
  PA_REQUIRE(slices >= 1 && total > 0 && parts && out, "sum_slices: bad operands");
  const unsigned blocks = (unsigned)((total / 4 + 1 + 255) / 256);
  if (out_dtype == kBF16) {
    hipLaunchKernelGGL(sum_slices_kernel<bf16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, parts, (bf16*)out, slices,
                       (size_t)total);
  } else if (out_dtype == kF32) {
    hipLaunchKernelGGL(sum_slices_kernel<float>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, parts, (float*)out,
                       slices, (size_t)total);
  } else {
    return pa::fail("sum_slices: unknown element type code %d", out_dtype);
  }
  return check_launch("sum_slices");
}
