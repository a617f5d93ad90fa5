// Mapped convolution over images of very few channels (first layers: grey, RGB, RGB-D), float32.
//
// The matrix-unit kernels (conv_fused.hip, conv_window_gemm.hip) contract 32 gather-side
// channels per chunk; with Cg <= 4 a chunk is at most an eighth full, and both the gathers and
// the MFMAs of the padding are wasted.  Here the reduction index (c, k) is packed instead:
//
//   small_forward_kernel   pix[b][n][m] = bias[n] + sum_{c,k} Wm[n][c][k] * col[b][(c,k)][m]
//       one thread per pixel gathers its Cg * K column values once into registers and forms
//       every output channel from them with weights read through the scalar unit
//   small_wgrad_kernel     gW[n][c][k] += sum_{b,m} pix[b][n][m] * col[b][(c,k)][m]
//       v_mfma_f32_32x32x2_f32 with the pixel as reduction index: per tile of 64 pixels the
//       column values of all (c, k) go to LDS once; lane l supplies pix[n = 32 a + l % 32][m]
//       as A and the column value of (c, k) = 32 b + l % 32 at pixel m as B
//
// col[b][(c,k)][m] = sum over the points and taps of sample k of pixel m of
// coefficient * img[b][c][tap], as in common/mapped_im2col.h:13-63 of the reference.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "conv_small.hpp"
#include "sdk_host.hpp"
#include "sdk_taps.hpp"

namespace sdk {
namespace {

constexpr int kSmThreads = 256;

// Kernel launch with dynamic LDS as an expression (for the dispatch macros).
template <typename... KArgs, typename... Args>
inline void launch_lds(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t smem,
                       hipStream_t stream, Args... args) {
  kernel<<<grid, block, smem, stream>>>(args...);
}

using floatx16 = __attribute__((__vector_size__(16 * sizeof(float)))) float;

// Keeps a loaded value in a register here and now: without it the compiler moves the load
// behind the test of the tap it belongs to, one branch, one load and one wait per tap.
__device__ __forceinline__ void pin(float& x) { asm volatile("" : "+v"(x)); }

// Column values of G consecutive samples (first: sample0; only the first `valid` exist, the
// others repeat the last) of one pixel for CG channels: v[g][c].  All map reads of the group
// are issued together, then all image reads, then the blend.
template <int INTERP, bool WEIGHTED, int CG, int G>
__device__ __forceinline__ void column_group(const float* __restrict__ img_b, size_t HW,
                                             const float* __restrict__ map,
                                             const float* __restrict__ wts, size_t sample0,
                                             int valid, int P, int H, int W, int Cg,
                                             float (&v)[G][CG]) {
  constexpr int N = PointTaps<float, INTERP>::N;
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int c = 0; c < CG; ++c) v[g][c] = 0.0f;
  const int q = WEIGHTED ? P : 1;
  for (int p = 0; p < q; ++p) {
    float mx[G], my[G], wt[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const size_t s = (sample0 + (g < valid ? g : valid - 1)) * q + p;
      mx[g] = map[s * 2];
      my[g] = map[s * 2 + 1];
      wt[g] = WEIGHTED ? wts[s] : 1.0f;
    }
    PointTaps<float, INTERP> t[G];
    float d[G][N][CG];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      t[g].set(mx[g], my[g], H, W);
#pragma unroll
      for (int i = 0; i < N; ++i) {
        const size_t o = t[g].off[i] >= 0 ? (size_t)t[g].off[i] : 0;
#pragma unroll
        for (int c = 0; c < CG; ++c) d[g][i][c] = img_b[(size_t)(c < Cg ? c : 0) * HW + o];
      }
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int i = 0; i < N; ++i)
#pragma unroll
        for (int c = 0; c < CG; ++c) pin(d[g][i][c]);
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
      for (int i = 0; i < N; ++i) {
        const float co = WEIGHTED ? wt[g] * t[g].w[i] : t[g].w[i];
        const bool on = t[g].off[i] >= 0 && co != 0.0f;
#pragma unroll
        for (int c = 0; c < CG; ++c)
          v[g][c] = __builtin_fmaf(on ? co : 0.0f, on ? d[g][i][c] : 0.0f, v[g][c]);
      }
    }
  }
}

// The same for G separate (sample, channel plane) items, one channel each: v[g].  An item
// with plane == nullptr yields 0.
template <int INTERP, bool WEIGHTED, int G>
__device__ __forceinline__ void column_items(const float* const (&plane)[G],
                                             const size_t (&sample)[G],
                                             const float* __restrict__ map,
                                             const float* __restrict__ wts,
                                             const float* __restrict__ safe, int P, int H, int W,
                                             float (&v)[G]) {
  constexpr int N = PointTaps<float, INTERP>::N;
#pragma unroll
  for (int g = 0; g < G; ++g) v[g] = 0.0f;
  const int q = WEIGHTED ? P : 1;
  for (int p = 0; p < q; ++p) {
    float mx[G], my[G], wt[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const size_t s = sample[g] * q + p;
      mx[g] = map[s * 2];
      my[g] = map[s * 2 + 1];
      wt[g] = WEIGHTED ? wts[s] : 1.0f;
    }
    PointTaps<float, INTERP> t[G];
    float d[G][N];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      t[g].set(mx[g], my[g], H, W);
      const float* pl = plane[g] != nullptr ? plane[g] : safe;
#pragma unroll
      for (int i = 0; i < N; ++i) d[g][i] = pl[t[g].off[i] >= 0 ? (size_t)t[g].off[i] : 0];
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int i = 0; i < N; ++i) pin(d[g][i]);
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
      for (int i = 0; i < N; ++i) {
        const float co = WEIGHTED ? wt[g] * t[g].w[i] : t[g].w[i];
        const bool on = plane[g] != nullptr && t[g].off[i] >= 0 && co != 0.0f;
        v[g] = __builtin_fmaf(on ? co : 0.0f, on ? d[g][i] : 0.0f, v[g]);
      }
    }
  }
}

// The weight matrix Wm[Cp][Cg][K] into LDS as wl[Cp][CG][KMAX], zero where c >= Cg or k >= K, so
// the loops over (c, k) need no guards and address with constants.  Every lane reads the same
// element at a time, which the LDS serves as a broadcast.
template <int CG, int KMAX>
__device__ __forceinline__ void stage_weights(const float* __restrict__ Wm, int Cp, int Cg, int K,
                                              float* __restrict__ wl) {
  for (int e = threadIdx.x; e < Cp * CG * KMAX; e += blockDim.x) {
    const int k = e % KMAX, c = (e / KMAX) % CG, n = e / (KMAX * CG);
    wl[e] = (c < Cg && k < K) ? Wm[((size_t)n * Cg + c) * K + k] : 0.0f;
  }
  __syncthreads();
}

// grid (pixel blocks, batch); KMAX bounds K (register array).
template <int INTERP, bool WEIGHTED, int CG, int KMAX>
__global__ __launch_bounds__(kSmThreads) void small_forward_kernel(
    const float* __restrict__ img, const float* __restrict__ map, const float* __restrict__ wts,
    const float* __restrict__ Wm, const float* __restrict__ bias, float* __restrict__ pix, int Cg,
    int H, int W, int Cp, int M, int K, int P) {
  extern __shared__ __align__(16) float wl[];
  stage_weights<CG, KMAX>(Wm, Cp, Cg, K, wl);
  const int m = blockIdx.x * blockDim.x + threadIdx.x;
  if (m >= M) return;
  const size_t HW = (size_t)H * W;
  const float* img_b = img + (size_t)blockIdx.y * Cg * HW;
  constexpr int G = 3;                      // samples whose reads are in flight together
  constexpr int KPAD = (KMAX + G - 1) / G * G;
  float col[KPAD][CG];
#pragma unroll
  for (int k0 = 0; k0 < KPAD; k0 += G) {
    if (k0 < K) {
      float grp[G][CG];
      column_group<INTERP, WEIGHTED, CG, G>(img_b, HW, map, wts, (size_t)m * K + k0,
                                            min(G, K - k0), P, H, W, Cg, grp);
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int c = 0; c < CG; ++c) col[k0 + g][c] = grp[g][c];
    } else {
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int c = 0; c < CG; ++c) col[k0 + g][c] = 0.0f;
    }
  }
  float* out = pix + (size_t)blockIdx.y * Cp * M + m;
  for (int n = 0; n < Cp; ++n) {
    const float* wrow = wl + n * (CG * KMAX);
    float acc = bias != nullptr ? bias[n] : 0.0f;
#pragma unroll
    for (int c = 0; c < CG; ++c) {
#pragma unroll
      for (int k = 0; k < KMAX; ++k) acc = __builtin_fmaf(wrow[c * KMAX + k], col[k][c], acc);
    }
    out[(size_t)n * M] = acc;
  }
}

// img[b][c][tap] += coefficient * sum_n Wm[n][c][k] * pix[b][n][m] over the taps of (m, k): the
// transpose of the forward.  One thread per pixel forms its Cg * K products with the weights
// in LDS and splats them with float atomics; img must hold the values to add to.
template <int INTERP, bool WEIGHTED, int CG, int KMAX>
__global__ __launch_bounds__(kSmThreads) void small_scatter_kernel(
    const float* __restrict__ pix, const float* __restrict__ map, const float* __restrict__ wts,
    const float* __restrict__ Wm, float* __restrict__ img, int Cg, int H, int W, int Cp, int M,
    int K, int P) {
  extern __shared__ __align__(16) float wl[];
  stage_weights<CG, KMAX>(Wm, Cp, Cg, K, wl);
  const int m = blockIdx.x * blockDim.x + threadIdx.x;
  if (m >= M) return;
  const size_t HW = (size_t)H * W;
  float* img_b = img + (size_t)blockIdx.y * Cg * HW;
  const float* in = pix + (size_t)blockIdx.y * Cp * M + m;
  float t[KMAX][CG];
#pragma unroll
  for (int k = 0; k < KMAX; ++k)
#pragma unroll
    for (int c = 0; c < CG; ++c) t[k][c] = 0.0f;
  for (int n = 0; n < Cp; ++n) {
    const float g = in[(size_t)n * M];
    const float* wrow = wl + n * (CG * KMAX);
#pragma unroll
    for (int c = 0; c < CG; ++c) {
#pragma unroll
      for (int k = 0; k < KMAX; ++k) t[k][c] = __builtin_fmaf(wrow[c * KMAX + k], g, t[k][c]);
    }
  }
  const int q = WEIGHTED ? P : 1;
  PointTaps<float, INTERP> tp;
  for (int p = 0; p < q; ++p) {
    // the map entries of all samples first (one round trip), then taps and atomics
    float mx[KMAX], my[KMAX], wt[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const size_t s = ((size_t)m * K + (k < K ? k : K - 1)) * q + p;
      mx[k] = map[s * 2];
      my[k] = map[s * 2 + 1];
      wt[k] = WEIGHTED ? wts[s] : 1.0f;
    }
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      pin(mx[k]);
      pin(my[k]);
      pin(wt[k]);
    }
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      if (k < K) {
        tp.set(mx[k], my[k], H, W);
#pragma unroll
        for (int i = 0; i < PointTaps<float, INTERP>::N; ++i) {
          const float co = WEIGHTED ? wt[k] * tp.w[i] : tp.w[i];
          if (tp.off[i] >= 0 && co != 0.0f) {
#pragma unroll
            for (int c = 0; c < CG; ++c)
              if (c < Cg) atomic_add_noret(img_b + (size_t)c * HW + tp.off[i], co * t[k][c]);
          }
        }
      }
    }
  }
}

// Workgroup = 4 waves, one batch element (grid (blocks, batch)), tiles of 64 pixels dealt
// round-robin.  NB: 32-row blocks of pixel-side channels (Cp <= 32 NB); CB: blocks of 32 columns
// (c, k) (Cg * K <= 32 CB).  Per tile every thread computes eight column values (so their map
// and image reads are in flight together) into an LDS tile, the pixel-side values are copied
// beside it, and wave w multiplies pixels 16 w .. 16 w + 15.  The waves' accumulators (NB * CB
// of 16 registers) are summed in LDS at the end and leave the workgroup as one float atomic per
// element of gW.  gbias (optional): the bias gradient, the sum of the pixel-side rows the
// kernel has in LDS anyway, one atomic per channel and workgroup (gbias must start from zero).
constexpr int kSmTile = 64;       // pixels per tile
constexpr int kSmLd = kSmTile + 1;   // row stride of the LDS tiles (floats): rows on distinct banks

template <int INTERP, bool WEIGHTED, int NB, int CB>
__global__ __launch_bounds__(kSmThreads) void small_wgrad_kernel(
    const float* __restrict__ pix, const float* __restrict__ img, const float* __restrict__ map,
    const float* __restrict__ wts, float* __restrict__ gW, float* __restrict__ gbias, int Cg,
    int H, int W, int Cp, int M, int K, int P) {
  constexpr int COLS = 32 * CB, ROWS = 32 * NB;
  float row_sum = 0.0f;   // thread n < ROWS: pixel-side row n over this workgroup's tiles
  constexpr int TILE_FLOATS = (COLS + ROWS) * kSmLd, SUM_FLOATS = ROWS * COLS;
  __shared__ float lds[TILE_FLOATS > SUM_FLOATS ? TILE_FLOATS : SUM_FLOATS];
  float* colT = lds;                  // [COLS][kSmLd]
  float* pixT = lds + COLS * kSmLd;   // [ROWS][kSmLd]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nl = lane & 31, h = lane >> 5;
  const size_t HW = (size_t)H * W;
  const float* img_b = img + (size_t)blockIdx.y * Cg * HW;
  const float* pix_b = pix + (size_t)blockIdx.y * Cp * M;
  const int CK = Cg * K;
  floatx16 acc[NB][CB];
#pragma unroll
  for (int a = 0; a < NB; ++a)
#pragma unroll
    for (int b = 0; b < CB; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;

  const int tiles = (M + kSmTile - 1) / kSmTile;
  for (int t = blockIdx.x; t < tiles; t += gridDim.x) {
    const int m0 = t * kSmTile;
    // ---- column values: thread -> pixel tid % 64, columns tid / 64 + 4 i
    {
      const int p = tid & (kSmTile - 1), m = m0 + p;
      // (eight items at a time: their reads are in flight together)
#pragma unroll
      for (int i0 = 0; i0 < COLS / 4; i0 += 8) {
        const float* plane[8];
        size_t sample[8];
        float val[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int col = (tid >> 6) + 4 * (i0 + i);
          const bool live = m < M && col < CK;
          const int c = live ? col / K : 0, k = live ? col - c * K : 0;
          plane[i] = live ? img_b + (size_t)c * HW : nullptr;
          sample[i] = (size_t)(live ? m : 0) * K + k;
        }
        column_items<INTERP, WEIGHTED, 8>(plane, sample, map, wts, img_b, P, H, W, val);
#pragma unroll
        for (int i = 0; i < 8; ++i) colT[((tid >> 6) + 4 * (i0 + i)) * kSmLd + p] = val[i];
      }
      // ---- pixel-side values: rows tid / 64 + 4 i (coalesced along the pixels)
#pragma unroll
      for (int i = 0; i < ROWS / 4; ++i) {
        const int n = (tid >> 6) + 4 * i;
        pixT[n * kSmLd + p] = (m < M && n < Cp) ? pix_b[(size_t)n * M + m] : 0.0f;
      }
    }
    __syncthreads();
    if (gbias != nullptr && tid < ROWS) {
      float s = 0.0f;
#pragma unroll 8
      for (int p = 0; p < kSmTile; ++p) s += pixT[tid * kSmLd + p];
      row_sum += s;
    }
    // ---- wave w: pixels 16 w + 2 s + h, s = 0..7
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int p = 16 * wave + 2 * s + h;
      float bv[CB];
#pragma unroll
      for (int b = 0; b < CB; ++b) bv[b] = colT[(32 * b + nl) * kSmLd + p];
#pragma unroll
      for (int a = 0; a < NB; ++a) {
        const float av = pixT[(32 * a + nl) * kSmLd + p];
#pragma unroll
        for (int b = 0; b < CB; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv[b], acc[a][b], 0, 0, 0);
      }
    }
    __syncthreads();   // the tiles are rewritten by the next round
  }
  // ---- sum the four waves' accumulators in LDS (over the tiles' space), then one atomic per
  // element.  D[row][column]: register v of lane l holds row 8 (v / 4) + 4 (l / 32) + v % 4,
  // column l % 32.
  float* sum = lds;   // [ROWS][COLS]
  for (int e = tid; e < SUM_FLOATS; e += kSmThreads) sum[e] = 0.0f;
  __syncthreads();
#pragma unroll
  for (int a = 0; a < NB; ++a)
#pragma unroll
    for (int b = 0; b < CB; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int n = 32 * a + 8 * (v >> 2) + 4 * h + (v & 3);
        atomicAdd(&sum[n * COLS + 32 * b + nl], acc[a][b][v]);
      }
  __syncthreads();
  for (int e = tid; e < SUM_FLOATS; e += kSmThreads) {
    const int n = e / COLS, col = e - n * COLS;
    if (n < Cp && col < CK) atomic_add_noret(gW + (size_t)n * CK + col, sum[e]);
  }
  if (gbias != nullptr && tid < Cp) atomic_add_noret(gbias + tid, row_sum);
}

}  // namespace

bool small_conv_supported(const ConvGeom& g) {
  return g.Cg >= 1 && g.Cg <= 4 && g.K >= 1 && g.K <= 25 && g.Cp >= 1 && g.Cp <= 128 &&
         g.B <= 65535 && (int64_t)g.Cg * g.H * g.W < ((int64_t)1 << 31) &&
         (int64_t)g.M * g.K * (g.P > 0 ? g.P : 1) * 2 < ((int64_t)1 << 31);
}

static int padded_blocks(int64_t n) {
  const int b = (int)ceil_div(n, 32);
  return b <= 2 ? b : 4;
}
bool small_wgrad_supported(const ConvGeom& g) {
  // accumulators of a wave: 16 registers per (row block, column block)
  return small_conv_supported(g) && padded_blocks(g.Cp) * padded_blocks((int64_t)g.Cg * g.K) <= 8;
}

int small_forward(const ConvGeom& g, const float* img, const float* map, const float* wts,
                  const float* Wm, const float* bias, float* pix, hipStream_t stream) {
  // few pixels: small workgroups, so that they spread over the CUs
  const int threads = (int64_t)g.M * g.B < 256 * 256 ? 64 : kSmThreads;
  const dim3 grid((unsigned)ceil_div(g.M, threads), (unsigned)g.B);
#define SF(CGv, KMv)                                                                            \
  SDK_DISPATCH_INTERP(g.interp, g.P,                                                            \
                      (launch_lds((small_forward_kernel<INTERP, WEIGHTED, CGv, KMv>),           \
                                          grid, dim3(threads),                                  \
                                          sizeof(float) * (size_t)g.Cp * CGv * KMv, stream, img, map, wts, Wm, \
                                          bias, pix, g.Cg, g.H, g.W, g.Cp, g.M, g.K, g.P)))
  if (g.K <= 9) {
    if (g.Cg <= 1) SF(1, 9); else if (g.Cg <= 3) SF(3, 9); else SF(4, 9);
  } else {
    if (g.Cg <= 1) SF(1, 25); else if (g.Cg <= 3) SF(3, 25); else SF(4, 25);
  }
#undef SF
  SDK_LAUNCH_CHECK("small_forward");
  return SDK_OK;
}

int small_scatter(const ConvGeom& g, const float* pix, const float* map, const float* wts,
                  const float* Wm, float* img, hipStream_t stream) {
  const int threads = (int64_t)g.M * g.B < 256 * 256 ? 64 : kSmThreads;
  const dim3 grid((unsigned)ceil_div(g.M, threads), (unsigned)g.B);
#define SS(CGv, KMv)                                                                            \
  SDK_DISPATCH_INTERP(g.interp, g.P,                                                            \
                      (launch_lds((small_scatter_kernel<INTERP, WEIGHTED, CGv, KMv>),           \
                                          grid, dim3(threads),                                  \
                                          sizeof(float) * (size_t)g.Cp * CGv * KMv, stream, pix, map, wts, Wm, \
                                          img, g.Cg, g.H, g.W, g.Cp, g.M, g.K, g.P)))
  if (g.K <= 9) {
    if (g.Cg <= 1) SS(1, 9); else if (g.Cg <= 3) SS(3, 9); else SS(4, 9);
  } else {
    if (g.Cg <= 1) SS(1, 25); else if (g.Cg <= 3) SS(3, 25); else SS(4, 25);
  }
#undef SS
  SDK_LAUNCH_CHECK("small_scatter");
  return SDK_OK;
}

int small_wgrad(const ConvGeom& g, const float* pix, const float* map, const float* wts,
                const float* img, float* gW, hipStream_t stream, float* gbias) {
  const int NB = (int)ceil_div(g.Cp, 32), CB = (int)ceil_div(g.Cg * g.K, 32);
  const int64_t tiles = ceil_div(g.M, kSmTile);
  // at most about two workgroups per CU over the whole grid: each ends with one atomic per
  // element of gW
  const int64_t want = std::max<int64_t>(1, ceil_div(512, g.B));
  const dim3 grid((unsigned)std::min<int64_t>(tiles, want), (unsigned)g.B);
#define SW(NBv, CBv)                                                                            \
  SDK_DISPATCH_INTERP(g.interp, g.P,                                                            \
                      (launch((small_wgrad_kernel<INTERP, WEIGHTED, NBv, CBv>), grid,           \
                              dim3(kSmThreads), stream, pix, img, map, wts, gW, gbias, g.Cg,    \
                              g.H, g.W, g.Cp, g.M, g.K, g.P)))
#define SWN(CBv)                                                               \
  do {                                                                         \
    if (NB <= 1) SW(1, CBv); else if (NB == 2) SW(2, CBv); else SW(4, CBv);    \
  } while (0)
  if (CB <= 1) SWN(1); else if (CB == 2) SWN(2); else SWN(4);
#undef SWN
#undef SW
  SDK_LAUNCH_CHECK("small_wgrad");
  return SDK_OK;
}

}  // namespace sdk
