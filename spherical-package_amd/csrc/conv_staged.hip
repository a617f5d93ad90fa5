// LDS-staged fused convolution kernels for gfx950 (float32 tensors, fp32 MFMA).
//
// gather_gemm:  pix[b][n, m] = sum_{c,k} Wm[n,(c,k)] * gather(img[b,c], tap(m,k)) + bias[n]
//
// A 256-thread workgroup owns a 2-D tile of 128 map pixels and NB*32 output
// channels.  Each of its 4 wavefronts owns 32 of the pixels and all NB*32
// channels (NB MFMA accumulators of 32 x 32).  Per chunk of kCC image channels
// the tile's image window is staged in LDS (conv_staged.hpp); then, for every
// kernel sample k, each lane turns its pixel's sample points into taps, gathers
// the column values of its pixel from LDS straight into the MFMA B-operand
// registers (lane l: pixel l%32, channel parity l/32) and multiplies with weight
// fragments loaded as one 16-byte read per lane from a pre-permuted weight
// copy.  No column tile and no barrier inside the k loop.
//
// MFMA 32x32x2 f32 register layout (wave64, lane l):
//   A operand: A[i = l % 32][k = l / 32]        B operand: B[k = l / 32][j = l % 32]
//   D, 16 registers v: D[i = 8*(v/4) + 4*(l/32) + v%4][j = l % 32]
#include <hip/hip_runtime.h>

#include "conv_fused.hpp"
#include "conv_staged.hpp"
#include "sdk_host.hpp"
#include "sdk_mfma.hpp"

namespace sdk {


constexpr int kStThreads = 256;

__device__ __forceinline__ int st_mfma_row(int v, int lane) {
  return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
}

__device__ __forceinline__ int st_xcd_band(int bid, int n) {
  constexpr int X = 8;
  const int per = n / X;
  if (bid >= per * X) return bid;
  return (bid % X) * per + bid / X;
}

// Weight copy for gather_gemm: Wp[k][c][nt][(n % 32) * NB + (n / 32) % NB] for
// n-tiles of NB*32 channels, zero padded to CgP x (n_tiles * NB * 32).
__global__ __launch_bounds__(kStThreads) void permute_weight_gather_kernel(
    const float* __restrict__ Wm, float* __restrict__ out, int Cp, int Cg, int K, int CgP,
    int n_tiles, int NB) {
  const int TN = NB * 32;
  const size_t total = (size_t)K * CgP * n_tiles * TN;
  for (size_t e = (size_t)blockIdx.x * kStThreads + threadIdx.x; e < total;
       e += (size_t)gridDim.x * kStThreads) {
    const int inner = (int)(e % TN);
    const int nt = (int)((e / TN) % n_tiles);
    const int c = (int)((e / ((size_t)TN * n_tiles)) % CgP);
    const int k = (int)(e / ((size_t)TN * n_tiles * CgP));
    const int n = nt * TN + (inner % NB) * 32 + inner / NB;
    out[e] = (n < Cp && c < Cg) ? Wm[(size_t)n * Cg * K + (size_t)c * K + k] : 0.0f;
  }
}

// Stages channels [c0, c0 + kCC) of the tile's window: region[cl * RSp + e].
__device__ __forceinline__ void load_region(const float* __restrict__ img_b, size_t HW, int Cg,
                                            int c0, const Region& rg,
                                            const int* __restrict__ src,
                                            float* __restrict__ region) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  constexpr int PER_WAVE = kCC / 4;
  for (int e = lane; e < rg.RS; e += 64) {
    const int o = src[e];
    float v[PER_WAVE];
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) {
      const int c = c0 + wave * PER_WAVE + j;
      v[j] = (o >= 0 && c < Cg) ? img_b[(size_t)c * HW + o] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) region[(wave * PER_WAVE + j) * rg.RSp + e] = v[j];
  }
}

template <int INTERP, bool WEIGHTED, int NB>
__global__ __launch_bounds__(kStThreads) void staged_gather_gemm_kernel(
    const float* __restrict__ img, const float* __restrict__ map, const float* __restrict__ wts,
    const float* __restrict__ Wp, const float* __restrict__ bias, float* __restrict__ pix, int Cg,
    int H, int W, int Cp, int K, int P, int CgP, int n_tiles, PixelTiling pt) {
  __shared__ float region[kCC * (kRegionCap + 1)];
  __shared__ int tc_e[4 * kTapRows * 32];
  __shared__ float tc_co[4 * kTapRows * 32];
  __shared__ int tc_rs[4 * (kTapKMax + 1)];
  __shared__ int tc_ns[4 * kTapKMax];
  __shared__ int src[kRegionCap];
  __shared__ int bb[4];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5;
  const int tile = st_xcd_band(blockIdx.x, pt.tiles_x * pt.tiles_y * n_tiles);
  const int nt = tile % n_tiles, ptile = tile / n_tiles;
  const int ty0 = (ptile / pt.tiles_x) * pt.TY(), tx0 = (ptile % pt.tiles_x) << pt.tx_shift;
  const int p_local = wave * 32 + (lane & 31);
  const int oy = ty0 + (p_local >> pt.tx_shift), ox = tx0 + (p_local & (pt.TX() - 1));
  const bool pix_ok = oy < pt.OH && ox < pt.OW;
  const int m = oy * pt.OW + ox;
  const int M = pt.OH * pt.OW;
  const size_t HW = (size_t)H * W;
  const float* img_b = img + (size_t)blockIdx.y * Cg * HW;
  const int q = WEIGHTED ? P : 1;
  constexpr int TN = NB * 32;
  constexpr int NT = Taps2D<INTERP>::N;

  const Region rg = find_region<INTERP, WEIGHTED>(map, wts, pt, ty0, tx0, oy, ox, pix_ok, K, P, H,
                                                  W, bb, tc_ns);
  build_region_lut(rg, H, W, src);
  const TapCache tc = build_tap_cache<INTERP, WEIGHTED>(map, wts, pt, oy, ox, pix_ok, K, P, H, W,
                                                        rg, tc_ns, tc_e, tc_co, tc_rs);

  floatx16 acc[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;

  for (int c0 = 0; c0 < CgP; c0 += kCC) {
    __syncthreads();  // previous chunk's readers are done
    load_region(img_b, HW, Cg, c0, rg, src, region);
    __syncthreads();
    // this lane's column rows inside the chunk: 2*step + half
    const float* reg_half = region + half * rg.RSp;
    for (int k = 0; k < K; ++k) {
      float col[kCC / 2];
#pragma unroll
      for (int s = 0; s < kCC / 2; ++s) col[s] = 0.0f;
      // adds one tap (encoded index e, coefficient co) of this lane's pixel to its column rows
      auto gather = [&](int e, float co) {
        if (__all(e >= 0 || co == 0.0f)) {
          const int ee = e >= 0 ? e : 0;
#pragma unroll
          for (int s = 0; s < kCC / 2; ++s) col[s] += co * reg_half[2 * s * rg.RSp + ee];
        } else {
          // some lane's tap lies outside the staged window
#pragma unroll
          for (int s = 0; s < kCC / 2; ++s) {
            float d;
            if (e >= 0) {
              d = reg_half[2 * s * rg.RSp + e];
            } else {
              const int c = c0 + 2 * s + half;
              d = (co != 0.0f && c < Cg) ? img_b[(size_t)c * HW + (-e - 1)] : 0.0f;
            }
            col[s] += co * d;
          }
        }
      };
      if (k < tc.kc) {
        const int r1 = tc.rs[k + 1];
        for (int r = tc.rs[k]; r < r1; ++r)
          gather(tc.e[r * 32 + (lane & 31)], tc.co[r * 32 + (lane & 31)]);
      } else {
        const size_t sbase = ((size_t)(pix_ok ? m : 0) * K + k) * q;
        Taps2D<INTERP> t;
        for (int p = 0; p < q; ++p) {
          t.set(map[(sbase + p) * 2], map[(sbase + p) * 2 + 1], H, W,
                WEIGHTED ? wts[sbase + p] : 1.0f);
#pragma unroll
          for (int i = 0; i < NT; ++i) {
            const float co = pix_ok ? t.w[i] : 0.0f;
            if (__any(co != 0.0f)) gather(rg.encode(t.y[i], t.x[i], W), co);
          }
        }
      }
      // weights: one 16-byte fragment per lane and step, rows c0 + 2*step + half
      const float* wrow = Wp + (((size_t)k * CgP + c0 + half) * n_tiles + nt) * TN + (lane & 31) * NB;
#pragma unroll
      for (int s = 0; s < kCC / 2; ++s) {
        float a[NB];
        const float* wp = wrow + (size_t)(2 * s) * n_tiles * TN;
        if constexpr (NB == 4) {
          const float4 f = *reinterpret_cast<const float4*>(wp);
          a[0] = f.x; a[1] = f.y; a[2] = f.z; a[3] = f.w;
        } else if constexpr (NB == 2) {
          const float2 f = *reinterpret_cast<const float2*>(wp);
          a[0] = f.x; a[1] = f.y;
        } else {
          a[0] = *wp;
        }
#pragma unroll
        for (int i = 0; i < NB; ++i)
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], col[s], acc[i], 0, 0, 0);
      }
    }
  }

  // epilogue: + bias, store; lanes own consecutive pixels of the tile
  if (pix_ok) {
    float* pix_b = pix + (size_t)blockIdx.y * Cp * M;
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int n = nt * TN + 32 * i + st_mfma_row(v, lane);
        if (n < Cp) pix_b[(size_t)n * M + m] = acc[i][v] + (bias ? bias[n] : 0.0f);
      }
  }
}

// ---------------------------------------------------------------------------
// gemm_scatter:  img[b,c] += scatter_{tap(m,k)}( sum_n Wm[n,(c,k)] * pix[b][n,m] )
//
// Same tile / wave / lane ownership as gather_gemm.  The pixel-side operand of
// a lane's 32 pixels (all Cp <= 2*NS channels) stays in registers as MFMA B
// fragments for the whole kernel.  For every chunk of kCC image channels and
// every kernel sample k one 32 x 32 accumulator per wave receives
// D[c][m] = sum_n W[n,(c,k)] pix[n,m]; each lane then splats its accumulator
// rows through its pixel's taps into the LDS window (lds_add_f32; global
// atomics only for taps outside the window).  After the K samples the window
// is flushed to the image with one atomic per element and cleared.
//
// Weight copy Ws[k][chunk][g][half][c % 32][j]: value for n = 2*(4g + j) + half,
// so a lane fetches the A fragments of four consecutive MFMA steps as 16 bytes.
// ---------------------------------------------------------------------------
// With bf16 != 0 the order is Ws[k][chunk][t][half][c % 32][j], n = 16*t + 8*half + j: the
// eight values a lane packs into one bf16 A fragment are 32 contiguous bytes.
__global__ __launch_bounds__(kStThreads) void permute_weight_scatter_kernel(
    const float* __restrict__ Wm, float* __restrict__ out, int Cp, int Cg, int K, int chunks,
    int NS, int bf16) {
  const size_t per_k = (size_t)chunks * NS * 64;
  const size_t total = (size_t)K * per_k;
  for (size_t e = (size_t)blockIdx.x * kStThreads + threadIdx.x; e < total;
       e += (size_t)gridDim.x * kStThreads) {
    int j, cl, half, g, chunk, k, n;
    if (bf16) {
      j = (int)(e & 7);
      cl = (int)((e >> 3) & 31);
      half = (int)((e >> 8) & 1);
      const size_t rest = e >> 9;             // (k * chunks + chunk) * (NS/8) + t
      g = (int)(rest % (NS / 8));
      chunk = (int)((rest / (NS / 8)) % chunks);
      k = (int)(rest / ((size_t)(NS / 8) * chunks));
      n = 16 * g + 8 * half + j;
    } else {
      j = (int)(e & 3);
      cl = (int)((e >> 2) & 31);
      half = (int)((e >> 7) & 1);
      const size_t rest = e >> 8;             // (k * chunks + chunk) * (NS/4) + g
      g = (int)(rest % (NS / 4));
      chunk = (int)((rest / (NS / 4)) % chunks);
      k = (int)(rest / ((size_t)(NS / 4) * chunks));
      n = 2 * (4 * g + j) + half;
    }
    const int c = chunk * kCC + cl;
    out[e] = (n < Cp && c < Cg) ? Wm[(size_t)n * Cg * K + (size_t)c * K + k] : 0.0f;
  }
}

template <int INTERP, bool WEIGHTED, int NS, bool BF16>
__global__ __launch_bounds__(kStThreads) void staged_gemm_scatter_kernel(
    const float* __restrict__ pix, const float* __restrict__ map, const float* __restrict__ wts,
    const float* __restrict__ Ws, float* __restrict__ img, int Cg, int H, int W, int Cp, int K,
    int P, int chunks, PixelTiling pt) {
  __shared__ float region[kCC * (kRegionCap + 1)];
  __shared__ int tc_e[4 * kTapRows * 32];
  __shared__ float tc_co[4 * kTapRows * 32];
  __shared__ int tc_rs[4 * (kTapKMax + 1)];
  __shared__ int tc_ns[4 * kTapKMax];
  __shared__ int src[kRegionCap];
  __shared__ int bb[4];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5;
  const int ptile = st_xcd_band(blockIdx.x, pt.tiles_x * pt.tiles_y);
  const int ty0 = (ptile / pt.tiles_x) * pt.TY(), tx0 = (ptile % pt.tiles_x) << pt.tx_shift;
  const int p_local = wave * 32 + (lane & 31);
  const int oy = ty0 + (p_local >> pt.tx_shift), ox = tx0 + (p_local & (pt.TX() - 1));
  const bool pix_ok = oy < pt.OH && ox < pt.OW;
  const int m = oy * pt.OW + ox;
  const int M = pt.OH * pt.OW;
  const size_t HW = (size_t)H * W;
  float* img_b = img + (size_t)blockIdx.y * Cg * HW;
  const float* pix_b = pix + (size_t)blockIdx.y * Cp * M;
  const int q = WEIGHTED ? P : 1;
  constexpr int NT = Taps2D<INTERP>::N;

  const Region rg = find_region<INTERP, WEIGHTED>(map, wts, pt, ty0, tx0, oy, ox, pix_ok, K, P, H,
                                                  W, bb, tc_ns);
  build_region_lut(rg, H, W, src);
  const TapCache tc = build_tap_cache<INTERP, WEIGHTED>(map, wts, pt, oy, ox, pix_ok, K, P, H, W,
                                                        rg, tc_ns, tc_e, tc_co, tc_rs);

  // pixel-side operand, resident in registers.  fp32: step s holds channel 2*s + half;
  // bf16: fragment t holds channels 16*t + 8*half + 0..7, two per register.
  float bfrag[BF16 ? 1 : NS];
  Bf16Frag bfrag16[BF16 ? NS / 8 : 1];
  if constexpr (BF16) {
#pragma unroll
    for (int t = 0; t < NS / 8; ++t) {
      float f[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int n = 16 * t + 8 * half + j;
        f[j] = (pix_ok && n < Cp) ? pix_b[(size_t)n * M + m] : 0.0f;
      }
      bfrag16[t] = pack_bf16x8(f);
    }
  } else {
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int n = 2 * s + half;
      bfrag[s] = (pix_ok && n < Cp) ? pix_b[(size_t)n * M + m] : 0.0f;
    }
  }
  for (int e = tid; e < kCC * rg.RSp; e += kStThreads) region[e] = 0.0f;
  __syncthreads();

  for (int chunk = 0; chunk < chunks; ++chunk) {
    const int c0 = chunk * kCC;
    for (int k = 0; k < K; ++k) {
      floatx16 acc;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
      const float4* wp = reinterpret_cast<const float4*>(
                             Ws + ((size_t)k * chunks + chunk) * NS * 64) + half * 32 + (lane & 31);
      if constexpr (BF16) {
        // per fragment t: 64 lanes x 8 floats = 128 float4; this lane's pair starts at
        // (half * 32 + lane % 32) * 2
        const float4* wb = reinterpret_cast<const float4*>(
                               Ws + ((size_t)k * chunks + chunk) * NS * 64) +
                           (half * 32 + (lane & 31)) * 2;
#pragma unroll
        for (int t = 0; t < NS / 8; ++t) {
          const float4 lo = wb[t * 128], hi = wb[t * 128 + 1];
          const float f[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
          acc = mfma_bf16(pack_bf16x8(f), bfrag16[t], acc);
        }
      } else {
#pragma unroll
        for (int g = 0; g < NS / 4; ++g) {
          const float4 a = wp[g * 64];
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, bfrag[4 * g + 0], acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, bfrag[4 * g + 1], acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, bfrag[4 * g + 2], acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, bfrag[4 * g + 3], acc, 0, 0, 0);
        }
      }
      // splat: accumulator register v of this lane is channel c0 + row(v), pixel m
      auto splat = [&](int e, float co) {
        if (co != 0.0f) {
          if (e >= 0) {
            float* dst = region + (4 * half) * rg.RSp + e;
            int offs[16];
            float vals[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              offs[v] = (8 * (v >> 2) + (v & 3)) * rg.RSp;
              vals[v] = co * acc[v];
            }
            lds_add_f32_batch<16>(dst, offs, vals);
          } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              const int c = c0 + st_mfma_row(v, lane);
              if (c < Cg) atomic_add_noret(img_b + (size_t)c * HW + (-e - 1), co * acc[v]);
            }
          }
        }
      };
      if (k < tc.kc) {
        const int r1 = tc.rs[k + 1];
        for (int r = tc.rs[k]; r < r1; ++r) splat(tc.e[r * 32 + (lane & 31)], tc.co[r * 32 + (lane & 31)]);
      } else if (pix_ok) {
        const size_t sbase = ((size_t)m * K + k) * q;
        Taps2D<INTERP> t;
        for (int p = 0; p < q; ++p) {
          t.set(map[(sbase + p) * 2], map[(sbase + p) * 2 + 1], H, W,
                WEIGHTED ? wts[sbase + p] : 1.0f);
#pragma unroll
          for (int i = 0; i < NT; ++i)
            if (__any(t.w[i] != 0.0f)) splat(rg.encode(t.y[i], t.x[i], W), t.w[i]);
        }
      }
    }
    // flush this chunk's window to the image and clear it
    __syncthreads();
    {
      constexpr int PER_WAVE = kCC / 4;
      for (int e = lane; e < rg.RS; e += 64) {
        const int o = src[e];
#pragma unroll
        for (int j = 0; j < PER_WAVE; ++j) {
          const int cl = wave * PER_WAVE + j;
          const float v = region[cl * rg.RSp + e];
          region[cl * rg.RSp + e] = 0.0f;
          if (o >= 0 && c0 + cl < Cg && v != 0.0f)
            atomic_add_noret(img_b + (size_t)(c0 + cl) * HW + o, v);
        }
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// Host side.
// ---------------------------------------------------------------------------
static PixelTiling make_tiling(const ConvGeom& g) {
  PixelTiling pt;
  pt.OW = g.OW;
  pt.OH = g.M / g.OW;
  pt.tx_shift = (pt.OH >= 8) ? 4 : (pt.OH >= 4 ? 5 : (pt.OH >= 2 ? 6 : 7));
  pt.tiles_x = (int)ceil_div(pt.OW, pt.TX());
  pt.tiles_y = (int)ceil_div(pt.OH, pt.TY());
  return pt;
}

bool staged_supported(const ConvGeom& g) {
  return g.OW >= 1 && g.M % g.OW == 0 && g.B <= 65535;
}

bool scatter_staged_supported(const ConvGeom& g) { return staged_supported(g) && g.Cp <= 128; }

size_t staged_workspace_bytes(const ConvGeom& g) {
  const size_t CgP = (size_t)(g.Cg + kCC - 1) / kCC * kCC;
  const size_t CpP = (size_t)(g.Cp + 127) / 128 * 128;
  return (size_t)g.K * CgP * CpP * sizeof(float);
}

int staged_gather_gemm(const ConvGeom& g, const float* img, const float* map, const float* wts,
                       const float* Wm, const float* bias, float* pix, float* workspace,
                       hipStream_t stream) {
  const PixelTiling pt = make_tiling(g);
  const int NB = g.Cp > 64 ? 4 : (g.Cp > 32 ? 2 : 1);
  const int TN = NB * 32;
  const int n_tiles = (int)ceil_div(g.Cp, TN);
  const int CgP = (int)ceil_div(g.Cg, kCC) * kCC;
  {
    const size_t total = (size_t)g.K * CgP * n_tiles * TN;
    const int blocks = (int)std::min<size_t>((total + kStThreads - 1) / kStThreads, 2048);
    launch(permute_weight_gather_kernel, dim3(blocks), dim3(kStThreads), stream, Wm, workspace,
           g.Cp, g.Cg, g.K, CgP, n_tiles, NB);
    SDK_LAUNCH_CHECK("permute_weight_gather");
  }
  const dim3 grid((unsigned)(pt.tiles_x * pt.tiles_y * n_tiles), (unsigned)g.B);
#define SG(NBv)                                                                                 \
  SDK_DISPATCH_INTERP(g.interp, g.P,                                                            \
                      (launch(staged_gather_gemm_kernel<INTERP, WEIGHTED, NBv>, grid,           \
                              dim3(kStThreads), stream, img, map, wts, (const float*)workspace, \
                              bias, pix, g.Cg, g.H, g.W, g.Cp, g.K, g.P, CgP, n_tiles, pt)))
  if (NB == 4) SG(4); else if (NB == 2) SG(2); else SG(1);
#undef SG
  SDK_LAUNCH_CHECK("staged_gather_gemm");
  return SDK_OK;
}

int staged_gemm_scatter(const ConvGeom& g, bool bf16, const float* pix, const float* map,
                        const float* wts, const float* Wm, float* img, float* workspace,
                        hipStream_t stream) {
  const PixelTiling pt = make_tiling(g);
  const int NS = g.Cp > 64 ? 64 : (g.Cp > 32 ? 32 : 16);   // MFMA steps: 2 channels each
  const int chunks = (int)ceil_div(g.Cg, kCC);
  {
    const size_t total = (size_t)g.K * chunks * NS * 64;
    const int blocks = (int)std::min<size_t>((total + kStThreads - 1) / kStThreads, 2048);
    launch(permute_weight_scatter_kernel, dim3(blocks), dim3(kStThreads), stream, Wm, workspace,
           g.Cp, g.Cg, g.K, chunks, NS, bf16 ? 1 : 0);
    SDK_LAUNCH_CHECK("permute_weight_scatter");
  }
  const dim3 grid((unsigned)(pt.tiles_x * pt.tiles_y), (unsigned)g.B);
#define SS(NSv, BFv)                                                                                  \
  SDK_DISPATCH_INTERP(g.interp, g.P,                                                             \
                      (launch(staged_gemm_scatter_kernel<INTERP, WEIGHTED, NSv, BFv>, grid,      \
                              dim3(kStThreads), stream, pix, map, wts, (const float*)workspace,  \
                              img, g.Cg, g.H, g.W, g.Cp, g.K, g.P, chunks, pt)))
  if (bf16) { if (NS == 64) SS(64, true); else if (NS == 32) SS(32, true); else SS(16, true); }
  else { if (NS == 64) SS(64, false); else if (NS == 32) SS(32, false); else SS(16, false); }
#undef SS
  SDK_LAUNCH_CHECK("staged_gemm_scatter");
  return SDK_OK;
}

}  // namespace sdk
