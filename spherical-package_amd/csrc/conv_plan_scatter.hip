// Plan-driven MFMA -> scatter kernel for gfx950 (float32 tensors):
//
//   img[b,c] += scatter_{tap(m,k)}( sum_n Wm[n,(c,k)] * pix[b][n,m] )
//
// used for conv backward-input and transposed-conv forward.
//
// MFMA 32x32x2 f32 register layout (wave64, lane l):
//   A operand: A[i = l % 32][k = l / 32]        B operand: B[k = l / 32][j = l % 32]
//   D, 16 registers v: D[i = 8*(v/4) + 4*(l/32) + v%4][j = l % 32]
#include <hip/hip_runtime.h>

#include "conv_fused.hpp"
#include "conv_window.hpp"
#include "conv_plan.hpp"
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

// Weight copy for the scatter kernel.  fp32: Ws[k][chunk][g][half][c % 32][j] holds the
// value for n = 2*(4g + j) + half, so a lane fetches the A fragments of four consecutive
// MFMA steps as 16 bytes.  bf16: Ws[k][chunk][t][half][c % 32][j], n = 16*t + 8*half + j: the
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

// ---------------------------------------------------------------------------
// planned_gemm_scatter.  A 256-thread workgroup owns one 2-D tile of 128 map
// pixels of one batch element; each of its 4 waves owns 32 of the pixels.  The
// pixel-side operand of a lane's pixel (all Cp <= 2*NS channels) stays in
// registers as MFMA B fragments for the whole kernel.  For every chunk of kCC
// image channels and every kernel sample k one 32 x 32 accumulator per wave
// receives D[c][m] = sum_n W[n,(c,k)] pix[n,m]; each lane then splats its
// accumulator rows through the plan rows of its pixel (conv_plan.hpp) into the
// tile's image window in LDS (64-bit compare-and-swap adds on channel pairs;
// global atomics only for taps outside the window).  After the K samples the
// window is flushed to the image with one atomic per element and cleared.
// Window and rows come from the plan: no tap arithmetic here, and the rows of
// sample k+1 and the first weight fragments of the next block are fetched while
// sample k is processed.
// ---------------------------------------------------------------------------
template <int NS, bool BF16>
__global__ __launch_bounds__(kStThreads, 2) void planned_gemm_scatter_kernel(
    const float* __restrict__ pix, const int* __restrict__ hdr, const int* __restrict__ ns,
    const int2* __restrict__ taps, const float* __restrict__ Ws, float* __restrict__ img, int Cg,
    int H, int W, int Cp, int K, int S, int chunks, PixelTiling pt, const int* __restrict__ gate,
    const int* __restrict__ big_lut) {
  if (gate != nullptr && *gate == 0) return;   // another kernel has done the work
  // window, channel pairs interleaved: value of (channel c, element e) at
  // region[((c / 2) * RSp + e) * 2 + c % 2], so two channels share an 8-byte word
  __shared__ __align__(8) float region[kCC * (kRegionCap + 1)];
  __shared__ int src[kRegionCap];
  __shared__ int ns_l[kPlanKMax];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5;
  const int tile = st_xcd_band(blockIdx.x, pt.tiles_x * pt.tiles_y);
  const int ty0 = (tile / pt.tiles_x) * pt.TY(), tx0 = (tile % pt.tiles_x) << pt.tx_shift;
  const int p_local = wave * 32 + (lane & 31);
  const int oy = ty0 + (p_local >> pt.tx_shift), ox = tx0 + (p_local & (pt.TX() - 1));
  const bool pix_ok = oy < pt.OH && ox < pt.OW;
  const int m = oy * pt.OW + ox;
  const int M = pt.OH * pt.OW;
  const size_t HW = (size_t)H * W;
  float* img_b = img + (size_t)blockIdx.y * Cg * HW;
  const float* pix_b = pix + (size_t)blockIdx.y * Cp * M;

  Region rg;
  rg.ry0 = hdr[tile * kHdrStride + 0];
  rg.rx0 = hdr[tile * kHdrStride + 1];
  rg.RH = hdr[tile * kHdrStride + 2];
  rg.RW = hdr[tile * kHdrStride + 3];
  rg.RS = rg.RH * rg.RW;
  rg.RSp = rg.RS | 1;
  load_region_lut(hdr + (size_t)tile * kHdrStride, rg.RS, src);
  for (int k = tid; k < K; k += kStThreads) ns_l[k] = ns[(size_t)tile * K + k];
  // plan rows of this tile: uniform base, 32-bit lane offsets
  const char* tile_taps = reinterpret_cast<const char*>(taps + (size_t)tile * K * S * 128);
  // a big tile is taken like any other tile outside its window: its rows name ranks
  const bool big_tile = big_lut != nullptr && hdr[tile * kHdrStride + 7] != 0;
  const int* big_l = big_lut + (big_tile ? (size_t)tile * kBigStride : 0);
  auto plan_row = [&](int k, int r) -> int2 {
    const char* row = tile_taps + (size_t)(k * S + r) * (128 * sizeof(int2));
    int2 ec = *reinterpret_cast<const int2*>(row + (unsigned)p_local * (unsigned)sizeof(int2));
    if (__int_as_float(ec.y) != 0.0f) ec.x = plan_row_at(ec.x, big_tile, big_l);
    return ec;
  };

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

  // rows of the first sample
  int2 cur[4];
  int cur_n = ns_l[0];
#pragma unroll
  for (int r = 0; r < 4; ++r) cur[r] = (r < cur_n) ? plan_row(0, r) : make_int2(0, 0);

  // this lane's 16-byte weight fragments of block (k, chunk); fp32: fragment g at [g * 64],
  // bf16: fragment pair t at [t * 128], [t * 128 + 1]
  auto weight_block = [&](int k, int chunk) -> const float4* {
    const float4* blk = reinterpret_cast<const float4*>(Ws + ((size_t)k * chunks + chunk) * NS * 64);
    return blk + (BF16 ? (half * 32 + (lane & 31)) * 2 : half * 32 + (lane & 31));
  };
  constexpr int kPre = 4;
  float4 wpre[kPre];
  {
    const float4* w0 = weight_block(0, 0);
#pragma unroll
    for (int i = 0; i < kPre; ++i) wpre[i] = BF16 ? w0[(i >> 1) * 128 + (i & 1)] : w0[i * 64];
  }

  for (int chunk = 0; chunk < chunks; ++chunk) {
    const int c0 = chunk * kCC;
    for (int k = 0; k < K; ++k) {
      // ---- rows of the next sample (of the next chunk's first sample after the last one)
      const int kn = (k + 1 < K) ? k + 1 : 0;
      const int nxt_n = ns_l[kn];
      int2 nxt[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) nxt[r] = (r < nxt_n) ? plan_row(kn, r) : make_int2(0, 0);

      floatx16 acc;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
      // weights: 16-byte fragments; the first kPre of a block were fetched during the
      // previous sample's splat, the rest arrive while the first MFMAs run
      const float4* wblk = weight_block(k, chunk);
      if constexpr (BF16) {
        float4 w[NS / 4];
#pragma unroll
        for (int i = 0; i < NS / 4; ++i) w[i] = (i < kPre) ? wpre[i] : wblk[(i >> 1) * 128 + (i & 1)];
#pragma unroll
        for (int t = 0; t < NS / 8; ++t) {
          const float4 lo = w[2 * t], hi = w[2 * t + 1];
          const float f[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
          acc = mfma_bf16(pack_bf16x8(f), bfrag16[t], acc);
        }
      } else {
        // two independent accumulator chains (even / odd step groups), summed at the end
        floatx16 acc2;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc2[v] = 0.0f;
#pragma unroll
        for (int g = 0; g < NS / 4; ++g) {
          const float4 a = (g < kPre) ? wpre[g] : wblk[g * 64];
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, bfrag[4 * g + 0], acc, 0, 0, 0);
          acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, bfrag[4 * g + 1], acc2, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, bfrag[4 * g + 2], acc, 0, 0, 0);
          acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, bfrag[4 * g + 3], acc2, 0, 0, 0);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] += acc2[v];
      }
      // first fragments of the next block (next sample, or first sample of the next chunk)
      {
        const int ck = (k + 1 < K) ? chunk : min(chunk + 1, chunks - 1);
        const float4* wn = weight_block(kn, ck);
#pragma unroll
        for (int i = 0; i < kPre; ++i) wpre[i] = BF16 ? wn[(i >> 1) * 128 + (i & 1)] : wn[i * 64];
      }
      // splat: accumulator register v of this lane is channel c0 + row(v), pixel m
      auto splat = [&](int e, float co) {
        if (co != 0.0f) {
          if (e >= 0) {
            // registers v = 4q + 2pr, +1 are channels 8q + 4*half + 2pr, +1: pair 4q + 2*half + pr
            float2* dst = reinterpret_cast<float2*>(region) + (2 * half) * rg.RSp + e;
#pragma unroll
            for (int hv = 0; hv < 2; ++hv) {   // two batches of 4 pairs keep the register count down
              int offs[4];
              float va[4], vb[4];
#pragma unroll
              for (int u = 0; u < 4; ++u) {
                const int q = 2 * hv + (u >> 1), pr = u & 1;
                offs[u] = (4 * q + pr) * rg.RSp;
                va[u] = co * acc[4 * q + 2 * pr];
                vb[u] = co * acc[4 * q + 2 * pr + 1];
              }
              lds_add_f32x2_batch<4>(dst, offs, va, vb);
            }
          } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              const int c = c0 + st_mfma_row(v, lane);
              if (c < Cg) atomic_add_noret(img_b + (size_t)c * HW + (-e - 1), co * acc[v]);
            }
          }
        }
      };
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (r < cur_n) splat(cur[r].x, __int_as_float(cur[r].y));
      for (int r = 4; r < cur_n; ++r) {
        const int2 ec = plan_row(k, r);
        splat(ec.x, __int_as_float(ec.y));
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) cur[r] = nxt[r];
      cur_n = nxt_n;
    }
    // flush this chunk's window to the image and clear it
    __syncthreads();
    {
      constexpr int PAIRS = kCC / 8;   // channel pairs per wave
      float2* r2 = reinterpret_cast<float2*>(region);
      for (int e = lane; e < rg.RS; e += 64) {
        const int o = src[e];
#pragma unroll
        for (int j = 0; j < PAIRS; ++j) {
          const int pc = wave * PAIRS + j, cl = 2 * pc;
          const float2 v = r2[pc * rg.RSp + e];
          r2[pc * rg.RSp + e] = make_float2(0.0f, 0.0f);
          if (o >= 0 && c0 + cl < Cg && v.x != 0.0f)
            atomic_add_noret(img_b + (size_t)(c0 + cl) * HW + o, v.x);
          if (o >= 0 && c0 + cl + 1 < Cg && v.y != 0.0f)
            atomic_add_noret(img_b + (size_t)(c0 + cl + 1) * HW + o, v.y);
        }
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// Host side.
// ---------------------------------------------------------------------------
size_t staged_workspace_bytes(const ConvGeom& g) {
  const size_t CgP = (size_t)(g.Cg + kCC - 1) / kCC * kCC;
  const size_t CpP = (size_t)(g.Cp + 127) / 128 * 128;
  return (size_t)g.K * CgP * CpP * sizeof(float);
}

bool planned_scatter_supported(const ConvGeom& g) {
  return plan_supported(g) && g.Cp <= 128 && g.B <= 65535;
}

// workspace: permuted weights (staged_workspace_bytes, 256-byte aligned) followed by the plan
int planned_gemm_scatter(const ConvGeom& g, bool bf16, const float* pix, const float* map,
                         const float* wts, const float* Wm, float* img, float* workspace,
                         const int* gate, hipStream_t stream, SharedPlan* shared) {
  const int NS = g.Cp > 64 ? 64 : (g.Cp > 32 ? 32 : 16);   // MFMA steps: 2 channels each
  const int chunks = (int)ceil_div(g.Cg, kCC);
  {
    const size_t total = (size_t)g.K * chunks * NS * 64;
    const int blocks = (int)std::min<size_t>((total + kStThreads - 1) / kStThreads, 2048);
    launch(permute_weight_scatter_kernel, dim3(blocks), dim3(kStThreads), stream, Wm, workspace,
           g.Cp, g.Cg, g.K, chunks, NS, bf16 ? 1 : 0);
    SDK_LAUNCH_CHECK("permute_weight_scatter");
  }
  Plan plan;
  char* plan_ws = reinterpret_cast<char*>(workspace) + ((staged_workspace_bytes(g) + 255) & ~(size_t)255);
  // a plan that only this (gated) kernel reads is built under the same gate; one that is
  // handed on to the weight gradient is built in any case
  int rc = build_plan(g, map, wts, plan_ws, stream, &plan, shared != nullptr ? nullptr : gate,
                      shared != nullptr);
  if (rc) return rc;
  if (shared != nullptr) {
    shared->plan = plan;
    shared->valid = true;
  }
  const dim3 grid((unsigned)plan.tiles, (unsigned)g.B);
#define PS(NSv, BFv)                                                                             \
  launch(planned_gemm_scatter_kernel<NSv, BFv>, grid, dim3(kStThreads), stream, pix, plan.hdr,   \
         plan.ns, plan.taps, (const float*)workspace, img, g.Cg, g.H, g.W, g.Cp, g.K, plan.S,    \
         chunks, plan.pt, gate, plan.big_lut)
  if (bf16) { if (NS == 64) PS(64, true); else if (NS == 32) PS(32, true); else PS(16, true); }
  else { if (NS == 64) PS(64, false); else if (NS == 32) PS(32, false); else PS(16, false); }
#undef PS
  SDK_LAUNCH_CHECK("planned_gemm_scatter");
  return SDK_OK;
}

}  // namespace sdk
