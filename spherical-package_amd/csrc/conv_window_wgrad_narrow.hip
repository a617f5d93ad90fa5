// Weight gradient of mapped convolution from an LDS window for narrow layers (at most 64
// pixel-side channels) with nearest taps and no interpolation weights: neighbour lists of a
// mesh, integer grids (gfx950, float32, fp32 MFMA).
//
//   gW[n][c][k] += sum_{b, m} pix[b][n][m] * img[b][c][tap(m, k)]
//
// A column value is a single window element with coefficient one: a 16-bit window offset per
// (sample, pixel), read four steps at a time, and one 4-byte LDS read for the value.  A wave
// can therefore feed a matrix instruction from every operand it builds (the kernel for wide
// layers needs four per operand to pay for the blend) and the work is split so that every wave
// issues the same number:
//
//   workgroup = 32 image channels x NBW blocks of 32 pixel-side channels x all K samples x one
//               batch element x every groups-th tile of the list
//   wave w    = samples 4 i + w (i < KF, "full" samples, K = 4 KF + R) for all NBW row blocks,
//               and of each of the R remaining samples row block w % NBW on the steps s with
//               s % (4 / NBW) == w / NBW: a quarter of that sample's work
//
// The reduction index of v_mfma_f32_32x32x2_f32 is the pixel.  A tile is staged in two halves
// of 64 pixels; step s of a half contracts its pixels m = 32 (l / 32) + s, lane l supplying row
// n = l % 32 of the pixel-side tile as A and channel c = l % 32 of the column tile as B.  Plan
// rows and values are read a group of four steps ahead of their MFMAs.  Everything a tile needs
// from global memory is requested while the MFMAs before it run (the next half's pixel-side
// values and plan rows during each half, the offsets of the next tile's window during the first
// half, the window itself, into registers, during the second), so the only exposed round trips
// are those of a workgroup's first tile.  The accumulators stay in registers over all tiles and
// leave the workgroup once, into a partial-sum buffer that the reduce kernel adds up.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "conv_fused.hpp"
#include "conv_plan.hpp"
#include "conv_window.hpp"
#include "sdk_host.hpp"
#include "sdk_mfma.hpp"

namespace sdk {

namespace {

constexpr int kWnThreads = 256;
constexpr int kWnE = 36;   // floats per window element: 32 channels + 4 of skew
constexpr int kWnH = 64;   // pixels per stage: half a tile
constexpr int kWnG = 68;   // floats per row of the pixel-side tile: 64 pixels + 4 of skew

template <int KF, int R, int NBW, int MM>
__global__ __launch_bounds__(kWnThreads, 2) void window_wgrad_narrow_kernel(
    const float* __restrict__ pix, const float* __restrict__ img, const int* __restrict__ hdr,
    const int* __restrict__ ns, const int2* __restrict__ taps, const int* __restrict__ list,
    const int* __restrict__ count, float* __restrict__ partial, int Cg, int H, int W, int Cp,
    PixelTiling pt, int groups, int batches, int c_chunks) {
  constexpr int CAP = kRegionCap;
  constexpr int K = 4 * KF + R;
  constexpr int ROWS = 32 * NBW;
  constexpr int NPH = 4 / NBW;    // step phases a remaining sample is split into
  constexpr int TPG = 4 / NPH;    // steps of a group of four on which a wave has its share
  constexpr int NACC = KF * NBW + R;
  constexpr int PPT = 8 * NBW;    // pixels of a stage's pixel-side tile staged per thread
  __shared__ __align__(16) float region[(CAP + 1) * kWnE];
  __shared__ __align__(16) float gt[ROWS * kWnG];
  __shared__ __align__(16) unsigned short rowsL[K * kWnH];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 31, h = lane >> 5;
  // Workgroup ids go round-robin over the 8 XCDs.  All workgroups of one tile run (every batch
  // element and channel chunk) read the same plan rows, those of one batch element the same
  // pixel-side tiles: they take consecutive slots of one XCD and meet in its L2.
  const int kinds = c_chunks * batches;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int kind = slot % kinds, group = (slot / kinds) * 8 + xcd;
  if (group >= groups) return;
  const int cc = kind % c_chunks, batch = kind / c_chunks;
  const int c0 = cc * kCC;
  const int M = pt.OH * pt.OW;
  const size_t HW = (size_t)H * W;
  const float* img_b = img + ((size_t)batch * Cg) * HW;
  const float* pix_b = pix + ((size_t)batch * Cp) * M;

  floatx16 acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;

  // B values: window element at byte offset o -> channel j at regb + o
  const char* regb = reinterpret_cast<const char*>(region) + 4 * j;
  // pixel-side tile staging role: row n_s, pixels px_s .. px_s + PPT - 1 of the stage
  const int n_s = tid / (kWnH / PPT), px_s = (tid % (kWnH / PPT)) * PPT;
  const bool n_ok = n_s < Cp;
  const float* pix_row = pix_b + (size_t)(n_ok ? n_s : 0) * M;
  // window staging role: channels 8 wave .. 8 wave + 7 of the elements lane, lane + 64, ...
  constexpr int ITER = (CAP + 63) / 64;
  const int cw = c0 + 8 * wave;
  const char* cbase = reinterpret_cast<const char*>(img_b + (size_t)min(cw, Cg - 1) * HW);
  const unsigned plane = (unsigned)HW * 4u;

  // ---- staging pieces
  int so[ITER];
  float sv[ITER][8];
  auto fetch_offsets = [&](int tile_) {
    const int* lut = hdr + (size_t)tile_ * kHdrStride;
    const int RSn = lut[2] * lut[3];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int e = lane + 64 * it;
      const int d = lut[kHdrLut + min(e, CAP - 1)];
      so[it] = e < RSn ? d : -1;
    }
  };
  auto fetch_window = [&]() {
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        // (slots past the window's end are never stored; channels past Cg read the last one,
        // their columns are dropped with the sums: plain loads from a valid address)
        sv[it][i] = *reinterpret_cast<const float*>(
            cbase + (unsigned)min(i, Cg - 1 - min(cw, Cg - 1)) * plane +
            (unsigned)max(so[it], 0) * 4u);
      }
    }
  };
  auto store_window = [&](int RS) {
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int e = lane + 64 * it;
      if (e < RS) {
        float4* d4 = reinterpret_cast<float4*>(region + e * kWnE + 8 * wave);
        d4[0] = make_float4(sv[it][0], sv[it][1], sv[it][2], sv[it][3]);
        d4[1] = make_float4(sv[it][4], sv[it][5], sv[it][6], sv[it][7]);
      }
    }
  };
  constexpr int NRW = (K * kWnH + kWnThreads - 1) / kWnThreads;
  // plan rows this thread stages per half: entry idx = tid + 256 u = (k, m)
  unsigned row_off[NRW], row_k[NRW];
#pragma unroll
  for (int u = 0; u < NRW; ++u) {
    const int idx = min(kWnThreads * u + tid, K * kWnH - 1);
    row_k[u] = idx >> 6;
    row_off[u] = (idx >> 6) * 128 + (idx & 63);
  }
  typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));
  float pf[PPT];
  int pvalid = 0;   // how many of pf's pixels exist (all of them: pf holds their values)
  int2 pr[NRW];
  int pn[NRW];
  // first pixel of this thread's run in half q_ of a tile, and how many of the run exist
  auto run_of = [&](int tile_, int q_, int* oy, int* ox) {
    const int ty0 = (tile_ / pt.tiles_x) * pt.TY(), tx0 = (tile_ % pt.tiles_x) << pt.tx_shift;
    const int p0 = kWnH * q_ + px_s;
    *oy = ty0 + (p0 >> pt.tx_shift);
    *ox = tx0 + (p0 & (pt.TX() - 1));
    return (n_ok && *oy < pt.OH) ? max(0, min(pt.OW - *ox, PPT)) : 0;
  };
  auto fetch_half = [&](int tile_, int q_) {
    // The run lies in one row of the grid.  A complete run is requested as 16-byte pieces from
    // wherever it starts; any other (the right edge of the grid, rows past Cp) is left to
    // store_half and this request reads the start of the tensor instead.
    int oy, ox;
    pvalid = run_of(tile_, q_, &oy, &ox);
    const float* rowp = pvalid == PPT ? pix_row + (size_t)oy * pt.OW + ox : pix_b;
#pragma unroll
    for (int i = 0; i < PPT / 4; ++i) {
      const float4u v4 = *reinterpret_cast<const float4u*>(rowp + 4 * i);
      pf[4 * i] = v4.x; pf[4 * i + 1] = v4.y; pf[4 * i + 2] = v4.z; pf[4 * i + 3] = v4.w;
    }
    // (uniform base, per-thread constant offset)
    const int2* tp = taps + ((size_t)tile_ * K * 128 + kWnH * q_);
    const int* np = ns + (size_t)tile_ * K;
#pragma unroll
    for (int u = 0; u < NRW; ++u) {
      pr[u] = tp[row_off[u]];
      pn[u] = np[row_k[u]];
    }
  };
  // gt[n][m]; rowsL[k * 64 + m] = window byte offset of the tap, of the zero element for
  // pixels without one
  auto store_half = [&](int tile_, int q_, int RS) {
    float o[PPT];
#pragma unroll
    for (int i = 0; i < PPT; ++i) o[i] = pf[i];
    if (pvalid != PPT) {
#pragma unroll
      for (int i = 0; i < PPT; ++i) o[i] = 0.0f;
      if (pvalid > 0) {
        int oy, ox;
        run_of(tile_, q_, &oy, &ox);
        const float* rowp = pix_row + (size_t)oy * pt.OW + ox;
#pragma unroll
        for (int i = 0; i < PPT; ++i)
          if (i < pvalid) o[i] = rowp[i];
      }
    }
    float4* dst = reinterpret_cast<float4*>(gt + n_s * kWnG + px_s);
#pragma unroll
    for (int i = 0; i < PPT / 4; ++i)
      dst[i] = make_float4(o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]);
#pragma unroll
    for (int u = 0; u < NRW; ++u) {
      const int idx = kWnThreads * u + tid;
      if (idx < K * kWnH) {
        const bool on = pn[u] >= 1 && __int_as_float(pr[u].y) != 0.0f;
        rowsL[idx] = (unsigned short)((on ? pr[u].x : RS) * (kWnE * 4));
      }
    }
  };

  const int cnt = *count;
  if (cnt == 0) return;   // (the summing kernel sees the same count and adds nothing)
  // The workgroups of one XCD take neighbouring tiles of the list at the same time: their
  // windows share cache lines, which then meet in that XCD's L2.
  const int first_ti = (group & 7) * (groups >> 3) + (group >> 3);
  if (first_ti < cnt) {
    const int first = list[first_ti];
    fetch_offsets(first);
    fetch_half(first, 0);
    fetch_window();
  }
  // this wave's share of the remaining samples: row block, step phase
  const int blk_w = wave % NBW, phase = wave / NBW;
  for (int ti = first_ti; ti < cnt; ti += groups) {
    const int tile = list[ti];
    const int* lut = hdr + (size_t)tile * kHdrStride;
    const int RS = lut[2] * lut[3];
    const bool has_next = ti + groups < cnt;
    const int tile_next = has_next ? list[ti + groups] : tile;

    __syncthreads();   // every wave is done with the previous tile
    if (tid < kWnE) region[RS * kWnE + tid] = 0.0f;   // the zero element inactive rows point at
    store_window(RS);

#pragma unroll 1
    for (int q = 0; q < 2; ++q) {
      if (q > 0) __syncthreads();   // the previous half's reads of gt / rowsL are done
      store_half(tile, q, RS);
      __syncthreads();   // (for q == 0 this also publishes the window)
      // requests for what comes next, answered while this half's MFMAs run
      if (has_next) {
        if (q == 0) fetch_offsets(tile_next);
        else fetch_window();
      }
      if (q == 0 || has_next) fetch_half(q == 0 ? tile : tile_next, q ^ 1);

      if constexpr (MM == kMmF32) {
        // ---- eight groups of four MFMA steps; plan rows two groups ahead, values one.  A wave's
        // share of the remaining samples (row block blk_w, steps phase + NPH t of every group)
        // is addressed through per-wave base pointers, so all waves run the same code.
        {
          constexpr int KFa = KF > 0 ? KF : 1, Ra = R > 0 ? R : 1;
          const unsigned short* rows_h = rowsL + 32 * h;
          const unsigned short* rows_r = rows_h + 4 * KF * kWnH + phase;
          const float* gt_r = gt + (32 * blk_w + j) * kWnG + 32 * h + phase;
          uint2 Rn[KFa];             // four steps' offsets of a full sample, 16 bits each
          unsigned Rr[Ra][TPG];      // offsets of this wave's steps of a remaining sample
          float val[KFa][4], valr[Ra][TPG];
          auto rows_issue = [&](int grp) {
            const int gq = grp < 8 ? grp : 7;
#pragma unroll
            for (int i = 0; i < KF; ++i)
              Rn[i] = *reinterpret_cast<const uint2*>(rows_h + (4 * i + wave) * kWnH + 4 * gq);
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
              for (int t = 0; t < TPG; ++t) Rr[r][t] = rows_r[r * kWnH + 4 * gq + NPH * t];
          };
          auto at = [&](const uint2& w, int step) {
            const unsigned d = step < 2 ? w.x : w.y;
            return *reinterpret_cast<const float*>(regb + ((step & 1) ? d >> 16 : d & 0xffffu));
          };
          auto vals_issue = [&]() {
#pragma unroll
            for (int i = 0; i < KF; ++i)
#pragma unroll
              for (int st = 0; st < 4; ++st) val[i][st] = at(Rn[i], st);
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
              for (int t = 0; t < TPG; ++t)
                valr[r][t] = *reinterpret_cast<const float*>(regb + Rr[r][t]);
          };
          rows_issue(0);
          vals_issue();    // group 0
          rows_issue(1);
#pragma unroll
          for (int grp = 0; grp < 8; ++grp) {
            float4 A[NBW];
            float Ar[TPG];
#pragma unroll
            for (int a = 0; a < NBW; ++a)
              A[a] = *reinterpret_cast<const float4*>(gt + (32 * a + j) * kWnG + 32 * h + 4 * grp);
            if constexpr (R > 0) {
#pragma unroll
              for (int t = 0; t < TPG; ++t) Ar[t] = gt_r[4 * grp + NPH * t];
            }
            float b[KFa][4], br[Ra][TPG];
#pragma unroll
            for (int i = 0; i < KF; ++i)
#pragma unroll
              for (int s = 0; s < 4; ++s) b[i][s] = val[i][s];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
              for (int t = 0; t < TPG; ++t) br[r][t] = valr[r][t];
            if (grp < 7) {
              vals_issue();            // group grp + 1
              rows_issue(grp + 2);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
#pragma unroll
              for (int i = 0; i < KF; ++i) {
#pragma unroll
                for (int a = 0; a < NBW; ++a) {
                  const float av = s == 0 ? A[a].x : (s == 1 ? A[a].y : (s == 2 ? A[a].z : A[a].w));
                  acc[i * NBW + a] =
                      __builtin_amdgcn_mfma_f32_32x32x2f32(av, b[i][s], acc[i * NBW + a], 0, 0, 0);
                }
              }
              if constexpr (R > 0) {
                if (s % NPH == NPH - 1) {
                  const int t = s / NPH;
#pragma unroll
                  for (int r = 0; r < R; ++r)
                    acc[KF * NBW + r] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                        Ar[t], br[r][t], acc[KF * NBW + r], 0, 0, 0);
                }
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      } else {
        // ---- bf16 matrix unit (operands rounded to bf16, or split into three bf16 pieces): one
        // instruction contracts 16 pixels, lane (j, h) supplying its row / channel for the eight
        // pixels 8 h .. 8 h + 7 of a group of 16.  A lane reads its eight window offsets of a
        // sample as one 16-byte read and the eight values after them; a wave's share of the
        // remaining samples is row block blk_w on every NPH-th group.
        const unsigned short* rows_g = rowsL + 8 * h;
#pragma unroll 1
        for (int grp = 0; grp < 4; ++grp) {
          auto b_values = [&](int k, float (&f)[8]) {
            const uint4 w = *reinterpret_cast<const uint4*>(rows_g + k * kWnH + 16 * grp);
            const unsigned d[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              f[2 * i] = *reinterpret_cast<const float*>(regb + (d[i] & 0xffffu));
              f[2 * i + 1] = *reinterpret_cast<const float*>(regb + (d[i] >> 16));
            }
          };
          auto a_values = [&](int row, float (&f)[8]) {
            const float4* ap = reinterpret_cast<const float4*>(gt + row * kWnG + 16 * grp + 8 * h);
            const float4 lo = ap[0], hi = ap[1];
            f[0] = lo.x; f[1] = lo.y; f[2] = lo.z; f[3] = lo.w;
            f[4] = hi.x; f[5] = hi.y; f[6] = hi.z; f[7] = hi.w;
          };
          Bf16Frag a16[NBW];
          Bf16Split a3[MM == kMmSplit ? NBW : 1];
          const bool mine = R > 0 && (grp % NPH) == phase;   // this group carries the wave's share
          if (KF > 0 || mine) {
#pragma unroll
            for (int a = 0; a < NBW; ++a) {
              float f[8];
              a_values(32 * a + j, f);
              if constexpr (MM == kMmSplit) a3[a] = split_bf16x8(f);
              else a16[a] = pack_bf16x8(f);
            }
          }
#pragma unroll
          for (int i = 0; i < KF; ++i) {
            float f[8];
            b_values(4 * i + wave, f);
            if constexpr (MM == kMmSplit) {
              const Bf16Split b3 = split_bf16x8(f);
#pragma unroll
              for (int a = 0; a < NBW; ++a) acc[i * NBW + a] = mfma_split(a3[a], b3, acc[i * NBW + a]);
            } else {
              const Bf16Frag b16 = pack_bf16x8(f);
#pragma unroll
              for (int a = 0; a < NBW; ++a) acc[i * NBW + a] = mfma_bf16(a16[a], b16, acc[i * NBW + a]);
            }
          }
          if (mine) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
              float f[8];
              b_values(4 * KF + r, f);
              if constexpr (MM == kMmSplit) {
                const Bf16Split b3 = split_bf16x8(f);
                // (the row block is the wave's: a select between the two fragments)
                acc[KF * NBW + r] = NBW == 1 || blk_w == 0
                                        ? mfma_split(a3[0], b3, acc[KF * NBW + r])
                                        : mfma_split(a3[NBW - 1], b3, acc[KF * NBW + r]);
              } else {
                const Bf16Frag b16 = pack_bf16x8(f);
                acc[KF * NBW + r] = NBW == 1 || blk_w == 0
                                        ? mfma_bf16(a16[0], b16, acc[KF * NBW + r])
                                        : mfma_bf16(a16[NBW - 1], b16, acc[KF * NBW + r]);
              }
            }
          }
        }
      }
    }
  }

  // ---- every accumulator register is stored as it lies (register-major, thread fastest)
  float* dst = partial + (size_t)blockIdx.x * (NACC * 16 * kWnThreads) + tid;
#pragma unroll
  for (int i = 0; i < NACC; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) dst[(i * 16 + v) * kWnThreads] = acc[i][v];
}

// Sums the accumulator copies of window_wgrad_narrow_kernel and adds them to gW.  Block
// (x, y, z): accumulator register x of thread threadIdx.x, channel chunk y, over every z-th of
// the batches * groups workgroups of that chunk.  (The shares of a remaining sample held by
// different waves meet in gW.)
__global__ __launch_bounds__(kWnThreads) void window_wgrad_narrow_reduce_kernel(
    const float* __restrict__ partial, float* __restrict__ gW, int Cg, int Cp, int K, int NBW,
    int groups, int batches, int c_chunks, const int* __restrict__ count) {
  if (*count == 0) return;   // nothing was summed
  const int tid = threadIdx.x, reg = blockIdx.x, cc = blockIdx.y;
  const int kinds = c_chunks * batches;
  const int total = batches * groups;
  const size_t per_wg = (size_t)gridDim.x * kWnThreads;
  // four reads in flight per thread (a plain loop waits for each in turn)
  auto at = [&](int i) {
    const int ic = min(i, total - 1);
    const int b = ic / groups, grp = ic % groups;
    const int kind = b * c_chunks + cc;
    const size_t wg = ((size_t)(grp >> 3) * kinds + kind) * 8 + (grp & 7);
    const float v = partial[wg * per_wg + (size_t)reg * kWnThreads + tid];
    return i < total ? v : 0.0f;
  };
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  const int step = gridDim.z;
  for (int i = blockIdx.z; i < total; i += 4 * step) {
    const float v0 = at(i), v1 = at(i + step), v2 = at(i + 2 * step), v3 = at(i + 3 * step);
    s0 += v0;
    s1 += v1;
    s2 += v2;
    s3 += v3;
  }
  const float s = (s0 + s1) + (s2 + s3);
  const int wave = tid >> 6, lane = tid & 63, j = lane & 31, h = lane >> 5;
  const int v = reg & 15, blk = reg >> 4;
  const int KF = K / 4;
  int k, a;
  if (blk < KF * NBW) {
    k = 4 * (blk / NBW) + wave;
    a = blk % NBW;
  } else {
    k = 4 * KF + (blk - KF * NBW);
    a = wave % NBW;
  }
  const int n = 32 * a + 8 * (v >> 2) + 4 * h + (v & 3);
  const int c = cc * kCC + j;
  if (c < Cg && n < Cp && k < K) atomic_add_noret(gW + (size_t)n * Cg * K + (size_t)c * K + k, s);
}

struct WnGrid {
  int c_chunks, groups, nreg;
  int64_t kinds, slots;
};
// about two workgroups per CU
WnGrid wn_grid(const ConvGeom& g, int tiles) {
  WnGrid w;
  w.c_chunks = (int)ceil_div(g.Cg, kCC);
  w.kinds = (int64_t)w.c_chunks * g.B;
  const int64_t want = std::max<int64_t>(8, ceil_div(ceil_div(512, w.kinds), 8) * 8);
  w.groups = (int)std::min<int64_t>(ceil_div(tiles, 8) * 8, want);
  w.slots = (int64_t)w.groups * w.kinds;
  w.nreg = ((g.K / 4) * (g.Cp > 32 ? 2 : 1) + g.K % 4) * 16;
  return w;
}
}  // namespace

bool window_wgrad_narrow_supported(const ConvGeom& g, int mm) {
  // (nearest taps without interpolation weights: one plan row per sample, coefficient one)
  (void)mm;   // every matrix arithmetic
  if (!(planned_wgrad_supported(g) && g.interp == 0 && g.P == 0 && g.K >= 1 &&
        g.K <= 10 && g.Cp <= 64 && (int64_t)g.H * g.W <= ((int64_t)1 << 24)))
    return false;
  // a thread's run of sixteen pixels of the pixel-side tile lies in one row of the grid and in
  // the tensor
  return g.OW >= 16 && plan_tiling(g.M / g.OW, g.OW).TX() >= 16;
}

size_t window_wgrad_narrow_partial_bytes(const ConvGeom& g) {
  const PixelTiling pt = plan_tiling(g.M / g.OW, g.OW);
  const WnGrid w = wn_grid(g, pt.tiles_x * pt.tiles_y);
  return (size_t)w.slots * w.nreg * kWnThreads * sizeof(float);
}

int window_wgrad_narrow(const ConvGeom& g, int mm, const Plan& plan, const TileLists& tl,
                        const float* pix, const float* img, float* gW, float* partial,
                        hipStream_t stream) {
  const WnGrid w = wn_grid(g, plan.tiles);
  if (w.slots >= ((int64_t)1 << 31))
    return fail(SDK_ERR_UNSUPPORTED, "window_wgrad_narrow: grid too large");
  const int NBW = g.Cp > 32 ? 2 : 1;
  const dim3 grid((unsigned)w.slots);
#define WN3(KFv, Rv, NBWv, MMv)                                                                \
  launch(window_wgrad_narrow_kernel<KFv, Rv, NBWv, MMv>, grid, dim3(kWnThreads), stream, pix,   \
         img, plan.hdr, plan.ns, plan.taps, tl.inside, tl.count, partial, g.Cg, g.H, g.W, g.Cp, \
         plan.pt, w.groups, (int)g.B, w.c_chunks)
#define WN2(KFv, Rv, NBWv)                                       \
  do {                                                           \
    if (mm == kMmBf16) WN3(KFv, Rv, NBWv, kMmBf16);              \
    else if (mm == kMmSplit) WN3(KFv, Rv, NBWv, kMmSplit);       \
    else WN3(KFv, Rv, NBWv, kMmF32);                             \
  } while (0)
#define WN(KFv, Rv)                                        \
  do {                                                     \
    if (NBW == 2) WN2(KFv, Rv, 2); else WN2(KFv, Rv, 1);   \
  } while (0)
  switch (g.K) {
    case 1: WN(0, 1); break;
    case 2: WN(0, 2); break;
    case 3: WN(0, 3); break;
    case 4: WN(1, 0); break;
    case 5: WN(1, 1); break;
    case 6: WN(1, 2); break;
    case 7: WN(1, 3); break;
    case 8: WN(2, 0); break;
    case 9: WN(2, 1); break;
    default: WN(2, 2); break;
  }
#undef WN
#undef WN2
#undef WN3
  SDK_LAUNCH_CHECK("window_wgrad_narrow");
  const int total = (int)g.B * w.groups;
  const int parts = (int)std::min<int64_t>(std::min(total, 16),
                                           ceil_div(2048, (int64_t)w.nreg * w.c_chunks));
  launch(window_wgrad_narrow_reduce_kernel,
         dim3((unsigned)w.nreg, (unsigned)w.c_chunks, (unsigned)std::max(parts, 1)),
         dim3(kWnThreads), stream, (const float*)partial, gW, g.Cg, g.Cp, g.K, NBW, w.groups,
         (int)g.B, w.c_chunks, tl.count);
  SDK_LAUNCH_CHECK("window_wgrad_narrow_reduce");
  return SDK_OK;
}

}  // namespace sdk
