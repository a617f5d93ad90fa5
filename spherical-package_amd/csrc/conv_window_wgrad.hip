// Weight gradient of mapped convolution from an LDS window, driven by a tap plan (gfx950,
// float32 tensors, fp32 MFMA):
//
//   gW[n][c][k] += sum_{b, m} pix[b][n][m] * col[b][(c, k)][m]
//   col[b][(c, k)][m] = sum_r coefficient(m, k, r) * img[b][c][tap(m, k, r)]
//
// for the tiles of a plan (conv_plan.hpp) whose taps all lie inside the tile's image window
// and whose samples have at most four plan rows.  The reduction index of the MFMA is the
// pixel: v_mfma_f32_32x32x2_f32 step s contracts the two pixels m = s and m = 16 + s of a
// quarter tile (32 pixels), lane l supplying row n = l % 32 of the pixel-side tile as A and
// channel c = l % 32 of the column tile as B, each for pixel 16 (l / 32) + s.
//
//   workgroup = 32 image channels (one chunk) x 128 pixel-side channels x all K samples x one
//               batch element x every groups-th tile of the list
//   wave w    = samples w KP .. w KP + KP - 1 for all four 32-row blocks of n ("full" samples,
//               K = 4 KP + R), and row block w for each of the R remaining samples
//
// so a wave builds the column values of its own samples itself, straight into B operands:
// per step and sample two LDS reads fetch the four plan rows of the lane's pixel (window byte
// offset, coefficient; the same address across a half wave), four LDS reads the window values
// of the lane's channel, four multiply-adds blend them.  Nothing is exchanged between waves
// and there is no barrier inside a quarter tile.  The pixel-side tile (128 x 32 values) and the
// quarter's plan rows are staged in LDS once per quarter, the window once per tile.  The
// accumulators ((4 KP + R) x 16 registers) stay in registers over all tiles and leave the
// workgroup once, into a partial-sum buffer that window_wgrad_reduce_kernel adds up.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "conv_fused.hpp"
#include "conv_plan.hpp"
#include "conv_window.hpp"
#include "sdk_host.hpp"
#include "sdk_mfma.hpp"

namespace sdk {

namespace {

constexpr int kWwThreads = 256;
constexpr int kWwE = 36;   // floats per window element: 32 channels + 4 of skew
constexpr int kWwG = 36;   // floats per row of the pixel-side tile: 32 pixels + 4 of skew
constexpr int kWwQ = 32;   // pixels per quarter tile
constexpr int kWwRows = 4; // plan rows per sample this kernel applies

// CAP: elements of the LDS window.  kRegionCap: the tiles of `list` lie inside their window.
// kBigCap: `list` holds big tiles, whose window is their list in big_lut; one workgroup per CU.
// With one wave per SIMD nothing else covers a global read, so that variant requests ahead what
// it has registers for: the pixel-side tile and the plan rows of the next quarter, and the
// offsets of the next tile's window, before a quarter's MFMAs.
// ONE: every sample of the plan has a single row (nearest taps without interpolation weights);
// the step loop then reads and applies that row alone instead of four, three of them padding.
template <int KP, int R, int CAP, int MM, bool ONE = false>
__global__ __launch_bounds__(kWwThreads, CAP > kRegionCap ? 1 : 2) void window_wgrad_kernel(
    const float* __restrict__ pix, const float* __restrict__ img, const int* __restrict__ hdr,
    const int* __restrict__ ns, const int2* __restrict__ taps, const int* __restrict__ list,
    const int* __restrict__ count, float* __restrict__ partial, int Cg, int H, int W, int Cp,
    int S, PixelTiling pt, int groups, int batches, int c_chunks, int n_tiles, int vec4,
    const int* __restrict__ big_lut) {
  constexpr int K = 4 * KP + R;
  constexpr bool BIG = CAP > kRegionCap;
  // (with two workgroups per CU the registers are not there: the requests spill and the kernel
  // takes half as long again)
  constexpr bool PIPE = BIG;
  __shared__ __align__(16) float region[(CAP + 1) * kWwE];
  __shared__ __align__(16) float gt[128 * kWwG];
  __shared__ __align__(16) int2 rowsL[K * kWwQ * kWwRows];
  __shared__ int src[BIG ? 1 : CAP];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // (a scalar for the compiler)
  const int j = lane & 31, h = lane >> 5;
  // Workgroup ids go round-robin over the 8 XCDs.  All workgroups of one tile run (every
  // batch element and channel chunk) read the same plan rows, those of one batch element the
  // same pixel-side tiles: they take consecutive slots of one XCD and meet in its L2.
  const int kinds = c_chunks * n_tiles * batches;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int kind = slot % kinds, group = (slot / kinds) * 8 + xcd;
  if (group >= groups) return;
  const int nt = kind % n_tiles, cc = (kind / n_tiles) % c_chunks;
  const int batch = kind / (n_tiles * c_chunks);
  const int c0 = cc * kCC, n0 = nt * 128;
  const int M = pt.OH * pt.OW;
  const size_t HW = (size_t)H * W;
  const float* img_b = img + ((size_t)batch * Cg) * HW;
  const float* pix_b = pix + ((size_t)batch * Cp) * M;

  floatx16 accF[KP > 0 ? KP : 1][4];
  floatx16 accR[R > 0 ? R : 1];
#pragma unroll
  for (int i = 0; i < (KP > 0 ? KP : 1); ++i)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) accF[i][a][v] = 0.0f;
#pragma unroll
  for (int i = 0; i < (R > 0 ? R : 1); ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) accR[i][v] = 0.0f;

  // B values: window element at byte offset o -> channel j at regb + o
  const char* regb = reinterpret_cast<const char*>(region) + 4 * j;
  // pixel-side tile staging role: row n_s, pixels 16 hr_s .. 16 hr_s + 15 of the quarter
  const int n_s = tid >> 1, hr_s = tid & 1;
  const bool n_ok = n0 + n_s < Cp;
  const float* pix_row = pix_b + (size_t)(n_ok ? n0 + n_s : 0) * M;

  // ---- staging pieces.  Window: wave w stages channels 8w .. 8w+7 of every element; a lane
  // owns elements lane, lane + 64, ... and has all its loads in flight before the first LDS write.
  constexpr int ITER = (CAP + 63) / 64;
  const int cw = c0 + 8 * wave;
  const char* cbase = reinterpret_cast<const char*>(img_b + (size_t)min(cw, Cg - 1) * HW);
  const unsigned plane = (unsigned)HW * 4u;
  // wv[it][i] = channel cw + i of the element at flat offset wo[it] (-1: none)
  auto fetch_window = [&](const int (&wo)[ITER], float (&wv)[ITER][8]) {
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        // Plain loads from a valid address, nothing that could become a branch around a load
        // (with a condition on the load the generated code took one of the eight of every
        // round behind a branch and waited for it there: five round trips per window instead
        // of one).  Slots past the window's end are never stored, the columns of channels
        // past Cg are dropped with the sums, and elements a box window has outside the image
        // (offset -1) are zeroed where they are stored.
        const unsigned ch = __builtin_amdgcn_readfirstlane(
            (unsigned)min(i, Cg - 1 - min(cw, Cg - 1)) * plane);
        wv[it][i] = *reinterpret_cast<const float*>(cbase + ch + (unsigned)max(wo[it], 0) * 4u);
      }
    }
  };
  auto store_window = [&](int RS, const int (&wo)[ITER], const float (&wv)[ITER][8]) {
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int e = lane + 64 * it;
      if (e < RS) {
        float4* d4 = reinterpret_cast<float4*>(region + e * kWwE + 8 * wave);
        if (wo[it] >= 0) {
          d4[0] = make_float4(wv[it][0], wv[it][1], wv[it][2], wv[it][3]);
          d4[1] = make_float4(wv[it][4], wv[it][5], wv[it][6], wv[it][7]);
        } else {
          d4[0] = make_float4(0.f, 0.f, 0.f, 0.f);
          d4[1] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
    }
  };
  // Quarter q of a tile: this thread's 16 values of the pixel-side tile (row n_s, pixels
  // 16 hr_s .. + 15) and its share of the plan rows, entry idx = tid + 256 u = (k, r, m), with
  // the rows its sample has (the row itself is read whether it exists or not, clamped to S).
  constexpr int TOTAL = K * kWwRows * kWwQ;
  constexpr int NR = (TOTAL + kWwThreads - 1) / kWwThreads;
  unsigned row_off[NR], row_k[NR];
#pragma unroll
  for (int u = 0; u < NR; ++u) {
    const int idx = min(kWwThreads * u + tid, TOTAL - 1);
    const int k = idx >> 7, r = (idx >> 5) & 3, m = idx & 31;
    row_k[u] = k;
    row_off[u] = (k * S + min(r, S - 1)) * 128 + m;
  }
  auto fetch_quarter = [&](int tile_, int q_, float4 (&gq)[4], int2 (&pr)[NR], int (&pn)[NR]) {
    const int ty0_ = (tile_ / pt.tiles_x) * pt.TY(), tx0_ = (tile_ % pt.tiles_x) << pt.tx_shift;
    const int p0 = kWwQ * q_ + 16 * hr_s;
    if (vec4) {
      const int oy = ty0_ + (p0 >> pt.tx_shift), ox = tx0_ + (p0 & (pt.TX() - 1));
      const float* rowp = pix_row + (size_t)oy * pt.OW + ox;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        gq[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (n_ok && oy < pt.OH && ox + 4 * i < pt.OW)
          gq[i] = *reinterpret_cast<const float4*>(rowp + 4 * i);
      }
    } else {
      float f[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int p = p0 + i;
        const int oy = ty0_ + (p >> pt.tx_shift), ox = tx0_ + (p & (pt.TX() - 1));
        const bool ok = n_ok && oy < pt.OH && ox < pt.OW;
        const float d = pix_row[ok ? (size_t)oy * pt.OW + ox : 0];
        f[i] = ok ? d : 0.0f;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) gq[i] = make_float4(f[4 * i], f[4 * i + 1], f[4 * i + 2], f[4 * i + 3]);
    }
    // (uniform bases, per-thread constant offsets: no 64-bit address arithmetic per entry)
    const int2* tp = taps + ((size_t)tile_ * K * S * 128 + kWwQ * q_);
    const int* np = ns + (size_t)tile_ * K;
#pragma unroll
    for (int u = 0; u < NR; ++u) {
      pr[u] = tp[row_off[u]];
      pn[u] = np[row_k[u]];
    }
  };
  auto store_quarter = [&](int RS, const float4 (&gq)[4], const int2 (&pr)[NR],
                           const int (&pn)[NR]) {
    float4* dst = reinterpret_cast<float4*>(gt + n_s * kWwG + 16 * hr_s);
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[i] = gq[i];
#pragma unroll
    for (int u = 0; u < NR; ++u) {
      const int idx = kWwThreads * u + tid;
      if (idx < TOTAL) {
        const int k = idx >> 7, r = (idx >> 5) & 3, m = idx & 31;
        const bool on = r < min(pn[u], min(S, kWwRows)) && __int_as_float(pr[u].y) != 0.0f;
        rowsL[(k * kWwQ + m) * kWwRows + r] =
            make_int2((on ? pr[u].x : RS) * (kWwE * 4), on ? pr[u].y : 0);
      }
    }
  };
  // what the big variant holds ahead: the coming quarter, the offsets of the next tile's window
  float4 pg[4];
  int2 pr[NR];
  int pn[NR];
  int wo[BIG ? ITER : 1];
  // offsets of the window elements this lane stages for big tile `tile_`
  auto fetch_offsets = [&](int tile_) {
    const int* bl = big_lut + (size_t)tile_ * kBigStride;
    const int RSn = min(bl[0], CAP);
#pragma unroll
    for (int it = 0; it < (BIG ? ITER : 1); ++it) {
      const int e = lane + 64 * it;
      wo[it] = e < RSn ? bl[kBigLut + e] : -1;
    }
  };

  const int cnt = *count;
  if (cnt == 0) return;   // (the summing kernel sees the same count and adds nothing)
  // The workgroups of one XCD take neighbouring tiles of the list at the same time: their
  // windows share cache lines, which then meet in that XCD's L2.
  const int first_ti = (group & 7) * (groups >> 3) + (group >> 3);
  if constexpr (PIPE) {
    if (first_ti < cnt) {
      const int first = list[first_ti];
      if constexpr (BIG) fetch_offsets(first);
      fetch_quarter(first, 0, pg, pr, pn);
    }
  }
  for (int ti = first_ti; ti < cnt; ti += groups) {
    const int tile = list[ti];
    int RS;
    const int* lut;
    if constexpr (BIG) {
      lut = big_lut + (size_t)tile * kBigStride;
      RS = min(lut[0], CAP);
    } else {
      lut = hdr + (size_t)tile * kHdrStride;
      RS = lut[2] * lut[3];
    }
    const bool has_next = ti + groups < cnt;
    const int tile_next = has_next ? list[ti + groups] : tile;

    __syncthreads();   // every wave is done with the previous tile
    if (tid < kWwE) region[RS * kWwE + tid] = 0.0f;   // the zero element inactive rows point at
    if constexpr (BIG) {
      float sv[ITER][8];
      fetch_window(wo, sv);
      store_window(RS, wo, sv);
    } else {
      for (int e = tid; e < RS; e += kWwThreads) src[e] = lut[kHdrLut + e];
      __syncthreads();
      int so[ITER];
      float sv[ITER][8];
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        const int e = lane + 64 * it;
        so[it] = e < RS ? src[e] : -1;
      }
      fetch_window(so, sv);
      store_window(RS, so, sv);
    }

#pragma unroll 1
    for (int q = 0; q < 4; ++q) {
      if (q > 0) __syncthreads();   // the previous quarter's reads of gt / rowsL are done
      if constexpr (PIPE) {
        store_quarter(RS, pg, pr, pn);
      } else {
        // ---- pixel-side tile of the quarter: gt[n][m], m = 16 hr + i; plan rows of the
        // quarter: rowsL[(k * 32 + m) * 4 + r] = (window byte offset, coefficient)
        fetch_quarter(tile, q, pg, pr, pn);
        store_quarter(RS, pg, pr, pn);
      }
      __syncthreads();   // (for q == 0 this also publishes the window)
      if constexpr (PIPE) {
        // requests for what comes next, answered while this quarter's MFMAs run
        if (q < 3) fetch_quarter(tile, q + 1, pg, pr, pn);
        else if (has_next) {
          fetch_quarter(tile_next, 0, pg, pr, pn);
          if constexpr (BIG) fetch_offsets(tile_next);
        }
      }

      if constexpr (MM == kMmF32) {
      // ---- 16 MFMA steps over the quarter's pixels m = 16 h + s, as a three-stage pipeline:
      // while the MFMAs of step s issue, the window values of step s + 1 and the plan rows of
      // step s + 2 are in flight, so no LDS round trip stands between two steps' MFMAs.
      constexpr int KW = KP + R;   // columns (samples) this wave builds per step
      int4 R01[KW], R23[KW];       // plan rows, two steps ahead
      float co[KW][4], val[KW][4]; // coefficients and window values, one step ahead
      float bcur[KW];
      const int2* rows_h = rowsL + (16 * h) * kWwRows;
#define SDK_ROWS_ISSUE(stepv)                                                        \
  do {                                                                               \
    const int st = (stepv) < 16 ? (stepv) : 15;                                      \
    _Pragma("unroll") for (int c = 0; c < KW; ++c) {                                 \
      const int k = c < KP ? wave * KP + c : 4 * KP + (c - KP);                      \
      const int4* rp = reinterpret_cast<const int4*>(rows_h + (k * kWwQ + st) * kWwRows); \
      if constexpr (ONE) {                                                           \
        const int2 r0 = *reinterpret_cast<const int2*>(rp);                          \
        R01[c].x = r0.x;                                                             \
        R01[c].y = r0.y;                                                             \
      } else {                                                                       \
        R01[c] = rp[0];                                                              \
        R23[c] = rp[1];                                                              \
      }                                                                              \
    }                                                                                \
  } while (0)
#define SDK_VALS_ISSUE()                                                             \
  do {                                                                               \
    _Pragma("unroll") for (int c = 0; c < KW; ++c) {                                 \
      val[c][0] = *reinterpret_cast<const float*>(regb + R01[c].x);                  \
      co[c][0] = __int_as_float(R01[c].y);                                           \
      if constexpr (!ONE) {                                                          \
        val[c][1] = *reinterpret_cast<const float*>(regb + R01[c].z);                \
        val[c][2] = *reinterpret_cast<const float*>(regb + R23[c].x);                \
        val[c][3] = *reinterpret_cast<const float*>(regb + R23[c].z);                \
        co[c][1] = __int_as_float(R01[c].w);                                         \
        co[c][2] = __int_as_float(R23[c].y);                                         \
        co[c][3] = __int_as_float(R23[c].w);                                         \
      }                                                                              \
    }                                                                                \
  } while (0)
#define SDK_BLEND(dst)                                                               \
  do {                                                                               \
    _Pragma("unroll") for (int c = 0; c < KW; ++c) {                                 \
      float bv = co[c][0] * val[c][0];                                               \
      if constexpr (!ONE) {                                                          \
        bv = __builtin_fmaf(co[c][1], val[c][1], bv);                                \
        bv = __builtin_fmaf(co[c][2], val[c][2], bv);                                \
        bv = __builtin_fmaf(co[c][3], val[c][3], bv);                                \
      }                                                                              \
      dst[c] = bv;                                                                   \
    }                                                                                \
  } while (0)
      SDK_ROWS_ISSUE(0);
      SDK_VALS_ISSUE();    // step 0
      SDK_ROWS_ISSUE(1);
      SDK_BLEND(bcur);     // step 0
      SDK_VALS_ISSUE();    // step 1
      SDK_ROWS_ISSUE(2);
      float4 A[4], Aw;
#pragma unroll
      for (int step = 0; step < 16; ++step) {
        if ((step & 3) == 0) {
#pragma unroll
          for (int a = 0; a < 4; ++a)
            A[a] = *reinterpret_cast<const float4*>(gt + (32 * a + j) * kWwG + 16 * h + step);
          Aw = *reinterpret_cast<const float4*>(gt + (32 * wave + j) * kWwG + 16 * h + step);
        }
        const int ss = step & 3;
        const float a0 = ss == 0 ? A[0].x : (ss == 1 ? A[0].y : (ss == 2 ? A[0].z : A[0].w));
        const float a1 = ss == 0 ? A[1].x : (ss == 1 ? A[1].y : (ss == 2 ? A[1].z : A[1].w));
        const float a2 = ss == 0 ? A[2].x : (ss == 1 ? A[2].y : (ss == 2 ? A[2].z : A[2].w));
        const float a3 = ss == 0 ? A[3].x : (ss == 1 ? A[3].y : (ss == 2 ? A[3].z : A[3].w));
        const float aw = ss == 0 ? Aw.x : (ss == 1 ? Aw.y : (ss == 2 ? Aw.z : Aw.w));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < KP; ++kk) {
          accF[kk][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, bcur[kk], accF[kk][0], 0, 0, 0);
          accF[kk][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, bcur[kk], accF[kk][1], 0, 0, 0);
          accF[kk][2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a2, bcur[kk], accF[kk][2], 0, 0, 0);
          accF[kk][3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a3, bcur[kk], accF[kk][3], 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
          accR[r] = __builtin_amdgcn_mfma_f32_32x32x2f32(aw, bcur[KP + r], accR[r], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (step < 15) {
          SDK_BLEND(bcur);                      // step + 1
          if (step < 14) SDK_VALS_ISSUE();      // step + 2
          if (step < 13) SDK_ROWS_ISSUE(step + 3);
        }
      }
#undef SDK_ROWS_ISSUE
#undef SDK_VALS_ISSUE
#undef SDK_BLEND
      } else {
        // ---- bf16 matrix unit (operands rounded to bf16, or split into three bf16 pieces):
        // one instruction contracts 16 pixels, lane (j, h) supplying its row / channel for the
        // eight pixels 8 h .. 8 h + 7 of the group.  A lane therefore builds eight column values
        // per sample and instruction from the window (the same reads and multiply-adds per
        // pixel as above) and takes its eight values of a row of the pixel-side tile as two
        // 16-byte reads.  The matrix unit is a small part of the time here; the kernel is bound
        // by the operand construction.
        constexpr int KW = KP + R;
#pragma unroll 1
        for (int grp = 0; grp < 2; ++grp) {
          const int m0 = 16 * grp + 8 * h;   // first of this lane's eight pixels of the quarter
          Bf16Frag b16[KW];
          Bf16Split b3[MM == kMmSplit ? KW : 1];
#pragma unroll
          for (int c = 0; c < KW; ++c) {
            const int k = c < KP ? wave * KP + c : 4 * KP + (c - KP);
            const int4* rp = reinterpret_cast<const int4*>(rowsL + (k * kWwQ + m0) * kWwRows);
            float bv[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              const int4 r01 = rp[2 * i], r23 = rp[2 * i + 1];
              const float v0 = *reinterpret_cast<const float*>(regb + r01.x);
              const float v1 = *reinterpret_cast<const float*>(regb + r01.z);
              const float v2 = *reinterpret_cast<const float*>(regb + r23.x);
              const float v3 = *reinterpret_cast<const float*>(regb + r23.z);
              float t = __int_as_float(r01.y) * v0;
              t = __builtin_fmaf(__int_as_float(r01.w), v1, t);
              t = __builtin_fmaf(__int_as_float(r23.y), v2, t);
              bv[i] = __builtin_fmaf(__int_as_float(r23.w), v3, t);
            }
            if constexpr (MM == kMmSplit) b3[c] = split_bf16x8(bv);
            else b16[c] = pack_bf16x8(bv);
          }
          // A fragments: rows 32 a + j (and 32 wave + j for the remaining samples)
          auto a_values = [&](int row, float (&f)[8]) {
            const float4* ap = reinterpret_cast<const float4*>(gt + row * kWwG + m0);
            const float4 lo = ap[0], hi = ap[1];
            f[0] = lo.x; f[1] = lo.y; f[2] = lo.z; f[3] = lo.w;
            f[4] = hi.x; f[5] = hi.y; f[6] = hi.z; f[7] = hi.w;
          };
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            if constexpr (KP > 0) {
              float f[8];
              a_values(32 * a + j, f);
              if constexpr (MM == kMmSplit) {
                const Bf16Split a3 = split_bf16x8(f);
#pragma unroll
                for (int kk = 0; kk < KP; ++kk) accF[kk][a] = mfma_split(a3, b3[kk], accF[kk][a]);
              } else {
                const Bf16Frag a16 = pack_bf16x8(f);
#pragma unroll
                for (int kk = 0; kk < KP; ++kk) accF[kk][a] = mfma_bf16(a16, b16[kk], accF[kk][a]);
              }
            }
          }
          if constexpr (R > 0) {
            float f[8];
            a_values(32 * wave + j, f);
            if constexpr (MM == kMmSplit) {
              const Bf16Split a3 = split_bf16x8(f);
#pragma unroll
              for (int r = 0; r < R; ++r) accR[r] = mfma_split(a3, b3[KP + r], accR[r]);
            } else {
              const Bf16Frag a16 = pack_bf16x8(f);
#pragma unroll
              for (int r = 0; r < R; ++r) accR[r] = mfma_bf16(a16, b16[KP + r], accR[r]);
            }
          }
        }
      }
    }
  }

  // ---- every accumulator register is stored as it lies (register-major, thread fastest)
  constexpr int NREG = (4 * KP + R) * 16;
  float* dst = partial + (size_t)blockIdx.x * (NREG * kWwThreads) + tid;
#pragma unroll
  for (int kk = 0; kk < KP; ++kk)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) dst[((kk * 4 + a) * 16 + v) * kWwThreads] = accF[kk][a][v];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int v = 0; v < 16; ++v) dst[((KP * 4 + r) * 16 + v) * kWwThreads] = accR[r][v];
}

// Sums the accumulator copies of window_wgrad_kernel and adds them to gW.  Block (x, y, z):
// accumulator register x of thread threadIdx.x, for the workgroup kind y = (channel chunk,
// row tile), over every z-th of the batches * groups workgroups of that kind.
__global__ __launch_bounds__(kWwThreads) void window_wgrad_reduce_kernel(
    const float* __restrict__ partial, float* __restrict__ gW, int Cg, int Cp, int K, int KP,
    int R, int groups, int batches, int c_chunks, int n_tiles, const int* __restrict__ count) {
  if (*count == 0) return;   // nothing was summed
  const int tid = threadIdx.x, reg = blockIdx.x;
  const int nt = blockIdx.y % n_tiles, cc = blockIdx.y / n_tiles;
  const int kinds = c_chunks * n_tiles * batches;
  const int total = batches * groups;
  const size_t per_wg = (size_t)(4 * KP + R) * 16 * kWwThreads;
  // four reads in flight per thread (a plain loop waits for each in turn)
  auto at = [&](int i) {
    const int ic = min(i, total - 1);
    const int b = ic / groups, grp = ic % groups;
    const int kind = (b * c_chunks + cc) * n_tiles + nt;
    const size_t wg = ((size_t)(grp >> 3) * kinds + kind) * 8 + (grp & 7);
    const float v = partial[wg * per_wg + (size_t)reg * kWwThreads + tid];
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
  int k, a;
  if (blk < 4 * KP) {
    k = wave * KP + blk / 4;
    a = blk & 3;
  } else {
    k = 4 * KP + (blk - 4 * KP);
    a = wave;
  }
  const int n = nt * 128 + 32 * a + 8 * (v >> 2) + 4 * h + (v & 3);
  const int c = cc * kCC + j;
  if (c < Cg && n < Cp && k < K) atomic_add_noret(gW + (size_t)n * Cg * K + (size_t)c * K + k, s);
}

struct WwGrid {
  int c_chunks, n_tiles, groups, nreg;
  int64_t kinds, slots;
};
// big: the launch over the big tiles (one workgroup per CU).
WwGrid ww_grid(const ConvGeom& g, int tiles, bool big) {
  WwGrid w;
  w.c_chunks = (int)ceil_div(g.Cg, kCC);
  w.n_tiles = (int)ceil_div(g.Cp, 128);
  w.kinds = (int64_t)w.c_chunks * w.n_tiles * g.B;
  // tile runs: a multiple of 8 (one set per XCD), about two workgroups per CU overall (one
  // for the big windows)
  const int64_t want = std::max<int64_t>(8, ceil_div(ceil_div(big ? 256 : 512, w.kinds), 8) * 8);
  w.groups = (int)std::min<int64_t>(ceil_div(tiles, 8) * 8, want);
  w.slots = (int64_t)w.groups * w.kinds;
  w.nreg = g.K * 16;
  return w;
}
}  // namespace

bool window_wgrad_big_supported(const ConvGeom& g, int mm) {
  (void)mm;   // every matrix arithmetic
  return planned_wgrad_supported(g) && g.K >= 1 && g.K <= 10 && g.Cp >= 1 &&
         (int64_t)g.H * g.W <= ((int64_t)1 << 24);
}

bool window_wgrad_supported(const ConvGeom& g, int mm) {
  // (every wave multiplies four 32-row blocks: with 64 rows or fewer half of that is padding.
  // On tiles inside an ordinary window the plan-driven kernel, which splits the pixels
  // instead, is then the faster one; on big tiles, which it reads from global memory, the
  // padded window kernel still is, down to a few rows: 3 x 3 bilinear at stride 2 on a
  // 64 x 128 grid, 4 x 128 -> 64 channels: 346 against 162 us; 128 -> 13 channels: the whole
  // backward call 0.49 against 0.29 ms.)
  return window_wgrad_big_supported(g, mm) && g.Cp > 64;
}

size_t window_wgrad_partial_bytes(const ConvGeom& g) {
  if (g.B == 0) return 0;
  // (one buffer serves whichever window kernels the call runs, one after the other)
  const size_t narrow =
      window_wgrad_narrow_supported(g, kMmF32) ? window_wgrad_narrow_partial_bytes(g) : 0;
  if (!window_wgrad_big_supported(g, kMmF32)) return narrow;
  const PixelTiling pt = plan_tiling(g.M / g.OW, g.OW);
  const int tiles = pt.tiles_x * pt.tiles_y;
  const WwGrid w = ww_grid(g, tiles, false), wb = ww_grid(g, tiles, true);
  return std::max(narrow,
                  (size_t)std::max(w.slots, wb.slots) * w.nreg * kWwThreads * sizeof(float));
}

int window_wgrad(const ConvGeom& g, int mm, const Plan& plan, const TileLists& tl,
                 const float* pix, const float* img, float* gW, float* partial,
                 hipStream_t stream, bool big) {
  if (big && plan.big_lut == nullptr) return SDK_OK;
  const WwGrid w = ww_grid(g, plan.tiles, big);
  const int* list = big ? tl.big : tl.inside;
  const int* count = big ? tl.count + 2 : tl.count;
  if (w.slots >= ((int64_t)1 << 31)) return fail(SDK_ERR_UNSUPPORTED, "window_wgrad: grid too large");
  const int TX = plan.pt.TX();
  const int vec4 = (g.OW % 4 == 0 && TX >= 16 && reinterpret_cast<uintptr_t>(pix) % 16 == 0) ? 1 : 0;
  const dim3 grid((unsigned)w.slots);
  const int KP = g.K / 4, R = g.K % 4;
#define WW3(KPv, Rv, CAPv, MMv)                                                                  \
  launch(window_wgrad_kernel<KPv, Rv, CAPv, MMv>, grid, dim3(kWwThreads), stream, pix, img,      \
         plan.hdr, plan.ns, plan.taps, list, count, partial, g.Cg, g.H, g.W, g.Cp, plan.S,       \
         plan.pt, w.groups, (int)g.B, w.c_chunks, w.n_tiles, vec4, plan.big_lut)
#define WW3ONE(KPv, Rv, CAPv)                                                                    \
  launch(window_wgrad_kernel<KPv, Rv, CAPv, kMmF32, true>, grid, dim3(kWwThreads), stream, pix,   \
         img, plan.hdr, plan.ns, plan.taps, list, count, partial, g.Cg, g.H, g.W, g.Cp, plan.S,   \
         plan.pt, w.groups, (int)g.B, w.c_chunks, w.n_tiles, vec4, plan.big_lut)
#define WW2(KPv, Rv, CAPv)                                                       \
  do {                                                                           \
    if (mm == kMmBf16) WW3(KPv, Rv, CAPv, kMmBf16);                              \
    else if (mm == kMmSplit) WW3(KPv, Rv, CAPv, kMmSplit);                       \
    else if (plan.S == 1) WW3ONE(KPv, Rv, CAPv);                                 \
    else WW3(KPv, Rv, CAPv, kMmF32);                                             \
  } while (0)
#define WW(KPv, Rv)                                                   \
  do {                                                                \
    if (big) WW2(KPv, Rv, kBigCap); else WW2(KPv, Rv, kRegionCap);    \
  } while (0)
  switch (g.K) {
    case 1: WW(0, 1); break;
    case 2: WW(0, 2); break;
    case 3: WW(0, 3); break;
    case 4: WW(1, 0); break;
    case 5: WW(1, 1); break;
    case 6: WW(1, 2); break;
    case 7: WW(1, 3); break;
    case 8: WW(2, 0); break;
    case 9: WW(2, 1); break;
    default: WW(2, 2); break;
  }
#undef WW
#undef WW2
#undef WW3
#undef WW3ONE
  SDK_LAUNCH_CHECK(big ? "window_wgrad(big)" : "window_wgrad");
  const int kinds0 = w.c_chunks * w.n_tiles, total = (int)g.B * w.groups;
  const int parts = (int)std::min<int64_t>(std::min(total, 16),
                                           ceil_div(2048, (int64_t)w.nreg * kinds0));
  launch(window_wgrad_reduce_kernel, dim3((unsigned)w.nreg, (unsigned)kinds0, (unsigned)std::max(parts, 1)),
         dim3(kWwThreads), stream, (const float*)partial, gW, g.Cg, g.Cp, g.K, KP, R, w.groups,
         (int)g.B, w.c_chunks, w.n_tiles, count);
  SDK_LAUNCH_CHECK("window_wgrad_reduce");
  return SDK_OK;
}

}  // namespace sdk
