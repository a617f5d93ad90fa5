// The inverse direction of mapped convolution (backward-input, transposed forward) for maps
// whose image is finer than their pixel grid: up-sampling transposed layers, strided layers.
//
//   img[b][c][u] = bias[c] + sum over the taps (m, k, r) -> u of
//                  coefficient(m, k, r) * sum_n Wm[n][c][k] * pix[b][n][m]
//
// Contracting first at the pixel grid's resolution and splatting the products afterwards
// (ext_modules/src/cpp/mapped_transposed_convolution_layer.cpp:8-60: a matrix product into
// columns, then common/mapped_im2col.h:89-158) takes M * K * Cp * Cg multiply-adds; gathering
// first and contracting per image element, as the window kernels do, takes H * W * K * Cp * Cg:
// four times as many where the image has four times the pixels.  The price is the column
// matrix in memory, B * Cg * K * M values written and read once, which a map of about unit
// scale cannot pay (configuration 4: 4.8 GB per pass) and an up-sampling one can
// (configuration 5's transposed layer: 73 MB).
//
//   product_gemm_kernel   col[b][m][k][c] = sum_n pix[b][n][m] * Wm[n][(c, k)]   (fp32 MFMA)
//   col2im_from_lists     the splat as a gather over the inverted map (mapped_gather_scatter.hip):
//                         no atomics, no fill, bias added where an element is written
#include <hip/hip_runtime.h>

#include <algorithm>

#include "conv_product.hpp"
#include "sdk_host.hpp"
#include "sdk_mfma.hpp"

namespace sdk {
namespace {

constexpr int kPgThreads = 256;
constexpr int kPgTile = 128;        // pixels m and columns (k, c) of a workgroup's tile
constexpr int kPgChunk = 32;        // pixel-side channels n per pass
constexpr int kPgLd = kPgTile + 4;  // row stride of the LDS tiles (floats, 16-byte rows)

typedef float vec4 __attribute__((ext_vector_type(4)));

// col[b][m][k][c] = sum_n pix[b][n][m] * Wm[n][c * K + k]: the product transposed, so that the
// Cg channels of a sample lie side by side (the splat reads them as one run per sample) and a
// lane's 32 neighbours store 32 consecutive floats.  Columns j = k * Cg + c.
// grid (strips of pixel tiles, column tiles, batch).  The reduction is short (Cp pixel-side
// channels), so a workgroup keeps its 128 columns of the weights in LDS for all of them (NC
// chunks of 32) and walks the pixel tiles of its strip: per tile the Cp x 128 pixel values go
// to LDS, each wave multiplies its 64 x 64 quarter (v_mfma_f32_32x32x2_f32, lane l supplying
// pixel / column l % 32 for the reduction index 2 s + l / 32) and stores it; the next tile's
// values are requested before the MFMAs.  Tiles inside the matrix read 16 bytes per lane from
// any 4-byte boundary; the tile on its edge reads element by element from clamped addresses
// (the choice is uniform over the workgroup: per-lane conditions around the reads end up as a
// branch and a wait per read).  (Every lane reading its own operand values from memory a tile
// ahead, with no pixel tile in LDS and no barrier, took 195 instead of 139 us at configuration
// 5: 256 registers and spills.)
template <int NC>
__global__ __launch_bounds__(kPgThreads, 2) void product_gemm_kernel(
    const float* __restrict__ Wm, const float* __restrict__ pix, float* __restrict__ col, int Cg,
    int K, int M, int Cp, int m_tiles) {
  __shared__ __attribute__((aligned(16))) float At[NC * kPgChunk * kPgLd];   // [n][pixel]
  __shared__ __attribute__((aligned(16))) float Bt[NC * kPgChunk * kPgLd];   // [n][column]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j = lane & 31, h = lane >> 5;
  const int R = Cg * K;
  const int j0 = blockIdx.y * kPgTile;
  const float* pix_b = pix + (size_t)blockIdx.z * Cp * M;
  float* col_b = col + (size_t)blockIdx.z * M * R;
  const int wr = (wave >> 1) * 64, wc = (wave & 1) * 64;
  // staging role: rows n = tid / 32 + 8 i, elements 4 (tid % 32) .. + 3
  const int sn = tid >> 5, se = 4 * (tid & 31);
  constexpr int NI = NC * kPgChunk / 8;   // rows per thread

  // ---- the weights: column j -> Wm[n][c * K + k]; rows past Cp multiply as zeros
  {
    int wcol[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int jj = min(j0 + se + e, R - 1);
      wcol[e] = (jj % Cg) * K + jj / Cg;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = sn + 8 * i;
      const float* wrow = Wm + (size_t)min(n, Cp - 1) * R;
      vec4 w;
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = n < Cp ? wrow[wcol[e]] : 0.0f;
      *reinterpret_cast<vec4*>(Bt + n * kPgLd + se) = w;
    }
  }

  vec4 ga[NI];
  auto fetch = [&](int m0) {
    const bool inside = m0 + kPgTile <= M;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const float* prow = pix_b + (size_t)min(sn + 8 * i, Cp - 1) * M;
      if (inside) {
        __builtin_memcpy(&ga[i], prow + m0 + se, sizeof(vec4));
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) ga[i][e] = prow[min(m0 + se + e, M - 1)];
      }
    }
  };
  int tile = blockIdx.x;
  if (tile < m_tiles) fetch(tile * kPgTile);
  for (; tile < m_tiles; tile += gridDim.x) {
    const int m0 = tile * kPgTile;
    __syncthreads();   // the previous tile's reads are done (and, the first time, Bt is written)
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const vec4 z = {0.f, 0.f, 0.f, 0.f};
      *reinterpret_cast<vec4*>(At + (sn + 8 * i) * kPgLd + se) = sn + 8 * i < Cp ? ga[i] : z;
    }
    __syncthreads();
    if (tile + (int)gridDim.x < m_tiles) fetch((tile + gridDim.x) * kPgTile);

    floatx16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;
    // (the operands of step s + 1 are read from LDS before the MFMAs of step s are issued)
    constexpr int STEPS = NC * kPgChunk / 2;
    const float* ar = At + h * kPgLd + wr + j;
    const float* br = Bt + h * kPgLd + wc + j;
    float a0 = ar[0], a1 = ar[32], b0 = br[0], b1 = br[32];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int sn1 = s + 1 < STEPS ? s + 1 : s;
      const float na0 = ar[2 * sn1 * kPgLd], na1 = ar[2 * sn1 * kPgLd + 32];
      const float nb0 = br[2 * sn1 * kPgLd], nb1 = br[2 * sn1 * kPgLd + 32];
      __builtin_amdgcn_sched_barrier(0);
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      a0 = na0;
      a1 = na1;
      b0 = nb0;
      b1 = nb1;
    }
    // D[pixel][column]: register v of lane l holds pixel 8 (v / 4) + 4 (l / 32) + v % 4 of
    // its 32, column l % 32
    // (tiles inside the matrix store without tests, walking one pointer down the rows)
    const bool whole = m0 + kPgTile <= M && j0 + kPgTile <= R;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int jj = j0 + wc + 32 * b + j;
        float* out = col_b + (size_t)(m0 + wr + 32 * a + 4 * h) * R + jj;
        if (whole) {
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              *out = acc[a][b][4 * g4 + e];
              out += R;
            }
            out += 4 * (size_t)R;
          }
        } else {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int dm = 8 * (v >> 2) + (v & 3);
            if (m0 + wr + 32 * a + 4 * h + dm < M && jj < R) out[(size_t)dm * R] = acc[a][b][v];
          }
        }
      }
  }
}

// Column matrices of at most this many bytes take the route (beyond, the gather form's extra
// matrix work costs less than the traffic).
constexpr size_t kProductMaxBytes = (size_t)1 << 30;

size_t col_bytes(const ConvGeom& g) {
  return sizeof(float) * (size_t)g.B * g.Cg * g.K * g.M;
}

// The batch goes through in slices of this many elements: a slice's column matrix (at most
// kProductSliceBytes where one element's fits) is still in the 256 MB memory-side cache when the
// launch behind the one that wrote it reads it back.  (Level-7 icosphere up-sampling, 4 x 64
// channels, 293 MB of columns: 0.253 ms in one piece, 0.239 in two, 0.276 in four, whose launches
// no longer fill the GPU.)
constexpr size_t kProductSliceBytes = (size_t)160 << 20;
int slice_batches(const ConvGeom& g) {
  const size_t per_b = sizeof(float) * (size_t)g.Cg * g.K * g.M;
  return (int)std::max<size_t>(1, std::min<size_t>((size_t)g.B, kProductSliceBytes / std::max<size_t>(per_b, 1)));
}
size_t slice_bytes(const ConvGeom& g) {
  return sizeof(float) * (size_t)slice_batches(g) * g.Cg * g.K * g.M;
}

}  // namespace

bool product_route_map(const ConvGeom& g) {
  return g.interp == 0 && g.P == 0 && g.M >= 1 && g.K >= 1 &&
         (int64_t)g.H * g.W >= 2 * (int64_t)g.M && (int64_t)g.M * g.K * 2 < ((int64_t)1 << 31) &&
         col2im_lists_bytes(g.H, g.W, g.M, g.K, g.P, g.interp) != 0;
}

bool product_route(const ConvGeom& g) {
  return product_route_map(g) && g.B >= 1 && g.B <= 65535 && g.Cp >= 16 && g.Cp <= 64 &&
         g.Cg >= 5 &&
         (int64_t)g.Cg * g.K <= 65535 * (int64_t)kPgTile &&
         (int64_t)g.B * g.Cg < ((int64_t)1 << 31) && col_bytes(g) <= kProductMaxBytes;
}

size_t product_workspace_bytes(const ConvGeom& g) {
  if (!product_route(g)) return 0;
  return ((slice_bytes(g) + 255) & ~(size_t)255) +
         col2im_lists_bytes(g.H, g.W, g.M, g.K, g.P, g.interp);
}

int product_gemm_scatter(const ConvGeom& g, const float* pix, const float* map, const float* wts,
                         const float* Wm, const float* bias, float* img, void* workspace,
                         hipStream_t stream, const void* kept_lists) {
  float* col = static_cast<float*>(workspace);
  void* own_lists = static_cast<char*>(workspace) + ((slice_bytes(g) + 255) & ~(size_t)255);
  const int R = g.Cg * g.K;
  const void* lists = kept_lists;
  if (lists == nullptr) {
    const int rc = col2im_lists_build(map, wts, own_lists, g.H, g.W, g.M, g.K, g.P, g.interp,
                                      stream);
    if (rc) return rc;
    lists = own_lists;
  }
  // (one column buffer serves every slice of the batch in turn)
  const int bs = slice_batches(g);
  const int m_tiles = (int)ceil_div(g.M, kPgTile);
  const int nc = (int)ceil_div(g.Cp, kPgChunk);
  for (int b0 = 0; b0 < g.B; b0 += bs) {
    const int nb = std::min<int>(bs, g.B - b0);
    // strips: one round of two workgroups per CU over the whole grid
    const int64_t others = ceil_div(R, kPgTile) * nb;
    const int strips = (int)std::max<int64_t>(1, std::min<int64_t>(m_tiles, ceil_div(512, others)));
    const dim3 grid((unsigned)strips, (unsigned)ceil_div(R, kPgTile), (unsigned)nb);
    const float* pix_s = pix + (size_t)b0 * g.Cp * g.M;
    float* img_s = img + (size_t)b0 * g.Cg * g.H * g.W;
#define PG(NCv)                                                                               \
  launch(product_gemm_kernel<NCv>, grid, dim3(kPgThreads), stream, Wm, pix_s, col, g.Cg, g.K, \
         g.M, g.Cp, m_tiles)
    if (nc <= 1) PG(1); else PG(2);
#undef PG
    SDK_LAUNCH_CHECK("mapped_conv(products)");
    const int rc = col2im_from_lists(col, bias, img_s, lists, nb * g.Cg, g.Cg, g.H, g.W, g.M,
                                     g.K, g.P, g.interp, stream);
    if (rc) return rc;
  }
  return SDK_OK;
}

}  // namespace sdk
