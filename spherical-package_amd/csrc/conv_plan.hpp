// Tap plan: the sample map of one convolution call, resolved once per call into
// per-tile lists of (window index, coefficient) pairs that every batch element
// and channel chunk reuses.
//
// The pixel grid is cut into 2-D tiles of 128 pixels (PixelTiling).  For tile t, with
// h = hdr + kHdrStride * t (conv_window.hpp):
//   h[0..3]          window of the image the tile's taps fall into: first row,
//                    first column, rows, columns (columns wrap modulo W).  When the
//                    bounding box of the taps is too large for a window but the taps touch
//                    at most kRegionCap distinct elements, the window is the sorted list of
//                    those elements instead (a "listed" window: 0, 0, 1, count)
//   h[4]             1 when every active tap of the tile lies inside that window
//   h[5]             the largest ns of the tile's samples (plan_kernel only)
//   h[6]             1 for a listed window
//   h[7]             1 for a big tile (below)
//   h[8 + e]         flat image offset of window element e (-1: outside the image)
//   ns[t*K + k]      rows of kernel sample k: the largest number of active taps
//                    any pixel of the tile has for that sample
//   taps[((t*K + k)*S + r)*128 + p]   row r < ns of pixel p (tile-local index):
//                    .x >= 0: element index inside the window (row * columns + column,
//                             or the rank in the list)
//                    .x <  0: -(flat offset inside the image plane) - 1 (outside the window)
//                    .y: float bits of the coefficient (interpolation weight times
//                    point weight); pixels with fewer taps are padded with 0.
// S = points per sample * taps per point bounds the rows of one sample.
//
// Big tiles.  A tile whose taps fit no window (h[4] would be 0) but touch at most kBigCap
// distinct elements is described a second way, for kernels that give a window most of a CU's
// LDS: with bl = big_lut + kBigStride * t,
//   bl[0]                  number of distinct elements
//   bl[8 + e]              flat image offset of element e, ascending
//   bl[8 + kBigCap + e]    what .x of a tap on element e would be in the ordinary encoding
// and the .x of its rows in taps is the rank of the tap's element in that list.  h[0..6] and
// the window LUT stay what they would be without this; a kernel that does not run big tiles
// from a big window turns a rank back into the ordinary encoding with plan_row_at below.
#pragma once
#include <hip/hip_runtime.h>

#include "conv_internal.hpp"
#include "conv_window.hpp"

namespace sdk {

constexpr int kPlanKMax = 256;  // kernel samples a plan can hold

struct Plan {
  PixelTiling pt;
  int tiles, S;
  const int* hdr;
  const int* ns;
  const int2* taps;
  const int* big_lut;   // nullptr: the plan has no big tiles
};

// The ordinary encoding (window index, or -(flat offset) - 1) of a plan row's .x for a kernel
// that treats tile t as a tile outside its window: x itself unless t is a big tile.
// big: h[7] != 0; bl: big_lut + kBigStride * t.
__device__ __forceinline__ int plan_row_at(int x, bool big, const int* __restrict__ bl) {
  return big ? bl[kBigLut + kBigCap + x] : x;
}

PixelTiling plan_tiling(int OH, int OW);
bool plan_supported(const ConvGeom& g);
size_t plan_bytes(const ConvGeom& g);

// Builds the plan of (g, map, wts) in `workspace` (plan_bytes(g) bytes, 16-byte aligned).
// gate: optional device flag; with one, the plan is built only if *gate != 0 (its only reader
// is gated the same way).  with_big = false: the plan has no big tiles (plan->big_lut = nullptr).
int build_plan(const ConvGeom& g, const float* map, const float* wts, void* workspace,
               hipStream_t stream, Plan* plan, const int* gate = nullptr, bool with_big = true);

// gW = sum_b pix[b] x im2col(img[b])^T from a plan; gW must be zero on entry.
// partial: planned_wgrad_partial_bytes(g) bytes (when that is not 0) in which the workgroups
// leave their sums for a second, summing kernel; nullptr: they add to gW themselves.
// The plan's tiles by class, on the device (conv_window_gemm.hip), each in ascending order:
// those whose taps all lie inside their window and the others (count[0], count[1] entries);
// the others again as big tiles and the remainder (count[2], count[3]); and, when the lists
// were built with small_cap > 0 (kProductCap for an inverse plan, whose small windows can run
// in the product form below), `inside` again as the tiles with a window of at most small_cap
// elements and the remainder (count[4], count[5]); and every tile that is not a big tile
// (count[6]).
struct TileLists {
  const int* inside;
  const int* rest;
  const int* big;
  const int* rest_small;
  const int* product;
  const int* inside_large;
  const int* not_big;
  const int* count;
};
// max_rows > 0: tiles with a sample of more than max_rows plan rows (h[5]) are neither inside
// nor big.
size_t tile_lists_bytes(const ConvGeom& g);
int build_tile_lists(const Plan& plan, void* workspace, hipStream_t stream, TileLists* out,
                     int max_rows = 0, int small_cap = 0);

// pix[b] = Wm x im2col(img[b]) + bias on the tiles of tl.inside, gathered from an LDS window.
// g: the contraction's geometry (gather side = img).  swapped: Wm is [Cg, Cp * K] instead of
// [Cp, Cg * K].  weights: window_gemm_weight_bytes(g) bytes of scratch for the re-laid-out
// weight matrix.  gate (optional): the kernel runs only if *gate == 0.
// kListBig: `weights` must hold what an earlier call for one of the other lists left there
// (same g, mm, Wm).
bool window_gemm_supported(const ConvGeom& g);
size_t window_gemm_weight_bytes(const ConvGeom& g);
// which: the tiles of tl.inside, tl.big, or tl.inside_large (what window_product leaves).
constexpr int kListInside = 0, kListBig = 1, kListInsideLarge = 2;
int window_gemm(const ConvGeom& g, int mm, const Plan& plan, const TileLists& tl,
                const float* img, const float* Wm, bool swapped, const float* bias, float* pix,
                float* weights, const int* gate, hipStream_t stream, int which = kListInside);

// Product form of the same contraction for the tiles of tl.product of an inverse plan (image
// tiles whose sources are at most kProductCap pixels: up-sampling and strided maps): per sample
// the weights are applied at the source pixels and the image pixels gather the products from
// LDS, which is half the matrix work of gathering first or less.  fp32 MFMA; g.Cg <= 256.
// weights: what window_gemm(..., kListInsideLarge) left for the same g, Wm.
constexpr int kProductCap = 64;
bool window_product_supported(const ConvGeom& g, int mm);
int window_product(const ConvGeom& g, const Plan& plan, const TileLists& tl, const float* img,
                   const float* bias, float* pix, const float* weights, const int* gate,
                   hipStream_t stream);

// The scatter of geometry g regrouped by target as a plan over tiles of the image grid, whose
// windows lie in the pixel grid; valid only if *gate == 0 after it was built (a target with
// more than kInversePlanRows sources per sample raises it).  The raw lists (source pixel,
// coefficient; rows of 128 tile pixels like the plan's) serve the global-gather kernel.
constexpr int kInversePlanRows = 16;
struct InversePlan {
  Plan plan;
  int* gate;
  const int* raw_off;
  const float* raw_co;
};
size_t inverse_plan_bytes(const ConvGeom& g);
int build_inverse_plan(const ConvGeom& g, const float* map, const float* wts, void* workspace,
                       hipStream_t stream, InversePlan* out);
// Pointers into a workspace build_inverse_plan filled for the same geometry.
void load_inverse_plan(const ConvGeom& g, void* workspace, InversePlan* out);
// Likewise for build_plan and build_tile_lists.
void load_plan(const ConvGeom& g, void* workspace, Plan* out);
void load_tile_lists(const Plan& plan, void* workspace, TileLists* out);

bool planned_wgrad_supported(const ConvGeom& g);
size_t planned_wgrad_partial_bytes(const ConvGeom& g);
// tile_list / tile_count (optional, device): only the listed tiles are summed.
int planned_wgrad(const ConvGeom& g, int mm, const Plan& plan, const float* pix,
                  const float* img, float* gW, float* partial, hipStream_t stream,
                  const int* tile_list = nullptr, const int* tile_count = nullptr);

// The same sums over the tiles of tl.inside, from an LDS window with the column values built
// straight into MFMA operands (conv_window_wgrad.hip; K <= 10, at most four plan rows per
// sample: build the lists with max_rows = 4; mm: the matrix arithmetic).  partial: window_wgrad_partial_bytes(g).
bool window_wgrad_supported(const ConvGeom& g, int mm);
// ... for the big tiles alone (window_wgrad(..., big = true)): also layers of at most 64
// pixel-side channels, whose other tiles are faster in the plan-driven kernel.
bool window_wgrad_big_supported(const ConvGeom& g, int mm);
// ... and for layers of at most 64 pixel-side channels with nearest taps and no interpolation
// weights (mm: the matrix arithmetic): the tiles of tl.inside; partial:
// window_wgrad_narrow_partial_bytes(g), which window_wgrad_partial_bytes(g) returns for them.
bool window_wgrad_narrow_supported(const ConvGeom& g, int mm);
size_t window_wgrad_narrow_partial_bytes(const ConvGeom& g);
int window_wgrad_narrow(const ConvGeom& g, int mm, const Plan& plan, const TileLists& tl,
                        const float* pix, const float* img, float* gW, float* partial,
                        hipStream_t stream);

size_t window_wgrad_partial_bytes(const ConvGeom& g);
// big: the sums over the tiles of tl.big, from their big windows.
int window_wgrad(const ConvGeom& g, int mm, const Plan& plan, const TileLists& tl,
                 const float* pix, const float* img, float* gW, float* partial,
                 hipStream_t stream, bool big = false);

}  // namespace sdk
