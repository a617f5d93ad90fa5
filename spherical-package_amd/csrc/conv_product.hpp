// The inverse direction of mapped convolution as a matrix product at the pixel grid's
// resolution followed by a gather of the products (conv_product.hip), float32.
#pragma once
#include <hip/hip_runtime.h>

#include "conv_internal.hpp"

namespace sdk {

// Maps that may take the route (H, W, M, K, P and interp of g): single nearest taps (every
// product is then read once; a blended sample's would be read by each of its taps), the image
// with at least twice the pixels of the map's grid.
bool product_route_map(const ConvGeom& g);
// Calls that take it: such a map, at least five image channels, 16 to 64 on the pixel side,
// a column matrix [B, M * K, Cg] below 1 GiB.
bool product_route(const ConvGeom& g);
// Workspace of the route: the column matrix, then the inverted map (0: not taken).
size_t product_workspace_bytes(const ConvGeom& g);
// img[b][c][u] = bias[c] (or 0) + the splat of Wm^T x pix[b]; every element of img is written.
// lists: the map's inverted lists from a kept plan (col2im_lists_build), or nullptr: they are
// then built in the workspace.
int product_gemm_scatter(const ConvGeom& g, const float* pix, const float* map, const float* wts,
                         const float* Wm, const float* bias, float* img, void* workspace,
                         hipStream_t stream, const void* lists = nullptr);

// The splat of a column matrix col[b][m * K + k][c] (channels last) onto planes / channels
// images of `channels` planes as a gather over the inverted map, mapped_gather_scatter.hip:
// img[b][c][u] = bias[c] (bias may be nullptr) + sum over the taps (m, k, r) -> u of
// coefficient * col[b][m * K + k][c].  The lists depend on the map alone.
size_t col2im_lists_bytes(int H, int W, int M, int K, int P, int interp);   // 0: too large
int col2im_lists_build(const float* map, const float* wts, void* lists, int H, int W, int M,
                       int K, int P, int interp, hipStream_t stream);
int col2im_from_lists(const float* col, const float* bias, float* img, const void* lists,
                      int64_t planes, int channels, int H, int W, int M, int K, int P, int interp,
                      hipStream_t stream);

}  // namespace sdk
