/*
 * sdk_mapped_ops.h - C ABI of the MI355X (gfx950) mapped-operation backend.
 *
 * One shared library, libsdk_mapped_ops.so, built from hand-written HIP
 * kernels.  Every entry point takes plain device pointers, sizes and a HIP
 * stream; no torch (or any other framework) type crosses this boundary.
 *
 * The entry points are what the reference package's per-family pybind11
 * extension modules (package `_spherical_distortion_ext`, reference setup.py:62-199)
 * bind for the device side of this path: each comment cites the reference
 * interface the function replaces (paths relative to the reference tree).
 *
 * Conventions
 *   - All tensors are dense, row-major ("contiguous NCHW"); device memory.
 *   - sample_map holds (x, y) pairs in pixel units, x = column, y = row, with
 *     the data's floating type.  Unweighted layout [..., 2] is selected by
 *     num_interp_pts == 0; weighted layout [..., P, 2] with interp_weights
 *     [..., P] by num_interp_pts == P >= 1 (interp_weights must be non-NULL).
 *   - interp: 0 nearest (round half away from zero, no wrap), 1 bilinear
 *     (out-of-range taps read as zero / are dropped), 2 bispherical (bilinear
 *     whose columns wrap modulo the width; rows are still bounds-checked).
 *     Any other value behaves as nearest, like the reference's switch default
 *     (ext_modules/include/core/resample.h:48-50, :72-76).
 *   - dtype: SDK_F32 or SDK_F64 for data, map and weights alike.
 *   - Outputs are fully written by the call (scatter targets are zero-filled
 *     first, on the same stream); inputs are never modified.
 *   - All work is enqueued on `stream` (a hipStream_t, NULL = default stream)
 *     and the call returns without synchronising.
 *   - Return value: SDK_OK (0) or a negative sdk_status; sdk_last_error()
 *     gives the message of the calling thread's most recent failure.  The
 *     reference prints and calls std::exit(-1) on a device error
 *     (ext_modules/include/cuda_helper.h:5-10); this library returns instead.
 *   - A plane (H*W, or OH*OW) must have fewer than 2^31 elements.
 */
#ifndef SDK_MAPPED_OPS_H_
#define SDK_MAPPED_OPS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum sdk_status {
  SDK_OK = 0,
  SDK_ERR_INVALID_ARGUMENT = -1, /* NULL pointer, bad size, unknown dtype */
  SDK_ERR_UNSUPPORTED = -2,      /* valid request this build cannot serve */
  SDK_ERR_WORKSPACE = -3,        /* workspace missing or too small */
  SDK_ERR_DEVICE = -4            /* HIP runtime reported an error */
} sdk_status;

typedef enum sdk_dtype { SDK_F32 = 0, SDK_F64 = 1 } sdk_dtype;

/* ext_modules/include/enums.h:12-16 (exported by include/layers/enum_export.h:10-18) */
typedef enum sdk_interp { SDK_NEAREST = 0, SDK_BILINEAR = 1, SDK_BISPHERICAL = 2 } sdk_interp;

/* Arithmetic / kernel choice of the dense contraction inside the convolution entry points.
 * SDK_COMPUTE_NATIVE:  the tensors' own type; float32 runs the fused gather + fp32-MFMA kernels.
 * SDK_COMPUTE_BF16:    operands rounded to bf16, fp32 accumulation (SDK_F32 only).
 * SDK_COMPUTE_UNFUSED: separate im2col/col2im and plain-FMA GEMM kernels through a column
 *                      workspace (always used for SDK_F64; kept selectable as a cross-check).
 * SDK_COMPUTE_SPLIT:   float32 results from the bf16 matrix unit: every float32 operand is split
 *                      exactly into three bf16 pieces and six of the nine piece products (all but
 *                      those below 2^-23 of the product) are accumulated in fp32.  Same accuracy
 *                      as SDK_COMPUTE_NATIVE (measured against float64: 1.4e-6 vs 1.3e-6 of the
 *                      largest output at 1152 terms per sum), faster, because the fp32 matrix
 *                      instructions compete with the gather arithmetic for the same lanes and
 *                      the bf16 ones do not.  Shapes or types the split kernels do not cover
 *                      run as SDK_COMPUTE_NATIVE. */
typedef enum sdk_compute {
  SDK_COMPUTE_NATIVE = 0,
  SDK_COMPUTE_BF16 = 1,
  SDK_COMPUTE_UNFUSED = 2,
  SDK_COMPUTE_SPLIT = 3
} sdk_compute;

typedef void* sdk_stream_t; /* hipStream_t */

const char* sdk_last_error(void);
int sdk_version(void);

/* ------------------------------------------------------------------------- *
 * Resampling.
 * ------------------------------------------------------------------------- */

/* Gather: out[b,c,my,mx] = interp(image[b,c], sample_map[my,mx]).
 * image [B,C,H,W]; sample_map [MH,MW,(P,)2]; out [B,C,MH,MW].
 * Replaces `_resample.resample_from_map` / `_weighted_resample.weighted_resample_from_map`
 * (ext_modules/include/layers/resample_layer.h:62-80,
 *  ext_modules/include/layers/weighted_resample_layer.h:76-101;
 *  device side ext_modules/src/cuda/resample_layer.cu, include/cuda/resample.cuh:50-81, :127-164). */
int sdk_resample_from_map(const void* image, const void* sample_map, const void* interp_weights,
                          void* out, int64_t batch, int64_t channels, int64_t height,
                          int64_t width, int64_t map_height, int64_t map_width,
                          int32_t num_interp_pts, int32_t interp, int32_t dtype,
                          sdk_stream_t stream);

/* Scatter: out (zero-filled) accumulates input[b,c,my,mx] at sample_map[my,mx].
 * input [B,C,MH,MW]; out [B,C,H,W].  If weight_sum is non-NULL it receives, as
 * one [H,W] plane, the same scatter applied to an all-ones input plane (the
 * per-pixel sum of splat weights; batch- and channel-invariant).
 * Replaces `_resample.resample_to_map` / `_weighted_resample.weighted_resample_to_map`
 * (ext_modules/include/layers/resample_layer.h:40-60,
 *  ext_modules/include/layers/weighted_resample_layer.h:49-74;
 *  device side include/cuda/resample.cuh:14-47, :87-124).
 *
 * workspace (optional, may be NULL): sdk_resample_to_map_workspace_bytes() bytes of device
 * scratch.  With it the map is first inverted on the device (per target pixel the list of
 * (source pixel, weight) pairs, up to 16); the scatter then runs as a gather without float
 * atomics and without the zero fill.  If a target collects more than 16 sources the call
 * falls back, on the device, to the atomic scatter. */
size_t sdk_resample_to_map_workspace_bytes(int64_t height, int64_t width, int32_t dtype);
int sdk_resample_to_map(const void* input, const void* sample_map, const void* interp_weights,
                        void* out, void* weight_sum, void* workspace, size_t workspace_bytes,
                        int64_t batch, int64_t channels, int64_t map_height, int64_t map_width,
                        int64_t height, int64_t width, int32_t num_interp_pts, int32_t interp,
                        int32_t dtype, sdk_stream_t stream);

/* sdk_resample_to_map followed by sdk_normalize_by_weight_sum in one call:
 * out[b,c] = splat(input[b,c]) / (weight_sum + eps), weight_sum [H,W] (required) = the splat of
 * an all-ones plane.  With the workspace the division happens where the splat is gathered, so
 * `out` is written once.  Replaces the reference's splat + weight-sum splat + division
 * (layers/functional/sphere_ops.py:74-80, eps 1e-12; resample entry points as above). */
int sdk_resample_to_map_normalized(const void* input, const void* sample_map,
                                   const void* interp_weights, void* out, void* weight_sum,
                                   void* workspace, size_t workspace_bytes, double eps,
                                   int64_t batch, int64_t channels, int64_t map_height,
                                   int64_t map_width, int64_t height, int64_t width,
                                   int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                   sdk_stream_t stream);

/* data[p, i] /= (weight_sum[i] + eps) for p < planes, i < plane_size, in place.
 * The reference does this in Python for its weighted splat
 * (layers/functional/sphere_ops.py:74-80, eps 1e-12). */
int sdk_normalize_by_weight_sum(void* data, const void* weight_sum, double eps, int64_t planes,
                                int64_t plane_size, int32_t dtype, sdk_stream_t stream);

/* The adjoint of sdk_mapped_max_unpool: out[b,c,oy,ox] = the image interpolated at the sample
 * indices[b,c,oy,ox] names (0 for an index outside the map).  image [B,C,H,W]; indices, out
 * [B,C,OH,OW].  This is the gradient of unpooling with respect to the pooled values, which a
 * working `MappedMaxUnpool` layer needs; the reference's version of that layer
 * (layers/functional/mapped_pooling.py:156-199, :235-242) refers to undefined names and cannot
 * run, so this entry point has no reference kernel: it is the transpose of
 * common/mapped_max_pool.h:60-78, :136-171. */
int sdk_mapped_gather_at_index(const void* image, const int64_t* indices, const void* sample_map,
                               const void* interp_weights, void* out, int64_t batch,
                               int64_t channels, int64_t height, int64_t width,
                               int64_t out_height, int64_t out_width, int64_t kernel_size,
                               int32_t num_interp_pts, int32_t interp, int32_t dtype,
                               sdk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * UV resampling (tangent images back to one image).
 * textures [B,C,NT,TH,TW]; quad_idx [H,W] int64 names, per image pixel, one of the NT textures;
 * tex_uv [H,W,2] = (u, v) in that texture's pixel coordinates (x first).  Interpolation taps stay
 * inside the named texture (bispherical wraps u within TW).  A quad_idx outside [0, NT)
 * contributes nothing (the reference reads out of bounds there).
 * ------------------------------------------------------------------------- */

/* Gather: out[b,c,y,x] = interp(textures[b,c,quad_idx[y,x]], tex_uv[y,x]).  out [B,C,H,W].
 * Replaces `_uv_resample.resample_from_uv_maps`
 * (ext_modules/include/layers/uv_resample_layer.h:76-99; body
 *  ext_modules/include/common/resample.h:132-158; host loop src/cpp/uv_resample_layer.cpp:41-72). */
int sdk_resample_from_uv_maps(const void* textures, const int64_t* quad_idx, const void* tex_uv,
                              void* out, int64_t batch, int64_t channels, int64_t num_textures,
                              int64_t tex_height, int64_t tex_width, int64_t height,
                              int64_t width, int32_t interp, int32_t dtype, sdk_stream_t stream);

/* Its adjoint: textures (zero-filled) accumulate input[b,c,y,x] at (quad_idx, tex_uv)[y,x].
 * input [B,C,H,W]; textures [B,C,NT,TH,TW].  Replaces `_uv_resample.resample_to_uv_maps`
 * (uv_resample_layer.h:48-74; body common/resample.h:160-187; src/cpp/uv_resample_layer.cpp:7-39).
 * workspace (optional, may be NULL): sdk_resample_to_uv_maps_workspace_bytes() bytes of device
 * scratch (4 bytes per image pixel + at most 260 per texture).  With it the image pixels are
 * bucketed by texture on the device and every texture is summed in on-chip memory and written
 * once, without atomics in memory and without a zero fill; the query returns 0 (and the call then needs no
 * workspace) when a texture does not fit there (TH*TW*sizeof > 64 KiB).  Without it: zero fill
 * and atomic adds. */
size_t sdk_resample_to_uv_maps_workspace_bytes(int64_t num_textures, int64_t tex_height,
                                               int64_t tex_width, int64_t height, int64_t width,
                                               int32_t dtype);
int sdk_resample_to_uv_maps(const void* input, const int64_t* quad_idx, const void* tex_uv,
                            void* textures, void* workspace, size_t workspace_bytes,
                            int64_t batch, int64_t channels, int64_t num_textures,
                            int64_t tex_height, int64_t tex_width, int64_t height, int64_t width,
                            int32_t interp, int32_t dtype, sdk_stream_t stream);
/* The buckets depend on quad_idx alone and can be kept between calls (the reference has no
 * counterpart: uv_resample_layer.h:48-74 is stateless).  _plan_build fills a caller-owned
 * buffer of sdk_resample_to_uv_maps_workspace_bytes() bytes (not 0); _planned is
 * sdk_resample_to_uv_maps with that buffer, which it only reads, in place of the workspace:
 * it launches the texture sums alone. */
int sdk_resample_to_uv_maps_plan_build(const int64_t* quad_idx, void* plan, size_t plan_bytes,
                                       int64_t num_textures, int64_t tex_height,
                                       int64_t tex_width, int64_t height, int64_t width,
                                       int32_t dtype, sdk_stream_t stream);
int sdk_resample_to_uv_maps_planned(const void* input, const int64_t* quad_idx, const void* tex_uv,
                                    void* textures, const void* plan, size_t plan_bytes,
                                    int64_t batch, int64_t channels, int64_t num_textures,
                                    int64_t tex_height, int64_t tex_width, int64_t height,
                                    int64_t width, int32_t interp, int32_t dtype,
                                    sdk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Voting resample (integer labels).  input [B,C,IH,IW] int64 labels in [0, num_candidates);
 * sample_map [IH,IW,2] int64 (x, y) target of every input pixel; out [B,C,OH,OW] int64 = for
 * every output pixel the label most of its sources carry (the first such label on a tie, 0
 * where no source lands).  Targets outside the output and labels outside the range cast no
 * vote.  With channels > 1 the reference offsets channel c's votes by c*OH*OW histogram elements
 * instead of c whole histograms, so votes of different channels share cells; that indexing is
 * reproduced (label images have one channel).  Replaces `_voting_resample.voting_resample_to_map`
 * (ext_modules/include/layers/voting_resample_layer.h:31-53; body
 *  core/interpolation.h:249-265, common/resample.h:109-130; histogram + argmax
 *  src/cpp/voting_resample_layer.cpp:8-37).
 * workspace (required): at least sdk_voting_resample_workspace_bytes() bytes, 16-byte aligned:
 * the vote histogram of one batch element, 4 bytes per (channel, output pixel, candidate); a
 * workspace n times that size lets n batch elements be processed per pass.
 * ------------------------------------------------------------------------- */
size_t sdk_voting_resample_workspace_bytes(int64_t channels, int64_t out_height,
                                           int64_t out_width, int64_t num_candidates);
int sdk_voting_resample_to_map(const int64_t* input, const int64_t* sample_map, int64_t* out,
                               void* workspace, size_t workspace_bytes, int64_t batch,
                               int64_t channels, int64_t in_height, int64_t in_width,
                               int64_t out_height, int64_t out_width, int64_t num_candidates,
                               sdk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Sample maps computed on the device (the reference builds them on the host with tensor
 * operations).  Maps are written in the layout every entry point above reads: (x, y) pairs in
 * pixel coordinates of an equirectangular image, lon = -pi + 2 pi x / W, lat = -pi/2 + pi y / (H-1).
 * ------------------------------------------------------------------------- */
typedef enum sdk_projection {
  SDK_MAP_GRID = 0,                   /* pixel grid offsets: layers/util/mapping_functions.py:43-75 */
  SDK_MAP_INVERSE_GNOMONIC = 1,       /* tangent-plane kernel projected back: :78-120 */
  SDK_MAP_INVERSE_EQUIRECTANGULAR = 2 /* longitude step widened by 1 / cos(lat): :123-160 */
} sdk_projection;

/* sample_map [ceil(H/stride), ceil(W/stride), kernel_h*kernel_w, 2]: for every stride-th pixel of an
 * H x W equirectangular image the kernel_h x kernel_w kernel about it (row-major, sample
 * (i, j) offset by (j - kernel_w/2, i - kernel_h/2) * dilation image steps), projected as
 * `projection` says; longitudes wrapped into the image for the two inverse projections.
 * Replaces `grid_projection_map`, `inverse_gnomonic_projection_map`,
 * `inverse_equirectangular_projection_map` (layers/util/mapping_functions.py:43-160, with
 * grids.py:5-25 and conversions.py:24-52). */
int sdk_equirect_kernel_map(void* sample_map, int64_t height, int64_t width, int64_t kernel_h,
                            int64_t kernel_w, int64_t stride, int64_t dilation,
                            int32_t projection, int32_t dtype, sdk_stream_t stream);

/* out [num_points, kernel_h*kernel_w, 2]: a gnomonic kernel_h x kernel_w kernel with angular
 * steps (res_lon, res_lat) about each of the points lonlat [num_points, 2] (lon, lat), returned
 * in (lon, lat) when image_height == 0, else in pixel coordinates of an image_height x
 * image_width equirectangular image.  Replaces `gnomonic_kernel`
 * (layers/util/icosahedron_functions.py:47-103) followed by `convert_spherical_to_image`
 * (layers/util/conversions.py:33-52), the pair the tangent-image and icosphere map builders use
 * (layers/util/tangent_images.py:59-88). */
int sdk_gnomonic_kernel_at(const void* lonlat, void* out, int64_t num_points, int64_t kernel_h,
                           int64_t kernel_w, double res_lat, double res_lon, int64_t image_height,
                           int64_t image_width, int32_t dtype, sdk_stream_t stream);

/* From a map of single points to the weighted (P = 4) form: out_map [num_samples, 4, 2] = the four
 * pixel centres around each sample of sample_map [num_samples, 2] (integer coordinates, column
 * wrapped, row clamped to the image), out_weights [num_samples, 4] proportional to
 * 1 / (great-circle distance + eps), normalised to sum to one.  The benchmark's large weighted
 * convolution is defined on such a map; the reference has no builder for it (its weighted maps
 * come from mesh code), so the kernel follows the definition, not a reference routine. */
int sdk_four_nearest_weighted_map(const void* sample_map, void* out_map, void* out_weights,
                                  int64_t num_samples, int64_t height, int64_t width, double eps,
                                  int32_t dtype, sdk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Mapped im2col / col2im (batched).
 * col[b, c*K + k, pix] with pix = y_out*OW + x_out, out_pixels = OH*OW.
 * sample_map [OH,OW,K,(P,)2].
 * Replace the device launchers MappedIm2Col2D / MappedCol2Im2D (+Weighted)
 * (ext_modules/include/cuda/mapped_im2col.cuh:28-49, :67-94, :113-136, :158-184),
 * which the reference calls once per batch element.
 * ------------------------------------------------------------------------- */
int sdk_mapped_im2col(const void* image, const void* sample_map, const void* interp_weights,
                      void* columns, int64_t batch, int64_t channels, int64_t height,
                      int64_t width, int64_t out_pixels, int64_t kernel_size,
                      int32_t num_interp_pts, int32_t interp, int32_t dtype, sdk_stream_t stream);

/* image [B,C,H,W] is zero-filled by the call, then accumulated into. */
int sdk_mapped_col2im(const void* columns, const void* sample_map, const void* interp_weights,
                      void* image, int64_t batch, int64_t channels, int64_t height,
                      int64_t width, int64_t out_pixels, int64_t kernel_size,
                      int32_t num_interp_pts, int32_t interp, int32_t dtype, sdk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Mapped max pooling.
 * ------------------------------------------------------------------------- */

/* out[b,c,oy,ox] = max_k interp(input[b,c], sample_map[oy,ox,k]) with strict `>`
 * (first maximum wins, NaN never wins) starting from -FLT_MAX;
 * indices[b,c,oy,ox] (int64) = flat element offset, inside sample_map, of the
 * winning sample's x coordinate (of its first interpolation point when
 * weighted), or -1 when no sample exceeded the start value.
 * Replaces `_mapped_max_pooling.mapped_max_pool` /
 * `_weighted_mapped_max_pooling.weighted_mapped_max_pool`
 * (ext_modules/include/layers/mapped_max_pooling_layer.h:42-62,
 *  weighted_mapped_max_pooling_layer.h:42-66; body
 *  ext_modules/include/common/mapped_max_pool.h:13-57, :81-133, device branch). */
int sdk_mapped_max_pool(const void* input, const void* sample_map, const void* interp_weights,
                        void* out, int64_t* indices, int64_t batch, int64_t channels,
                        int64_t height, int64_t width, int64_t out_height, int64_t out_width,
                        int64_t kernel_size, int32_t num_interp_pts, int32_t interp,
                        int32_t dtype, sdk_stream_t stream);

/* Mapped average pool: out[b,c,oy,ox] = (sum over the K samples of the interpolated input) / K,
 * summed in ascending sample order.  Replaces `_mapped_avg_pooling.mapped_avg_pool` /
 * `_weighted_mapped_avg_pooling.weighted_mapped_avg_pool`
 * (ext_modules/include/layers/mapped_avg_pooling_layer.h, weighted_mapped_avg_pooling_layer.h;
 *  body common/mapped_avg_pool.h:13-40, :70-105). */
int sdk_mapped_avg_pool(const void* input, const void* sample_map, const void* interp_weights,
                        void* out, int64_t batch, int64_t channels, int64_t height, int64_t width,
                        int64_t out_height, int64_t out_width, int64_t kernel_size,
                        int32_t num_interp_pts, int32_t interp, int32_t dtype,
                        sdk_stream_t stream);

/* Its adjoint: grad_input [B,C,H,W] (fully written by the call) receives grad_output / K
 * splatted at every one of the K samples of its pixel.  `workspace` as for
 * sdk_resample_to_map (sdk_resample_to_map_workspace_bytes(height, width, dtype)): with it the
 * splat runs as a gather over the inverted map, without it (NULL, 0) with float atomics.
 * Replaces `_mapped_avg_pooling.mapped_avg_unpool` / `weighted_mapped_avg_unpool`
 * (same headers; body common/mapped_avg_pool.h:42-68, :107-140). */
int sdk_mapped_avg_unpool(const void* grad_output, const void* sample_map,
                          const void* interp_weights, void* grad_input, void* workspace,
                          size_t workspace_bytes, int64_t batch, int64_t channels, int64_t height,
                          int64_t width, int64_t out_height, int64_t out_width,
                          int64_t kernel_size, int32_t num_interp_pts, int32_t interp,
                          int32_t dtype, sdk_stream_t stream);

/* grad_input [B,C,H,W] (fully written by the call) receives grad_output[b,c,oy,ox]
 * splatted at the sample the stored index names, with the same interpolation.
 * Negative or out-of-range indices contribute nothing.
 *
 * `workspace` is optional device scratch of sdk_mapped_max_unpool_workspace_bytes()
 * bytes (it depends on the input plane only: 32 bytes per 2048 input pixels,
 * 12 bytes per band of 32 KB of image rows and, while that stays below 32 MiB,
 * 40 KB per band for the band's pooled pixels with their taps resolved;
 * 1.3 MB for a 256 x 512 plane).  With it the
 * call works by pieces of the input plane, whole rows (float32, single nearest
 * taps, kernel_size 4 or 9, width a multiple of 4) or tiles: the pooled pixels
 * that can reach a piece are found from the map, their contributions are summed
 * in on-chip memory and every input pixel is written once with a plain store.
 * Without it (NULL, or too small), or when the map or the indices do not fit
 * that scheme (the pooled pixels that can reach one piece of the input are too
 * many or spread too far apart, or an index names a sample of another pooled
 * pixel than its own), the call zero-fills grad_input and scatters with atomic
 * adds, as the reference does; the choice is made on the device, the result is
 * the same.
 * Replaces `_mapped_max_pooling.mapped_max_unpool` /
 * `_weighted_mapped_max_pooling.weighted_mapped_max_unpool`
 * (ext_modules/include/layers/mapped_max_pooling_layer.h:64-88,
 *  weighted_mapped_max_pooling_layer.h:68-99; body common/mapped_max_pool.h:60-78, :136-171). */
size_t sdk_mapped_max_unpool_workspace_bytes(int64_t height, int64_t width, int32_t dtype);
int sdk_mapped_max_unpool(const void* grad_output, const int64_t* indices, const void* sample_map,
                          const void* interp_weights, void* grad_input, void* workspace,
                          size_t workspace_bytes, int64_t batch, int64_t channels, int64_t height,
                          int64_t width, int64_t out_height, int64_t out_width,
                          int64_t kernel_size, int32_t num_interp_pts, int32_t interp,
                          int32_t dtype, sdk_stream_t stream);

/* sdk_mapped_max_unpool for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments and results as sdk_mapped_max_unpool without the workspace pair:
 * the scratch (256 + 32 bytes per 2048-pixel tile of the input plane for the tile windows,
 * 48 KB for the row-band table behind them) is a 311 552-byte array inside the library, one
 * copy per GPU, held until the process ends.  The
 * call allocates and frees nothing.  Limit: the input plane may have at most
 * SDK_MAPPED_MAX_UNPOOL_STATIC_MAX_TILES tiles, ceil(width / TW) * ceil(height / (2048 / TW))
 * with TW = 128 (wider for planes lower than 16 rows, narrower for planes under 65 columns),
 * i.e. any plane up to 4096 x 4096; a larger one returns SDK_ERR_WORKSPACE with a message.
 * Every call on one GPU uses that GPU's array (the part it needs is cleared by a fill kernel at
 * the start of the call): calls that overlap on one GPU, on different streams or from different
 * threads, race; calls on one stream are ordered and safe.  The first call on a device looks up
 * the array's address (hipGetSymbolAddress) and should happen outside a graph capture. */
#define SDK_MAPPED_MAX_UNPOOL_STATIC_MAX_TILES 8192
int sdk_mapped_max_unpool_static(const void* grad_output, const int64_t* indices,
                                 const void* sample_map, const void* interp_weights,
                                 void* grad_input, int64_t batch, int64_t channels,
                                 int64_t height, int64_t width, int64_t out_height,
                                 int64_t out_width, int64_t kernel_size, int32_t num_interp_pts,
                                 int32_t interp, int32_t dtype, sdk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Mapped convolution.  weight [Cout, Cin, K]; bias [Cout];
 * input [B,Cin,H,W]; sample_map [OH,OW,K,(P,)2]; output [B,Cout,OH,OW].
 *
 * Every convolution entry point needs device scratch (re-laid-out weights for
 * the fused kernels, one batch element's column matrix for the unfused path):
 * ask sdk_mapped_conv_workspace_bytes() (same arguments for the forward,
 * backward and transposed entry points of one layer call; map_height x map_width
 * is the grid of the sample map: OH x OW, resp. IH x IW for the transposed
 * layer; image_height x image_width is the image the map points into: the
 * input of a mapped convolution, the output of a transposed one) and pass at
 * least that many bytes, 256-byte aligned.  Besides the
 * weights the scratch holds the call's tap plan (the sample map resolved into
 * window indices and coefficients), up to
 * 8 * map pixels * kernel_size * points * taps-per-point bytes, and the weight
 * gradient's per-workgroup partial sums (at most 160 MB; larger ones are not
 * reserved and that call adds to grad_weight directly).
 * ------------------------------------------------------------------------- */
size_t sdk_mapped_conv_workspace_bytes(int64_t batch, int64_t in_channels, int64_t out_channels,
                                       int64_t image_height, int64_t image_width,
                                       int64_t map_height, int64_t map_width,
                                       int64_t kernel_size,
                                       int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                       int32_t compute);

/* output[b] = weight[Cout, Cin*K] x im2col(input[b]) + bias.
 * Replaces `_mapped_convolution.mapped_conv_forward` /
 * `_weighted_mapped_convolution.weighted_mapped_conv_forward`
 * (ext_modules/include/layers/mapped_convolution_layer.h:62-87,
 *  weighted_mapped_convolution_layer.h:69-101; device side
 *  ext_modules/src/cuda/mapped_convolution_layer.cu:16-74). */
int sdk_mapped_conv_forward(const void* input, const void* sample_map, const void* interp_weights,
                            const void* weight, const void* bias, void* output, void* workspace,
                            size_t workspace_bytes, int64_t batch, int64_t in_channels,
                            int64_t height, int64_t width, int64_t out_channels,
                            int64_t out_height, int64_t out_width, int64_t kernel_size,
                            int32_t num_interp_pts, int32_t interp, int32_t dtype,
                            int32_t compute, sdk_stream_t stream);

/* grad_input[b] = col2im(weight^T x grad_output[b]).
 * Replaces cuda::MappedConvBackwardInput, first half of `mapped_conv_backward`
 * (ext_modules/include/layers/mapped_convolution_layer.h:89-134;
 *  ext_modules/src/cuda/mapped_convolution_layer.cu:76-133). */
int sdk_mapped_conv_backward_input(const void* grad_output, const void* sample_map,
                                   const void* interp_weights, const void* weight,
                                   void* grad_input, void* workspace, size_t workspace_bytes,
                                   int64_t batch, int64_t in_channels, int64_t height,
                                   int64_t width, int64_t out_channels, int64_t out_height,
                                   int64_t out_width, int64_t kernel_size,
                                   int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                   int32_t compute, sdk_stream_t stream);

/* grad_weight[Cout, Cin*K] = sum_b grad_output[b] x im2col(input[b])^T.
 * Replaces cuda::MappedConvBackwardWeight
 * (ext_modules/src/cuda/mapped_convolution_layer.cu:135-194). */
int sdk_mapped_conv_backward_weight(const void* grad_output, const void* sample_map,
                                    const void* interp_weights, const void* input,
                                    void* grad_weight, void* workspace, size_t workspace_bytes,
                                    int64_t batch, int64_t in_channels, int64_t height,
                                    int64_t width, int64_t out_channels, int64_t out_height,
                                    int64_t out_width, int64_t kernel_size,
                                    int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                    int32_t compute, sdk_stream_t stream);

/* grad_bias[c] = sum over batch and pixels of grad_output[b,c,:]
 * (`grad_output.sum({0, 2, 3})`, ext_modules/include/layers/mapped_convolution_layer.h:130). */
int sdk_bias_grad(const void* grad_output, void* grad_bias, int64_t batch, int64_t channels,
                  int64_t pixels, int32_t dtype, sdk_stream_t stream);

/* All three gradients of one layer call: grad_input, grad_weight and grad_bias as the
 * three entry points above compute them, with the map resolved once for both contractions.
 * Replaces `_mapped_convolution.mapped_conv_backward` /
 * `_weighted_mapped_convolution.weighted_mapped_conv_backward`, which return the three
 * tensors from one call (ext_modules/include/layers/mapped_convolution_layer.h:89-134,
 *  weighted_mapped_convolution_layer.h:103-153).
 * When grad_output holds 384 MiB or more, the bias gradient (bound by HBM) runs on a stream of
 * the library's own, forked from `stream` before the two contractions (bound by the matrix
 * unit) and joined behind them; everything the call launches is complete when the work queued
 * on `stream` behind the call starts.  While `stream` is being captured into a graph, and for
 * smaller tensors, all of it runs on `stream`.  The same holds for
 * sdk_mapped_transposed_conv_backward. */
int sdk_mapped_conv_backward(const void* grad_output, const void* sample_map,
                             const void* interp_weights, const void* input, const void* weight,
                             void* grad_input, void* grad_weight, void* grad_bias,
                             void* workspace, size_t workspace_bytes, int64_t batch,
                             int64_t in_channels, int64_t height, int64_t width,
                             int64_t out_channels, int64_t out_height, int64_t out_width,
                             int64_t kernel_size, int32_t num_interp_pts, int32_t interp,
                             int32_t dtype, int32_t compute, sdk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Mapped transposed convolution.  weight [Cin, Cout, K]; bias [Cout];
 * input [B,Cin,IH,IW]; sample_map [IH,IW,K,(P,)2] pointing into the
 * [OH,OW] output; output [B,Cout,OH,OW].
 * Replace `_mapped_transposed_convolution.mapped_transposed_conv_forward/_backward`
 * and the weighted twins
 * (ext_modules/include/layers/mapped_transposed_convolution_layer.h:62-93, :95-140;
 *  device side ext_modules/src/cuda/mapped_transposed_convolution_layer.cu:53-223).
 * ------------------------------------------------------------------------- */
int sdk_mapped_transposed_conv_forward(const void* input, const void* sample_map,
                                       const void* interp_weights, const void* weight,
                                       const void* bias, void* output, void* workspace,
                                       size_t workspace_bytes, int64_t batch,
                                       int64_t in_channels, int64_t in_height, int64_t in_width,
                                       int64_t out_channels, int64_t out_height,
                                       int64_t out_width, int64_t kernel_size,
                                       int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                       int32_t compute, sdk_stream_t stream);

int sdk_mapped_transposed_conv_backward_input(const void* grad_output, const void* sample_map,
                                              const void* interp_weights, const void* weight,
                                              void* grad_input, void* workspace,
                                              size_t workspace_bytes, int64_t batch,
                                              int64_t in_channels, int64_t in_height,
                                              int64_t in_width, int64_t out_channels,
                                              int64_t out_height, int64_t out_width,
                                              int64_t kernel_size, int32_t num_interp_pts,
                                              int32_t interp, int32_t dtype, int32_t compute,
                                              sdk_stream_t stream);

int sdk_mapped_transposed_conv_backward_weight(const void* grad_output, const void* sample_map,
                                               const void* interp_weights, const void* input,
                                               void* grad_weight, void* workspace,
                                               size_t workspace_bytes, int64_t batch,
                                               int64_t in_channels, int64_t in_height,
                                               int64_t in_width, int64_t out_channels,
                                               int64_t out_height, int64_t out_width,
                                               int64_t kernel_size, int32_t num_interp_pts,
                                               int32_t interp, int32_t dtype, int32_t compute,
                                               sdk_stream_t stream);

/* All three gradients of one transposed layer call.  Replaces
 * `_mapped_transposed_convolution.mapped_transposed_conv_backward` and its weighted twin
 * (ext_modules/include/layers/mapped_transposed_convolution_layer.h:92-140). */
int sdk_mapped_transposed_conv_backward(const void* grad_output, const void* sample_map,
                                        const void* interp_weights, const void* input,
                                        const void* weight, void* grad_input, void* grad_weight,
                                        void* grad_bias, void* workspace, size_t workspace_bytes,
                                        int64_t batch, int64_t in_channels, int64_t in_height,
                                        int64_t in_width, int64_t out_channels,
                                        int64_t out_height, int64_t out_width,
                                        int64_t kernel_size, int32_t num_interp_pts,
                                        int32_t interp, int32_t dtype, int32_t compute,
                                        sdk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Plans: what the convolution kernels derive from the sample map alone, kept
 * between calls.  The reference is stateless (every call of
 * ext_modules/src/cuda/mapped_convolution_layer.cu:16-194 re-reads the map); a
 * layer's map is constant over a training run, so the tap plan (the map
 * resolved into window indices and coefficients per pixel tile, with the lists
 * of tiles by kind) and its inverse (per image pixel the pixels that sample
 * it) can be built once into caller-owned device memory:
 *
 *   sdk_mapped_conv_plan_bytes(...)   size of the buffer, 0 when this geometry
 *                                     has no plan (then use the plain entry points)
 *   sdk_mapped_conv_plan_build(...)   fills it from sample_map / interp_weights
 *   sdk_..._planned(...)              the entry point of the same name with
 *                                     (plan, plan_bytes) after the workspace
 *                                     pair; identical results
 *
 * A plan depends on the map, on the size of the image it points into
 * (image_height x image_width), on the map's grid (map_height x map_width),
 * kernel_size, num_interp_pts and interp; not on batch size, channel counts,
 * weights or the compute mode, and one plan serves a mapped convolution and a
 * mapped transposed convolution over the same map.  The buffer must be
 * 256-byte aligned, is only read by the planned calls, and must be rebuilt
 * when the map's contents change.  float32 tensors only (dtype = SDK_F32).
 * ------------------------------------------------------------------------- */
size_t sdk_mapped_conv_plan_bytes(int64_t image_height, int64_t image_width, int64_t map_height,
                                  int64_t map_width, int64_t kernel_size, int32_t num_interp_pts,
                                  int32_t interp, int32_t dtype);
int sdk_mapped_conv_plan_build(const void* sample_map, const void* interp_weights, void* plan,
                               size_t plan_bytes, int64_t image_height, int64_t image_width,
                               int64_t map_height, int64_t map_width, int64_t kernel_size,
                               int32_t num_interp_pts, int32_t interp, int32_t dtype,
                               sdk_stream_t stream);
int sdk_mapped_conv_forward_planned(const void* input, const void* sample_map, const void*
    interp_weights, const void* weight, const void* bias, void* output, void* workspace, size_t
    workspace_bytes, void* plan, size_t plan_bytes, int64_t batch, int64_t in_channels, int64_t
    height, int64_t width, int64_t out_channels, int64_t out_height, int64_t out_width, int64_t
    kernel_size, int32_t num_interp_pts, int32_t interp, int32_t dtype, int32_t compute,
    sdk_stream_t stream);
int sdk_mapped_conv_backward_input_planned(const void* grad_output, const void* sample_map, const
    void* interp_weights, const void* weight, void* grad_input, void* workspace, size_t
    workspace_bytes, void* plan, size_t plan_bytes, int64_t batch, int64_t in_channels, int64_t
    height, int64_t width, int64_t out_channels, int64_t out_height, int64_t out_width, int64_t
    kernel_size, int32_t num_interp_pts, int32_t interp, int32_t dtype, int32_t compute,
    sdk_stream_t stream);
int sdk_mapped_conv_backward_weight_planned(const void* grad_output, const void* sample_map, const
    void* interp_weights, const void* input, void* grad_weight, void* workspace, size_t
    workspace_bytes, void* plan, size_t plan_bytes, int64_t batch, int64_t in_channels, int64_t
    height, int64_t width, int64_t out_channels, int64_t out_height, int64_t out_width, int64_t
    kernel_size, int32_t num_interp_pts, int32_t interp, int32_t dtype, int32_t compute,
    sdk_stream_t stream);
int sdk_mapped_conv_backward_planned(const void* grad_output, const void* sample_map, const void*
    interp_weights, const void* input, const void* weight, void* grad_input, void* grad_weight,
    void* grad_bias, void* workspace, size_t workspace_bytes, void* plan, size_t plan_bytes,
    int64_t batch, int64_t in_channels, int64_t height, int64_t width, int64_t out_channels,
    int64_t out_height, int64_t out_width, int64_t kernel_size, int32_t num_interp_pts, int32_t
    interp, int32_t dtype, int32_t compute, sdk_stream_t stream);
int sdk_mapped_transposed_conv_forward_planned(const void* input, const void* sample_map, const
    void* interp_weights, const void* weight, const void* bias, void* output, void* workspace,
    size_t workspace_bytes, void* plan, size_t plan_bytes, int64_t batch, int64_t in_channels,
    int64_t in_height, int64_t in_width, int64_t out_channels, int64_t out_height, int64_t
    out_width, int64_t kernel_size, int32_t num_interp_pts, int32_t interp, int32_t dtype, int32_t
    compute, sdk_stream_t stream);
int sdk_mapped_transposed_conv_backward_input_planned(const void* grad_output, const void*
    sample_map, const void* interp_weights, const void* weight, void* grad_input, void* workspace,
    size_t workspace_bytes, void* plan, size_t plan_bytes, int64_t batch, int64_t in_channels,
    int64_t in_height, int64_t in_width, int64_t out_channels, int64_t out_height, int64_t
    out_width, int64_t kernel_size, int32_t num_interp_pts, int32_t interp, int32_t dtype, int32_t
    compute, sdk_stream_t stream);
int sdk_mapped_transposed_conv_backward_weight_planned(const void* grad_output, const void*
    sample_map, const void* interp_weights, const void* input, void* grad_weight, void* workspace,
    size_t workspace_bytes, void* plan, size_t plan_bytes, int64_t batch, int64_t in_channels,
    int64_t in_height, int64_t in_width, int64_t out_channels, int64_t out_height, int64_t
    out_width, int64_t kernel_size, int32_t num_interp_pts, int32_t interp, int32_t dtype, int32_t
    compute, sdk_stream_t stream);
int sdk_mapped_transposed_conv_backward_planned(const void* grad_output, const void* sample_map,
    const void* interp_weights, const void* input, const void* weight, void* grad_input, void*
    grad_weight, void* grad_bias, void* workspace, size_t workspace_bytes, void* plan, size_t
    plan_bytes, int64_t batch, int64_t in_channels, int64_t in_height, int64_t in_width, int64_t
    out_channels, int64_t out_height, int64_t out_width, int64_t kernel_size, int32_t
    num_interp_pts, int32_t interp, int32_t dtype, int32_t compute, sdk_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Plans of the scatter direction.  The optional workspaces of
 * sdk_resample_to_map / sdk_resample_to_map_normalized, sdk_mapped_avg_unpool
 * and sdk_mapped_max_unpool hold what those calls derive from the map alone
 * (the inverted map: per target pixel its sources; the pooled window of every
 * image tile).  A caller whose map stays the same builds that once into its
 * own device memory ("plan", as large as the workspace of the same call) and
 * passes it to the *_planned entry point, which skips the rebuild and gives
 * the same results.  The reference has no counterpart (its entry points,
 * ext_modules/include/layers/resample_layer.h:40-60,
 * mapped_avg_pooling_layer.h, mapped_max_pooling_layer.h:64-88, are stateless).
 *
 * sdk_resample_to_map_plan_build: plan_bytes >=
 *   sdk_resample_to_map_workspace_bytes(height, width, dtype).  kernel_size = 1
 *   for a resampling map [map_height, map_width, (P,) 2]; for average
 *   unpooling pass the pooled grid as map_height x map_width and the map's K.
 *   An average-unpooling plan also holds, behind the lists, the pooled window
 *   of every image tile (as sdk_mapped_max_unpool's plan does): where every
 *   window has at most 8192 pooled pixels the planned call sums each tile in
 *   LDS from its window and the lists are neither filled nor read; otherwise
 *   it gathers through the lists.
 * sdk_resample_plan_complete: synchronises `stream` and sets *complete to a
 *   bit mask.  Bit 0 (value 1): the planned call needs no fallback (every
 *   target's list holds all its sources, at most 16 each, or the lists are not
 *   used).  Bit 1 (value 2): the tiled average unpooling runs.  The planned
 *   calls take that mask as plan_complete: with bit 0 set they launch the
 *   gather (or the tiled kernel) alone (sample_map / interp_weights are then
 *   not read by sdk_resample_to_map_planned and may be NULL; the average
 *   unpooling always reads them); with 0 they launch every stage, each gated on
 *   the device, and the fallback (fill, atomic scatter, division) runs only if
 *   the plan is incomplete.  Passing a set bit for a plan that did not report
 *   it gives wrong results (sources that did not fit are dropped).
 * sdk_resample_to_map_planned: normalize = 0 is sdk_resample_to_map (weight_sum
 *   optional), normalize = 1 sdk_resample_to_map_normalized (weight_sum
 *   required, eps used).
 * sdk_mapped_max_unpool_plan_build / _planned: plan_bytes >=
 *   sdk_mapped_max_unpool_workspace_bytes(height, width, dtype).  The first
 *   256 bytes of this plan are the call's fallback flag and are rewritten by
 *   every planned call: calls that share one plan must not overlap.
 * sdk_mapped_max_unpool_plan_bands: synchronises `stream` and sets *bands to 1
 *   if the plan's map lets one kernel do the whole call (float32, unweighted
 *   nearest taps, every pooled row reaching few image rows), else to 0.
 * sdk_mapped_max_unpool_planned_bands: sdk_mapped_max_unpool_planned for a plan
 *   on which that query returned 1 (with 0 the result is undefined): the same
 *   result with two launches in place of five.  Unweighted maps only, so it
 *   takes no interp_weights / num_interp_pts.  It leaves the plan's flag
 *   cleared itself instead of clearing it up front.
 * ------------------------------------------------------------------------- */
int sdk_resample_to_map_plan_build(const void* sample_map, const void* interp_weights, void* plan,
                                   size_t plan_bytes, int64_t map_height, int64_t map_width,
                                   int64_t height, int64_t width, int64_t kernel_size,
                                   int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                   sdk_stream_t stream);
int sdk_resample_plan_complete(const void* plan, size_t plan_bytes, sdk_stream_t stream,
                               int32_t* complete);
int sdk_resample_to_map_planned(const void* input, const void* sample_map,
                                const void* interp_weights, void* out, void* weight_sum,
                                void* plan, size_t plan_bytes, int32_t plan_complete,
                                int32_t normalize, double eps, int64_t batch, int64_t channels,
                                int64_t map_height, int64_t map_width, int64_t height,
                                int64_t width, int32_t num_interp_pts, int32_t interp,
                                int32_t dtype, sdk_stream_t stream);
int sdk_mapped_avg_unpool_planned(const void* grad_output, const void* sample_map,
                                  const void* interp_weights, void* grad_input, void* plan,
                                  size_t plan_bytes, int32_t plan_complete, int64_t batch,
                                  int64_t channels, int64_t height, int64_t width,
                                  int64_t out_height, int64_t out_width, int64_t kernel_size,
                                  int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                  sdk_stream_t stream);
int sdk_mapped_max_unpool_plan_build(const void* sample_map, void* plan, size_t plan_bytes,
                                     int64_t height, int64_t width, int64_t out_height,
                                     int64_t out_width, int64_t kernel_size,
                                     int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                     sdk_stream_t stream);
int sdk_mapped_max_unpool_planned(const void* grad_output, const int64_t* indices,
                                  const void* sample_map, const void* interp_weights,
                                  void* grad_input, void* plan, size_t plan_bytes, int64_t batch,
                                  int64_t channels, int64_t height, int64_t width,
                                  int64_t out_height, int64_t out_width, int64_t kernel_size,
                                  int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                  sdk_stream_t stream);
int sdk_mapped_max_unpool_plan_bands(const void* plan, size_t plan_bytes, int64_t height,
                                     int64_t width, int32_t dtype, sdk_stream_t stream,
                                     int32_t* bands);
int sdk_mapped_max_unpool_planned_bands(const void* grad_output, const int64_t* indices,
                                        const void* sample_map, void* grad_input, void* plan,
                                        size_t plan_bytes, int64_t batch, int64_t channels,
                                        int64_t height, int64_t width, int64_t out_height,
                                        int64_t out_width, int64_t kernel_size, int32_t interp,
                                        int32_t dtype, sdk_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SDK_MAPPED_OPS_H_ */
