// Sample maps computed on the device: the kernel maps of an equirectangular image (grid,
// inverse gnomonic and inverse equirectangular projection of a kh x kw tangent-plane kernel
// about every pixel) and gnomonic kernels about arbitrary points of the sphere.  The reference
// builds these on the host with tensor operations (layers/util/mapping_functions.py:16-160,
// layers/util/icosahedron_functions.py:47-103, layers/util/conversions.py:24-76,
// layers/util/grids.py:5-25); here one thread computes one sample, in the map's own precision
// and in the reference's order of operations, so a float32 map differs from the reference's
// only by the last bits of the transcendental functions.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "sdk_host.hpp"

namespace sdk {

constexpr int kMapBlock = 256;
constexpr double kPi = 3.14159265358979323846;

__device__ __forceinline__ float m_sin(float v) { return sinf(v); }
__device__ __forceinline__ double m_sin(double v) { return sin(v); }
__device__ __forceinline__ float m_cos(float v) { return cosf(v); }
__device__ __forceinline__ double m_cos(double v) { return cos(v); }
__device__ __forceinline__ float m_atan(float v) { return atanf(v); }
__device__ __forceinline__ double m_atan(double v) { return atan(v); }
__device__ __forceinline__ float m_asin(float v) { return asinf(v); }
__device__ __forceinline__ double m_asin(double v) { return asin(v); }
__device__ __forceinline__ float m_atan2(float a, float b) { return atan2f(a, b); }
__device__ __forceinline__ double m_atan2(double a, double b) { return atan2(a, b); }
__device__ __forceinline__ float m_sqrt(float v) { return sqrtf(v); }
__device__ __forceinline__ double m_sqrt(double v) { return sqrt(v); }
__device__ __forceinline__ float m_fmod(float a, float b) { return fmodf(a, b); }
__device__ __forceinline__ double m_fmod(double a, double b) { return fmod(a, b); }

// Element i of `steps` evenly spaced values from lo to hi, as the tensor library the reference
// runs on computes them: from the lower end in the first half, from the upper end in the second.
template <typename T>
__device__ __forceinline__ T linspace_at(T lo, T hi, int steps, int i) {
  const T step = (hi - lo) / T(steps - 1);
  return i < steps / 2 ? lo + step * T(i) : hi - step * T(steps - i - 1);
}

// Remainder with the sign of the divisor (the `%` of the reference's tensors).
template <typename T>
__device__ __forceinline__ T floor_mod(T a, T b) {
  T m = m_fmod(a, b);
  if (m != T(0) && ((b < T(0)) != (m < T(0)))) m += b;
  return m;
}

// (new_hi - new_lo) * (v - old_lo) / (old_hi - old_lo) + new_lo with new_lo = 0
// (layers/util/conversions.py:24-30); longitude -> column, latitude -> row (:33-52).
template <typename T>
__device__ __forceinline__ T lon_to_x(T lon, int W) {
  return T(W) * (lon - T(-kPi)) / T(kPi - (-kPi));
}
template <typename T>
__device__ __forceinline__ T lat_to_y(T lat, int H) {
  return T(H - 1) * (lat - T(-kPi / 2)) / T(kPi / 2 - (-kPi / 2));
}

// Inverse gnomonic projection of the tangent-plane point (dx, dy) about (lon, lat)
// (layers/util/mapping_functions.py:99-104, layers/util/icosahedron_functions.py:86-91).
template <typename T>
__device__ __forceinline__ void inverse_gnomonic(T lon, T lat, T dx, T dy, T& out_lon, T& out_lat) {
  const T rho = m_sqrt(dx * dx + dy * dy);
  const T nu = m_atan(rho);
  out_lat = m_asin(m_cos(nu) * m_sin(lat) + dy * m_sin(nu) * m_cos(lat) / rho);
  out_lon = lon + m_atan2(dx * m_sin(nu), rho * m_cos(lat) * m_cos(nu) - dy * m_sin(lat) * m_sin(nu));
}

// out [OH, OW, kh*kw, 2], OH = ceil(H / stride), OW = ceil(W / stride).
// PROJ 0: grid (mapping_functions.py:43-75), 1: inverse gnomonic (:78-120),
// 2: inverse equirectangular (:123-160).
template <typename T, int PROJ>
__global__ __launch_bounds__(kMapBlock) void equirect_kernel_map_kernel(
    T* __restrict__ out, int H, int W, int kh, int kw, int stride, int dilation, int OW,
    size_t total, double res_lon, double res_lat) {
  const size_t idx = (size_t)blockIdx.x * kMapBlock + threadIdx.x;
  if (idx >= total) return;
  const int K = kh * kw;
  const int k = (int)(idx % K);
  const size_t pix = idx / K;
  const int x = (int)(pix % OW) * stride, y = (int)(pix / OW) * stride;
  const int ci = k / kw - kh / 2, cj = k % kw - kw / 2;
  // kernel differentials: products in double, stored in the map's precision (:30-37)
  const T dlon = (T)((double)(cj * dilation) * res_lon);
  const T dlat = (T)((double)(ci * dilation) * -res_lat);
  const T lon = linspace_at<T>(T(-kPi), T(kPi), W + 1, x);      // grids.py:19-21
  const T lat = linspace_at<T>(T(-kPi / 2), T(kPi / 2), H, y);  // grids.py:22-23
  T mlon, mlat;
  if constexpr (PROJ == 0) {
    mlat = lat + dlat;
    mlon = lon + dlon;
  } else {
    if constexpr (PROJ == 1) {
      inverse_gnomonic(lon, lat, dlon, dlat, mlon, mlat);
      if (k == K / 2) {   // the (0, 0) sample, whose projection divides by zero (:106-108)
        mlat = lat;
        mlon = lon;
      }
    } else {
      mlat = lat + dlat;
      mlon = lon + dlon / m_cos(mlat);
    }
    mlon = floor_mod(mlon + T(kPi), T(2 * kPi)) - T(kPi);   // longitudinal wrap-around
  }
  out[idx * 2] = lon_to_x(mlon, W);
  out[idx * 2 + 1] = lat_to_y(mlat, H);
}

// Gnomonic kh x kw kernels about n given points: out [n, kh*kw, 2] in (lon, lat), or in pixel
// coordinates of an img_h x img_w equirectangular image when img_h > 0
// (layers/util/icosahedron_functions.py:47-103, then conversions.py:33-52).
template <typename T>
__global__ __launch_bounds__(kMapBlock) void gnomonic_kernel_at_kernel(
    const T* __restrict__ lonlat, T* __restrict__ out, size_t total, int kh, int kw,
    double res_lat, double res_lon, int img_h, int img_w) {
  const size_t idx = (size_t)blockIdx.x * kMapBlock + threadIdx.x;
  if (idx >= total) return;
  const int K = kh * kw;
  const int k = (int)(idx % K);
  const size_t p = idx / K;
  const int i = k / kw, j = k % kw;
  T dx = (T)((j - kw / 2) * res_lon);
  T dy = (T)((i - kh / 2) * res_lat);
  if (kh % 2 == 0) dy += (T)(res_lat / 2);   // even kernels are centred between samples
  if (kw % 2 == 0) dx += (T)(res_lon / 2);
  const T lon = lonlat[p * 2], lat = lonlat[p * 2 + 1];
  T olon, olat;
  inverse_gnomonic(lon, lat, dx, dy, olon, olat);
  const bool centre = k == (kh / 2) * kw + kw / 2;
  if (kh % 2 == 1 && centre) olat = lat;
  if (kw % 2 == 1 && centre) olon = lon;
  olon = floor_mod(olon + T(kPi), T(2 * kPi)) - T(kPi);
  out[idx * 2] = img_h > 0 ? lon_to_x(olon, img_w) : olon;
  out[idx * 2 + 1] = img_h > 0 ? lat_to_y(olat, img_h) : olat;
}

// The four pixel centres around every sample and weights proportional to the inverse
// great-circle distance to them, normalised to sum to one: the weighted (P = 4) form of a map
// for an equirectangular image (columns wrap, rows clamp).  The distance comes from the
// haversine form, 2 asin sqrt(sin^2(dlat / 2) + cos lat0 cos lat1 sin^2(dlon / 2)), with the
// angle differences taken from the coordinate differences and cos(lat) as sin(pi y / (H - 1)):
// exactly 0 for a sample on a pixel centre and for any two points of a pole row, and relative
// accuracy for neighbours a pixel apart, where the arccosine of a dot product would keep half
// its digits in float32 (the weights 1 / (d + eps) are sensitive to d at the scale of eps).
__device__ __forceinline__ float m_sinpi(float v) { return sinpif(v); }
__device__ __forceinline__ double m_sinpi(double v) { return sinpi(v); }

template <typename T>
__global__ __launch_bounds__(kMapBlock) void four_nearest_weighted_kernel(
    const T* __restrict__ map, T* __restrict__ out_map, T* __restrict__ out_w, size_t count, int H,
    int W, T eps) {
  const size_t i = (size_t)blockIdx.x * kMapBlock + threadIdx.x;
  if (i >= count) return;
  const T x = map[i * 2], y = map[i * 2 + 1];
  const T x1 = floor(x);
  T y1 = floor(y);
  y1 = y1 < T(0) ? T(0) : (y1 > T(H - 1) ? T(H - 1) : y1);
  const T y2 = y1 + T(1) > T(H - 1) ? T(H - 1) : y1 + T(1);
  const T xs[4] = {x1, x1 + T(1), x1, x1 + T(1)};
  const T ys[4] = {y1, y1, y2, y2};
  const T c0 = m_sinpi(y / T(H - 1));
  T w[4], total = T(0);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const T sa = m_sinpi(T(0.5) * (y - ys[k]) / T(H - 1));
    const T so = m_sinpi((x - xs[k]) / T(W));
    T hav = sa * sa + c0 * m_sinpi(ys[k] / T(H - 1)) * so * so;
    hav = hav < T(0) ? T(0) : (hav > T(1) ? T(1) : hav);
    const T d = T(2) * m_asin(m_sqrt(hav));
    w[k] = T(1) / (d + eps);
    total += w[k];
    out_map[(i * 4 + k) * 2] = floor_mod(xs[k], T(W));
    out_map[(i * 4 + k) * 2 + 1] = ys[k];
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) out_w[i * 4 + k] = w[k] / total;
}

}  // namespace sdk

using namespace sdk;

extern "C" {

int sdk_equirect_kernel_map(void* sample_map, int64_t height, int64_t width, int64_t kernel_h,
                            int64_t kernel_w, int64_t stride, int64_t dilation,
                            int32_t projection, int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(sample_map, "equirect_kernel_map: NULL pointer");
  SDK_REQUIRE(height >= 2 && width >= 1 && height < ((int64_t)1 << 30) &&
                  width < ((int64_t)1 << 30),
              "equirect_kernel_map: image %lld x %lld (height must be at least 2)",
              (long long)height, (long long)width);
  SDK_REQUIRE(kernel_h >= 1 && kernel_w >= 1 && kernel_h * kernel_w <= 4096,
              "equirect_kernel_map: kernel %lld x %lld", (long long)kernel_h, (long long)kernel_w);
  SDK_REQUIRE(stride >= 1 && dilation >= 1, "equirect_kernel_map: stride and dilation must be >= 1");
  SDK_REQUIRE(projection >= 0 && projection <= 2, "equirect_kernel_map: unknown projection %d",
              (int)projection);
  const int64_t OH = ceil_div(height, stride), OW = ceil_div(width, stride);
  const size_t total = (size_t)OH * OW * kernel_h * kernel_w;
  SDK_REQUIRE(ceil_div((int64_t)total, kMapBlock) < ((int64_t)1 << 31),
              "equirect_kernel_map: map too large");
  SDK_REQUIRE(dilation * std::max(kernel_h, kernel_w) < ((int64_t)1 << 30),
              "equirect_kernel_map: dilation too large");
  // angular resolution of the image (grids.py:5-10)
  const double res_lon = 2 * kPi / (double)width;
  const double res_lat = kPi / (double)(height - 1);
  const dim3 grid((unsigned)ceil_div((int64_t)total, kMapBlock));
#define EKM(PROJv)                                                                               \
  SDK_DISPATCH_DTYPE(dtype, (launch(equirect_kernel_map_kernel<T, PROJv>, grid, dim3(kMapBlock), \
                                    (hipStream_t)stream, (T*)sample_map, (int)height, (int)width, \
                                    (int)kernel_h, (int)kernel_w, (int)stride, (int)dilation,    \
                                    (int)OW, total, res_lon, res_lat)))
  if (projection == 0) EKM(0); else if (projection == 1) EKM(1); else EKM(2);
#undef EKM
  SDK_LAUNCH_CHECK("equirect_kernel_map");
  return SDK_OK;
}

int sdk_gnomonic_kernel_at(const void* lonlat, void* out, int64_t num_points, int64_t kernel_h,
                           int64_t kernel_w, double res_lat, double res_lon, int64_t image_height,
                           int64_t image_width, int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(num_points >= 0, "gnomonic_kernel_at: negative size");
  SDK_REQUIRE(kernel_h >= 1 && kernel_w >= 1 && kernel_h * kernel_w <= 4096,
              "gnomonic_kernel_at: kernel %lld x %lld", (long long)kernel_h, (long long)kernel_w);
  SDK_REQUIRE(image_height == 0 || (image_height >= 2 && image_width >= 1 &&
                                    image_height < ((int64_t)1 << 30) &&
                                    image_width < ((int64_t)1 << 30)),
              "gnomonic_kernel_at: image %lld x %lld", (long long)image_height,
              (long long)image_width);
  if (num_points == 0) return SDK_OK;
  SDK_REQUIRE(lonlat && out, "gnomonic_kernel_at: NULL pointer");
  const size_t total = (size_t)num_points * kernel_h * kernel_w;
  SDK_REQUIRE(ceil_div((int64_t)total, kMapBlock) < ((int64_t)1 << 31),
              "gnomonic_kernel_at: map too large");
  const dim3 grid((unsigned)ceil_div((int64_t)total, kMapBlock));
  SDK_DISPATCH_DTYPE(dtype, (launch(gnomonic_kernel_at_kernel<T>, grid, dim3(kMapBlock),
                                    (hipStream_t)stream, (const T*)lonlat, (T*)out, total,
                                    (int)kernel_h, (int)kernel_w, res_lat, res_lon,
                                    (int)image_height, (int)image_width)));
  SDK_LAUNCH_CHECK("gnomonic_kernel_at");
  return SDK_OK;
}

int sdk_four_nearest_weighted_map(const void* sample_map, void* out_map, void* out_weights,
                                  int64_t num_samples, int64_t height, int64_t width, double eps,
                                  int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(num_samples >= 0, "four_nearest_weighted_map: negative size");
  SDK_REQUIRE(height >= 2 && width >= 1 && height < ((int64_t)1 << 24) &&
                  width < ((int64_t)1 << 24),
              "four_nearest_weighted_map: image %lld x %lld", (long long)height, (long long)width);
  SDK_REQUIRE(eps > 0.0, "four_nearest_weighted_map: eps must be positive");
  if (num_samples == 0) return SDK_OK;
  SDK_REQUIRE(sample_map && out_map && out_weights, "four_nearest_weighted_map: NULL pointer");
  SDK_REQUIRE(ceil_div(num_samples, kMapBlock) < ((int64_t)1 << 31),
              "four_nearest_weighted_map: too many samples");
  const dim3 grid((unsigned)ceil_div(num_samples, kMapBlock));
  SDK_DISPATCH_DTYPE(dtype, (launch(four_nearest_weighted_kernel<T>, grid, dim3(kMapBlock),
                                    (hipStream_t)stream, (const T*)sample_map, (T*)out_map,
                                    (T*)out_weights, (size_t)num_samples, (int)height, (int)width,
                                    (T)eps)));
  SDK_LAUNCH_CHECK("four_nearest_weighted_map");
  return SDK_OK;
}

}  // extern "C"
