// Generic (any floating type, any shape) convolution path: mapped im2col /
// col2im kernels chained with a plain LDS-tiled FMA GEMM, one batch element at
// a time through a caller-provided column workspace.  This is the route for
// float64 (the type of the reference's own known-answer tests) and for shapes
// the fused MFMA kernels do not cover; it is also what the fused kernels are
// cross-checked against on the GPU.
#include <hip/hip_runtime.h>

#include "conv_internal.hpp"
#include "sdk_host.hpp"
#include "sdk_taps.hpp"

namespace sdk {

constexpr int kTile = 64;   // C tile is kTile x kTile per 256-thread block
constexpr int kStep = 16;   // reduction step staged through LDS

// C[i,j] (op)= sum_l A(i,l) * B(l,j) with arbitrary element strides.
// grid.z = split of the reduction range; with splits > 1 (or accumulate) the
// partial tile is added atomically onto C, otherwise stored (+ row bias).
template <typename T>
__global__ __launch_bounds__(256) void gemm_strided_kernel(
    const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
    const T* __restrict__ row_bias, int m, int n, int k, int64_t sai, int64_t sal, int64_t sbl,
    int64_t sbj, int64_t sci, int k_per_split, int atomic_out) {
  __shared__ T As[kStep][kTile + 1];
  __shared__ T Bs[kStep][kTile + 1];
  const int tid = threadIdx.x;
  const int ti = tid / 16, tj = tid % 16;  // 16 x 16 threads, 4 x 4 outputs each
  const int i0 = blockIdx.y * kTile, j0 = blockIdx.x * kTile;
  const int kbeg = blockIdx.z * k_per_split;
  const int kend = min(k, kbeg + k_per_split);
  T acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = T(0);

  for (int k0 = kbeg; k0 < kend; k0 += kStep) {
    // Stage kStep x kTile slices of A and B (4 elements per thread each).  The
    // thread->element order follows the faster-varying stride of each operand.
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = tid + r * 256;
      int l, i;
      if (sal == 1) { l = e % kStep; i = e / kStep; } else { i = e % kTile; l = e / kTile; }
      const int gi = i0 + i, gl = k0 + l;
      As[l][i] = (gi < m && gl < kend) ? A[(int64_t)gi * sai + (int64_t)gl * sal] : T(0);
      int j;
      if (sbl == 1) { l = e % kStep; j = e / kStep; } else { j = e % kTile; l = e / kTile; }
      const int gj = j0 + j;
      const int gl2 = k0 + l;
      Bs[l][j] = (gj < n && gl2 < kend) ? B[(int64_t)gl2 * sbl + (int64_t)gj * sbj] : T(0);
    }
    __syncthreads();
#pragma unroll
    for (int l = 0; l < kStep; ++l) {
      T a[4], b[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        a[r] = As[l][ti + 16 * r];
        b[r] = Bs[l][tj + 16 * r];
      }
#pragma unroll
      for (int x = 0; x < 4; ++x)
#pragma unroll
        for (int y = 0; y < 4; ++y) acc[x][y] += a[x] * b[y];
    }
    __syncthreads();
  }
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const int gi = i0 + ti + 16 * x;
    if (gi >= m) continue;
#pragma unroll
    for (int y = 0; y < 4; ++y) {
      const int gj = j0 + tj + 16 * y;
      if (gj >= n) continue;
      T* dst = C + (int64_t)gi * sci + gj;
      if (atomic_out)
        atomic_add_noret(dst, acc[x][y]);
      else
        *dst = acc[x][y] + (row_bias ? row_bias[gi] : T(0));
    }
  }
}

template <typename T>
static int gemm_strided(const T* A, const T* B, T* C, const T* row_bias, int m, int n, int k,
                        int64_t sai, int64_t sal, int64_t sbl, int64_t sbj, int64_t sci,
                        int splits, bool accumulate, hipStream_t stream) {
  if (m == 0 || n == 0) return SDK_OK;
  splits = max(1, min(splits, (int)ceil_div(k, kStep)));
  int kps = (int)ceil_div(k, splits);
  kps = (int)ceil_div(kps, kStep) * kStep;
  splits = (int)ceil_div(k, kps);
  const dim3 grid((unsigned)ceil_div(n, kTile), (unsigned)ceil_div(m, kTile), (unsigned)splits);
  launch(gemm_strided_kernel<T>, grid, dim3(256), stream, A, B, C, row_bias, m, n,
                     k, sai, sal, sbl, sbj, sci, kps, (splits > 1 || accumulate) ? 1 : 0);
  SDK_LAUNCH_CHECK("gemm_strided");
  return SDK_OK;
}

// img plane fill: dst[(b*C + c)*n + i] = bias ? bias[c] : 0.
template <typename T>
__global__ __launch_bounds__(256) void plane_fill_kernel(T* __restrict__ dst,
                                                         const T* __restrict__ bias, int C,
                                                         size_t n, const int* __restrict__ gate) {
  if (gate != nullptr && *gate == 0) return;
  const size_t plane = blockIdx.y;
  const T v = bias ? bias[plane % C] : T(0);
  T* p = dst + plane * n;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    p[i] = v;
}

template <typename T>
int plane_fill(T* dst, const T* bias, int64_t planes, int C, size_t n, hipStream_t stream,
               const int* gate) {
  if (planes == 0 || n == 0) return SDK_OK;
  if (!bias) return zero_fill_gated(dst, sizeof(T) * (size_t)planes * n, stream, gate);
  if (planes > 65535) return fail(SDK_ERR_UNSUPPORTED, "plane_fill: too many planes");
  const dim3 grid((unsigned)std::min<int64_t>(ceil_div((int64_t)n, 256), 64), (unsigned)planes);
  launch(plane_fill_kernel<T>, grid, dim3(256), stream, dst, bias, C, n, gate);
  SDK_LAUNCH_CHECK("plane_fill");
  return SDK_OK;
}
template int plane_fill<float>(float*, const float*, int64_t, int, size_t, hipStream_t, const int*);
template int plane_fill<double>(double*, const double*, int64_t, int, size_t, hipStream_t,
                                const int*);

template <typename T>
int generic_gather_gemm(const ConvGeom& g, const T* img, const T* map, const T* wts, const T* Wm,
                        const T* bias, T* pix, T* workspace, hipStream_t stream) {
  const int CK = g.Cg * g.K;
  const size_t img_b = (size_t)g.Cg * g.H * g.W, pix_b = (size_t)g.Cp * g.M;
  for (int64_t b = 0; b < g.B; ++b) {
    int rc = launch_mapped_im2col<T>(img + b * img_b, map, wts, workspace, g.Cg, g.H, g.W, g.M,
                                     g.K, g.P, g.interp, stream);
    if (rc) return rc;
    // pix[b][Cp, M] = Wm[Cp, CK] x col[CK, M] + bias
    rc = gemm_strided<T>(Wm, workspace, pix + b * pix_b, bias, g.Cp, g.M, CK, CK, 1, g.M, 1, g.M,
                         1, false, stream);
    if (rc) return rc;
  }
  return SDK_OK;
}

template <typename T>
int generic_gemm_scatter(const ConvGeom& g, const T* pix, const T* map, const T* wts, const T* Wm,
                         const T* bias, T* img, T* workspace, hipStream_t stream) {
  const int CK = g.Cg * g.K;
  const size_t img_b = (size_t)g.Cg * g.H * g.W, pix_b = (size_t)g.Cp * g.M;
  int rc = plane_fill<T>(img, bias, g.B * g.Cg, g.Cg, (size_t)g.H * g.W, stream);
  if (rc) return rc;
  for (int64_t b = 0; b < g.B; ++b) {
    // col[CK, M] = Wm^T[CK, Cp] x pix[b][Cp, M]
    rc = gemm_strided<T>(Wm, pix + b * pix_b, workspace, (const T*)nullptr, CK, g.M, g.Cp, 1, CK,
                         g.M, 1, g.M, 1, false, stream);
    if (rc) return rc;
    rc = launch_mapped_col2im<T>(workspace, map, wts, img + b * img_b, g.Cg, g.H, g.W, g.M, g.K,
                                 g.P, g.interp, stream);
    if (rc) return rc;
  }
  return SDK_OK;
}

template <typename T>
int generic_gather_wgrad(const ConvGeom& g, const T* pix, const T* map, const T* wts, const T* img,
                         T* gW, T* workspace, hipStream_t stream) {
  const int CK = g.Cg * g.K;
  const size_t img_b = (size_t)g.Cg * g.H * g.W, pix_b = (size_t)g.Cp * g.M;
  int rc = zero_fill(gW, sizeof(T) * (size_t)g.Cp * CK, stream);
  if (rc) return rc;
  const int tiles = (int)(ceil_div(CK, kTile) * ceil_div(g.Cp, kTile));
  const int splits = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(g.M, 256),
                                                               ceil_div(2048, tiles)));
  for (int64_t b = 0; b < g.B; ++b) {
    rc = launch_mapped_im2col<T>(img + b * img_b, map, wts, workspace, g.Cg, g.H, g.W, g.M, g.K,
                                 g.P, g.interp, stream);
    if (rc) return rc;
    // gW[Cp, CK] += pix[b][Cp, M] x col[CK, M]^T
    rc = gemm_strided<T>(pix + b * pix_b, workspace, gW, (const T*)nullptr, g.Cp, CK, g.M, g.M, 1,
                         1, g.M, CK, splits, true, stream);
    if (rc) return rc;
  }
  return SDK_OK;
}

#define SDK_INSTANTIATE(T)                                                                       \
  template int generic_gather_gemm<T>(const ConvGeom&, const T*, const T*, const T*, const T*,   \
                                      const T*, T*, T*, hipStream_t);                            \
  template int generic_gemm_scatter<T>(const ConvGeom&, const T*, const T*, const T*, const T*,  \
                                       const T*, T*, T*, hipStream_t);                           \
  template int generic_gather_wgrad<T>(const ConvGeom&, const T*, const T*, const T*, const T*,  \
                                       T*, T*, hipStream_t);
SDK_INSTANTIATE(float)
SDK_INSTANTIATE(double)

// ---------------------------------------------------------------------------
// grad_bias[c] = sum_{b,i} gout[b,c,i].  grid (C, B * slices): every block reduces one
// contiguous slice of one plane (b, c), with 16-byte loads where the slice allows, and adds
// its partial sum atomically.
// ---------------------------------------------------------------------------
// NOLDS: every wave adds its partial sum itself (four atomics per block instead of one, 0.15
// against 0.12 ms at 8 x 128 x 256 x 512 when the kernel runs alone).  That form is for a
// combined backward call, where this kernel runs beside contraction kernels whose workgroups
// fill a CU's LDS: a block holding even one LDS granule would keep one of them out.
template <typename T, bool NOLDS>
__global__ __launch_bounds__(256) void bias_grad_kernel(const T* __restrict__ gout,
                                                        T* __restrict__ gbias, int C, int M,
                                                        int slices, int per_block) {
  const int c = blockIdx.x;
  const int b = blockIdx.y / slices, sl = blockIdx.y % slices;
  const int beg = sl * per_block, end = min(M, beg + per_block);
  const T* p = gout + ((size_t)b * C + c) * M;
  constexpr int V = 16 / (int)sizeof(T);   // elements per 16-byte load
  T acc = T(0);
  // elements up to the first 16-byte boundary (planes whose size is not a multiple of four
  // elements start anywhere), 16-byte loads from there, then what is left
  const int mis = (int)(((reinterpret_cast<uintptr_t>(p) + (size_t)beg * sizeof(T)) & 15) / sizeof(T));
  const int head = min(end - beg, mis ? V - mis : 0);
  if ((int)threadIdx.x < head) acc += p[beg + threadIdx.x];
  const int vbeg = beg + head;
  T a0 = T(0), a1 = T(0), a2 = T(0), a3 = T(0);
  const int nv = (end - vbeg) / V;
  if constexpr (V == 4) {
    // four loads in flight per thread (one per iteration waits for each in turn)
    const float4* pv = reinterpret_cast<const float4*>(p + vbeg);
    int i = threadIdx.x;
    for (; i + 768 < nv; i += 1024) {
      const float4 v0 = pv[i], v1 = pv[i + 256], v2 = pv[i + 512], v3 = pv[i + 768];
      a0 += (v0.x + v1.x) + (v2.x + v3.x);
      a1 += (v0.y + v1.y) + (v2.y + v3.y);
      a2 += (v0.z + v1.z) + (v2.z + v3.z);
      a3 += (v0.w + v1.w) + (v2.w + v3.w);
    }
    for (; i < nv; i += 256) {
      const float4 v = pv[i];
      a0 += v.x;
      a1 += v.y;
      a2 += v.z;
      a3 += v.w;
    }
  } else {
    for (int i = threadIdx.x; i < nv; i += 256) {
      const double2 v = reinterpret_cast<const double2*>(p + vbeg)[i];
      a0 += v.x;
      a1 += v.y;
    }
  }
  acc += (a0 + a1) + (a2 + a3);
  for (int i = vbeg + nv * V + threadIdx.x; i < end; i += 256) acc += p[i];
  // wave64 butterfly, then one LDS slot per wave (or one atomic per wave)
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
  if constexpr (NOLDS) {
    if ((threadIdx.x & 63) == 0) atomic_add_noret(gbias + c, acc);
  } else {
    __shared__ T part[4];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) atomic_add_noret(gbias + c, part[0] + part[1] + part[2] + part[3]);
  }
}

template <typename T>
int launch_bias_grad(const T* gout, T* gbias, int64_t B, int64_t C, int64_t M,
                     hipStream_t stream, bool no_lds) {
  int rc = zero_fill(gbias, sizeof(T) * (size_t)C, stream);
  if (rc) return rc;
  if (B * M == 0 || C == 0) return SDK_OK;
  // about 8192 blocks overall, at least 16384 elements each; slices of a multiple of 4 elements
  int64_t slices = std::min<int64_t>(std::max<int64_t>(1, ceil_div(8192, C * B)),
                                     std::max<int64_t>(1, M / 16384));
  int64_t per_block = ceil_div(ceil_div(M, slices), 4) * 4;
  slices = ceil_div(M, per_block);
  if (B * slices > 65535)
    return fail(SDK_ERR_UNSUPPORTED, "bias_grad: batch %lld too large", (long long)B);
  const dim3 grid((unsigned)C, (unsigned)(B * slices));
  if (no_lds)
    launch(bias_grad_kernel<T, true>, grid, dim3(256), stream, gout, gbias, (int)C, (int)M,
           (int)slices, (int)per_block);
  else
    launch(bias_grad_kernel<T, false>, grid, dim3(256), stream, gout, gbias, (int)C, (int)M,
           (int)slices, (int)per_block);
  SDK_LAUNCH_CHECK("bias_grad");
  return SDK_OK;
}

int bias_grad(const void* grad_output, void* grad_bias, int64_t batch, int64_t channels,
              int64_t pixels, int32_t dtype, hipStream_t stream, bool beside_contractions) {
  SDK_REQUIRE(grad_output && grad_bias, "bias_grad: NULL pointer");
  SDK_REQUIRE(batch >= 0 && channels >= 0 && pixels >= 0 && pixels < ((int64_t)1 << 31) &&
                  batch * pixels < ((int64_t)1 << 40) && channels <= 2147483647,
              "bias_grad: bad size");
  SDK_DISPATCH_DTYPE(dtype, return launch_bias_grad<T>((const T*)grad_output, (T*)grad_bias, batch,
                                                        channels, pixels, stream,
                                                        beside_contractions));
  return SDK_OK;
}

}  // namespace sdk

extern "C" int sdk_bias_grad(const void* grad_output, void* grad_bias, int64_t batch,
                             int64_t channels, int64_t pixels, int32_t dtype,
                             sdk_stream_t stream) {
  return sdk::bias_grad(grad_output, grad_bias, batch, channels, pixels, dtype,
                        (hipStream_t)stream, false);
}
