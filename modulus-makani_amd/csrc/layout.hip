// Layout passes between the reference coefficient layout (complex64 [rows][lmax][mmax],
// m fastest -- what RealSHT.forward returns and InverseRealSHT.forward / the dhconv einsum
// consume, makani/models/common/spectral_convolution.py:131-141) and the order-major
// "spectral" layout float [mmax][lmax][ld] the contraction kernels work on.
#include "sfno_internal.h"

namespace sfno {

// grid (ceil(mmax/32), lmax, ceil(rows/32)), block (32, 8)
__global__ __launch_bounds__(256) void spectral_to_coeffs_kernel(const float* __restrict__ spec, float2* __restrict__ coeffs, int64_t rows,
                                                                 int lmax, int mmax, int ld, int tri) {
    __shared__ float2 tile[32][33];
    const int tx = threadIdx.x, ty = threadIdx.y;
    const int m0 = blockIdx.x * 32, l = blockIdx.y;
    const int64_t r0 = (int64_t)blockIdx.z * 32;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int mm = ty + 8 * i, m = m0 + mm;
        const int64_t r = r0 + tx;
        float2 v = make_float2(0.f, 0.f);
        if (m < mmax && r < rows && (!tri || m <= l)) v = *reinterpret_cast<const float2*>(spec + ((int64_t)m * lmax + l) * ld + 2 * r);
        tile[mm][tx] = v;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int rr = ty + 8 * i, m = m0 + tx;
        const int64_t r = r0 + rr;
        if (r < rows && m < mmax) coeffs[(r * lmax + l) * mmax + m] = tile[tx][rr];
    }
}

__global__ __launch_bounds__(256) void coeffs_to_spectral_kernel(const float2* __restrict__ coeffs, float* __restrict__ spec, int64_t rows,
                                                                 int lmax, int mmax, int ld, int tri) {
    __shared__ float2 tile[32][33];
    const int tx = threadIdx.x, ty = threadIdx.y;
    const int m0 = blockIdx.x * 32, l = blockIdx.y;
    if (tri && m0 > l) return;          // a tile entirely above the diagonal holds nothing to move
    const int64_t r0 = (int64_t)blockIdx.z * 32;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int rr = ty + 8 * i, m = m0 + tx;
        const int64_t r = r0 + rr;
        float2 v = make_float2(0.f, 0.f);
        // orders above the degree are not moved in triangular mode: do not read them either
        if (r < rows && m < mmax && (!tri || m <= l)) v = coeffs[(r * lmax + l) * mmax + m];
        tile[rr][tx] = v;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int mm = ty + 8 * i, m = m0 + mm;
        const int64_t r = r0 + tx;
        // channel slots between 2*rows and ld are padding: keep them zero
        if (m < mmax && 2 * r < ld && (!tri || m <= l)) {
            float2 v = r < rows ? tile[tx][mm] : make_float2(0.f, 0.f);
            *reinterpret_cast<float2*>(spec + ((int64_t)m * lmax + l) * ld + 2 * r) = v;
        }
    }
}

static bool grid_ok(int64_t rows, int lmax) { return rows > 0 && lmax > 0 && lmax <= 65535 && (rows + 31) / 32 <= 65535; }

int coeffs_to_spectral_launch(const float2* coeffs, float* spec, int64_t rows, int lmax, int mmax, int ld, int tri, hipStream_t s) {
    if (!grid_ok(rows, lmax) || mmax <= 0 || ld < 2 * rows) return SFNO_EINVAL;
    // the z range covers the padded channel slots too (ld/2 >= rows)
    dim3 grid((mmax + 31) / 32, lmax, (unsigned)((ld / 2 + 31) / 32));
    hipLaunchKernelGGL(coeffs_to_spectral_kernel, grid, dim3(32, 8), 0, s, coeffs, spec, rows, lmax, mmax, ld, tri);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int spectral_to_coeffs_launch(const float* spec, float2* coeffs, int64_t rows, int lmax, int mmax, int ld, int tri, hipStream_t s) {
    if (!grid_ok(rows, lmax) || mmax <= 0 || ld < 2 * rows) return SFNO_EINVAL;
    dim3 grid((mmax + 31) / 32, lmax, (unsigned)((rows + 31) / 32));
    hipLaunchKernelGGL(spectral_to_coeffs_kernel, grid, dim3(32, 8), 0, s, spec, coeffs, rows, lmax, mmax, ld, tri);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
