// Layout passes between the reference coefficient layout (complex64 [rows][lmax][mmax],
// m fastest -- what RealSHT.forward returns and InverseRealSHT.forward / the dhconv einsum
// consume, makani/models/common/spectral_convolution.py:131-141) and the order-major
// "spectral" layout float [mmax][lmax][ld] the contraction kernels work on.
#include "sfno_internal.h"

namespace sfno {

// Workgroups are handed to the 8 XCDs round-robin by linear id.  A tile is 32 orders x 32 rows of one degree; its
// 256-byte pieces of the reference layout start wherever (r lmax + l) mmax + m0 falls, so neighbouring order tiles
// share 128-byte lines.  All order tiles of one (degree, row tile) therefore run back to back on one XCD, where
// the shared lines meet in that XCD's L2; degrees go to the XCDs round-robin.
// grid = 8 * mtiles * ceil(lmax/8) * rtiles workgroups, block (32, 8)
__device__ __forceinline__ bool map_tile(int mtiles, int lmax, int& m0, int& l, int64_t& r0) {
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    const int l8 = (lmax + 7) / 8;
    const int t = q / mtiles;
    m0 = (q - t * mtiles) * 32;
    l = (t % l8) * 8 + xcd;
    r0 = (int64_t)(t / l8) * 32;
    return l < lmax;
}

__global__ __launch_bounds__(256) void spectral_to_coeffs_kernel(const float* __restrict__ spec, float2* __restrict__ coeffs, int64_t rows,
                                                                 int lmax, int mmax, int ld, int tri, int mtiles) {
    __shared__ float2 tile[32][33];
    const int tx = threadIdx.x, ty = threadIdx.y;
    int m0, l;
    int64_t r0;
    if (!map_tile(mtiles, lmax, m0, l, r0)) return;
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
                                                                 int lmax, int mmax, int ld, int tri, int mtiles) {
    __shared__ float2 tile[32][33];
    const int tx = threadIdx.x, ty = threadIdx.y;
    int m0, l;
    int64_t r0;
    if (!map_tile(mtiles, lmax, m0, l, r0)) return;
    if (tri && m0 > l) return;          // a tile entirely above the diagonal holds nothing to move
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

// number of workgroups for `rtiles` row tiles, or 0 if the grid does not fit
static unsigned tile_blocks(int lmax, int mmax, int64_t rtiles) {
    if (lmax <= 0 || mmax <= 0 || rtiles <= 0) return 0;
    const int64_t n = 8 * (int64_t)((mmax + 31) / 32) * ((lmax + 7) / 8) * rtiles;
    return n > 0x7fffffffLL ? 0 : (unsigned)n;
}

int coeffs_to_spectral_launch(const float2* coeffs, float* spec, int64_t rows, int lmax, int mmax, int ld, int tri, hipStream_t s) {
    if (rows <= 0 || ld < 2 * rows) return SFNO_EINVAL;
    // the row tiles cover the padded channel slots too (ld/2 >= rows)
    const unsigned blocks = tile_blocks(lmax, mmax, (ld / 2 + 31) / 32);
    if (!blocks) return SFNO_EINVAL;
    hipLaunchKernelGGL(coeffs_to_spectral_kernel, dim3(blocks), dim3(32, 8), 0, s, coeffs, spec, rows, lmax, mmax, ld, tri, (mmax + 31) / 32);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int spectral_to_coeffs_launch(const float* spec, float2* coeffs, int64_t rows, int lmax, int mmax, int ld, int tri, hipStream_t s) {
    if (rows <= 0 || ld < 2 * rows) return SFNO_EINVAL;
    const unsigned blocks = tile_blocks(lmax, mmax, (rows + 31) / 32);
    if (!blocks) return SFNO_EINVAL;
    hipLaunchKernelGGL(spectral_to_coeffs_kernel, dim3(blocks), dim3(32, 8), 0, s, spec, coeffs, rows, lmax, mmax, ld, tri, (mmax + 31) / 32);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
