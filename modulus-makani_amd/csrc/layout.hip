// Layout passes between the reference coefficient layout (complex64 [rows][lmax][mmax],
// m fastest -- what RealSHT.forward returns and InverseRealSHT.forward / the dhconv einsum
// consume, makani/models/common/spectral_convolution.py:131-141) and the order-major
// "spectral" layout float [mmax][lmax][ld] the contraction kernels work on.
#include "sfno_internal.h"

namespace sfno {

// A tile is 64 orders x 80 complex rows of one degree: on the order-major side 64 pieces of up to 640 contiguous bytes
// (the whole padded row for up to 80 channels), on the reference side 80 runs of 512 contiguous bytes, which start
// wherever (r lmax + l) mmax + m0 falls, so neighbouring order tiles share 128-byte lines.  Workgroups are handed to the
// 8 XCDs round-robin by linear id: all order tiles of one (degree, row tile) run back to back on one XCD, where the
// shared lines meet in that XCD's L2; degrees go to the XCDs round-robin.  Every global load of a tile is issued
// before its first LDS store.
// grid = 8 * mtiles * ceil(lmax/8) * rtiles workgroups of 256 threads
constexpr int LT_M = 64;                    // orders per tile
constexpr int LT_R = 80;                    // complex rows per tile
constexpr int LT_Q = LT_R / 2;              // groups of four floats per order
constexpr int LT_PITCH = 2 * LT_R + 2;      // floats per order in LDS: a wavefront's 8-byte accesses along the orders spread over all banks
constexpr int LT_T = 256;
constexpr int LT_ITQ = LT_M * LT_Q / LT_T;  // 10 groups of four per thread
constexpr int LT_ITR = LT_M * LT_R / LT_T;  // 20 complex values per thread
static_assert(LT_M * LT_Q % LT_T == 0 && LT_M * LT_R % LT_T == 0, "the tile divides evenly among the threads");

struct LayoutTile {
    int m0, l, r0;          // first order, degree, first row
    int nr;                 // rows of the tensor in this tile (the reference side)
    int nq;                 // groups of four floats per order that lie inside ld (the order-major side)
    int mcount, mdata;      // orders inside mmax; of those, the ones that carry data (m <= l in triangular mode)
};

__device__ __forceinline__ bool map_tile(int mtiles, int64_t rows, int lmax, int mmax, int ld, int tri, LayoutTile& t) {
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    const int l8 = (lmax + 7) / 8;
    const int u = q / mtiles;
    t.m0 = (q - u * mtiles) * LT_M;
    t.l = (u % l8) * 8 + xcd;
    t.r0 = (u / l8) * LT_R;
    if (t.l >= lmax) return false;
    const int64_t left = rows - t.r0;
    t.nr = left < 0 ? 0 : left < LT_R ? (int)left : LT_R;
    const int fl = ld - 2 * t.r0;           // a multiple of four: ld is a multiple of 16, r0 of 80
    t.nq = fl < 2 * LT_R ? fl / 4 : LT_Q;
    t.mcount = mmax - t.m0 < LT_M ? mmax - t.m0 : LT_M;
    const int below = t.l - t.m0 + 1;
    t.mdata = !tri ? t.mcount : below < 0 ? 0 : below < t.mcount ? below : t.mcount;
    return true;
}

__global__ __launch_bounds__(LT_T) void spectral_to_coeffs_kernel(const float* __restrict__ spec, float2* __restrict__ coeffs, int64_t rows, int lmax,
                                                                  int mmax, int ld, int tri, int mtiles) {
    __shared__ __align__(16) float tile[LT_M * LT_PITCH];
    const int tid = threadIdx.x;
    LayoutTile t;
    if (!map_tile(mtiles, rows, lmax, mmax, ld, tri, t)) return;
    if (t.mdata > 0) {                      // (uniform over the workgroup) a tile above the diagonal is zeros: nothing to read
        float4 v[LT_ITQ];
#pragma unroll
        for (int it = 0; it < LT_ITQ; ++it) {
            const int idx = tid + it * LT_T, mm = idx / LT_Q, qd = idx - mm * LT_Q;
            v[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (mm < t.mdata && qd < t.nq) v[it] = *reinterpret_cast<const float4*>(spec + ((int64_t)(t.m0 + mm) * lmax + t.l) * ld + 2 * t.r0 + 4 * qd);
        }
#pragma unroll
        for (int it = 0; it < LT_ITQ; ++it) {
            const int idx = tid + it * LT_T, mm = idx / LT_Q, qd = idx - mm * LT_Q;
            float2* dst = reinterpret_cast<float2*>(tile + mm * LT_PITCH + 4 * qd);
            dst[0] = make_float2(v[it].x, v[it].y);
            dst[1] = make_float2(v[it].z, v[it].w);
        }
        __syncthreads();
    }
    const int mm = tid & (LT_M - 1);
    if (mm >= t.mcount) return;
    const bool data = mm < t.mdata;
    float2* dst = coeffs + ((int64_t)t.r0 * lmax + t.l) * mmax + t.m0 + mm;
    const float* src = tile + mm * LT_PITCH;
#pragma unroll 4
    for (int r = tid / LT_M; r < t.nr; r += LT_T / LT_M) {
        float2 v = make_float2(0.f, 0.f);
        if (data) v = *reinterpret_cast<const float2*>(src + 2 * r);
        dst[(int64_t)r * lmax * mmax] = v;
    }
}

__global__ __launch_bounds__(LT_T) void coeffs_to_spectral_kernel(const float2* __restrict__ coeffs, float* __restrict__ spec, int64_t rows, int lmax,
                                                                  int mmax, int ld, int tri, int mtiles) {
    __shared__ __align__(16) float tile[LT_M * LT_PITCH];
    const int tid = threadIdx.x;
    LayoutTile t;
    if (!map_tile(mtiles, rows, lmax, mmax, ld, tri, t)) return;
    if (t.mdata <= 0) return;               // orders above the degree are not moved in triangular mode: nothing to read or write
    {
        const int mm = tid & (LT_M - 1);
        const bool in = mm < t.mdata;
        const float2* src = coeffs + ((int64_t)t.r0 * lmax + t.l) * mmax + t.m0 + mm;
        float2 v[LT_ITR];
#pragma unroll
        for (int it = 0; it < LT_ITR; ++it) {
            const int r = tid / LT_M + it * (LT_T / LT_M);
            // row slots between the tensor's rows and ld / 2 are padding: they are written as zeros
            v[it] = make_float2(0.f, 0.f);
            if (in && r < t.nr) v[it] = src[(int64_t)r * lmax * mmax];
        }
#pragma unroll
        for (int it = 0; it < LT_ITR; ++it) {
            const int r = tid / LT_M + it * (LT_T / LT_M);
            *reinterpret_cast<float2*>(tile + mm * LT_PITCH + 2 * r) = v[it];
        }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < LT_ITQ; ++it) {
        const int idx = tid + it * LT_T, mm = idx / LT_Q, qd = idx - mm * LT_Q;
        if (mm < t.mdata && qd < t.nq) {
            const float2* src = reinterpret_cast<const float2*>(tile + mm * LT_PITCH + 4 * qd);
            const float2 a = src[0], b = src[1];
            *reinterpret_cast<float4*>(spec + ((int64_t)(t.m0 + mm) * lmax + t.l) * ld + 2 * t.r0 + 4 * qd) = make_float4(a.x, a.y, b.x, b.y);
        }
    }
}

// number of workgroups for `rtiles` row tiles, or 0 if the grid does not fit
static unsigned tile_blocks(int lmax, int mmax, int64_t rtiles) {
    if (lmax <= 0 || mmax <= 0 || rtiles <= 0) return 0;
    const int64_t n = 8 * (int64_t)((mmax + LT_M - 1) / LT_M) * ((lmax + 7) / 8) * rtiles;
    return n > 0x7fffffffLL ? 0 : (unsigned)n;
}

int coeffs_to_spectral_launch(const float2* coeffs, float* spec, int64_t rows, int lmax, int mmax, int ld, int tri, hipStream_t s) {
    if (rows <= 0 || ld < 2 * rows || ld % 16) return SFNO_EINVAL;
    // the row tiles cover the padded channel slots too (ld/2 >= rows)
    const unsigned blocks = tile_blocks(lmax, mmax, (ld / 2 + LT_R - 1) / LT_R);
    if (!blocks) return SFNO_EINVAL;
    hipLaunchKernelGGL(coeffs_to_spectral_kernel, dim3(blocks), dim3(LT_T), 0, s, coeffs, spec, rows, lmax, mmax, ld, tri, (mmax + LT_M - 1) / LT_M);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int spectral_to_coeffs_launch(const float* spec, float2* coeffs, int64_t rows, int lmax, int mmax, int ld, int tri, hipStream_t s) {
    if (rows <= 0 || ld < 2 * rows || ld % 16) return SFNO_EINVAL;
    const unsigned blocks = tile_blocks(lmax, mmax, (rows + LT_R - 1) / LT_R);
    if (!blocks) return SFNO_EINVAL;
    hipLaunchKernelGGL(spectral_to_coeffs_kernel, dim3(blocks), dim3(LT_T), 0, s, spec, coeffs, rows, lmax, mmax, ld, tri, (mmax + LT_M - 1) / LT_M);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
