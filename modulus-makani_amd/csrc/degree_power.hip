// Per-degree power of spherical harmonic coefficients held in the spectral layout float [mmax][lmax][ld]
// ((re, im) of channel row r at 2r, 2r+1; only entries with l >= m exist):
//     power[r][l] = |c[r,l,0]|^2 + 2 sum_{0 < m <= min(l, mmax-1)} |c[r,l,m]|^2
// This is what GeometricH1Loss reduces its transform output to before weighting the degrees with l(l+1)
// (makani/utils/losses.py:301-305 and 320-331), computed here straight from the output of the Legendre analysis,
// without the pass to the reference coefficient layout.  The gradient kernel writes the spectral-layout cotangent
// the adjoint analysis consumes.  Both are bound by the one pass over the coefficients.
#include "sfno_internal.h"

namespace sfno {
namespace {

constexpr int DP_R = 64;    // channel rows per workgroup (consecutive threads: consecutive 8-byte elements)
constexpr int DP_M = 4;     // orders summed in parallel

// grid (lmax, ceil(rows / DP_R)), block (DP_R, DP_M)
__global__ __launch_bounds__(DP_R * DP_M) void degree_power_kernel(const float* __restrict__ spec, float* __restrict__ power, int64_t rows, int lmax,
                                                                  int mmax, int ld) {
    __shared__ float part[DP_M][DP_R];
    const int l = blockIdx.x;
    const int64_t r = (int64_t)blockIdx.y * DP_R + threadIdx.x;
    const int mtop = min(l, mmax - 1);
    float acc = 0.f;
    if (r < rows) {
        for (int m = threadIdx.y; m <= mtop; m += DP_M) {
            const float2 c = *reinterpret_cast<const float2*>(spec + ((int64_t)m * lmax + l) * ld + 2 * r);
            const float p = fmaf(c.x, c.x, c.y * c.y);
            acc += m == 0 ? p : 2.f * p;
        }
    }
    part[threadIdx.y][threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.y == 0 && r < rows) {
        float s = part[0][threadIdx.x];
#pragma unroll
        for (int j = 1; j < DP_M; ++j) s += part[j][threadIdx.x];
        power[r * lmax + l] = s;
    }
}

// gspec[m][l][2r..2r+1] = w_m * 2 * gpower[r][l] * c[r,l,m]  (w_0 = 1, w_m = 2 otherwise); padding columns zero
// grid (lmax, ceil((ld/2) / DP_R)), block (DP_R, DP_M)
__global__ __launch_bounds__(DP_R * DP_M) void degree_power_grad_kernel(const float* __restrict__ spec, const float* __restrict__ gpower,
                                                                       float* __restrict__ gspec, int64_t rows, int lmax, int mmax, int ld) {
    const int l = blockIdx.x;
    const int64_t r = (int64_t)blockIdx.y * DP_R + threadIdx.x;
    if (2 * r >= ld) return;
    const int mtop = min(l, mmax - 1);
    const float g = r < rows ? 2.f * gpower[r * lmax + l] : 0.f;
    for (int m = threadIdx.y; m <= mtop; m += DP_M) {
        const int64_t at = ((int64_t)m * lmax + l) * ld + 2 * r;
        float2 o = make_float2(0.f, 0.f);
        if (r < rows) {
            const float2 c = *reinterpret_cast<const float2*>(spec + at);
            const float w = m == 0 ? g : 2.f * g;
            o = make_float2(w * c.x, w * c.y);
        }
        *reinterpret_cast<float2*>(gspec + at) = o;
    }
}

}  // namespace

int degree_power_launch(const float* spec, float* power, int64_t rows, int lmax, int mmax, int ld, hipStream_t s) {
    if (rows < 1 || lmax < 1 || mmax < 1 || ld < 2 * rows || (rows + DP_R - 1) / DP_R > 65535) return SFNO_EINVAL;
    hipLaunchKernelGGL(degree_power_kernel, dim3(lmax, (unsigned)((rows + DP_R - 1) / DP_R)), dim3(DP_R, DP_M), 0, s, spec, power, rows, lmax, mmax, ld);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int degree_power_grad_launch(const float* spec, const float* gpower, float* gspec, int64_t rows, int lmax, int mmax, int ld, hipStream_t s) {
    if (rows < 1 || lmax < 1 || mmax < 1 || ld < 2 * rows || (ld / 2 + DP_R - 1) / DP_R > 65535) return SFNO_EINVAL;
    hipLaunchKernelGGL(degree_power_grad_kernel, dim3(lmax, (unsigned)((ld / 2 + DP_R - 1) / DP_R)), dim3(DP_R, DP_M), 0, s, spec, gpower, gspec, rows,
                       lmax, mmax, ld);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
