// Gradient of the dhconv contraction with respect to its weight:
//     gw[i][o][l] = sum over rows k = (m, b) of conj(x[k][i]) * g[k][o]
// (the backward of einsum("bixy,iox->boxy") at makani/models/common/contractions.py:130-136 with
// respect to `bc`).  Per degree l this is four real GEMMs on v_mfma_f32_32x32x2_f32,
//     Re gw = Xr^T Gr + Xi^T Gi,      Im gw = Xr^T Gi - Xi^T Gr,
// whose K dimension is the rows k of the spectral layout.  Both operands come straight from global
// memory as (re, im) pairs: lanes 0-31 read row k and lanes 32-63 row k + 1, so one 8-byte load per
// lane feeds the k = 0 and k = 1 slices of an operand for 32 channels, and its two registers are
// the real-part operand and the imaginary-part operand.
//
// A workgroup is 8 wavefronts = the 8 degrees that share 64-byte lines of gw ([i][o][l], l fastest),
// all on the same 64 x 64 tile of (i, o).  The results meet in LDS and leave as whole lines.
#include "sfno_internal.h"

namespace sfno {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int WG_IB = 2;             // 32-channel blocks of i per wavefront
constexpr int WG_OB = 2;             // 32-channel blocks of o per wavefront
constexpr int WG_TI = 32 * WG_IB;    // i per workgroup
constexpr int WG_TO = 32 * WG_OB;    // o per workgroup
constexpr int WG_DEG = 8;            // degrees (wavefronts) per workgroup
constexpr int WG_UN = 4;             // row pairs per loop iteration
constexpr int WG_PITCH = WG_DEG + 1; // float2 per staged line of gw; odd so that the 32 lanes of a store hit 32 banks pairs

struct RowVals {
    float2 a[WG_UN][WG_IB];
    float2 b[WG_UN][WG_OB];
};

__global__ __launch_bounds__(64 * WG_DEG, 1) void dhconv_wgrad_kernel(DhconvWgradArgs p, int ni, int no) {
    __shared__ float2 stage[32 * WG_TO * WG_PITCH];

    // Workgroups are dealt to the 8 XCDs round-robin by linear id.  All tiles of one group of 8 degrees run
    // as neighbours in one XCD's queue, where they share the rows of X and G in that XCD's L2.  The groups go
    // to the XCDs highest degrees (most rows) first, in alternating direction round by round: the work of a
    // group grows linearly with its degree, and dealing every round in the same direction would give the
    // first XCD a quarter more rows than the average.
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    const int tiles = ni * no;
    const int t = q % tiles, gl = q / tiles;
    const int lg = (p.L + WG_DEG - 1) / WG_DEG - 1 - (gl * 8 + ((gl & 1) ? 7 - xcd : xcd));
    if (lg < 0) return;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int l = lg * WG_DEG + wave;
    const int i0 = (t / no) * WG_TI, o0 = (t % no) * WG_TO;
    const int I2 = 2 * p.I, O2 = 2 * p.O;
    const int h = lane >> 5, jj = lane & 31;

    int cola[WG_IB], colb[WG_OB];
#pragma unroll
    for (int ib = 0; ib < WG_IB; ++ib) cola[ib] = 2 * min(i0 + 32 * ib + jj, p.I - 1);
#pragma unroll
    for (int ob = 0; ob < WG_OB; ++ob) colb[ob] = 2 * min(o0 + 32 * ob + jj, p.O - 1);

    // a wavefront whose degree does not exist (last group when L is not a multiple of 8) has no rows
    const int nrows = l < p.L ? (p.tri ? min(l + 1, p.M) : p.M) * p.B : 0;
    const int64_t mstride_in = (int64_t)p.L * p.ld_in, mstride_out = (int64_t)p.L * p.ld_out;
    const float* __restrict__ X = p.X + (int64_t)min(l, p.L - 1) * p.ld_in;
    const float* __restrict__ G = p.G + (int64_t)min(l, p.L - 1) * p.ld_out;

    f32x16 re[WG_IB][WG_OB], im[WG_IB][WG_OB];
#pragma unroll
    for (int ib = 0; ib < WG_IB; ++ib)
#pragma unroll
        for (int ob = 0; ob < WG_OB; ++ob)
#pragma unroll
            for (int v = 0; v < 16; ++v) re[ib][ob][v] = im[ib][ob][v] = 0.f;

    // rows past the end are clamped to the last row and their X values zeroed
    auto load = [&](int k0, RowVals& r) {
#pragma unroll
        for (int u = 0; u < WG_UN; ++u) {
            const int k = min(k0 + 2 * u + h, nrows - 1);
            const int m = k / p.B, b = k - m * p.B;
            const float* xr = X + m * mstride_in + (int64_t)b * I2;
            const float* gr = G + m * mstride_out + (int64_t)b * O2;
#pragma unroll
            for (int ib = 0; ib < WG_IB; ++ib) r.a[u][ib] = *reinterpret_cast<const float2*>(xr + cola[ib]);
#pragma unroll
            for (int ob = 0; ob < WG_OB; ++ob) r.b[u][ob] = *reinterpret_cast<const float2*>(gr + colb[ob]);
        }
    };
    auto mac = [&](int k0, const RowVals& r) {
#pragma unroll
        for (int u = 0; u < WG_UN; ++u) {
            const unsigned live = k0 + 2 * u + h < nrows ? 0xffffffffu : 0u;
            float xr[WG_IB], xi[WG_IB], nxi[WG_IB];
#pragma unroll
            for (int ib = 0; ib < WG_IB; ++ib) {
                xr[ib] = __uint_as_float(__float_as_uint(r.a[u][ib].x) & live);
                xi[ib] = __uint_as_float(__float_as_uint(r.a[u][ib].y) & live);
                nxi[ib] = -xi[ib];
            }
            // two passes so that the two updates of one accumulator are 8 instructions apart
#pragma unroll
            for (int ob = 0; ob < WG_OB; ++ob)
#pragma unroll
                for (int ib = 0; ib < WG_IB; ++ib) {
                    re[ib][ob] = __builtin_amdgcn_mfma_f32_32x32x2f32(xr[ib], r.b[u][ob].x, re[ib][ob], 0, 0, 0);
                    im[ib][ob] = __builtin_amdgcn_mfma_f32_32x32x2f32(xr[ib], r.b[u][ob].y, im[ib][ob], 0, 0, 0);
                }
#pragma unroll
            for (int ob = 0; ob < WG_OB; ++ob)
#pragma unroll
                for (int ib = 0; ib < WG_IB; ++ib) {
                    re[ib][ob] = __builtin_amdgcn_mfma_f32_32x32x2f32(xi[ib], r.b[u][ob].y, re[ib][ob], 0, 0, 0);
                    im[ib][ob] = __builtin_amdgcn_mfma_f32_32x32x2f32(nxi[ib], r.b[u][ob].x, im[ib][ob], 0, 0, 0);
                }
        }
    };

    // the loads run one iteration ahead of the matrix instructions, into two register sets that swap roles
    if (nrows > 0) {
        constexpr int STEP = 2 * WG_UN;
        RowVals r0, r1;
        load(0, r0);
        for (int k0 = 0;;) {
            if (k0 + STEP < nrows) load(k0 + STEP, r1);
            mac(k0, r0);
            if ((k0 += STEP) >= nrows) break;
            if (k0 + STEP < nrows) load(k0 + STEP, r0);
            mac(k0, r1);
            if ((k0 += STEP) >= nrows) break;
        }
    }

    // The 8 wavefronts hold the same (i, o) tile for 8 consecutive degrees: one block of 32 i at a time they
    // write it to LDS as [i][o][degree], and the workgroup stores it as the 64-byte lines of gw.
    float2* __restrict__ gw = reinterpret_cast<float2*>(p.GW);
#pragma unroll
    for (int ib = 0; ib < WG_IB; ++ib) {
        if (ib) __syncthreads();
#pragma unroll
        for (int ob = 0; ob < WG_OB; ++ob)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int il = 8 * (v >> 2) + 4 * h + (v & 3), ol = 32 * ob + jj;
                stage[(il * WG_TO + ol) * WG_PITCH + wave] = make_float2(re[ib][ob][v], im[ib][ob][v]);
            }
        __syncthreads();
#pragma unroll 4
        for (int e = threadIdx.x; e < 32 * WG_TO * WG_DEG; e += 64 * WG_DEG) {
            const int line = e >> 3, d = e & 7;
            const int i = i0 + 32 * ib + (line >> 6), o = o0 + (line & (WG_TO - 1)), ll = lg * WG_DEG + d;
            if (i < p.I && o < p.O && ll < p.L) gw[((int64_t)i * p.O + o) * p.L + ll] = stage[line * WG_PITCH + d];
        }
    }
}

}  // namespace

int dhconv_wgrad_launch(const DhconvWgradArgs& a, hipStream_t s) {
    const int ni = (a.I + WG_TI - 1) / WG_TI, no = (a.O + WG_TO - 1) / WG_TO;
    const int64_t ngroups = (a.L + WG_DEG - 1) / WG_DEG;
    const int64_t blocks = 8 * ((ngroups + 7) / 8) * ni * no;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(dhconv_wgrad_kernel, dim3((unsigned)blocks), dim3(64 * WG_DEG), 0, s, a, ni, no);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
