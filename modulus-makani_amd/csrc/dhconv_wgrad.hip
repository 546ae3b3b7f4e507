// Gradient of the dhconv contraction with respect to its weight:
//     gw[i][o][l] = sum over rows k = (m, b) of conj(x[k][i]) * g[k][o]
// (the backward of einsum("bixy,iox->boxy") at makani/models/common/contractions.py:130-136 with
// respect to `bc`).  Per degree l this is a real GEMM on v_mfma_f32_32x32x2_f32 whose K dimension
// is (k, c), c = re/im of x:
//     D[i][n] = sum_k  X[k][2i] * Bop[(k,0)][n] + X[k][2i+1] * Bop[(k,1)][n],    n = 2o + (re|im of gw)
//     Bop[(k,0)][n] = G[k][n],   Bop[(k,1)][n] = n even ? G[k][n+1] : -G[k][n-1]
// so one MFMA consumes one spectral-layout row of X and of G, and both operands come straight from
// global memory: lanes 0-31 hold c = 0, lanes 32-63 hold c = 1, i.e. the A operand is 64 consecutive
// floats of the row and the B operand 32 floats with neighbouring lanes of the upper half swapped.
#include "sfno_internal.h"

namespace sfno {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int WG_IB = 2;   // 32-row blocks of i per wavefront
constexpr int WG_NB = 4;   // 32-column blocks of n per wavefront
constexpr int WG_TI = 2 * 32 * WG_IB;   // i per workgroup (2 wavefronts along i)
constexpr int WG_TN = 2 * 32 * WG_NB;   // n per workgroup (2 wavefronts along n)
constexpr int WG_UN = 4;   // rows k per loop iteration

struct RowVals {
    float a[WG_UN][WG_IB];
    float b[WG_UN][WG_NB];
};

__global__ __launch_bounds__(256, 2) void dhconv_wgrad_kernel(DhconvWgradArgs p, int ni, int nn) {
    // Workgroups are dealt to the 8 XCDs round-robin by linear id.  The 8 degrees that share a 64-byte
    // line of gw ([i][o][l], l fastest) run as neighbours in one XCD's queue so that their 8-byte stores
    // meet in that XCD's L2; groups of 8 degrees go to the XCDs round-robin, highest degrees (most rows) first.
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    const int tiles = ni * nn;
    const int j8 = q & 7, t = (q >> 3) % tiles, gl = (q >> 3) / tiles;
    const int l = p.L - 1 - ((gl * 8 + xcd) * 8 + j8);
    if (l < 0) return;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int i0 = (t / nn) * WG_TI + (wave >> 1) * 32 * WG_IB;
    const int n0 = (t % nn) * WG_TN + (wave & 1) * 32 * WG_NB;
    const int I2 = 2 * p.I, O2 = 2 * p.O;
    if (i0 >= p.I || n0 >= O2) return;
    const int c = lane >> 5, jj = lane & 31;

    int cola[WG_IB], colb[WG_NB];
    float sgn[WG_NB];
#pragma unroll
    for (int ib = 0; ib < WG_IB; ++ib) cola[ib] = 2 * min(i0 + 32 * ib + jj, p.I - 1) + c;
#pragma unroll
    for (int nb = 0; nb < WG_NB; ++nb) {
        const int n = n0 + 32 * nb + jj;
        colb[nb] = min(n ^ c, O2 - 1);
        sgn[nb] = (c && (n & 1)) ? -1.f : 1.f;
    }

    const int mv = p.tri ? min(l + 1, p.M) : p.M;
    const int nrows = mv * p.B;
    const int64_t mstride_in = (int64_t)p.L * p.ld_in, mstride_out = (int64_t)p.L * p.ld_out;
    const float* __restrict__ X = p.X + (int64_t)l * p.ld_in;
    const float* __restrict__ G = p.G + (int64_t)l * p.ld_out;

    f32x16 acc[WG_IB][WG_NB];
#pragma unroll
    for (int ib = 0; ib < WG_IB; ++ib)
#pragma unroll
        for (int nb = 0; nb < WG_NB; ++nb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[ib][nb][v] = 0.f;

    // rows past the end are clamped to the last row and their A values zeroed
    auto load = [&](int k0, RowVals& r) {
#pragma unroll
        for (int u = 0; u < WG_UN; ++u) {
            const int k = min(k0 + u, nrows - 1);
            const int m = k / p.B, b = k - m * p.B;
            const float* xr = X + m * mstride_in + (int64_t)b * I2;
            const float* gr = G + m * mstride_out + (int64_t)b * O2;
#pragma unroll
            for (int ib = 0; ib < WG_IB; ++ib) r.a[u][ib] = xr[cola[ib]];
#pragma unroll
            for (int nb = 0; nb < WG_NB; ++nb) r.b[u][nb] = gr[colb[nb]];
        }
    };
    auto mac = [&](int k0, const RowVals& r) {
#pragma unroll
        for (int u = 0; u < WG_UN; ++u) {
            const bool live = k0 + u < nrows;
#pragma unroll
            for (int nb = 0; nb < WG_NB; ++nb) {
                const float bv = r.b[u][nb] * sgn[nb];
#pragma unroll
                for (int ib = 0; ib < WG_IB; ++ib)
                    acc[ib][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(live ? r.a[u][ib] : 0.f, bv, acc[ib][nb], 0, 0, 0);
            }
        }
    };

    RowVals cur, nxt;
    load(0, cur);
    for (int k0 = 0; k0 < nrows; k0 += WG_UN) {
        const bool more = k0 + WG_UN < nrows;
        if (more) load(k0 + WG_UN, nxt);
        mac(k0, cur);
        if (more) cur = nxt;
    }

    float* __restrict__ gw = p.GW;
#pragma unroll
    for (int ib = 0; ib < WG_IB; ++ib)
#pragma unroll
        for (int nb = 0; nb < WG_NB; ++nb) {
            const int n = n0 + 32 * nb + jj;
            if (n >= O2) continue;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = i0 + 32 * ib + 8 * (v >> 2) + 4 * c + (v & 3);
                if (i < p.I) gw[(((int64_t)i * p.O + (n >> 1)) * p.L + l) * 2 + (n & 1)] = acc[ib][nb][v];
            }
        }
}

}  // namespace

int dhconv_wgrad_launch(const DhconvWgradArgs& a, hipStream_t s) {
    const int ni = (a.I + WG_TI - 1) / WG_TI, nn = (2 * a.O + WG_TN - 1) / WG_TN;
    const int64_t ngroups = (a.L + 7) / 8;
    const int64_t blocks = 8 * ((ngroups + 7) / 8) * ni * nn * 8;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(dhconv_wgrad_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a, ni, nn);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
