// Packed-operand batched GEMM on fp32 MFMA (v_mfma_f32_32x32x2_f32) for gfx950.
//
// Serves the three contractions of the SFNO spectral path:
//   PG_ANALYSIS  : spec[m][l][n]  = sum_k  W[m][l][k]   * xm[m][k][n]     (RealSHT.forward, Legendre stage)
//   PG_SYNTHESIS : xm[m][k][n]    = sum_l  P[m][l][k]   * spec[m][l][n]   (InverseRealSHT.forward, Legendre stage)
//   PG_DHCONV    : out[m][l][b][o'] = sum_i' in[m][l][b][i'] * W'[l][o'][i']  (contractions.py:130-136 as a real GEMM)
// The constant operand P (table / weight) is read exactly once per (batch, row block) as
// a contiguous stream of pre-swizzled MFMA fragments, straight from HBM into registers.
// The activation operand Q is staged through LDS in K-chunks of 16 and shared by the four
// wavefronts of a workgroup, each of which owns one 32-row block of P and all NT 32-wide
// column tiles of the workgroup's column range.
#include "sfno_internal.h"

namespace sfno {

typedef float floatx16 __attribute__((ext_vector_type(16)));

template <int MODE>
struct BatchGeom {
    int nrows;       // rows of the packed operand in this batch
    int klen;        // contraction length
    int ncols;       // columns of Q
    const float* q;  // Legendre modes: first Q row of the batch
    float* o;        // Legendre modes: first output row of the batch
};

template <int MODE>
__device__ __forceinline__ BatchGeom<MODE> batch_geom(const PgemmArgs& a, int b) {
    BatchGeom<MODE> g;
    if (MODE == PG_ANALYSIS) {
        g.nrows = a.lmax - b;
        g.klen = a.nlat;
        g.ncols = a.ld;
        g.q = a.Q + (int64_t)b * a.nlat * a.ld;
        g.o = a.Out + ((int64_t)b * a.lmax + b) * a.ld;
    } else if (MODE == PG_SYNTHESIS) {
        g.nrows = a.nlat;
        g.klen = a.lmax - b;
        g.ncols = a.ld;
        g.q = a.Q + ((int64_t)b * a.lmax + b) * a.ld;
        g.o = a.Out + (int64_t)b * a.nlat * a.ld;
    } else {
        g.nrows = a.O2;
        g.klen = a.I2;
        int mm = a.tri ? min(b + 1, a.M) : a.M;
        g.ncols = mm * a.B;
        g.q = a.Q;
        g.o = a.Out;
    }
    return g;
}

template <int NT, int MODE>
__global__ __launch_bounds__(256) void pgemm_kernel(PgemmArgs a) {
    constexpr int TN = 32 * NT;
    // Legendre modes store float4 rows (n contiguous); dhconv transposes k-contiguous
    // rows on the way in, an odd row pitch spreads those writes over the banks.
    constexpr int LDQ = (MODE == PG_DHCONV) ? TN + 1 : TN + ((TN % 64 == 0) ? 32 : 0);
    __shared__ __align__(16) float qs[2][PG_KC][LDQ];

    const int2 wi = a.work[blockIdx.x];
    const int b = wi.x;
    if (b < 0) return;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int n0 = blockIdx.y * TN;
    const BatchGeom<MODE> g = batch_geom<MODE>(a, b);
    if (n0 >= g.ncols) return;

    const int nrb = (g.nrows + PG_ROWS - 1) / PG_ROWS;
    const int nc = (g.klen + PG_KC - 1) / PG_KC;
    const int rb = wi.y + wave;
    const bool active = rb < nrb;
    const int tiles = min(NT, (g.ncols - n0 + 31) / 32);   // column tiles with any valid column

    const float4* ap = reinterpret_cast<const float4*>(a.A) + ((a.a_off[b] + (int64_t)(active ? rb : 0) * nc) * 128 + lane);

    floatx16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.0f;

    // ---- Q staging -------------------------------------------------------------------------
    constexpr int QV = (MODE == PG_DHCONV) ? NT : (NT + 1) / 2;   // vector loads per thread per chunk
    float4 qreg4[(MODE == PG_DHCONV) ? 1 : QV];
    float2 qreg2[(MODE == PG_DHCONV) ? QV : 1];

    auto q_load = [&](int c) {
        const int k0 = c * PG_KC;
        if (MODE == PG_DHCONV) {
#pragma unroll
            for (int u = 0; u < QV; ++u) {
                int e = tid + 256 * u;
                int kp = e & 7, col = e >> 3;
                int k = k0 + 2 * kp, n = n0 + col;
                float2 v = make_float2(0.f, 0.f);
                if (n < g.ncols && k < g.klen) {
                    int mm = n / a.B, bb = n - mm * a.B;
                    const float* src = g.q + ((int64_t)mm * a.L + b) * a.ld_in + (int64_t)bb * a.I2 + k;
                    v = *reinterpret_cast<const float2*>(src);
                }
                qreg2[u] = v;
            }
        } else {
#pragma unroll
            for (int u = 0; u < QV; ++u) {
                int e = tid + 256 * u;
                int row = e / (TN / 4), c4 = e - row * (TN / 4);
                int k = k0 + row, n = n0 + 4 * c4;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (e < 4 * TN && k < g.klen && n < g.ncols) v = *reinterpret_cast<const float4*>(g.q + (int64_t)k * a.ld + n);
                qreg4[u] = v;
            }
        }
    };
    auto q_store = [&](int buf) {
        if (MODE == PG_DHCONV) {
#pragma unroll
            for (int u = 0; u < QV; ++u) {
                int e = tid + 256 * u;
                int kp = e & 7, col = e >> 3;
                qs[buf][2 * kp][col] = qreg2[u].x;
                qs[buf][2 * kp + 1][col] = qreg2[u].y;
            }
        } else {
#pragma unroll
            for (int u = 0; u < QV; ++u) {
                int e = tid + 256 * u;
                int row = e / (TN / 4), c4 = e - row * (TN / 4);
                if (e < 4 * TN) *reinterpret_cast<float4*>(&qs[buf][row][4 * c4]) = qreg4[u];
            }
        }
    };

    float4 acur[2], anext[2];
    q_load(0);
    if (active && nc > 0) {
        acur[0] = ap[0];
        acur[1] = ap[64];
    }
    q_store(0);
    __syncthreads();

    const int kh = lane >> 5, cl = lane & 31;
    for (int c = 0; c < nc; ++c) {
        const int buf = c & 1;
        const bool more = c + 1 < nc;
        if (more) {
            q_load(c + 1);
            if (active) {
                anext[0] = ap[(int64_t)(c + 1) * 128];
                anext[1] = ap[(int64_t)(c + 1) * 128 + 64];
            }
        }
        if (active) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float af[4] = {acur[h].x, acur[h].y, acur[h].z, acur[h].w};
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const float* qrow = &qs[buf][8 * h + 2 * s + kh][cl];
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        if (t < tiles) {
                            float qv = qrow[32 * t];
                            if (MODE == PG_DHCONV)
                                acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(qv, af[s], acc[t], 0, 0, 0);
                            else
                                acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[s], qv, acc[t], 0, 0, 0);
                        }
                    }
                }
            }
        }
        if (more) q_store(buf ^ 1);
        __syncthreads();
        acur[0] = anext[0];
        acur[1] = anext[1];
    }

    if (!active) return;
    // ---- epilogue ------------------------------------------------------------------------------
    // D layout of the 32x32 MFMA: register v of lane j holds D[8*(v/4) + 4*(j/32) + v%4][j%32].
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        if (t >= tiles) continue;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int di = 8 * (v >> 2) + 4 * kh + (v & 3);
            if (MODE == PG_DHCONV) {
                // D rows = Q columns (order m, batch b), D cols = packed rows (output channel o')
                int n = n0 + 32 * t + di, oc = PG_ROWS * rb + cl;
                if (n < g.ncols && oc < g.nrows) {
                    int mm = n / a.B, bb = n - mm * a.B;
                    g.o[((int64_t)mm * a.L + b) * a.ld_out + (int64_t)bb * a.O2 + oc] = acc[t][v];
                }
            } else {
                int r = PG_ROWS * rb + di, n = n0 + 32 * t + cl;
                if (r < g.nrows && n < g.ncols) g.o[(int64_t)r * a.ld + n] = acc[t][v];
            }
        }
    }
}

template <int MODE>
static int launch_mode(const PgemmArgs& a, int n_work, int64_t ncols, hipStream_t s) {
    if (n_work <= 0 || ncols <= 0) return SFNO_OK;
    // widest column tile that wastes the fewest padded columns; wide tiles re-read P least
    static const int cand[] = {6, 5, 4, 8, 3, 2, 1};
    int best = 1;
    int64_t best_pad = INT64_MAX;
    for (int nt : cand) {
        if (MODE == PG_DHCONV && nt != 8 && ncols > 32 * nt) continue;
        int64_t pad = (ncols + 32 * nt - 1) / (32 * nt) * (32 * nt);
        if (pad < best_pad) { best_pad = pad; best = nt; }
    }
    dim3 block(256);
#define PG_CASE(NT_)                                                                        \
    case NT_: {                                                                             \
        dim3 grid(n_work, (unsigned)((ncols + 32 * NT_ - 1) / (32 * NT_)));                 \
        hipLaunchKernelGGL((pgemm_kernel<NT_, MODE>), grid, block, 0, s, a);                \
        break;                                                                              \
    }
    switch (best) {
        PG_CASE(1) PG_CASE(2) PG_CASE(3) PG_CASE(4) PG_CASE(5) PG_CASE(6) PG_CASE(8)
        default: return SFNO_EINVAL;
    }
#undef PG_CASE
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int pgemm_launch(int mode, const PgemmArgs& a, int n_work, int64_t ncols_max, hipStream_t s) {
    switch (mode) {
        case PG_ANALYSIS: return launch_mode<PG_ANALYSIS>(a, n_work, ncols_max, s);
        case PG_SYNTHESIS: return launch_mode<PG_SYNTHESIS>(a, n_work, ncols_max, s);
        case PG_DHCONV: return launch_mode<PG_DHCONV>(a, n_work, ncols_max, s);
    }
    return SFNO_EINVAL;
}

}  // namespace sfno
