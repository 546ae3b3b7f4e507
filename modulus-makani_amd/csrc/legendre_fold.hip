// Equator-folded Legendre contractions on fp32 MFMA (v_mfma_f32_32x32x2_f32), gfx950.
//
//   analysis : spec[m][l][n] = sum_k W[m][l][k] xm[m][k][n]     (RealSHT.forward, Legendre stage)
//   synthesis: xm[m][k][n]   = sum_l P[m][l][k] spec[m][l][n]   (InverseRealSHT.forward, Legendre stage)
//
// All supported latitude grids are symmetric about the equator and
// Pbar_l^m(pi - theta) = (-1)^(l+m) Pbar_l^m(theta).  With k' = nlat-1-k and K2 = ceil(nlat/2):
//   analysis : c[l] = sum_{k<K2} W[l][k] (X[k] + (-1)^(l+m) X[k'])      -> half the MACs per coefficient
//   synthesis: X[k] = E[k] + O[k], X[k'] = E[k] - O[k],  E/O = sum over l of even/odd l+m of P[l][k] c[l]
// A workgroup has four wavefronts = 2 parities x 2 row blocks of 32.  Per K-chunk of 16 it
// stages two 16-row panels in LDS (analysis: sums and differences of mirrored latitude rows;
// synthesis: even- and odd-parity degree rows), each wavefront streams its own pre-swizzled
// table fragments from HBM (see sfno_internal.h) and owns all NT 32-wide column tiles.
#include "sfno_internal.h"

namespace sfno {

typedef float floatx16 __attribute__((ext_vector_type(16)));

template <int NT, bool ANALYSIS>
__global__ __launch_bounds__(256) void legendre_fold_kernel(PgemmArgs a) {
    constexpr int TN = 32 * NT;
    constexpr int LDQ = TN + ((TN % 64 == 0) ? 32 : 0);
    // [buffer][parity][k][column]; reused for the parity exchange of the synthesis epilogue
    __shared__ __align__(16) float qs[2][2][PG_KC][LDQ];

    const int2 wi = a.work[blockIdx.x];
    const int m = wi.x;
    if (m < 0) return;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int par = wave >> 1, rb = wi.y + (wave & 1);
    const int n0 = blockIdx.y * TN;
    const int ld = a.ld, nlat = a.nlat, lmax = a.lmax;
    if (n0 >= ld) return;
    const int K2 = (nlat + 1) >> 1;
    const int nl0 = (lmax - m > 0) ? (lmax - m + 1) >> 1 : 0;          // degrees of parity 0: l = m, m+2, ...
    const int nl1 = (lmax - m - 1 > 0) ? (lmax - m) >> 1 : 0;          // parity 1: l = m+1, m+3, ...
    const int nlp = par ? nl1 : nl0;

    const int nrows = ANALYSIS ? nlp : K2;
    const int nrb = (nrows + PG_ROWS - 1) / PG_ROWS;
    const int nc = ANALYSIS ? (K2 + PG_KC - 1) / PG_KC : (nl0 + PG_KC - 1) / PG_KC;
    const bool active = rb < nrb;
    const int tiles = min(NT, (ld - n0 + 31) / 32);

    const float* xm_m = (ANALYSIS ? a.Q : a.Out) + (int64_t)m * nlat * ld;     // Fourier panel of order m
    const float* sp_m = (ANALYSIS ? a.Out : a.Q) + (int64_t)m * lmax * ld;     // spectral panel of order m
    const float4* ap = reinterpret_cast<const float4*>(a.A) + ((a.a_off[2 * m + par] + (int64_t)(active ? rb : 0) * nc) * 128 + lane);

    floatx16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.0f;

    constexpr int QV = (NT + 1) / 2;       // float4 per thread per 16-row panel
    float4 q0[QV], q1[QV];

    auto q_load = [&](int c) {
#pragma unroll
        for (int u = 0; u < QV; ++u) {
            const int e = tid + 256 * u;
            const int row = e / (TN / 4), c4 = e - row * (TN / 4);
            const int i = c * PG_KC + row, n = n0 + 4 * c4;
            float4 v0 = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
            if (e < 4 * TN && n < ld) {
                if (ANALYSIS) {
                    // i = latitude k; panel 0 = X[k] + X[k'], panel 1 = X[k] - X[k']
                    if (i < K2) {
                        const int kk = nlat - 1 - i;
                        const float4 x0 = *reinterpret_cast<const float4*>(xm_m + (int64_t)i * ld + n);
                        if (kk != i) {
                            const float4 x1 = *reinterpret_cast<const float4*>(xm_m + (int64_t)kk * ld + n);
                            v0 = make_float4(x0.x + x1.x, x0.y + x1.y, x0.z + x1.z, x0.w + x1.w);
                            v1 = make_float4(x0.x - x1.x, x0.y - x1.y, x0.z - x1.z, x0.w - x1.w);
                        } else {
                            v0 = x0;                      // the equator row is its own mirror image
                        }
                    }
                } else {
                    // i = index within a parity; panel 0 = degree m+2i, panel 1 = degree m+2i+1
                    const int l0 = m + 2 * i;
                    if (l0 < lmax) v0 = *reinterpret_cast<const float4*>(sp_m + (int64_t)l0 * ld + n);
                    if (l0 + 1 < lmax) v1 = *reinterpret_cast<const float4*>(sp_m + (int64_t)(l0 + 1) * ld + n);
                }
            }
            q0[u] = v0;
            q1[u] = v1;
        }
    };
    auto q_store = [&](int buf) {
#pragma unroll
        for (int u = 0; u < QV; ++u) {
            const int e = tid + 256 * u;
            const int row = e / (TN / 4), c4 = e - row * (TN / 4);
            if (e < 4 * TN) {
                *reinterpret_cast<float4*>(&qs[buf][0][row][4 * c4]) = q0[u];
                *reinterpret_cast<float4*>(&qs[buf][1][row][4 * c4]) = q1[u];
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
                    const float* qrow = &qs[buf][par][8 * h + 2 * s + kh][cl];
#pragma unroll
                    for (int t = 0; t < NT; ++t)
                        if (t < tiles) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[s], qrow[32 * t], acc[t], 0, 0, 0);
                }
            }
        }
        if (more) q_store(buf ^ 1);
        __syncthreads();
        acur[0] = anext[0];
        acur[1] = anext[1];
    }

    // D layout of the 32x32 MFMA: register v of lane j holds D[8*(v/4) + 4*(j/32) + v%4][j%32].
    if (ANALYSIS) {
        if (!active) return;
        float* out = a.Out + (int64_t)m * lmax * ld;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (t >= tiles) continue;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = PG_ROWS * rb + 8 * (v >> 2) + 4 * kh + (v & 3);
                const int n = n0 + 32 * t + cl;
                if (r < nrows && n < ld) out[(int64_t)(m + par + 2 * r) * ld + n] = acc[t][v];
            }
        }
    } else {
        // odd-parity wavefronts hand their sums to the even-parity wavefront of the same row block
        float* exch = &qs[0][0][0][0] + (wave & 1) * (NT * 16 * 64);
        if (par == 1 && active) {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int v = 0; v < 16; ++v) exch[(t * 16 + v) * 64 + lane] = acc[t][v];
        }
        __syncthreads();
        if (par == 0 && active) {
            float* out = a.Out + (int64_t)m * nlat * ld;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if (t >= tiles) continue;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int k = PG_ROWS * rb + 8 * (v >> 2) + 4 * kh + (v & 3);
                    const int n = n0 + 32 * t + cl;
                    const float e = acc[t][v], o = exch[(t * 16 + v) * 64 + lane];
                    if (k < K2 && n < ld) {
                        out[(int64_t)k * ld + n] = e + o;
                        const int kk = nlat - 1 - k;
                        if (kk != k) out[(int64_t)kk * ld + n] = e - o;
                    }
                }
            }
        }
    }
}

template <bool ANALYSIS>
static int launch_fold(const PgemmArgs& a, int n_work, hipStream_t s) {
    const int64_t ncols = a.ld;
    if (n_work <= 0 || ncols <= 0) return SFNO_OK;
    static const int cand[] = {6, 5, 4, 3, 2, 1};
    int best = 1;
    int64_t best_pad = INT64_MAX;
    for (int nt : cand) {
        int64_t pad = (ncols + 32 * nt - 1) / (32 * nt) * (32 * nt);
        if (pad < best_pad) { best_pad = pad; best = nt; }
    }
#define LF_CASE(NT_)                                                                                 \
    case NT_: {                                                                                      \
        dim3 grid(n_work, (unsigned)((ncols + 32 * NT_ - 1) / (32 * NT_)));                          \
        hipLaunchKernelGGL((legendre_fold_kernel<NT_, ANALYSIS>), grid, dim3(256), 0, s, a);         \
        break;                                                                                       \
    }
    switch (best) {
        LF_CASE(1) LF_CASE(2) LF_CASE(3) LF_CASE(4) LF_CASE(5) LF_CASE(6)
        default: return SFNO_EINVAL;
    }
#undef LF_CASE
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int legendre_fold_launch(bool analysis, const PgemmArgs& a, int n_work, hipStream_t s) {
    return analysis ? launch_fold<true>(a, n_work, s) : launch_fold<false>(a, n_work, s);
}

}  // namespace sfno
