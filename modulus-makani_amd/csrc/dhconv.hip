// dhconv on fp32 MFMA (v_mfma_f32_32x32x2_f32), gfx950.
//
//   y[b,o,l,m] = sum_i x[b,i,l,m] w[i,o,l]        (makani/models/common/contractions.py:130-136)
// runs as one real GEMM per degree l on the spectral layout,
//   out[(m,b)][o'] = sum_i' in[(m,b)][i'] * Wt[l][i'][o'],   i' = 2i + {re,im}, o' = 2o + {re,im},
// where Wt is the 2x2 real embedding of each complex weight: rows 2i, 2i+1 of column pair
// (2o, 2o+1) are (re, im) and (-im, re).
//
// A workgroup owns (degree l, block of 128 output columns o', group of 128 rows (m,b)).
// Each of its four wavefronts owns 32 rows: it reads its own activation rows straight from
// HBM/L2 into MFMA A-fragments (rows are contiguous along i' in the spectral layout) and
// keeps a 32 x 128 accumulator.  The weight chunk (16 i' x 128 o') is expanded from the
// packed complex weights into LDS once per chunk and shared by the four wavefronts as the
// B operand.  Wavefronts whose rows lie beyond the orders present at this degree (m > l)
// exit early, so the triangular structure costs no guarded matrix instructions.
#include "sfno_internal.h"

namespace sfno {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));

// grid = (8 * ceil(L/8) * nob, row groups); VEC4: 2*I is a multiple of 4 so activation rows can be read as float4
template <bool VEC4>
__global__ __launch_bounds__(256) void dhconv_kernel(DhconvArgs a) {
    constexpr int NT = DH_COLS / 32;                 // 4 column tiles per wavefront
    constexpr int LDW = DH_COLS + 32;                // pitch = 32 mod 64: the two half-waves read different banks
    __shared__ __align__(16) float ws[2][PG_KC][LDW];

    // Workgroups go to the 8 XCDs round-robin by linear id: all column blocks and row groups of a
    // degree share their activation panel, so a degree stays on one XCD.  Degrees are handed out
    // largest first: they have the most orders, hence the most rows.
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    const int lidx = (q / a.nob) * 8 + xcd, ob = q % a.nob;
    if (lidx >= a.L) return;
    const int l = a.L - 1 - lidx;
    // Wavefront w of every workgroup runs on SIMD w, and low degrees fill only the first row blocks:
    // rotate the block a wavefront takes from workgroup to workgroup so that no SIMD gets all the work.
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = (__builtin_amdgcn_readfirstlane(tid >> 6) + q + blockIdx.y) & 3;
    const int ncols = (a.tri ? min(l + 1, a.M) : a.M) * a.B;      // rows (m,b) present at this degree
    const int r0 = blockIdx.y * 128;
    if (r0 >= ncols) return;
    const bool active = r0 + 32 * wave < ncols;
    const int nc = a.nc;                                           // K chunks of 16 i' (8 complex input channels)
    const int kh = lane >> 5, cl = lane & 31;

    // my activation row (clamped: rows past the end repeat the last one and are not stored)
    const int n = min(r0 + 32 * wave + cl, ncols - 1);
    const int mm = n / a.B, bb = n - mm * a.B;
    const float* xrow = a.X + ((int64_t)mm * a.L + l) * a.ld_in + (int64_t)bb * a.I2;
    // packed weights of (l, ob): nc chunks of 8 x 64 complex, 16 bytes per thread and chunk
    const f4* wp = reinterpret_cast<const f4*>(a.W) + ((int64_t)l * a.nob + ob) * nc * 256 + tid;

    floatx16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.0f;

    // A fragments: lane (row, kh) holds i' = 16c + 8kh .. +7; k-step s of the chunk uses i' = 16c + 8kh + s
    // on both operands.  Reads are clamped into the row; the weights are zero beyond 2*I.
    auto x_load = [&](int c, f4 (&xr)[2]) {
        if (VEC4) {
            // a group of four i' is either entirely inside the row or entirely in the zero-weight padding
            const int k = 16 * c + 8 * kh;
            xr[0] = *reinterpret_cast<const f4*>(xrow + min(k, a.I2 - 4));
            xr[1] = *reinterpret_cast<const f4*>(xrow + min(k + 4, a.I2 - 4));
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = min(16 * c + 8 * kh + 2 * j, a.I2 - 2);
                const f2 v = *reinterpret_cast<const f2*>(xrow + k);
                xr[j >> 1][2 * (j & 1)] = v[0];
                xr[j >> 1][2 * (j & 1) + 1] = v[1];
            }
        }
    };
    // thread t expands complex pair (i = t/32, o = 2(t%32), 2(t%32)+1) of the chunk
    auto w_store = [&](int buf, f4 w) {
        const int ii = tid >> 5, o2 = tid & 31;
        *reinterpret_cast<f4*>(&ws[buf][2 * ii][4 * o2]) = w;
        const f4 r = {-w[1], w[0], -w[3], w[2]};
        *reinterpret_cast<f4*>(&ws[buf][2 * ii + 1][4 * o2]) = r;
    };
    auto compute = [&](int buf, const f4 (&xr)[2]) {
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const float* wrow = &ws[buf][8 * kh + s][cl];
            const float xv = xr[s >> 2][s & 3];
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(xv, wrow[32 * t], acc[t], 0, 0, 0);
        }
    };

    // software pipeline, one chunk deep; the explicit wait at the end of each iteration keeps
    // the wait-count bookkeeping of the next MFMA block empty
    f4 xcur[2], xnext[2], wnext;
    x_load(0, xcur);
    w_store(0, wp[0]);
    __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0)
    __syncthreads();
    for (int c = 0; c < nc; ++c) {
        const int buf = c & 1;
        const bool more = c + 1 < nc;
        if (more) {
            wnext = wp[(int64_t)(c + 1) * 256];
            x_load(c + 1, xnext);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (active) compute(buf, xcur);
        __builtin_amdgcn_sched_barrier(0);
        if (more) w_store(buf ^ 1, wnext);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        xcur[0] = xnext[0];
        xcur[1] = xnext[1];
    }

    if (!active) return;
    // D layout of the 32x32 MFMA: register v of lane j holds D[8*(v/4) + 4*(j/32) + v%4][j%32];
    // D rows = my 32 activation rows, D cols = output columns o'
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int nn = r0 + 32 * wave + 8 * (v >> 2) + 4 * kh + (v & 3);
        if (nn >= ncols) continue;
        const int m2 = nn / a.B, b2 = nn - m2 * a.B;
        float* orow = a.Y + ((int64_t)m2 * a.L + l) * a.ld_out + (int64_t)b2 * a.O2;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int oc = DH_COLS * ob + 32 * t + cl;
            if (oc < a.O2) orow[oc] = acc[t][v];
        }
    }
}

// packed[l][ob][c][ii][o] (complex) = w[8c + ii][64 ob + o][l], zero outside the weight
__global__ __launch_bounds__(256) void dhconv_pack_kernel(const float2* __restrict__ w, float2* __restrict__ packed, int I, int O, int L,
                                                          int nob, int nc) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = (int64_t)L * nob * nc * 512;
    if (idx >= total) return;
    const int o = (int)(idx & 63), ii = (int)((idx >> 6) & 7);
    int64_t rem = idx >> 9;
    const int c = (int)(rem % nc);
    rem /= nc;
    const int ob = (int)(rem % nob), l = (int)(rem / nob);
    const int i = 8 * c + ii, oo = 64 * ob + o;
    float2 v = make_float2(0.f, 0.f);
    if (i < I && oo < O) v = w[((int64_t)i * O + oo) * L + l];
    packed[idx] = v;
}

int dhconv_pack_launch(const float2* w, float* packed, int I, int O, int L, hipStream_t s) {
    const int nob = (2 * O + DH_COLS - 1) / DH_COLS, nc = (2 * I + PG_KC - 1) / PG_KC;
    const int64_t total = (int64_t)L * nob * nc * 512;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(dhconv_pack_kernel, dim3((unsigned)blocks), dim3(256), 0, s, w, reinterpret_cast<float2*>(packed), I, O, L, nob, nc);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int dhconv_launch(const DhconvArgs& a, hipStream_t s) {
    const int64_t rows_max = (int64_t)a.M * a.B;
    if (rows_max <= 0 || a.L <= 0) return SFNO_OK;
    dim3 grid((unsigned)((a.L + 7) / 8 * 8 * a.nob), (unsigned)((rows_max + 127) / 128));
    const bool vec4 = a.I2 % 4 == 0 && a.ld_in % 4 == 0;
    if (vec4)
        hipLaunchKernelGGL((dhconv_kernel<true>), grid, dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL((dhconv_kernel<false>), grid, dim3(256), 0, s, a);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
