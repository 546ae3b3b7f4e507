// Equator-folded Legendre contractions on the matrix cores of gfx950: fp32 results from the bf16 pipe (operands cut
// exactly into three bf16 planes, six v_mfma_f32_32x32x16_bf16 per K step; the default), the fp32 instruction
// v_mfma_f32_32x32x2_f32, or plain bf16 operands -- see MODE below.
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
typedef float f4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// MODE selects the arithmetic of the contraction:
// LF_FP32:  v_mfma_f32_32x32x2_f32 on the fp32 table stream.
// LF_BF16:  the table stream holds bf16 (8 per lane and chunk: lane (row, kg) has k = 16c + 8kg .. +7) and the
//   contraction runs on v_mfma_f32_32x32x16_bf16 with the panel values rounded to bf16 (nearest even) as they are
//   read from LDS; accumulation stays fp32.
// LF_SPLIT: fp32 operands on the bf16 matrix pipe.  An fp32 number is exactly the sum of three bf16 numbers (its
//   24 significant bits cut into 8 + 8 + 8 by truncation), so t * q = sum_ij t_i q_j; the six products with
//   i + j <= 2 are kept (each dropped one is below 2^-23 of the product, the size of an fp32 rounding), every kept
//   product is exact in the fp32 accumulator, and one K = 16 step costs 6 x 32 matrix-pipe cycles instead of the
//   8 x 64 of v_mfma_f32_32x32x2_f32.  The table is split on the host (three bf16 planes in the lane order of
//   LF_BF16), the panel values as they are read from LDS.  Non-finite inputs turn into NaN (inf - inf).
enum { LF_FP32 = 0, LF_BF16 = 1, LF_SPLIT = 2 };

// x = hi + mid + lo with 8 significant bits each; the pair (a, b) packed as two bf16 per plane
__device__ __forceinline__ void split3_pack(float a, float b, uint32_t& hi, uint32_t& mid, uint32_t& lo) {
    const uint32_t ab = __builtin_bit_cast(uint32_t, a), bb = __builtin_bit_cast(uint32_t, b);
    const float a1 = a - __builtin_bit_cast(float, ab & 0xffff0000u), b1 = b - __builtin_bit_cast(float, bb & 0xffff0000u);
    const uint32_t a1b = __builtin_bit_cast(uint32_t, a1), b1b = __builtin_bit_cast(uint32_t, b1);
    const float a2 = a1 - __builtin_bit_cast(float, a1b & 0xffff0000u), b2 = b1 - __builtin_bit_cast(float, b1b & 0xffff0000u);
    hi = __builtin_amdgcn_perm(bb, ab, 0x07060302u);
    mid = __builtin_amdgcn_perm(b1b, a1b, 0x07060302u);
    lo = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, b2), __builtin_bit_cast(uint32_t, a2), 0x07060302u);
}

// resident wavefronts per SIMD: set by the 16 NT accumulator registers and, in split mode, the three-plane fragments
constexpr int lf_occupancy(int nt, int mode) {
    if (mode == LF_SPLIT) return nt <= 3 ? 4 : 3;
    return nt <= 4 ? 4 : 3;
}

template <int NT, bool ANALYSIS, int MODE>
__global__ __launch_bounds__(256, lf_occupancy(NT, MODE)) void legendre_fold_kernel(PgemmArgs a) {
    constexpr bool BF16 = MODE == LF_BF16;
    constexpr int TN = 32 * NT;
    constexpr int LDQ = TN + ((TN % 64 == 0) ? 32 : 0);
    // [buffer][parity][k][column]; reused for the parity exchange of the synthesis epilogue
    __shared__ __align__(16) float qs[2][2][PG_KC][LDQ];

    // Workgroups go to the 8 XCDs round-robin by linear id and entry 8 i + x of the work list is meant for XCD x: the
    // column tiles of one entry run back to back on that XCD, where they share the entry's table fragments in L2.
    const int nct = (a.ld + 32 * NT - 1) / (32 * NT);
    const int qid = blockIdx.x >> 3;
    const int ct = qid % nct;
    const int2 wi = a.work[(qid / nct) * 8 + (blockIdx.x & 7)];
    const int m = wi.x;
    if (m < 0) return;
    // the wavefront index is uniform: keep it (and everything derived from it) in scalar registers
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    // wavefront w runs on SIMD w; alternate which SIMDs get the (possibly absent) second row block
    // and the (one row shorter) odd parity from workgroup to workgroup
    const int wslot = (wave + qid) & 3;
    const int par = wslot >> 1, rb = wi.y + (wslot & 1);
    const int n0 = ct * TN;
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

    const float* xm_m = (ANALYSIS ? a.Q : a.Out) + (int64_t)m * nlat * ld;     // Fourier panel of order m
    const float* sp_m = (ANALYSIS ? a.Out : a.Q) + (int64_t)m * lmax * ld;     // spectral panel of order m
    // wavefronts without a row block read the head of the table and discard it
    // 16 bytes per lane: fp32 blocks are two such pieces per chunk (128 per block), bf16 blocks one (64 per block)
    constexpr int NA = MODE == LF_BF16 ? 1 : MODE == LF_SPLIT ? 3 : 2;     // 16-byte pieces per lane and block
    constexpr int APB = 64 * NA;
    // Index entry of a row block: first block of its stream | leading chunks left out << 48 (their entries are negligible:
    // towards the poles the table falls off like sin^m(theta)).  The K loop of the workgroup starts at the smallest such
    // count of its (up to) four row blocks; a wavefront joins in at its own.
    auto entry_of = [&](int p_, int rb_) {
        const int nr = ANALYSIS ? (p_ ? nl1 : nl0) : K2;
        // an order without degrees (synthesis with mmax > lmax: nc = 0) has no entries; its rows are zero-filled below
        return (nc > 0 && rb_ * PG_ROWS < nr) ? a.a_off[a.a_off[2 * m + p_] + rb_] : (int64_t)nc << 48;
    };
    int cstart = nc;
#pragma unroll
    for (int s_ = 0; s_ < 4; ++s_) cstart = min(cstart, (int)(entry_of(s_ >> 1, wi.y + (s_ & 1)) >> 48));
    const int64_t my_entry = entry_of(par, rb);
    cstart = max(cstart, 0);
    const int c0w = min(max((int)(my_entry >> 48), 0), nc);   // nc for a wavefront without a row block or with nothing but negligible entries
    const float4* ap = reinterpret_cast<const float4*>(a.A) + ((c0w < nc ? my_entry & (((int64_t)1 << 48) - 1) : (int64_t)0) * APB + lane);

    floatx16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.0f;

    constexpr int QV = (NT + 1) / 2;       // float4 per thread per 16-row panel
    f4 q0[QV], q1[QV];

    // Loads are unconditional (indices clamped into the panel) and keep the raw rows in
    // registers; masking and the mirror sum/difference happen when the chunk is written to
    // LDS, one chunk of MFMAs later.
    // uniform panel base + 32-bit byte offset per lane (a panel is far smaller than 4 GiB): one address register per load
    const char* qpanel = reinterpret_cast<const char*>(ANALYSIS ? xm_m : sp_m);
    auto q_at = [&](int row, int n) { return *reinterpret_cast<const f4*>(qpanel + (size_t)(((uint32_t)row * (uint32_t)ld + (uint32_t)n) * 4u)); };
    auto q_load = [&](int c) {
#pragma unroll
        for (int u = 0; u < QV; ++u) {
            const int e = tid + 256 * u;
            const int row = e / (TN / 4), c4 = e - row * (TN / 4);
            const int i = c * PG_KC + row, n = min(n0 + 4 * c4, ld - 4);
            if (ANALYSIS) {
                const int k = min(i, K2 - 1);
                q0[u] = q_at(k, n);
                q1[u] = q_at(nlat - 1 - k, n);
            } else {
                q0[u] = q_at(min(m + 2 * i, lmax - 1), n);
                q1[u] = q_at(min(m + 2 * i + 1, lmax - 1), n);
            }
        }
    };
    auto q_store = [&](int buf, int c) {
        const f4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < QV; ++u) {
            const int e = tid + 256 * u;
            const int row = e / (TN / 4), c4 = e - row * (TN / 4);
            const int i = c * PG_KC + row;
            const bool col_ok = n0 + 4 * c4 < ld;
            if (e < 4 * TN) {
                f4 v0, v1;
                if (ANALYSIS) {
                    // i = latitude k; panel 0 = X[k] + X[k'], panel 1 = X[k] - X[k']; the equator row is its own mirror
                    const bool ok = col_ok && i < K2, mirror = (nlat - 1 - i) != i;
                    v0 = mirror ? q0[u] + q1[u] : q0[u];
                    v1 = mirror ? q0[u] - q1[u] : zero;
                    v0 = ok ? v0 : zero;
                    v1 = ok ? v1 : zero;
                } else {
                    // i = index within a parity; panel 0 = degree m+2i, panel 1 = degree m+2i+1
                    v0 = (col_ok && m + 2 * i < lmax) ? q0[u] : zero;
                    v1 = (col_ok && m + 2 * i + 1 < lmax) ? q1[u] : zero;
                }
                *reinterpret_cast<f4*>(&qs[buf][0][row][4 * c4]) = v0;
                *reinterpret_cast<f4*>(&qs[buf][1][row][4 * c4]) = v1;
            }
        }
    };
    const int kh = lane >> 5, cl = lane & 31;
    // One K-chunk of MFMAs.  No branches inside: columns past ld hold zeros in LDS and are
    // masked at the store, so the LDS reads can be issued well ahead of the matrix instructions.
    auto compute = [&](int buf, const f4 (&ar)[NA]) {
        if constexpr (MODE == LF_SPLIT) {
            const bf16x8 a0 = __builtin_bit_cast(bf16x8, ar[0]), a1 = __builtin_bit_cast(bf16x8, ar[1]), a2 = __builtin_bit_cast(bf16x8, ar[2]);
            const float* qbase = &qs[buf][par][8 * kh][cl];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                typedef uint32_t u4 __attribute__((ext_vector_type(4)));
                u4 h, mi, lo;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    uint32_t x, y, z;
                    split3_pack(qbase[2 * e * LDQ + 32 * t], qbase[(2 * e + 1) * LDQ + 32 * t], x, y, z);
                    h[e] = x; mi[e] = y; lo[e] = z;
                }
                const bf16x8 q0v = __builtin_bit_cast(bf16x8, h), q1v = __builtin_bit_cast(bf16x8, mi), q2v = __builtin_bit_cast(bf16x8, lo);
                // smallest terms first
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a2, q0v, acc[t], 0, 0, 0);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, q1v, acc[t], 0, 0, 0);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, q2v, acc[t], 0, 0, 0);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, q0v, acc[t], 0, 0, 0);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, q1v, acc[t], 0, 0, 0);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, q0v, acc[t], 0, 0, 0);
                // one tile at a time: the split values of several tiles in flight would not fit the registers
                __builtin_amdgcn_sched_barrier(0);
            }
        } else if constexpr (BF16) {
            // ar[0] carries 8 bf16 table values; every column tile gathers its 8 panel values along k
            const bf16x8 av = __builtin_bit_cast(bf16x8, ar[0]);
            const float* qbase = &qs[buf][par][8 * kh][cl];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                bf16x8 qv;
#pragma unroll
                for (int e = 0; e < 8; ++e) qv[e] = (__bf16)qbase[e * LDQ + 32 * t];
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, qv, acc[t], 0, 0, 0);
            }
        } else {
            // the panel values of k-step i+1 are read from LDS before the MFMAs of k-step i are issued
            float qv[2][NT];
            const float* qbase = &qs[buf][par][kh][cl];
#pragma unroll
            for (int t = 0; t < NT; ++t) qv[0][t] = qbase[32 * t];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (i + 1 < 8) {
                    const float* qrow = qbase + 2 * (i + 1) * LDQ;
#pragma unroll
                    for (int t = 0; t < NT; ++t) qv[(i + 1) & 1][t] = qrow[32 * t];
                }
                const float av = ar[i >> 2][i & 3];
#pragma unroll
                for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, qv[i & 1][t], acc[t], 0, 0, 0);
            }
        }
    };
    const f4* apv = reinterpret_cast<const f4*>(ap);
    auto a_load = [&](int c, f4 (&ar)[NA]) {
#pragma unroll
        for (int p = 0; p < NA; ++p) ar[p] = apv[(int64_t)max(c - c0w, 0) * APB + 64 * p];
    };

    // Software pipeline, one chunk deep: the loads of chunk c+1 (raw panel rows and table
    // fragments) are issued before the MFMAs of chunk c and are first touched after them.
    // The explicit wait for all of them at the end of the iteration keeps the wait-count
    // bookkeeping of the next iteration's MFMA block empty.
    f4 acur[NA], anext[NA];
    if (cstart < nc) {
        q_load(cstart);
        a_load(cstart, acur);
        q_store(cstart & 1, cstart);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0): the first table fragments too
    __syncthreads();
    for (int c = cstart; c < nc; ++c) {
        const int buf = c & 1;
        const bool more = c + 1 < nc;
        if (more) {
            q_load(c + 1);
            a_load(c + 1, anext);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (c >= c0w) compute(buf, acur);
        __builtin_amdgcn_sched_barrier(0);
        if (more) q_store(buf ^ 1, c + 1);
        __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0): everything issued above has landed
        __syncthreads();
#pragma unroll
        for (int p = 0; p < NA; ++p) acur[p] = anext[p];
    }

    // D layout of the 32x32 MFMA: register v of lane j holds D[8*(v/4) + 4*(j/32) + v%4][j%32].
    if (ANALYSIS) {
        if (!active) return;
        float* out = a.Out + (int64_t)m * lmax * ld;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = PG_ROWS * rb + 8 * (v >> 2) + 4 * kh + (v & 3);
                const int n = n0 + 32 * t + cl;
                if (r < nrows && n < ld) out[(int64_t)(m + par + 2 * r) * ld + n] = acc[t][v];
            }
        }
    } else {
        // odd-parity wavefronts hand their sums to the even-parity wavefront of the same row block
        float* exch = &qs[0][0][0][0] + (wslot & 1) * (NT * 16 * 64);
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

template <bool ANALYSIS, int MODE>
static int launch_fold(const PgemmArgs& a, int n_work, hipStream_t s) {
    const int64_t ncols = a.ld;
    if (n_work <= 0 || ncols <= 0) return SFNO_OK;
    // the kernel addresses a panel (one order: nlat or lmax rows of ld floats) with 32-bit byte offsets
    if ((int64_t)(a.nlat > a.lmax ? a.nlat : a.lmax) * a.ld >= ((int64_t)1 << 30)) return SFNO_EUNSUPPORTED;
    // prefer the least padding, then the widest tile count that still keeps four wavefronts per SIMD resident (4 tiles; 3
    // where the operands are split into planes: 384 channels measured 1-4 % faster as 8 x 3 tiles than as 6 x 4)
    static const int cand_plain[] = {4, 5, 3, 2, 1}, cand_split[] = {3, 4, 5, 2, 1};
    int best = 1;
    int64_t best_pad = INT64_MAX;
    for (int nt : (MODE == LF_SPLIT ? cand_split : cand_plain)) {
        int64_t pad = (ncols + 32 * nt - 1) / (32 * nt) * (32 * nt);
        if (pad < best_pad) { best_pad = pad; best = nt; }
    }
#define LF_CASE(NT_)                                                                                 \
    case NT_: {                                                                                      \
        const int64_t nwg = (int64_t)n_work * ((ncols + 32 * NT_ - 1) / (32 * NT_));                 \
        if (nwg > 0x7fffffffLL) return SFNO_EUNSUPPORTED;                                            \
        dim3 grid((unsigned)nwg);                                                                    \
        hipLaunchKernelGGL((legendre_fold_kernel<NT_, ANALYSIS, MODE>), grid, dim3(256), 0, s, a);   \
        break;                                                                                       \
    }
    switch (best) {
        LF_CASE(1) LF_CASE(2) LF_CASE(3) LF_CASE(4) LF_CASE(5)
        default: return SFNO_EINVAL;
    }
#undef LF_CASE
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int legendre_fold_launch(bool analysis, int format, const PgemmArgs& a, int n_work, hipStream_t s) {
    switch (format) {
        case PG_FORMAT_F16X2: return legendre_f16_launch(analysis, a, n_work, s);
        case PG_FORMAT_BF16: return analysis ? launch_fold<true, LF_BF16>(a, n_work, s) : launch_fold<false, LF_BF16>(a, n_work, s);
        case PG_FORMAT_SPLIT: return analysis ? launch_fold<true, LF_SPLIT>(a, n_work, s) : launch_fold<false, LF_SPLIT>(a, n_work, s);
        case PG_FORMAT_FP32: return analysis ? launch_fold<true, LF_FP32>(a, n_work, s) : launch_fold<false, LF_FP32>(a, n_work, s);
    }
    return SFNO_EINVAL;
}

}  // namespace sfno
