// Equator-folded Legendre contractions with fp32 accuracy on the fp16 matrix pipe of gfx950 (the default fp32 path):
//
//   analysis : spec[m][l][n] = sum_k W[m][l][k] xm[m][k][n]     (RealSHT.forward, Legendre stage)
//   synthesis: xm[m][k][n]   = sum_l P[m][l][k] spec[m][l][n]   (InverseRealSHT.forward, Legendre stage)
//
// Work decomposition, table streams, equator fold and the omitted polar chunks are those of legendre_fold.hip: a
// workgroup has four wavefronts = 2 parities x 2 row blocks of 32 table rows, owns NT 32-wide column tiles and walks K
// in chunks of 16.  What differs is the arithmetic.  An fp32 number scaled by a power of two into the range of fp16 is,
// to 22 of its 24 significant bits, the sum of two fp16 numbers; with both operands cut that way a product needs three
// v_mfma_f32_32x32x16_f16 (t0 q0 + t0 q1 + t1 q0; t1 q1 is below 2^-21 of the product), each exact in the fp32
// accumulator, where three exact bf16 parts need six.
//   table: cut on the host from the float64 value (both parts rounded to nearest, so 23 bits are kept), one power-of-two
//          scale per table row that brings the row's largest entry to [2^14, 2^15); 4 bytes per entry in the stream;
//   panel: cut once per workgroup by the threads that stage it (one thread per column, which holds the column's 16 rows
//          of the chunk: no cross-lane work) -- sums and differences of mirrored latitude rows (analysis) or the degree
//          rows of the two parities (synthesis) go to LDS as two fp16 planes in the order the matrix instruction wants
//          its B operand (16-byte fragment reads, no arithmetic in the matrix phase) -- with one power-of-two scale per column.  The scale of a column is found while the
//          column streams by: the staging threads keep a bound on its exponent, raise it (leaving a few bits of
//          headroom) when a chunk exceeds it and publish the bound with the chunk; a wavefront whose column's bound
//          moved rescales that column's partial sums, which is exact.
// Entries more than 2^17 below the largest entry of their column (row) keep fewer bits, so the error bound is
// 2^-21 |t q| + 2^-38 max|t| max|q| per product where fp32 arithmetic has 2^-24 |t q|; the transform's own longitude
// FFT has an error of that second kind already (relative to the largest value of a latitude row).
#include "sfno_internal.h"

namespace sfno {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __fp16 fp16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));
typedef unsigned int u2 __attribute__((ext_vector_type(2)));
typedef int i4 __attribute__((ext_vector_type(4)));

constexpr int LH_TOP = 14;             // scaled magnitudes stay below 2^(TOP + 1)
constexpr int LH_HEAD = 3;             // bits of headroom left when a column's exponent bound is raised
constexpr int LH_SH = LH_TOP + 127;    // scaled = x * 2^(SH - E), E = biased exponent bound of the column

// resident workgroups per CU: set by the 16 NT accumulator registers and the staged rows held across the matrix phase
constexpr int lh_occupancy(int nt, bool analysis) { return nt <= 4 ? 4 : analysis ? 2 : 3; }

__device__ __forceinline__ unsigned int lh_pk(float a, float b) { return __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_pkrtz(a, b)); }

template <int NT, bool ANALYSIS>
__global__ __launch_bounds__(256, lh_occupancy(NT, ANALYSIS)) void legendre_f16_kernel(PgemmArgs a) {
    constexpr int TN = 32 * NT;            // columns per workgroup
    constexpr int QN = TN / 4;             // column quads
    constexpr int QW = QN / 4;             // column quads staged per wavefront
    // LDS image of one (buffer, panel, plane): column c = 4 j + cc lives in class cc at slot j; a slot is the column's 16 k
    // values (32 bytes); classes are CS bytes apart with CS = 128 mod 256, and the two 16-byte halves of a slot swap places in
    // classes 2 and 3, so that the 16-byte fragment reads of 16 consecutive columns cover all banks
    constexpr int CS = QN * 32 + 128;
    constexpr int PLANE = 4 * CS;
    constexpr int PLANES = 2 * 2 * 2 * PLANE < 16384 ? 16384 : 2 * 2 * 2 * PLANE;      // [buffer][panel][plane]; at least the 16 KiB of the parity exchange
    __shared__ __align__(16) unsigned char planes[PLANES];
    __shared__ __align__(16) int expo[2][2][TN];   // [buffer][panel][column]: exponent bound the chunk was cut with

    // Workgroups go to the 8 XCDs round-robin by linear id and entry 8 i + x of the work list is meant for XCD x: the
    // column tiles of one entry run back to back on that XCD, where they share the entry's table fragments in L2.
    const int nct = (a.ld + TN - 1) / TN;
    const int qid = blockIdx.x >> 3;
    const int ct = qid % nct;
    // (the record is read through the scalar unit: one 64-byte request, wavefront-uniform)
    const __attribute__((address_space(4))) int64_t* wrec =
        reinterpret_cast<const __attribute__((address_space(4))) int64_t*>(reinterpret_cast<uintptr_t>(a.wrec)) + (int64_t)((qid / nct) * 8 + (blockIdx.x & 7)) * PG_WREC;
    int64_t rec[PG_WREC];
#pragma unroll
    for (int i = 0; i < PG_WREC; ++i) rec[i] = wrec[i];
    const int m = (int)rec[PG_WREC_M];
    if (m < 0) return;
    const int2 wi = make_int2(m, (int)rec[PG_WREC_RB]);
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
    // Index entry of a row block: first block of its stream | leading chunks left out << 48 (their entries are negligible:
    // towards the poles the table falls off like sin^m(theta)).  The K loop of the workgroup starts at the smallest such
    // count of its (up to) four row blocks; a wavefront joins in at its own.
    constexpr int APB = 128;               // 16-byte pieces per block: two planes x 64 lanes
    // (the work record holds the entries of the four streams -- nc << 48 for one that does not exist: an order without
    // degrees, synthesis with mmax > lmax, has none, its rows are zero-filled below -- and the parities' first positions)
    auto entry_pos = [&](int p_, int rb_) { return (p_ ? rec[PG_WREC_POS + 1] : rec[PG_WREC_POS]) + rb_; };
    int cstart = nc;
#pragma unroll
    for (int s_ = 0; s_ < 4; ++s_) cstart = min(cstart, (int)(rec[PG_WREC_ENTRY + s_] >> 48));
    const int64_t my_entry = par ? ((wslot & 1) ? rec[PG_WREC_ENTRY + 3] : rec[PG_WREC_ENTRY + 2]) : ((wslot & 1) ? rec[PG_WREC_ENTRY + 1] : rec[PG_WREC_ENTRY]);
    cstart = max(cstart, 0);
    const int c0w = min(max((int)(my_entry >> 48), 0), nc);   // nc for a wavefront without a row block or with nothing but negligible entries
    const f4* apv = reinterpret_cast<const f4*>(a.A) + ((c0w < nc ? my_entry & (((int64_t)1 << 48) - 1) : (int64_t)0) * APB + lane);

    floatx16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.0f;
    int erun[NT];                          // exponent bound my partial sums of tile t are scaled with (per lane = column)
#pragma unroll
    for (int t = 0; t < NT; ++t) erun[t] = 0;

    // ---- staging: thread = one column of the tile and RPT consecutive rows of the chunk, both panels.  Up to four tiles a
    // column is shared by two neighbouring lanes (8 rows each: all 256 threads at four tiles); five tiles give a thread the
    // column's 16 rows (160 threads, dealt out over the four wavefronts).
    constexpr int RPT = NT <= 4 ? 8 : 16;  // rows per thread
    constexpr int TPC = PG_KC / RPT;       // threads per column
    constexpr int CW = TN / 4;             // columns staged per wavefront
    const bool stager = lane < CW * TPC;
    const int scol = wave * CW + min(lane / TPC, CW - 1), shalf = lane % TPC;
    float q0[RPT], q1[RPT];
    int E0 = 0, E1 = 0;                    // exponent bounds of my column, panel 0 and 1 (equal in the lanes that share it)
    // uniform panel base + 32-bit byte offset per lane (a panel is far smaller than 4 GiB): one address register per load
    const char* qpanel = reinterpret_cast<const char*>(ANALYSIS ? xm_m : sp_m);
    const int sn = min(n0 + scol, ld - 1);
    const bool col_ok = n0 + scol < ld;
    auto q_at = [&](int row) { return *reinterpret_cast<const float*>(qpanel + (size_t)(((uint32_t)row * (uint32_t)ld + (uint32_t)sn) * 4u)); };
    // raw rows into registers (indices clamped into the panel); masking, the mirror sum/difference and the cut happen when
    // the chunk is written to LDS, one chunk of matrix instructions later
    auto q_load = [&](int c) {
        if (!stager) return;
#pragma unroll
        for (int rr = 0; rr < RPT; ++rr) {
            const int i = c * PG_KC + RPT * shalf + rr;
            if (ANALYSIS) {
                const int k = min(i, K2 - 1);
                q0[rr] = q_at(k);
                q1[rr] = q_at(nlat - 1 - k);
            } else {
                q0[rr] = q_at(min(m + 2 * i, lmax - 1));
                q1[rr] = q_at(min(m + 2 * i + 1, lmax - 1));
            }
        }
    };
    // my column's slot within a plane (class scol & 3, slot scol >> 2; the 16-byte halves swap in classes 2 and 3)
    const int st_lo = (scol & 3) * CS + (scol >> 2) * 32 + ((((scol & 3) >> 1) ^ (RPT == 8 ? shalf : 0)) * 16), st_hi = st_lo ^ 16;
    // one panel's values of my column: bound, scale, cut, one 16-byte write per plane and 8 rows
    auto cut_store = [&](unsigned char* pl0, const float (&v)[RPT], int& E) {
        float mx = __builtin_fabsf(v[0]);
#pragma unroll
        for (int rr = 1; rr < RPT; ++rr) mx = __builtin_fmaxf(mx, __builtin_fabsf(v[rr]));
        int mb = __builtin_bit_cast(int, mx);
        if (TPC == 2) mb = max(mb, __builtin_amdgcn_mov_dpp(mb, 0xB1, 0xF, 0xF, true));      // the neighbour's eight rows (quad_perm [1,0,3,2])
        const int eb = mb >> 23;
        E = eb > E ? eb + LH_HEAD : E;
        const int sh = LH_SH - E;
        u4 hi[RPT / 8], lo[RPT / 8];
#pragma unroll
        for (int e = 0; e < RPT / 2; ++e) {
            const float xa = __builtin_ldexpf(v[2 * e], sh), xb = __builtin_ldexpf(v[2 * e + 1], sh);
            const unsigned int h = lh_pk(xa, xb);
            float ra, rb2;
            // remainder = x - (float)h in one instruction each: the fp16 operand is read as it stands
            asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel_hi:[1,0,0]" : "=v"(ra) : "v"(h), "v"(xa));
            asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(rb2) : "v"(h), "v"(xb));
            hi[e >> 2][e & 3] = h;
            lo[e >> 2][e & 3] = lh_pk(ra, rb2);
        }
        *reinterpret_cast<u4*>(pl0 + st_lo) = hi[0];
        *reinterpret_cast<u4*>(pl0 + PLANE + st_lo) = lo[0];
        if constexpr (RPT == 16) {
            *reinterpret_cast<u4*>(pl0 + st_hi) = hi[1];
            *reinterpret_cast<u4*>(pl0 + PLANE + st_hi) = lo[1];
        }
    };
    auto q_store = [&](int buf, int c) {
        if (!stager) return;
        // chunks that touch neither end of the K range nor the column tail need no masks
        const bool plain = col_ok && (ANALYSIS ? (c + 1) * PG_KC < K2 : m + 2 * (c + 1) * PG_KC < lmax);
        if constexpr (ANALYSIS) {
            // i = latitude k; panel 0 = X[k] + X[k'], panel 1 = X[k] - X[k']; the equator row is its own mirror
            float v0[RPT], v1[RPT];
            if (plain) {
#pragma unroll
                for (int rr = 0; rr < RPT; ++rr) {
                    v0[rr] = q0[rr] + q1[rr];
                    v1[rr] = q0[rr] - q1[rr];
                }
            } else {
#pragma unroll
                for (int rr = 0; rr < RPT; ++rr) {
                    const int i = c * PG_KC + RPT * shalf + rr;
                    const bool ok = col_ok && i < K2, mirror = (nlat - 1 - i) != i;
                    v0[rr] = ok ? (mirror ? q0[rr] + q1[rr] : q0[rr]) : 0.f;
                    v1[rr] = ok && mirror ? q0[rr] - q1[rr] : 0.f;
                }
            }
            cut_store(planes + ((buf * 2 + 0) * 2) * PLANE, v0, E0);
            cut_store(planes + ((buf * 2 + 1) * 2) * PLANE, v1, E1);
        } else {
            // i = index within a parity; panel 0 = degree m+2i, panel 1 = degree m+2i+1.  What lies outside is zeroed in place (the
            // raw rows are not needed again), so that the common case carries no copies of the 32 values
            if (!plain) {
#pragma unroll
                for (int rr = 0; rr < RPT; ++rr) {
                    const int i = c * PG_KC + RPT * shalf + rr;
                    q0[rr] = (col_ok && m + 2 * i < lmax) ? q0[rr] : 0.f;
                    q1[rr] = (col_ok && m + 2 * i + 1 < lmax) ? q1[rr] : 0.f;
                }
            }
            cut_store(planes + ((buf * 2 + 0) * 2) * PLANE, q0, E0);
            cut_store(planes + ((buf * 2 + 1) * 2) * PLANE, q1, E1);
        }
        if (shalf == 0) {
            expo[buf][0][scol] = E0;
            expo[buf][1][scol] = E1;
        }
    };

    // ---- matrix phase --------------------------------------------------------------------------------------------------------
    const int kg = lane >> 5, cl = lane & 31;
    const int frag = (cl & 3) * CS + (cl >> 2) * 32 + ((kg ^ ((cl & 3) >> 1)) * 16);      // my fragment of tile 0 within a plane
    auto compute = [&](int buf, const f4 (&ar)[2]) {
        // follow the scales of my columns
        int enew[NT];
        bool moved = false;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            enew[t] = expo[buf][par][32 * t + cl];
            moved |= enew[t] != erun[t];
        }
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int d = erun[t] - enew[t];
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[t][v] = __builtin_ldexpf(acc[t][v], d);
                erun[t] = enew[t];
            }
        }
        const f16x8 a0 = __builtin_bit_cast(f16x8, ar[0]), a1 = __builtin_bit_cast(f16x8, ar[1]);
        const unsigned char* pb = planes + ((buf * 2 + par) * 2) * PLANE + frag;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const f16x8 b0 = *reinterpret_cast<const f16x8*>(pb + t * 256), b1 = *reinterpret_cast<const f16x8*>(pb + PLANE + t * 256);
            // smallest terms first
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b0, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b1, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b0, acc[t], 0, 0, 0);
        }
    };
    auto a_load = [&](int c, f4 (&ar)[2]) {
        // (chunks past the end repeat the last one: the stream of the next row block, or the end of the buffer, follows)
#pragma unroll
        for (int p = 0; p < 2; ++p) ar[p] = apv[(int64_t)max(min(c, nc - 1) - c0w, 0) * APB + 64 * p];
    };

    // Software pipeline, one chunk deep: the loads of the next chunk (raw panel rows and table fragments) are issued before
    // the matrix instructions of the current one and are first touched after them.  (Table fragments requested three chunks
    // ahead, in rotating register sets, changed nothing at any shape and cost a resident workgroup at four tiles.)
    // The analysis walks the latitudes from the equator to the pole: Fourier coefficients of order m fall off towards the
    // poles like sin^m(theta), so the first chunk sets the column scales and later ones rarely move them; the synthesis
    // walks the degrees upwards, the direction in which spectra decay.
    constexpr int cstep = ANALYSIS ? -1 : 1;
    const int cfirst = ANALYSIS ? nc - 1 : cstart;
    f4 acur[2], anext[2];
    if (cstart < nc) {
        q_load(cfirst);
        a_load(cfirst, acur);
        q_store(cfirst & 1, cfirst);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0): the first table fragments too
    __syncthreads();
    for (int c = cfirst, left = nc - cstart; left > 0; --left, c += cstep) {
        const int buf = c & 1;
        const bool more = left > 1;
        if (more) {
            q_load(c + cstep);
            a_load(c + cstep, anext);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (c >= c0w) compute(buf, acur);
        __builtin_amdgcn_sched_barrier(0);
        if (more) q_store(buf ^ 1, c + cstep);
        __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0): everything issued above has landed
        __syncthreads();
#pragma unroll
        for (int p = 0; p < 2; ++p) acur[p] = anext[p];
    }

    // ---- epilogue: undo the scales (row factor stored with the table, column bound erun), store ------------------------------
    // D layout of the 32x32 MFMA: register v of lane j holds D[8*(v/4) + 4*(j/32) + v%4][j%32].
    f4 rinv[4];
    if (active) {
        const float* rp = a.rinv + (entry_pos(par, rb) - 2 * (int64_t)a.mmax) * PG_ROWS + 4 * kg;
#pragma unroll
        for (int q = 0; q < 4; ++q) rinv[q] = *reinterpret_cast<const f4*>(rp + 8 * q);
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[t][v] = __builtin_ldexpf(acc[t][v], erun[t] - LH_SH) * rinv[v >> 2][v & 3];
    }
    if (ANALYSIS) {
        if (!active) return;
        float* out = a.Out + (int64_t)m * lmax * ld;
        if (PG_ROWS * (rb + 1) <= nrows && n0 + TN <= ld) {
            // no row or column of my tile needs a check: one address per row, the tiles at constant offsets from it
            float* o = out + (int64_t)(m + par + 2 * (PG_ROWS * rb + 4 * kg)) * ld + n0 + cl;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float* orow = o + (int64_t)(2 * (8 * (v >> 2) + (v & 3))) * ld;
#pragma unroll
                for (int t = 0; t < NT; ++t) orow[32 * t] = acc[t][v];
            }
            return;
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = PG_ROWS * rb + 8 * (v >> 2) + 4 * kg + (v & 3);
                const int n = n0 + 32 * t + cl;
                if (r < nrows && n < ld) out[(int64_t)(m + par + 2 * r) * ld + n] = acc[t][v];
            }
        }
    } else {
        // X[k] = E[k] + O[k] and X[k'] = E[k] - O[k]: the two wavefronts of a row block swap their sums through LDS, one column
        // tile at a time, and each stores one of the two rows -- the even-parity wavefront the northern row k, the odd-parity
        // one the mirrored row k' -- so that all four wavefronts share the stores
        static_assert(4 * 16 * 64 * 4 <= PLANES, "the parity exchange reuses the plane buffers");
        float* exch = reinterpret_cast<float*>(planes);
        float* mine = exch + wslot * (16 * 64) + lane;
        const float* theirs = exch + (wslot ^ 2) * (16 * 64) + lane;
        float* out = a.Out + (int64_t)m * nlat * ld;
        const int k0 = PG_ROWS * rb + 4 * kg;
        const bool whole = active && PG_ROWS * (rb + 1) <= K2 - 1 && n0 + TN <= ld;      // no row or column of my tile needs a check
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (t > 0) __syncthreads();               // the previous tile has been read
            if (active) {
#pragma unroll
                for (int v = 0; v < 16; ++v) mine[v * 64] = acc[t][v];
            }
            __syncthreads();
            if (whole) {
                // one address per wavefront tile, rows at multiples of +-ld from it, no checks
                float* o = out + (int64_t)(par ? nlat - 1 - k0 : k0) * ld + n0 + 32 * t + cl;
                const int64_t rstep = par ? -(int64_t)ld : (int64_t)ld;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float other = theirs[v * 64];
                    o[(8 * (v >> 2) + (v & 3)) * rstep] = par ? other - acc[t][v] : acc[t][v] + other;
                }
            } else if (active) {
                const int n = n0 + 32 * t + cl;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int k = k0 + 8 * (v >> 2) + (v & 3);
                    const float other = theirs[v * 64];
                    // even parity: E + O to row k; odd parity: E - O to row k' (the equator row is its own mirror and has O = 0)
                    const float x = par ? other - acc[t][v] : acc[t][v] + other;
                    const int row = par ? nlat - 1 - k : k;
                    if (k < K2 && n < ld && !(par && row == k)) out[(int64_t)row * ld + n] = x;
                }
            }
        }
    }
}

template <bool ANALYSIS>
static int launch_f16(const PgemmArgs& a, int n_work, hipStream_t s) {
    const int64_t ncols = a.ld;
    if (n_work <= 0 || ncols <= 0) return SFNO_OK;
    if (!a.rinv || !a.wrec) return SFNO_EINVAL;
    // the kernel addresses a panel (one order: nlat or lmax rows of ld floats) with 32-bit byte offsets
    if ((int64_t)(a.nlat > a.lmax ? a.nlat : a.lmax) * a.ld >= ((int64_t)1 << 30)) return SFNO_EUNSUPPORTED;
    // prefer the least padding, then the tile count listed first
    static const int cand[] = {4, 3, 5, 2, 1};
    int best = 1;
    int64_t best_pad = INT64_MAX;
    for (int nt : cand) {
        int64_t pad = (ncols + 32 * nt - 1) / (32 * nt) * (32 * nt);
        if (pad < best_pad) { best_pad = pad; best = nt; }
    }
#define LH_CASE(NT_)                                                                             \
    case NT_: {                                                                                  \
        const int64_t nwg = (int64_t)n_work * ((ncols + 32 * NT_ - 1) / (32 * NT_));             \
        if (nwg > 0x7fffffffLL) return SFNO_EUNSUPPORTED;                                        \
        dim3 grid((unsigned)nwg);                                                                \
        hipLaunchKernelGGL((legendre_f16_kernel<NT_, ANALYSIS>), grid, dim3(256), 0, s, a);      \
        break;                                                                                   \
    }
    switch (best) {
        LH_CASE(1) LH_CASE(2) LH_CASE(3) LH_CASE(4) LH_CASE(5)
        default: return SFNO_EINVAL;
    }
#undef LH_CASE
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int legendre_f16_launch(bool analysis, const PgemmArgs& a, int n_work, hipStream_t s) {
    return analysis ? launch_f16<true>(a, n_work, s) : launch_f16<false>(a, n_work, s);
}

}  // namespace sfno
