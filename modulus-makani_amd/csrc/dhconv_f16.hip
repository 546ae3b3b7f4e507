// dhconv with fp32 accuracy on the fp16 matrix pipe of gfx950 (the default fp32 path for even channel counts):
//
//   y[b,o,l,m] = sum_i x[b,i,l,m] w[i,o,l]        (makani/models/common/contractions.py:130-136)
//
// An fp32 number scaled by a power of two into the range of fp16 is, to 22 of its 24 significant bits, the sum of
// two fp16 numbers (11 significant bits each): x 2^s = h0 + h1.  With both operands cut that way
//   x w = (a0 b0 + a0 b1 + a1 b0) 2^-(s+t)  up to  a1 b1  (below 2^-21 of the product) and the two cut-off tails,
// three v_mfma_f32_32x32x16_f16 per K = 16 step into the fp32 accumulator, each product exact.
//
// Per degree l the contraction is four real GEMMs on the real and imaginary parts,
//   Yr = Xr Wr + (-Xi) Wi,   Yi = Xr Wi + Xi Wr,
// with rows (m, b) of the spectral layout as A operands (read straight from HBM/L2, de-interleaved and cut in
// registers; -Xi costs one sign flip per packed pair) and the weights as B operands: the packed stream holds, per
// (degree, block of 32 NTC output channels, chunk of 16 input channels), the image of one LDS stage -- (Wr, Wi) x two
// fp16 planes x output channel x 16 input channels -- which the wavefronts move with global_load_lds_dwordx4 into a
// ring of three stages, two chunks ahead of the matrix instructions.  8 bytes per complex weight, read once.
//
// Scales.  fp16 keeps 11 significant bits only above 2^-14, so every operand row is brought close to the top of the
// range (magnitudes below 2^15) by a power of two, which costs no accuracy and is undone when the result is stored:
//   weights: one scale per (degree, output channel), from the largest |Re|, |Im| over the input channels, chosen when
//            the weights are packed;
//   activations: one scale per row (m, l, b), found while the row streams by.  A wavefront owns 32 rows and reads
//            each in chunks of 16 complex values; it keeps a bound on the row's exponent that is raised (with a few
//            bits of headroom) when a chunk exceeds it, and then rescales the row's partial sums by the same power of two.
// Entries much smaller than the largest entry of their row (by more than 2^17) keep fewer bits: the error of a
// product is bounded by 2^-21 |x w| + 2^-38 max|x| max|w|, where fp32 arithmetic has 2^-24 |x w|.
#include "dhconv_map.h"
#include "sfno_internal.h"

namespace sfno {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __fp16 fp16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));

constexpr int DHF_KC = 16;             // complex input channels per chunk: one matrix K step per part
constexpr int DHF_TOP = 14;            // scaled magnitudes stay below 2^(TOP + 1)
constexpr int DHF_HEAD = 3;            // bits of headroom left when a row's exponent bound is raised
constexpr int DHF_SH = DHF_TOP + 127;  // scaled = x * 2^(SH - E), E = biased exponent bound of the row
constexpr int DHF_STAGES = 3;

__device__ __forceinline__ unsigned int pk_rtz(float a, float b) {
    return __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_pkrtz(a, b));
}
// 16 bytes per lane from global memory to LDS base + 16 lane (M0 carries the base; the compiler reserves M0 and does not
// accept it on a clobber list: nothing else in this file may depend on M0 -- no indexed register arrays, no LDS-DMA builtins)
__device__ __forceinline__ void dhf_dma16(const void* g, unsigned lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_byte_addr) : "memory");
}
// byte offset, within one (part, plane) of a stage, of the 16-byte piece (output channel o, half kg of the chunk):
// the halves swap places every 8 channels so that the 16-byte reads of 16 consecutive lanes cover all banks
__host__ __device__ constexpr int dhf_piece(int o, int kg) { return o * 32 + ((kg ^ ((o >> 3) & 1)) * 16); }

// grid = dh_blocks workgroups (see dh_map), row groups of 128; a.nob = ceil(O / (32 NTC)); requires 2*I % 4 == 0
template <int NTC>
__global__ __launch_bounds__(256, 2) void dhconv_f16_kernel(DhconvArgs a) {
    constexpr int CO = 32 * NTC;                     // complex output channels per workgroup
    constexpr int STAGE = 4 * CO * 32;               // bytes: (Wr, Wi) x 2 planes x CO x 16 fp16
    constexpr int ND = STAGE / 4096;                 // direct-to-LDS loads per wavefront and chunk
    constexpr int NX = 4;                            // activation loads per lane and chunk
    __shared__ __align__(16) unsigned char lds[DHF_STAGES * STAGE];

    int l, ob, r0, ncols, rot;
    if (!dh_map(a, 128, l, ob, r0, ncols, rot)) return;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wslot = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave = (wslot + rot) & 3;
    const bool active = r0 + 32 * wave < ncols;
    const int nc = a.nc;                                           // chunks of 16 complex input channels
    const int kg = lane >> 5, cl = lane & 31;
    const unsigned lds0 = (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)lds);

    const int n = min(r0 + 32 * wave + cl, ncols - 1);
    const int mm = n / a.B, bb = n - mm * a.B;
    const float* xrow = a.X + ((int64_t)mm * a.L + l) * a.ld_in + (int64_t)bb * a.I2;
    // packed weights of (l, ob): nc stage images; this wavefront moves bytes [ND wslot KiB, ND (wslot + 1) KiB) of each
    const unsigned char* wsrc = reinterpret_cast<const unsigned char*>(a.W) + ((int64_t)l * a.nob + ob) * nc * STAGE + wslot * (ND * 1024) + lane * 16;
    const unsigned wdst = lds0 + wslot * (ND * 1024);

    floatx16 yr[NTC], yi[NTC];
#pragma unroll
    for (int t = 0; t < NTC; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            yr[t][v] = 0.0f;
            yi[t][v] = 0.0f;
        }
    int E = 0;                 // biased exponent bound of my row (lanes cl and cl + 32 hold the same row and agree)
    int pend = 0;              // change of E by the last chunk that was cut, not yet applied to the partial sums

    // my 8 complex activations of chunk c: i = 16c + 8kg .. +7, (re, im) interleaved (clamped in groups of two complex
    // values; the weights are zero past I)
    auto x_load = [&](int c, f4 (&xr)[NX]) {
        const int k = 2 * DHF_KC * c + 16 * kg;
#pragma unroll
        for (int j = 0; j < NX; ++j) xr[j] = *reinterpret_cast<const f4*>(xrow + min(k + 4 * j, a.I2 - 4));
    };
    auto w_dma = [&](int c, int stage) {
#pragma unroll
        for (int j = 0; j < ND; ++j) dhf_dma16(wsrc + (int64_t)c * STAGE + j * 1024, wdst + stage * STAGE + j * 1024);
    };
    // exponent bound of the row after this chunk
    auto bound = [&](const f4 (&xr)[NX]) {
        float mx = 0.f;
#pragma unroll
        for (int j = 0; j < NX; ++j)
            mx = __builtin_fmaxf(__builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fabsf(xr[j][0]), __builtin_fabsf(xr[j][1]))),
                                 __builtin_fmaxf(__builtin_fabsf(xr[j][2]), __builtin_fabsf(xr[j][3])));
        const unsigned int mb = __builtin_bit_cast(unsigned int, mx);
        // the other half of the row's chunk sits 32 lanes away
        const auto sw = __builtin_amdgcn_permlane32_swap(mb, mb, false, false);
        const int eb = (int)(max(sw[0], sw[1]) >> 23);
        const int en = eb > E ? eb + DHF_HEAD : E;
        pend = E - en;
        E = en;
    };
    // planes of the chunk: pl[0], pl[1] = Xr (upper, lower part), pl[2], pl[3] = Xi; word e of a plane holds the channels
    // 2e, 2e + 1 of the lane's eight
    auto cut_quad = [&](const f4 (&xr)[NX], int e, u4 (&pl)[4]) {
        const f4 s = xr[e];
        const int sh = DHF_SH - E;
        const float ra = __builtin_ldexpf(s[0], sh), ia = __builtin_ldexpf(s[1], sh), rb = __builtin_ldexpf(s[2], sh), ib = __builtin_ldexpf(s[3], sh);
        const fp16x2 hr = __builtin_amdgcn_cvt_pkrtz(ra, rb), hi = __builtin_amdgcn_cvt_pkrtz(ia, ib);
        pl[0][e] = __builtin_bit_cast(unsigned int, hr);
        pl[1][e] = pk_rtz(__builtin_fmaf((float)hr[0], -1.0f, ra), __builtin_fmaf((float)hr[1], -1.0f, rb));
        pl[2][e] = __builtin_bit_cast(unsigned int, hi);
        pl[3][e] = pk_rtz(__builtin_fmaf((float)hi[0], -1.0f, ia), __builtin_fmaf((float)hi[1], -1.0f, ib));
    };
    // partial sums follow their row's scale: D row 8 (v / 4) + 4 kg + v % 4 belongs to the lanes of that number
    auto rescale = [&]() {
        if (__builtin_amdgcn_ballot_w64(pend != 0) == 0) return;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int d = __builtin_amdgcn_ds_bpermute(4 * (8 * (v >> 2) + 4 * kg + (v & 3)), pend);
#pragma unroll
            for (int t = 0; t < NTC; ++t) {
                yr[t][v] = __builtin_ldexpf(yr[t][v], d);
                yi[t][v] = __builtin_ldexpf(yi[t][v], d);
            }
        }
    };
    // one chunk of matrix instructions on stage `stage` with the planes pc
    const int frag = dhf_piece(cl, kg);
    auto contract = [&](int stage, const u4 (&pc)[4]) {
        const unsigned char* sb = lds + stage * STAGE + frag;
        const f16x8 xr0 = __builtin_bit_cast(f16x8, pc[0]), xr1 = __builtin_bit_cast(f16x8, pc[1]);
        const f16x8 xi0 = __builtin_bit_cast(f16x8, pc[2]), xi1 = __builtin_bit_cast(f16x8, pc[3]);
        // -Xi: one sign flip per packed pair
        const f16x8 ni0 = __builtin_bit_cast(f16x8, pc[2] ^ 0x80008000u), ni1 = __builtin_bit_cast(f16x8, pc[3] ^ 0x80008000u);
#pragma unroll
        for (int t = 0; t < NTC; ++t) {
            const f16x8 wr0 = *reinterpret_cast<const f16x8*>(sb + (0 * CO + 32 * t) * 32), wr1 = *reinterpret_cast<const f16x8*>(sb + (1 * CO + 32 * t) * 32);
            const f16x8 wi0 = *reinterpret_cast<const f16x8*>(sb + (2 * CO + 32 * t) * 32), wi1 = *reinterpret_cast<const f16x8*>(sb + (3 * CO + 32 * t) * 32);
            // smallest terms first; the two sums alternate so that no instruction waits for the one before it
            yr[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xr1, wr0, yr[t], 0, 0, 0);
            yi[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xr1, wi0, yi[t], 0, 0, 0);
            yr[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ni1, wi0, yr[t], 0, 0, 0);
            yi[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xi1, wr0, yi[t], 0, 0, 0);
            yr[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xr0, wr1, yr[t], 0, 0, 0);
            yi[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xr0, wi1, yi[t], 0, 0, 0);
            yr[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ni0, wi1, yr[t], 0, 0, 0);
            yi[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xi0, wr1, yi[t], 0, 0, 0);
            yr[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xr0, wr0, yr[t], 0, 0, 0);
            yi[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xr0, wi0, yi[t], 0, 0, 0);
            yr[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ni0, wi0, yr[t], 0, 0, 0);
            yi[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xi0, wr0, yi[t], 0, 0, 0);
        }
    };

    // Pipeline, three weight stages.  Iteration c: cut the activations of chunk c + 1 (requested during iteration c - 1;
    // the compiler's wait for them also covers this wavefront's pieces of the weights of chunk c + 1, which were requested
    // before them), barrier (every wavefront's pieces of chunk c + 1 have landed and every wavefront is done reading
    // chunk c - 1), request chunk c + 2 into the stage of chunk c - 1, contract chunk c, and let the partial sums follow
    // the scale chunk c + 1 was cut with.  The requests thus have one contraction (48 or 24 matrix instructions) to land.
    // Only the weight requests are written in assembly (the compiler would make every LDS read wait for them); their
    // wait is the explicit one before the barrier.
    f4 X0[NX], X1[NX];
    u4 P0[4], P1[4];
    if (active) x_load(0, X0);
    w_dma(0, 0);
    if (nc > 1) {
        if (active) x_load(1, X1);
        w_dma(1, 1);
    }
    if (active) {
        bound(X0);
#pragma unroll
        for (int e = 0; e < NX; ++e) cut_quad(X0, e, P0);
    }
    pend = 0;                                                       // nothing has been summed yet

    auto iter = [&](int c, int stage, const u4 (&pc)[4], u4 (&pn)[4], f4 (&xc)[NX], const f4 (&xn)[NX]) {
        const bool more1 = c + 1 < nc, more2 = c + 2 < nc;         // uniform over the workgroup
        if (active && more1) {
            bound(xn);
#pragma unroll
            for (int e = 0; e < NX; ++e) cut_quad(xn, e, pn);
        }
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if (more2) {
            // xc held chunk c, cut during the previous iteration
            if (active) x_load(c + 2, xc);
            w_dma(c + 2, stage == 0 ? 2 : stage - 1);
        }
        if (active) {
            contract(stage, pc);
            rescale();
            pend = 0;
        }
    };
    int c = 0, stage = 0;
    for (; c + 1 < nc; c += 2) {
        iter(c, stage, P0, P1, X0, X1);
        stage = stage == 2 ? 0 : stage + 1;
        iter(c + 1, stage, P1, P0, X1, X0);
        stage = stage == 2 ? 0 : stage + 1;
    }
    if (c < nc) iter(c, stage, P0, P1, X0, X1);

    if (!active) return;
    // Undo the scales: row by 2^(E - SH) (the partial sums carry the scale of the last cut), column by the factor stored
    // with the weights.
    float cinv[NTC];
#pragma unroll
    for (int t = 0; t < NTC; ++t) cinv[t] = a.cinv[(int64_t)l * (a.nob * CO) + CO * ob + 32 * t + cl];
    const int Efinal = E;
    const int nn0 = r0 + 32 * wave + 4 * kg;                       // my first row; the others are 8 (v / 4) + v % 4 further on
    if (a.B == 1 && r0 + 32 * wave + 32 <= ncols && 2 * (CO * ob + CO) <= a.O2) {
        // one sample and no row or channel of my tile outside the tensor: row = order, one address, constant steps
        float* o = a.Y + ((int64_t)nn0 * a.L + l) * a.ld_out + 2 * (CO * ob + cl);
        const int64_t rstep = (int64_t)a.L * a.ld_out;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int er = __builtin_amdgcn_ds_bpermute(4 * (8 * (v >> 2) + 4 * kg + (v & 3)), Efinal);
            float* orow = o + (8 * (v >> 2) + (v & 3)) * rstep;
#pragma unroll
            for (int t = 0; t < NTC; ++t)
                *reinterpret_cast<f2*>(orow + 64 * t) = f2{__builtin_ldexpf(yr[t][v], er - DHF_SH) * cinv[t], __builtin_ldexpf(yi[t][v], er - DHF_SH) * cinv[t]};
        }
        return;
    }
    if ((a.B & (a.B - 1)) == 0 && r0 + 32 * wave + 32 <= ncols && 2 * (CO * ob + CO) <= a.O2) {
        // a power-of-two number of samples, whole tile inside: (order, sample) of a row by shift and mask, no checks
        const int lb = 31 - __builtin_clz(a.B);
        float* o = a.Y + (int64_t)l * a.ld_out + 2 * (CO * ob + cl);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int er = __builtin_amdgcn_ds_bpermute(4 * (8 * (v >> 2) + 4 * kg + (v & 3)), Efinal);
            const int nn = nn0 + 8 * (v >> 2) + (v & 3);
            float* orow = o + (int64_t)(nn >> lb) * a.L * a.ld_out + (int64_t)(nn & (a.B - 1)) * a.O2;
#pragma unroll
            for (int t = 0; t < NTC; ++t)
                *reinterpret_cast<f2*>(orow + 64 * t) = f2{__builtin_ldexpf(yr[t][v], er - DHF_SH) * cinv[t], __builtin_ldexpf(yi[t][v], er - DHF_SH) * cinv[t]};
        }
        return;
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int er = __builtin_amdgcn_ds_bpermute(4 * (8 * (v >> 2) + 4 * kg + (v & 3)), Efinal);
        const int nn = nn0 + 8 * (v >> 2) + (v & 3);
        if (nn >= ncols) continue;
        const int m2 = nn / a.B, b2 = nn - m2 * a.B;
        float* orow = a.Y + ((int64_t)m2 * a.L + l) * a.ld_out + (int64_t)b2 * a.O2;
#pragma unroll
        for (int t = 0; t < NTC; ++t) {
            const int oc = 2 * (CO * ob + 32 * t + cl);
            if (oc < a.O2)
                *reinterpret_cast<f2*>(orow + oc) = f2{__builtin_ldexpf(yr[t][v], er - DHF_SH) * cinv[t], __builtin_ldexpf(yi[t][v], er - DHF_SH) * cinv[t]};
        }
    }
}

// cmax[l][o] = largest |Re|, |Im| of w[.][o][l] over the input channels (adjoint: of w[o][.][l], w being [O][I][L]).  A thread
// takes DHF_CMAX_I input channels of one (o, l) and joins the others with an integer atomic maximum on the bit pattern (the
// values are magnitudes: their order as unsigned integers is their order as floats, a NaN ranks above all and stays); cmax is
// cleared by the kernel in front.  grid (ceil(O L / 256), ceil(I / DHF_CMAX_I))
constexpr int DHF_CMAX_I = 16;
__global__ __launch_bounds__(256) void dhconv_colmax_clear_kernel(float* __restrict__ cmax, int64_t n) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < n) cmax[idx] = 0.f;
}
__global__ __launch_bounds__(256) void dhconv_colmax_kernel(const float2* __restrict__ w, float* __restrict__ cmax, int I, int O, int L, int adjoint) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;     // o * L + l
    if (idx >= (int64_t)O * L) return;
    const int o = (int)(idx / L), l = (int)(idx - (int64_t)o * L);
    const int i0 = blockIdx.y * DHF_CMAX_I, i1 = min(i0 + DHF_CMAX_I, I);
    float mx = 0.f;
#pragma unroll 4
    for (int i = i0; i < i1; ++i) {
        const float2 z = adjoint ? w[((int64_t)o * I + i) * L + l] : w[((int64_t)i * O + o) * L + l];
        mx = fmaxf(mx, fmaxf(fabsf(z.x), fabsf(z.y)));
    }
    atomicMax(reinterpret_cast<unsigned int*>(cmax) + ((int64_t)l * O + o), __float_as_uint(mx));
}

// Writes the stage images.  packed[l][ob][c] = [part (Re, Im)][plane][o (CO)][two 16-byte halves, see dhf_piece]: the half kg
// of channel o holds plane `plane` of part `part` of w[16c + 8kg + e][CO ob + o][l] * 2^s[l][o], e = 0..7, as fp16; plane 0 is
// the value rounded to fp16, plane 1 the rounded remainder; zero outside the weight (adjoint: the weight is conj(w[o][i][l]),
// w being [O][I][L]).  cinv[l][CO ob + o] = 2^-s.  The parameter has l fastest, the stream has it slowest: a workgroup moves
// the 16 x 32 channel pairs of one (c, ob, quarter of the channel block) for 8 degrees through LDS, reading 64 contiguous
// bytes per pair.  grid (nc * nob * (CO / 32), ceil(L / 8)), block 256
template <int NTC>
__global__ __launch_bounds__(256) void dhconv_pack_f16_kernel(const float2* __restrict__ w, const float* __restrict__ cmax, unsigned char* __restrict__ packed,
                                                              float* __restrict__ cinv, int I, int O, int L, int nob, int nc, int adjoint) {
    constexpr int CO = 32 * NTC, STAGE = 4 * CO * 32;
    __shared__ float2 tile[512][9];                  // [pair = ii * 32 + o][degree], padded
    const int q = blockIdx.x % NTC, c = (blockIdx.x / NTC) % nc, ob = blockIdx.x / (NTC * nc);
    const int l0 = blockIdx.y * 8;
    const int tid = threadIdx.x, dl = tid & 7;
#pragma unroll 4
    for (int pass = 0; pass < 16; ++pass) {
        const int pr = pass * 32 + (tid >> 3);       // eight lanes per pair: one 64-byte segment
        const int ii = pr >> 5, o = pr & 31;
        const int i = DHF_KC * c + ii, oo = CO * ob + 32 * q + o, l = l0 + dl;
        float2 z = make_float2(0.f, 0.f);
        if (i < I && oo < O && l < L) {
            if (adjoint) {
                z = w[((int64_t)oo * I + i) * L + l];
                z.y = -z.y;
            } else {
                z = w[((int64_t)i * O + oo) * L + l];
            }
        }
        tile[pr][dl] = z;
    }
    __syncthreads();
    // thread -> one 16-byte piece per degree: (part, plane, half kg, channel o)
    const int o = tid & 31, kg = (tid >> 5) & 1, plane = (tid >> 6) & 1, part = tid >> 7;
    const int oo = CO * ob + 32 * q + o;
    for (int d = 0; d < 8; ++d) {
        const int l = l0 + d;
        if (l >= L) break;
        // scale: the column's largest magnitude lands in [2^TOP, 2^(TOP+1))
        int sh = 0;
        if (oo < O) {
            const unsigned int mb = __builtin_bit_cast(unsigned int, cmax[(int64_t)l * O + oo]);
            if (mb != 0) sh = DHF_SH - (int)(mb >> 23);
        }
        if (c == 0 && tid < 32) cinv[(int64_t)l * (nob * CO) + CO * ob + 32 * q + o] = __builtin_ldexpf(1.0f, -sh);
        u4 piece;
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
            unsigned short h[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const float2 z = tile[(8 * kg + 2 * e2 + u) * 32 + o][d];
                const float v = __builtin_ldexpf(part ? z.y : z.x, sh);
                const _Float16 v0 = (_Float16)v;
                const _Float16 v1 = (_Float16)(v - (float)v0);
                h[u] = __builtin_bit_cast(unsigned short, plane ? v1 : v0);
            }
            piece[e2] = (unsigned int)h[0] | ((unsigned int)h[1] << 16);
        }
        unsigned char* dst = packed + (((int64_t)l * nob + ob) * nc + c) * STAGE + ((part * 2 + plane) * CO + 32 * q) * 32 + dhf_piece(o, kg);
        *reinterpret_cast<u4*>(dst) = piece;
    }
}

int dhconv_f16_ntc(int O) { return O > 64 ? 4 : 2; }

int dhconv_pack_f16_launch(const float2* w, void* packed, float* cinv, float* cmax, int I, int O, int L, int adjoint, hipStream_t s) {
    const int ntc = dhconv_f16_ntc(O);
    const int nob = (O + 32 * ntc - 1) / (32 * ntc), nc = (I + DHF_KC - 1) / DHF_KC;
    if ((int64_t)nob * nc * ntc > 0x7fffffffLL || (L + 7) / 8 > 65535) return SFNO_EUNSUPPORTED;
    const int64_t cols = (int64_t)O * L;
    if ((cols + 255) / 256 > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    if ((I + DHF_CMAX_I - 1) / DHF_CMAX_I > 65535) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(dhconv_colmax_clear_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, s, cmax, cols);
    hipLaunchKernelGGL(dhconv_colmax_kernel, dim3((unsigned)((cols + 255) / 256), (unsigned)((I + DHF_CMAX_I - 1) / DHF_CMAX_I)), dim3(256), 0, s, w, cmax, I,
                       O, L, adjoint);
    const dim3 grid((unsigned)(nob * nc * ntc), (unsigned)((L + 7) / 8));
    if (ntc == 4)
        hipLaunchKernelGGL((dhconv_pack_f16_kernel<4>), grid, dim3(256), 0, s, w, cmax, reinterpret_cast<unsigned char*>(packed), cinv, I, O, L, nob, nc, adjoint);
    else
        hipLaunchKernelGGL((dhconv_pack_f16_kernel<2>), grid, dim3(256), 0, s, w, cmax, reinterpret_cast<unsigned char*>(packed), cinv, I, O, L, nob, nc, adjoint);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int dhconv_f16_launch(const DhconvArgs& a, hipStream_t s) {
    const int64_t rows_max = (int64_t)a.M * a.B;
    if (rows_max <= 0 || a.L <= 0) return SFNO_OK;
    if (a.I2 % 4 != 0 || a.ld_in % 4 != 0 || !a.cinv) return SFNO_EUNSUPPORTED;
    const int64_t blocks = dh_blocks(a, 128);
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    if (dhconv_f16_ntc(a.O2 / 2) == 4)
        hipLaunchKernelGGL((dhconv_f16_kernel<4>), dim3((unsigned)blocks), dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL((dhconv_f16_kernel<2>), dim3((unsigned)blocks), dim3(256), 0, s, a);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
