// Pointwise (1x1 convolution) tail of the SFNO block on bf16 MFMA, for bf16 NCHW activations:
//   y[b][o][p] = epilogue( sum_k w[o][k] x[b][k][p] ),   p = pixel (h, w) flattened
// with bias, exact GELU and "+ scale * addend + shift" (instance norm of the addend folded into a
// per-(b, o) affine) fused into the epilogue, plus the two small passes an instance norm needs
// (row statistics -> scale/shift, and scale/shift + activation).  Replaces the nn.Conv2d(k=1) /
// nn.InstanceNorm2d / nn.GELU sequences of makani/models/networks/sfnonet.py:246-262 and
// makani/models/common/layers.py:86-133,136-216 when the activations are bf16.
//
// GEMM kernel.  v_mfma_f32_32x32x16_bf16 wants 8 consecutive k per lane for both operands, but the
// activations are pixel-contiguous.  No transposition is needed: a lane reads 2 consecutive pixels
// (4 bytes) of 8 consecutive k rows and regroups them with byte permutes into two B fragments, one
// per pixel of its pair; MFMA column q of N-tile t then stands for pixel 2q + t, so every lane ends up
// with 2 consecutive pixels of each output row and stores them as one 4-byte piece.
// Two kernels.  Convolutions with at most 96 output channels (pw_gemm_kernel): a wavefront owns 96 rows x 64
// pixels, eight wavefronts side by side along the pixels; weights come from global memory (L2 resident) as A
// fragments, packed so that a fragment is 1 KiB of consecutive memory, activations through a triple-buffered LDS
// stage, both prefetched in registers.  All others (pw_gemm_dma_kernel, further down): 384 rows x 256 pixels per
// workgroup with both operand streams loaded straight into LDS.
#include "sfno_internal.h"
#include <type_traits>

namespace sfno {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int PW_MT = 3;          // 32-row tiles per wavefront
constexpr int PW_ROWS = 32 * PW_MT;
constexpr int PW_KC = 16;         // k rows per MFMA K step
constexpr int PW_KS = 2;          // MFMA K steps per chunk (one LDS stage, one barrier)
constexpr int PW_KALIGN = 128;    // K is padded to whole unrolled loop bodies (PW_KC * prefetch distance)

__device__ __forceinline__ float bf16_to_f(unsigned short h) { return __uint_as_float((unsigned int)h << 16); }
__device__ __forceinline__ unsigned short f_to_bf16(float f) { return __builtin_bit_cast(unsigned short, (__bf16)f); }
// two floats rounded to nearest-even bf16 in one word, lo in the low half (the hardware conversion takes a pair: one
// instruction where two single conversions need a shift and an or as well)
__device__ __forceinline__ unsigned int bf16_pair(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    const floatx2 f = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(f, bf16x2));
}

// p[i] for a wavefront-uniform i, of an array the kernel never writes: read through the scalar unit, whose loads do not
// count against the vector memory counter
__device__ __forceinline__ float uniform_load(const float* p, int64_t i) {
    return reinterpret_cast<const __attribute__((address_space(4))) float*>(reinterpret_cast<uintptr_t>(p))[i];
}

// exact (erf) GELU for bf16 outputs.  gelu(x) = max(x, 0) - |x| erfc(|x| / sqrt 2) / 2 for both signs (no cancellation in
// the negative tail), and erfc is evaluated as 2^Q(|x|): log2 erfc(t / sqrt 2) is smooth, a degree-6 polynomial in t follows it
// to 1.1e-4 on [0, 6.5] (relative error of erfc 7e-5, a thirtieth of the half ulp of the bf16 result).  Beyond 6.5 t is
// clamped: the term is then below 3e-10 |x| / 6.5 in magnitude, where the formula x (1 + erf(x / sqrt 2)) / 2 in fp32
// arithmetic has long returned -0.  Ten full-rate instructions and one exp2, where a rational form needs a reciprocal as well.
__device__ __forceinline__ float gelu(float x) {
    // (the median of three stands for min and max: one instruction each, where fminf / fmaxf first canonicalise their operand)
    const float t = __builtin_amdgcn_fmed3f(fabsf(x), 0.f, 6.5f);
    float q = fmaf(t, 2.008575651e-05f, -5.615057212e-04f);
    q = fmaf(t, q, 6.880626770e-03f);
    q = fmaf(t, q, -5.027262948e-02f);
    q = fmaf(t, q, -4.624537704e-01f);
    q = fmaf(t, q, -1.149621597e+00f);
    // (the factor 1/2 rides in the exponent: the constant term is the fitted -1.062872110e-04 minus one)
    q = fmaf(t, q, -1.000106287211f);
    return fmaf(-fabsf(x), __builtin_amdgcn_exp2f(q), __builtin_amdgcn_fmed3f(x, 0.f, __builtin_inff()));
}

// WM = wavefronts along the output rows: 4 (x 2 along pixels: 384 rows x 128 pixels per workgroup) or
// 1 (x 8 along pixels: 96 rows x 512 pixels, for convolutions with few output channels)
// NT = pixels per lane = N tiles per wavefront: 2 (eight wavefronts of 96 x 64, two per SIMD) or 4 (four wavefronts of
// 96 x 128, one per SIMD, half the weight-fragment traffic per MFMA)
template <int WM, int NT>
__global__ __launch_bounds__(NT == 2 ? 512 : 256) void pw_gemm_kernel(PointwiseArgs a) {
    constexpr int NW = (NT == 2) ? 8 : 4;         // wavefronts per workgroup
    constexpr int PW_THREADS = 64 * NW;
    constexpr int PW_PX = 32 * NT;                // pixels per wavefront
    constexpr int WN = NW / WM;
    constexpr int WPX = WN * PW_PX;               // pixels per workgroup
    constexpr int PITCH = WPX * 2 + 16;           // bytes per LDS row
    constexpr int CK = PW_KC * PW_KS;             // k rows per chunk = per loop step
    constexpr int STAGE = CK * PITCH;
    constexpr int D = (WM == 4) ? 4 : 2;          // prefetch distance in chunks
    constexpr int XW = CK * WPX * 2 / (16 * PW_THREADS);   // 16-byte pieces of the activation chunk per thread
    static_assert(PW_KALIGN % (CK * D) == 0, "loop body divides the padded K");
    static_assert(CK * WPX * 2 == XW * 16 * PW_THREADS, "chunk split evenly over the threads");
    __shared__ __align__(16) unsigned char lds[3 * STAGE];

    const int xcd = blockIdx.x & 7, qid = blockIdx.x >> 3;
    const int ob = qid % a.n_oblk;
    const int64_t strip_lin = (int64_t)(qid / a.n_oblk) * 8 + xcd;
    if (strip_lin >= a.n_strips * a.B) return;
    const int b = (int)(strip_lin / a.n_strips);
    const int64_t pw0 = (strip_lin - (int64_t)b * a.n_strips) * WPX;      // first pixel of the workgroup

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int q = lane & 31, ko = lane >> 5;
    const int o0 = ob * (PW_ROWS * WM) + (wave / WN) * PW_ROWS;
    const int pxw = (wave % WN) * PW_PX;                                  // wavefront's pixel offset inside the stage

    // input channels k < K1 come from X, the others (if any) from X2: a convolution over the concatenation of two tensors
    const int K1 = a.X2 ? a.K1 : a.K;
    const unsigned short* __restrict__ X = a.X + (int64_t)b * K1 * a.P;
    const unsigned short* __restrict__ X2 = a.X2 ? a.X2 + (int64_t)b * (a.K - K1) * a.P : X;
    // this thread's 16-byte pieces (8 pixels of one k row) of an activation chunk of CK rows x WPX pixels
    int xr[XW], loff[XW];
    int64_t xoff[XW];
#pragma unroll
    for (int u = 0; u < XW; ++u) {
        const int e = tid + PW_THREADS * u;
        xr[u] = e / (WPX / 8);
        const int c8 = e - xr[u] * (WPX / 8);
        xoff[u] = min(pw0 + 8 * c8, a.P - 8);                             // past the end: valid pixels, masked at the store
        loff[u] = xr[u] * PITCH + 16 * c8;
    }
    // weight fragments: packed blocks of 32 rows x 16 k, 16 bytes per lane (see pointwise_pack_kernel)
    const int nc16 = a.Kpad / PW_KC;
    const unsigned short* wrow[PW_MT];
#pragma unroll
    for (int mt = 0; mt < PW_MT; ++mt) wrow[mt] = a.W + ((int64_t)(o0 / 32 + mt) * nc16 * 64 + lane) * 8;

    // Kpad is a multiple of CK * D: the unrolled loop below has no conditional steps, which keeps the
    // compiler's count of loads in flight exact (a skipped step would make it wait for nearly all of them)
    const int nchunks = a.Kpad / CK;
    u32x4 araw[D][PW_KS][PW_MT];
    u32x4 xraw[D][XW];

    auto load_a = [&](int c, u32x4 (&dst)[PW_KS][PW_MT]) {
        const int cc = min(c, nchunks - 1);
#pragma unroll
        for (int ks = 0; ks < PW_KS; ++ks)
#pragma unroll
            for (int mt = 0; mt < PW_MT; ++mt) dst[ks][mt] = *reinterpret_cast<const u32x4*>(wrow[mt] + (cc * PW_KS + ks) * 512);
    };
    auto load_x = [&](int c, u32x4 (&dst)[XW]) {
        const int cc = min(c, nchunks - 1);
#pragma unroll
        for (int u = 0; u < XW; ++u) {
            const int k = min(cc * CK + xr[u], a.K - 1);                  // rows past K meet zero weights
            dst[u] = *reinterpret_cast<const u32x4*>((k < K1 ? X + (int64_t)k * a.P : X2 + (int64_t)(k - K1) * a.P) + xoff[u]);
        }
    };
    auto store_x = [&](int stage, const u32x4 (&src)[XW]) {
#pragma unroll
        for (int u = 0; u < XW; ++u) *reinterpret_cast<u32x4*>(&lds[stage * STAGE + loff[u]]) = src[u];
    };

    f32x16 acc[PW_MT][NT];
#pragma unroll
    for (int mt = 0; mt < PW_MT; ++mt)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mt][t][v] = 0.f;

    // prologue: chunks 0 and 1 into LDS, chunks 2..D+1 of the activations and 0..D-1 of the weights in flight
    {
        u32x4 x0[XW], x1[XW];
        load_x(0, x0);
        load_x(1, x1);
#pragma unroll
        for (int d = 0; d < D; ++d) {
            load_x(d + 2, xraw[(d + 2) % D]);
            load_a(d, araw[d]);
        }
        store_x(0, x0);
        store_x(1, x1);
    }
    __syncthreads();

    // B fragments: lane = pixel group q (NT pixels), k rows 8 ko .. 8 ko + 7 of a 16-row sub-step.  The raw words of the next
    // sub-step are read while the MFMAs of the current one run (hence three stages: chunk c + 1 is read during chunk c).
    typedef unsigned int rw_t __attribute__((ext_vector_type(NT / 2)));
    const unsigned char* fragbase = &lds[0] + (8 * ko) * PITCH + (pxw + NT * q) * 2;
    rw_t rw[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) rw[r] = *reinterpret_cast<const rw_t*>(fragbase + r * PITCH);
    int s0 = 0;                                    // stage of chunk c
    for (int c0 = 0; c0 < nchunks; c0 += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            const int c = c0 + u;
            const int s1 = (s0 == 2) ? 0 : s0 + 1; // stage of chunk c + 1
            const int s2 = (s1 == 2) ? 0 : s1 + 1; // stage of chunk c + 2
#pragma unroll
            for (int ks = 0; ks < PW_KS; ++ks) {
                u32x4 bf[NT];
#pragma unroll
                for (int pp = 0; pp < NT / 2; ++pp)
#pragma unroll
                    for (int h = 0; h < 4; ++h) {
                        bf[2 * pp][h] = __builtin_amdgcn_perm(rw[2 * h + 1][pp], rw[2 * h][pp], 0x05040100u);
                        bf[2 * pp + 1][h] = __builtin_amdgcn_perm(rw[2 * h + 1][pp], rw[2 * h][pp], 0x07060302u);
                    }
                const unsigned char* fb = (ks + 1 < PW_KS) ? fragbase + s0 * STAGE + (ks + 1) * PW_KC * PITCH : fragbase + s1 * STAGE;
#pragma unroll
                for (int r = 0; r < 8; ++r) rw[r] = *reinterpret_cast<const rw_t*>(fb + r * PITCH);
#pragma unroll
                for (int mt = 0; mt < PW_MT; ++mt) {
                    const bf16x8 av = __builtin_bit_cast(bf16x8, araw[u][ks][mt]);
#pragma unroll
                    for (int t = 0; t < NT; ++t)
                        acc[mt][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, __builtin_bit_cast(bf16x8, bf[t]), acc[mt][t], 0, 0, 0);
                }
            }
            // hand chunk c + 2 to its stage, then refill the two register slots
            store_x(s2, xraw[(u + 2) % D]);
            load_x(c + 2 + D, xraw[(u + 2) % D]);
            load_a(c + D, araw[u]);
            __syncthreads();
            s0 = s1;
        }
    }

    // epilogue: lane holds rows 8 (v / 4) + 4 ko + v % 4 of each 32-row tile and pixels NT q .. NT q + NT - 1
    const int64_t px = pw0 + pxw + NT * q;
    if (px >= a.P) return;
    unsigned short* __restrict__ Y = a.Y + (int64_t)b * a.O * a.P;
    const unsigned short* __restrict__ R = a.addend ? a.addend + (int64_t)b * a.O * a.P : nullptr;
#pragma unroll
    for (int mt = 0; mt < PW_MT; ++mt) {
        rw_t rv[16];
        if (R) {
            // all addend loads of the tile first
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int o = min(o0 + 32 * mt + 8 * (v >> 2) + 4 * ko + (v & 3), a.O - 1);
                rv[v] = *reinterpret_cast<const rw_t*>(R + (int64_t)o * a.P + px);
            }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int o = o0 + 32 * mt + 8 * (v >> 2) + 4 * ko + (v & 3);
            if (o >= a.O) continue;
            const float bs = a.bias ? a.bias[o] : 0.f;
            float y[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) y[t] = acc[mt][t][v] + bs;
            if (a.act == SFNO_ACT_GELU) {
#pragma unroll
                for (int t = 0; t < NT; ++t) y[t] = gelu(y[t]);
            }
            if (R) {
                const float sc = a.add_scale ? a.add_scale[(int64_t)b * a.O + o] : 1.f;
                const float sh = a.add_shift ? a.add_shift[(int64_t)b * a.O + o] : 0.f;
#pragma unroll
                for (int pp = 0; pp < NT / 2; ++pp) {
                    y[2 * pp] += fmaf(sc, __uint_as_float(rv[v][pp] << 16), sh);
                    y[2 * pp + 1] += fmaf(sc, __uint_as_float(rv[v][pp] & 0xffff0000u), sh);
                }
            }
            rw_t out;
#pragma unroll
            for (int pp = 0; pp < NT / 2; ++pp) out[pp] = bf16_pair(y[2 * pp], y[2 * pp + 1]);
            *reinterpret_cast<rw_t*>(Y + (int64_t)o * a.P + px) = out;
        }
    }
}

// ---- tall variant with direct-to-LDS loads ----------------------------------------------------------
// For O > 96 the kernel above is bound by the weight fragments every wavefront pulls through L1 for only 6 MFMAs
// each.  This variant gives a wavefront 96 rows x 128 pixels (3 x 4 tiles, 192 accumulator registers), eight
// wavefronts per workgroup (384 rows x 256 pixels, half the weight traffic per pixel), and moves both operand
// streams with global_load_lds_dwordx4: lane i's 16 bytes land at LDS base + 16 i, no staging registers.
//
// One persistent workgroup per CU walks its tiles as one unbroken stream of 32-row K chunks, so the operands of the
// next tile are already in LDS when the stores of the current one leave.  A read only reaches the HBM rate with
// some 50 KB in flight per CU, and the memory counter of a wavefront retires in order, so a wavefront that waits for
// a weight block (an L2 hit) would also wait for every activation block it asked for earlier.  The two streams
// therefore belong to different wavefronts: wavefronts 0-3 fetch the weights into three stages of 24 KiB, wavefronts
// 4-7 the activations into five stages of 16 KiB; a stage is asked for again as soon as every wavefront has read it, so
// two to three weight chunks and four to five activation chunks (64-80 KiB) are on their way or waiting.  The loads are
// issued from inline assembly (the compiler would order every LDS read behind all outstanding direct-to-LDS loads)
// and the waits are written out by hand.  Other memory operations of a wavefront (the epilogue's stores and addend
// loads) are older than the loads a wait is meant for or younger than all of them; either way the wait covers
// at least the loads it is meant for.
constexpr int DM_MT = 3, DM_NT = 4;
constexpr int DM_ROWS = 4 * 32 * DM_MT;          // 384 rows per workgroup
constexpr int DM_PX = 2 * 32 * DM_NT;            // 256 pixels per workgroup
constexpr int DM_CK = 32;                        // k rows per chunk
constexpr int DM_ABYTES = 2 * (DM_ROWS / 32) * 1024;   // weight stage: 24 fragment blocks of 1 KiB
constexpr int DM_XBLK = 1024 + 16;               // two pixel rows of the chunk (2 x 512 bytes) + padding
constexpr int DM_XBYTES = (DM_CK / 2) * DM_XBLK; // activation stage
constexpr int DM_WSTAGES = 3, DM_XSTAGES = 5;    // chunks in LDS or on their way, per stream
constexpr int DM_XBASE = DM_WSTAGES * DM_ABYTES;
constexpr int DM_LDS = DM_XBASE + DM_XSTAGES * DM_XBYTES;
static_assert(DM_LDS <= 160 * 1024, "one workgroup per CU");

// M0 carries the LDS destination.  The compiler refuses "m0" in a clobber list (a reserved register), so nothing may
// keep a value in M0 across this call: the kernels that use it index no register array dynamically and use no
// readlane/movrel/sendmsg around it.
__device__ __forceinline__ void dma16(const void* g, unsigned lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_byte_addr) : "memory");
}

// Workgroup barrier of the streaming pipeline: the s_waitcnt in front of it names both counters it depends on (the
// vector-memory count that leaves later chunks in flight, and lgkmcnt(0) for this wavefront's LDS reads of the chunk
// that is about to be overwritten), so the barrier itself is the bare instruction and no fence lowering can add a
// full vmcnt(0) to it.
__device__ __forceinline__ void dm_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

// GELU: exact GELU on the output; ADD: "+ scale * addend + shift"
template <bool GELU, bool ADD>
__global__ __launch_bounds__(512) void pw_gemm_dma_kernel(PointwiseArgs a) {
    __shared__ __align__(16) unsigned char lds[DM_LDS];
    // tiles of this XCD, row block fastest: q -> (row block q % n_oblk, strip (q / n_oblk) * 8 + xcd); the workgroups of the
    // XCD deal them out round robin, so the row blocks of one strip run at the same time on one L2
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, nslot = gridDim.x >> 3;
    const int strips = (int)(a.n_strips * a.B);
    const int nq = xcd < strips ? (strips - xcd + 7) / 8 * a.n_oblk : 0;
    if (slot >= nq) return;
    const int ntl = (nq - slot + nslot - 1) / nslot;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wo = wave >> 1, wp = wave & 1;                    // 4 wavefronts along the rows x 2 along the pixels
    const int q = lane & 31, ko = lane >> 5;
    const unsigned lds0 = (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)lds);
    const bool wload = wave < 4;                                // this wavefront fetches weights (else activations)
    const int lw = wave & 3;

    const int nc16 = a.Kpad / PW_KC;
    const int nchunks = a.Kpad / DM_CK;
    const int64_t wrb = (int64_t)nc16 * 512;                   // ushorts between row blocks
    // input channels k < K1 come from X, the others (if any) from X2: a convolution over the concatenation of two tensors
    const int K1 = a.X2 ? a.K1 : a.K;

    const unsigned n_oblk = (unsigned)a.n_oblk, n_strips = (unsigned)a.n_strips;
    auto tile_of = [&](int qq, int& ob, int& b, int64_t& pw0) {
        const unsigned sl = (unsigned)qq / n_oblk * 8u + (unsigned)xcd;
        ob = (int)((unsigned)qq % n_oblk);
        b = (int)(sl / n_strips);
        pw0 = (int64_t)(sl - (unsigned)b * n_strips) * DM_PX;
    };

    // load stream of this wavefront: weight blocks (row blocks 3 lw .. 3 lw + 2 of both 16-row k steps), or activation blocks
    // 4 lw .. 4 lw + 3 (block xb = rows 2 xb, 2 xb + 1 of the chunk; lane = row (lane >> 5), 8 pixels (lane & 31))
    int iq = slot, ic = 0, isg = 0;                             // next chunk to ask for: tile, chunk, stage
    const unsigned short *sp0 = nullptr, *sp1 = nullptr;        // wavefront-uniform bases of the stream's tile
    int voff = lane * 8;                                        // lane's offset from them, in elements
    auto issue = [&]() -> bool {
        if (iq >= nq) return false;
        if (ic == 0) {
            int ob, b;
            int64_t pw0;
            tile_of(iq, ob, b, pw0);
            if (wload) {
                sp0 = a.W + ((int64_t)(ob * (DM_ROWS / 32) + 3 * lw) * nc16) * 512;
            } else {
                sp0 = a.X + (int64_t)b * K1 * a.P;
                sp1 = a.X2 ? a.X2 + (int64_t)b * (a.K - K1) * a.P : sp0;
                voff = (int)min(pw0 + 8 * (lane & 31), a.P - 8);
            }
        }
        if (wload) {
            const unsigned sb = lds0 + isg * DM_ABYTES + 3 * lw * 1024;
            const unsigned short* src = sp0 + (int64_t)ic * 1024 + voff;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int i = 0; i < 3; ++i) dma16(src + ks * 512 + i * wrb, sb + (ks * 12 + i) * 1024);
            isg = (isg == DM_WSTAGES - 1) ? 0 : isg + 1;
        } else {
            const unsigned sb = lds0 + DM_XBASE + isg * DM_XBYTES + 4 * lw * DM_XBLK;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // rows k0 and k0 + 1 for the two halves of the wavefront; rows past K meet zero weights
                const int k0 = min(ic * DM_CK + 8 * lw + 2 * i, a.K - 1), k1 = min(k0 + 1, a.K - 1);
                const unsigned short* r0 = k0 < K1 ? sp0 + (int64_t)k0 * a.P : sp1 + (int64_t)(k0 - K1) * a.P;
                const unsigned short* r1 = k1 < K1 ? sp0 + (int64_t)k1 * a.P : sp1 + (int64_t)(k1 - K1) * a.P;
                dma16((lane >> 5 ? r1 : r0) + voff, sb + i * DM_XBLK);
            }
            isg = (isg == DM_XSTAGES - 1) ? 0 : isg + 1;
        }
        if (++ic == nchunks) {
            ic = 0;
            iq += nslot;
        }
        return true;
    };

    f32x16 acc[DM_MT][DM_NT];

    // fill the pipeline: three weight chunks or five activation chunks, then chunk 0 must have landed
    bool full = true;
    for (int i = 0; i < (wload ? DM_WSTAGES : DM_XSTAGES); ++i) full = issue() && full;
    if (full)
        __builtin_amdgcn_s_waitcnt(0x007C);        // vmcnt(12) lgkmcnt(0): two chunks of weights, three of the four later activation chunks
    else
        __builtin_amdgcn_s_waitcnt(0x0070);        // vmcnt(0) lgkmcnt(0)
    dm_barrier();

    const unsigned char* abase = lds + (DM_MT * wo) * 1024 + lane * 16;
    const unsigned char* xbase = lds + DM_XBASE + (4 * ko) * DM_XBLK + wp * 256 + 8 * q;
    int sw = 0, sx = 0;
    // Operands of a 16-row k step: eight raw words of activations (rw), regrouped by byte permutes into the four B fragments
    // (bf), and three A fragments (af).  The LDS reads of the next k step are issued into rw and af as soon as the current
    // step has consumed them (rw after the permutes, af[mt] after the MFMAs of row tile mt), so they run under the MFMAs.
    u32x2 rw[8];
    u32x4 af[DM_MT], bf[DM_NT];
    auto load_rw = [&](const unsigned char* sxp, int ks) {
#pragma unroll
        for (int r = 0; r < 8; ++r) rw[r] = *reinterpret_cast<const u32x2*>(sxp + (8 * ks + (r >> 1)) * DM_XBLK + (r & 1) * 512);
    };
    auto load_af = [&](const unsigned char* sa, int ks, int mt) { af[mt] = *reinterpret_cast<const u32x4*>(sa + (ks * 12 + mt) * 1024); };
    auto regroup = [&]() {
#pragma unroll
        for (int pp = 0; pp < 2; ++pp)
#pragma unroll
            for (int h = 0; h < 4; ++h) {
                bf[2 * pp][h] = __builtin_amdgcn_perm(rw[2 * h + 1][pp], rw[2 * h][pp], 0x05040100u);
                bf[2 * pp + 1][h] = __builtin_amdgcn_perm(rw[2 * h + 1][pp], rw[2 * h][pp], 0x07060302u);
            }
    };
    // (the first k step of a tile starts its sums from the constant zero: no pass over the 192 accumulators between tiles)
    auto mfma_row = [&](int mt, bool first) {
        const bf16x8 av = __builtin_bit_cast(bf16x8, af[mt]);
        if (first) {
            const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < DM_NT; ++t)
                acc[mt][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, __builtin_bit_cast(bf16x8, bf[t]), zero, 0, 0, 0);
        } else {
#pragma unroll
            for (int t = 0; t < DM_NT; ++t)
                acc[mt][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, __builtin_bit_cast(bf16x8, bf[t]), acc[mt][t], 0, 0, 0);
        }
    };

    // Epilogue of one tile, a quarter of a row tile (eight rows, of which a lane has the four of its half ko) at a time.
    // Bias and the addend's scale and shift come through the scalar unit, the eight rows in one batch ahead of the four
    // stores: a vector load between the stores would make each store wait for the one before, since the wait for the load
    // covers every store issued before it.  The addend itself is read half a row tile ahead.
    auto epilogue = [&](auto whole, int o0, int ko4, int b, int64_t lane_off) {
        constexpr bool WHOLE = decltype(whole)::value;
        unsigned short* __restrict__ Y = a.Y + lane_off;
        const unsigned short* __restrict__ R = ADD ? a.addend + lane_off : nullptr;
        auto row_of = [&](int mt, int v) { return 32 * mt + 8 * (v >> 2) + (v & 3); };     // without the lane's 4 ko
        u32x2 rv[2][8];
        auto load_addend = [&](int mh) {
            if constexpr (ADD) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    int r = row_of(mh >> 1, 8 * (mh & 1) + j);
                    if (!WHOLE) r = min(r, a.O - 1 - o0 - ko4);
                    rv[mh & 1][j] = *reinterpret_cast<const u32x2*>(R + (int64_t)r * a.P);
                }
            }
        };
        // scalar loads one quarter ahead: those of quarter q + 1 are issued once those of quarter q have arrived (the wait of the
        // scalar unit is for all of its loads at once), and are under way while quarter q is converted and stored
        float ub[2][8], usc[2][8], ush[2][8];
        auto load_scalars = [&](int qq) {
            const int oq = o0 + row_of(qq >> 2, 4 * (qq & 3));   // rows oq .. oq + 7 (ko = 0: oq .. oq + 3)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int64_t u = WHOLE ? oq + i : min(oq + i, a.O - 1);
                ub[qq & 1][i] = a.bias ? uniform_load(a.bias, u) : 0.f;
                usc[qq & 1][i] = (ADD && a.add_scale) ? uniform_load(a.add_scale, (int64_t)b * a.O + u) : 1.f;
                ush[qq & 1][i] = (ADD && a.add_shift) ? uniform_load(a.add_shift, (int64_t)b * a.O + u) : 0.f;
            }
        };
        load_addend(0);
        load_scalars(0);
#pragma unroll
        for (int mh = 0; mh < 2 * DM_MT; ++mh) {
            const int mt = mh >> 1;
            if (!WHOLE && o0 + 32 * mt >= a.O) break;
            if (mh + 1 < 2 * DM_MT && (WHOLE || o0 + 32 * ((mh + 1) >> 1) < a.O)) load_addend(mh + 1);
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                const int qq = 2 * mh + g;
                const int v0 = 8 * (mh & 1) + 4 * g;
                const int oq = o0 + row_of(mt, v0);
                asm volatile("" ::"s"(ub[qq & 1][0]), "s"(ub[qq & 1][7]));       // the wait for this quarter's scalars goes here
                __builtin_amdgcn_sched_barrier(0);
                if (qq + 1 < 4 * DM_MT) load_scalars(qq + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    const int v = v0 + jj;
                    if (!WHOLE && oq + ko4 + jj >= a.O) continue;
                    const float bs = ko4 ? ub[qq & 1][4 + jj] : ub[qq & 1][jj];
                    float y[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) y[t] = acc[mt][t][v] + bs;
                    if constexpr (GELU) {
#pragma unroll
                        for (int t = 0; t < 4; ++t) y[t] = gelu(y[t]);
                    }
                    if constexpr (ADD) {
                        const float sc = ko4 ? usc[qq & 1][4 + jj] : usc[qq & 1][jj], sh = ko4 ? ush[qq & 1][4 + jj] : ush[qq & 1][jj];
                        const u32x2 r = rv[mh & 1][4 * g + jj];
#pragma unroll
                        for (int pp = 0; pp < 2; ++pp) {
                            y[2 * pp] += fmaf(sc, __uint_as_float(r[pp] << 16), sh);
                            y[2 * pp + 1] += fmaf(sc, __uint_as_float(r[pp] & 0xffff0000u), sh);
                        }
                    }
                    u32x2 out;
#pragma unroll
                    for (int pp = 0; pp < 2; ++pp) out[pp] = bf16_pair(y[2 * pp], y[2 * pp + 1]);
                    *reinterpret_cast<u32x2*>(Y + (int64_t)row_of(mt, v) * a.P) = out;
                }
            }
        }
    };

    for (int tl = 0; tl < ntl; ++tl) {
        const unsigned char* sa = abase + sw * DM_ABYTES;
        const unsigned char* sxp = xbase + sx * DM_XBYTES;
        load_rw(sxp, 0);
#pragma unroll
        for (int mt = 0; mt < DM_MT; ++mt) load_af(sa, 0, mt);
        for (int c = 0; c < nchunks; ++c) {
            // first k step of the chunk; the second one's operands follow it into the registers
            regroup();
            __builtin_amdgcn_sched_barrier(0);
            load_rw(sxp, 1);
#pragma unroll
            for (int mt = 0; mt < DM_MT; ++mt) {
                mfma_row(mt, c == 0);
                __builtin_amdgcn_sched_barrier(0);
                load_af(sa, 1, mt);
                __builtin_amdgcn_sched_barrier(0);
            }
            regroup();
            // Every wavefront has read all of this chunk.  The next chunk must have landed for every wavefront before it is
            // read; in flight may stay the loads of one weight chunk (6) or of three activation chunks (12), everything once
            // the stream has run dry.  Then this chunk's stages take the chunk three (five) further on.
            if (!full)
                __builtin_amdgcn_s_waitcnt(0x0070);    // vmcnt(0) lgkmcnt(0)
            else if (wload)
                __builtin_amdgcn_s_waitcnt(0x0076);    // vmcnt(6) lgkmcnt(0)
            else
                __builtin_amdgcn_s_waitcnt(0x007C);    // vmcnt(12) lgkmcnt(0)
            dm_barrier();
            full = issue();
            sw = (sw == DM_WSTAGES - 1) ? 0 : sw + 1;
            sx = (sx == DM_XSTAGES - 1) ? 0 : sx + 1;
            sa = abase + sw * DM_ABYTES;
            sxp = xbase + sx * DM_XBYTES;
            // second k step; the first one of the next chunk follows (after the last chunk of a tile these reads are
            // repeated behind the epilogue, which needs the registers)
            __builtin_amdgcn_sched_barrier(0);
            load_rw(sxp, 0);
#pragma unroll
            for (int mt = 0; mt < DM_MT; ++mt) {
                mfma_row(mt, false);
                __builtin_amdgcn_sched_barrier(0);
                load_af(sa, 0, mt);
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        // epilogue: lane holds rows 8 (v / 4) + 4 ko + v % 4 of each 32-row tile and pixels 4 q .. 4 q + 3
        int ob, b;
        int64_t pw0;
        tile_of(slot + tl * nslot, ob, b, pw0);
        // (derived afresh for every tile: hoisted out of the tile loop, the row offsets of a lane and its addresses would
        // occupy registers the accumulators need)
        int lane_ = lane;
        asm volatile("" : "+v"(lane_));
        const int ko4 = (lane_ >> 5) * 4;
        const int o0 = ob * DM_ROWS + wo * 32 * DM_MT;          // first row of the wavefront
        const int64_t px = pw0 + wp * 128 + 4 * (lane_ & 31);
        if (px < a.P && o0 < a.O) {
            const int64_t lane_off = ((int64_t)b * a.O + o0 + ko4) * a.P + px;      // lane's first row
            // whole wavefront tile inside the matrix: no row needs a check or a clamp
            if (o0 + 32 * DM_MT <= a.O)
                epilogue(std::true_type{}, o0, ko4, b, lane_off);
            else
                epilogue(std::false_type{}, o0, ko4, b, lane_off);
        }
    }
}

// packed[rb][c][lane][e] = bf16(w[32 rb + (lane & 31)][16 c + 8 (lane >> 5) + e]), zero outside the O x K weight:
// the A fragment of one wavefront for row block rb and chunk c is 1 KiB of consecutive memory
__global__ __launch_bounds__(256) void pointwise_pack_kernel(const float* __restrict__ w, unsigned short* __restrict__ packed, int O, int K, int nc,
                                                             int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int e = (int)(idx & 7), lane = (int)((idx >> 3) & 63);
    const int64_t blk = idx >> 9;
    const int c = (int)(blk % nc), rb = (int)(blk / nc);
    const int o = 32 * rb + (lane & 31), k = 16 * c + 8 * (lane >> 5) + e;
    packed[idx] = (o < O && k < K) ? f_to_bf16(w[(int64_t)o * K + k]) : (unsigned short)0;
}

// ---- instance-norm statistics ------------------------------------------------------------------
// partial[row][seg] = (sum d, sum d^2), d = x - x[row][0] (the pivot keeps the variance formula from cancelling)
constexpr int ST_THREADS = 256;
__global__ __launch_bounds__(ST_THREADS) void row_stats_partial_kernel(const unsigned short* __restrict__ x, float2* __restrict__ partial, int64_t P,
                                                                       int nseg) {
    const int64_t row = blockIdx.x;
    const int seg = blockIdx.y;
    const unsigned short* __restrict__ xr = x + row * P;
    const float pivot = bf16_to_f(xr[0]);
    const int64_t ngroups = P / 8;
    const int64_t g0 = ngroups * seg / nseg, g1 = ngroups * (seg + 1) / nseg;
    float s = 0.f, s2 = 0.f;
    for (int64_t g = g0 + threadIdx.x; g < g1; g += ST_THREADS) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(xr + 8 * g);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = __uint_as_float(v[i] << 16) - pivot, hi = __uint_as_float(v[i] & 0xffff0000u) - pivot;
            s += lo + hi;
            s2 = fmaf(lo, lo, fmaf(hi, hi, s2));
        }
    }
    if (seg == nseg - 1)
        for (int64_t i = 8 * ngroups + threadIdx.x; i < P; i += ST_THREADS) {
            const float d = bf16_to_f(xr[i]) - pivot;
            s += d;
            s2 = fmaf(d, d, s2);
        }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        s += __shfl_down(s, off, 64);
        s2 += __shfl_down(s2, off, 64);
    }
    __shared__ float2 red[ST_THREADS / 64];
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = make_float2(s, s2);
    __syncthreads();
    if (threadIdx.x == 0) {
        float2 t = red[0];
        for (int w = 1; w < ST_THREADS / 64; ++w) {
            t.x += red[w].x;
            t.y += red[w].y;
        }
        partial[row * nseg + seg] = t;
    }
}

// scale = gamma * rstd, shift = beta - mean * scale  (biased variance, as torch.nn.functional.instance_norm)
__global__ void row_stats_finalize_kernel(const unsigned short* __restrict__ x, const float2* __restrict__ partial, const float* __restrict__ gamma,
                                          const float* __restrict__ beta, float* __restrict__ scale, float* __restrict__ shift, int64_t rows,
                                          int channels, int64_t P, int nseg, float eps) {
    const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows) return;
    double s = 0.0, s2 = 0.0;
    for (int i = 0; i < nseg; ++i) {
        s += partial[row * nseg + i].x;
        s2 += partial[row * nseg + i].y;
    }
    const double n = (double)P;
    const double md = s / n;
    const double var = fmax(s2 / n - md * md, 0.0);
    const float mean = bf16_to_f(x[row * P]) + (float)md;
    const float rstd = (float)(1.0 / sqrt(var + (double)eps));
    const int c = (int)(row % channels);
    const float sc = (gamma ? gamma[c] : 1.f) * rstd;
    scale[row] = sc;
    shift[row] = (beta ? beta[c] : 0.f) - mean * sc;
}

// The same coefficients from per-latitude moments of the field (the inverse longitude kernel's by-product):
// stats[row][k] = (a_k, d_k), the mean over longitude of latitude row k and of its squared deviation from a_k.
// mean = avg_k a_k, variance = avg_k ((a_k - mean)^2 + d_k); one wavefront per row, sums in double.
__global__ __launch_bounds__(64) void lat_stats_finalize_kernel(const float2* __restrict__ stats, const float* __restrict__ gamma,
                                                                const float* __restrict__ beta, float* __restrict__ scale, float* __restrict__ shift,
                                                                int channels, int nlat, float eps) {
    const int64_t row = blockIdx.x;
    const float2* __restrict__ sr = stats + row * nlat;
    double s = 0.0;
    for (int k = threadIdx.x; k < nlat; k += 64) s += (double)sr[k].x;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    const double mean = s / nlat;
    double v = 0.0;
    for (int k = threadIdx.x; k < nlat; k += 64) {
        const float2 t = sr[k];
        const double d = (double)t.x - mean;
        v += d * d + (double)t.y;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    if (threadIdx.x == 0) {
        const float rstd = (float)(1.0 / sqrt(v / nlat + (double)eps));
        const int c = (int)(row % channels);
        const float sc = (gamma ? gamma[c] : 1.f) * rstd;
        scale[row] = sc;
        shift[row] = (beta ? beta[c] : 0.f) - (float)mean * sc;
    }
}

// y = act(scale[row] * x + shift[row]), bf16 -> bf16, 8 pixels per thread
__global__ __launch_bounds__(256) void scale_shift_act_kernel(const unsigned short* __restrict__ x, const float* __restrict__ scale,
                                                              const float* __restrict__ shift, unsigned short* __restrict__ y, int64_t P,
                                                              int64_t groups_per_row, int64_t total_groups, int act) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= total_groups) return;
    const int64_t row = g / groups_per_row;
    const int64_t i0 = row * P + 8 * (g - row * groups_per_row);
    const float sc = scale[row], sh = shift[row];
    const u32x4 v = *reinterpret_cast<const u32x4*>(x + i0);
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float lo = fmaf(sc, __uint_as_float(v[i] << 16), sh), hi = fmaf(sc, __uint_as_float(v[i] & 0xffff0000u), sh);
        if (act == SFNO_ACT_GELU) {
            lo = gelu(lo);
            hi = gelu(hi);
        }
        o[i] = bf16_pair(lo, hi);
    }
    *reinterpret_cast<u32x4*>(y + i0) = o;
}

}  // namespace

// compute units of the current device (256 when the query fails)
static int device_cus() {
    static int cached[64] = {};
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void)hipGetLastError(); return 256; }
    if (cached[dev] > 0) return cached[dev];
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) { (void)hipGetLastError(); return 256; }
    cached[dev] = cus;
    return cus;
}

// the kernel for O > 96 walks K in chunks of 32 rows and takes any number of them; the other one runs whole unrolled loop bodies
int pointwise_kpad(int K, int O) {
    const int align = O > PW_ROWS ? DM_CK : PW_KALIGN;
    return (K + align - 1) / align * align;
}
// rows are padded to whole workgroup tiles so that no fragment load needs a bound check
int pointwise_opad(int O) {
    const int tile = O > PW_ROWS ? 4 * PW_ROWS : PW_ROWS;
    return (O + tile - 1) / tile * tile;
}

int pointwise_pack_launch(const float* w, unsigned short* packed, int O, int K, hipStream_t s) {
    const int nc = pointwise_kpad(K, O) / PW_KC;
    const int64_t total = (int64_t)(pointwise_opad(O) / 32) * nc * 512;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(pointwise_pack_kernel, dim3((unsigned)blocks), dim3(256), 0, s, w, packed, O, K, nc, total);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int pointwise_gemm_launch(PointwiseArgs a, hipStream_t s) {
    a.Kpad = pointwise_kpad(a.K, a.O);
    if (a.P % 8 != 0 || a.K < 1 || a.O < 1 || a.B < 1 || a.P < 8) return SFNO_EUNSUPPORTED;
    const bool tall = a.O > PW_ROWS;              // several wavefronts share a pixel strip
    const int wm = tall ? 4 : 1;
    const bool dma = tall;                        // direct-to-LDS kernel for O > 96
    if (a.X2 && (a.K1 < 1 || a.K1 >= a.K)) return SFNO_EINVAL;
    const int wpx = dma ? DM_PX : 512;            // pixels per workgroup
    a.n_oblk = (a.O + PW_ROWS * wm - 1) / (PW_ROWS * wm);
    a.n_strips = (a.P + wpx - 1) / wpx;
    const int64_t strips = a.n_strips * a.B;
    const int64_t blocks = (strips + 7) / 8 * 8 * a.n_oblk;
    if (blocks > 0x7fffffffLL || (dma && a.P > 0x7fffffffLL)) return SFNO_EUNSUPPORTED;
    if (dma)       // persistent: one workgroup per CU (its LDS admits no second one), the same number on every XCD
    {
        const dim3 grid((unsigned)std::min<int64_t>(blocks, std::max(8, device_cus() / 8 * 8)));
        const bool g = a.act == SFNO_ACT_GELU, r = a.addend != nullptr;
        if (g && r) hipLaunchKernelGGL((pw_gemm_dma_kernel<true, true>), grid, dim3(512), 0, s, a);
        else if (g) hipLaunchKernelGGL((pw_gemm_dma_kernel<true, false>), grid, dim3(512), 0, s, a);
        else if (r) hipLaunchKernelGGL((pw_gemm_dma_kernel<false, true>), grid, dim3(512), 0, s, a);
        else hipLaunchKernelGGL((pw_gemm_dma_kernel<false, false>), grid, dim3(512), 0, s, a);
    }
    else
        hipLaunchKernelGGL((pw_gemm_kernel<1, 2>), dim3((unsigned)blocks), dim3(512), 0, s, a);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int row_stats_segments(int64_t rows, int64_t P) {
    // ~16 K elements per workgroup.  The split depends on the row length only, so that the sums of a row (and with them
    // every value downstream) do not change with the number of rows: a sample gives the same result alone and in a batch.
    (void)rows;
    return (int)std::max<int64_t>(1, std::min<int64_t>(P / 16384, 64));
}

int instance_norm_coeffs_launch(const unsigned short* x, const float* gamma, const float* beta, float* scale, float* shift, float2* partial,
                                int64_t rows, int channels, int64_t P, float eps, hipStream_t s) {
    if (rows < 1 || P < 1 || channels < 1 || rows > 0x7fffffffLL / 64) return SFNO_EUNSUPPORTED;
    if (P % 8 != 0) return SFNO_EUNSUPPORTED;     // 16-byte loads from every row start
    const int nseg = row_stats_segments(rows, P);
    hipLaunchKernelGGL(row_stats_partial_kernel, dim3((unsigned)rows, (unsigned)nseg), dim3(ST_THREADS), 0, s, x, partial, P, nseg);
    hipLaunchKernelGGL(row_stats_finalize_kernel, dim3((unsigned)((rows + 127) / 128)), dim3(128), 0, s, x, partial, gamma, beta, scale, shift, rows,
                       channels, P, nseg, eps);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int instance_norm_coeffs_lat_launch(const float2* stats, const float* gamma, const float* beta, float* scale, float* shift, int64_t rows, int channels,
                                    int nlat, float eps, hipStream_t s) {
    if (rows < 1 || rows > 0x7fffffffLL || channels < 1 || nlat < 1) return SFNO_EINVAL;
    hipLaunchKernelGGL(lat_stats_finalize_kernel, dim3((unsigned)rows), dim3(64), 0, s, stats, gamma, beta, scale, shift, channels, nlat, eps);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int scale_shift_act_launch(const unsigned short* x, const float* scale, const float* shift, unsigned short* y, int64_t rows, int64_t P, int act,
                           hipStream_t s) {
    if (rows < 1 || P < 8 || P % 8 != 0) return SFNO_EUNSUPPORTED;
    const int64_t gpr = P / 8, total = rows * gpr;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(scale_shift_act_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, scale, shift, y, P, gpr, total, act);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
