// Weight gradient of the 1x1 convolution on bf16 NCHW activations:
//
//   dW[o][k] = sum_{b,p} g[b][o][p] x[b][k][p],      db[o] = sum_{b,p} g[b][o][p]
//
// (what autograd derives for nn.Conv2d(kernel_size=1), makani/models/common/layers.py:95-116,160-216).  Both operands are
// pixel-contiguous and the sum runs over the pixels, so a row of g is an A operand and a row of x a B operand of
// v_mfma_f32_32x32x16_bf16 as they lie in memory: 8 consecutive pixels per lane, no transposition.  The bias gradient
// rides along as one more column: row K of x is taken to be all ones.
//
// A workgroup (eight wavefronts, 4 x 2) owns a 256 x 256 tile of dW and a contiguous share of the (sample, 32-pixel chunk)
// sequence.  Per chunk 256 rows of g and 256 rows of x (64 bytes each) go straight from memory into a ring of four LDS
// stages with global_load_lds_dwordx4, three chunks ahead of the matrix instructions (issued from inline assembly with a
// counted wait, as in the forward kernel); a lane fetches the 16-byte piece whose LDS slot it owns, and the pieces of a row
// are permuted by (row >> 1) & 3 so that the 16-byte fragment reads of eight consecutive rows cover all banks.  Pieces
// past the end of a sample come from a block of zeros, the bias column from a block of ones.  Each wavefront multiplies
// 64 x 128 (two A and four B fragments per 16 pixels for eight matrix instructions).  The shares' partial tiles go to a
// workspace [share][O][K + 1] and a second kernel adds them up in a fixed order: results do not depend on scheduling.
// All tiles of one share run on one XCD (workgroups are dealt to the XCDs round robin by linear id), where they meet
// the share's rows of g and x in L2.
#include "sfno_internal.h"

namespace sfno {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int WG_THREADS = 512;
constexpr int WG_TO = 256;            // rows of dW (output channels) per workgroup
constexpr int WG_TK = 256;            // columns of dW (input channels, + the bias column) per workgroup
constexpr int WG_PX = 32;             // pixels per chunk: four 16-byte pieces per row
constexpr int WG_ROWS = WG_TO + WG_TK;
constexpr int WG_STAGE = WG_ROWS * 2 * WG_PX;                 // bytes per LDS stage
constexpr int WG_STAGES = 4;
constexpr int WG_PIECES = WG_ROWS * (WG_PX / 8) / WG_THREADS; // 16-byte pieces per thread and chunk
constexpr int WG_RSTEP = WG_THREADS / (WG_PX / 8);            // rows between a thread's pieces
static_assert(WG_PX == 32, "four pieces per row: the permutation and the slot arithmetic below");
static_assert(WG_ROWS * (WG_PX / 8) % WG_THREADS == 0, "the chunk divides evenly among the threads");
static_assert(WG_TO * (WG_PX / 8) % WG_THREADS == 0, "a thread's piece j is a row of g for all threads or a row of x for all threads");
static_assert(WG_RSTEP % 8 == 0, "a thread's pieces share the permutation of their rows");
static_assert(WG_STAGES * WG_STAGE <= 160 * 1024, "one workgroup per CU");

// sources of the pieces that are not read from the tensors
__device__ __align__(16) const unsigned int wg_zero16[4] = {0u, 0u, 0u, 0u};
__device__ __align__(16) const unsigned int wg_ones16[4] = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};

// 16 bytes per lane from global memory to LDS base + 16 lane (M0 carries the base; the compiler reserves M0 and does not
// accept it on a clobber list: nothing else in this file may depend on M0)
__device__ __forceinline__ void wg_dma16(const void* g, unsigned lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_byte_addr) : "memory");
}

struct WgradShape {
    int n_ot, n_kt, splits;
    int64_t cps, chunks;               // chunks per sample, chunks in all
};

// how the launcher and the workspace query divide the work: shares of at least eight chunks, one workgroup per CU (all
// workgroups resident at once, the tiles of a share side by side on one XCD)
static WgradShape wgrad_shape(int O, int Kext, int B, int64_t P) {
    WgradShape s;
    s.n_ot = (O + WG_TO - 1) / WG_TO;
    s.n_kt = (Kext + WG_TK - 1) / WG_TK;
    s.cps = (P + WG_PX - 1) / WG_PX;
    s.chunks = s.cps * B;
    const int tiles = s.n_ot * s.n_kt;
    int64_t want = 256 / tiles / 8 * 8;
    if (want < 8) want = 8;
    const int64_t most = (s.chunks + 7) / 8;       // at least eight chunks per share
    if (want > most) want = most;
    if (want < 1) want = 1;
    s.splits = (int)want;
    return s;
}

struct WgradArgs {
    const unsigned short* G;           // bf16 [B][O][P]
    const unsigned short* X;           // bf16 [B][K][P]
    float* ws;                         // [splits][O][Kext]
    int O, K, Kext, B;
    int64_t P;
    int n_ot, n_kt, splits;
    int64_t cps, chunks;
};

// grid = 8 * ceil(splits / 8) * n_ot * n_kt workgroups of 512 threads
__global__ __launch_bounds__(WG_THREADS, 2) void pw_wgrad_kernel(WgradArgs a) {
    __shared__ __align__(16) unsigned char lds[WG_STAGES * WG_STAGE];
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    const int tiles = a.n_ot * a.n_kt;
    const int split = (q / tiles) * 8 + xcd, tile = q % tiles;
    if (split >= a.splits) return;
    const int o0 = (tile % a.n_ot) * WG_TO, k0 = (tile / a.n_ot) * WG_TK;
    const int64_t c_begin = (int64_t)split * a.chunks / a.splits, c_end = (int64_t)(split + 1) * a.chunks / a.splits;
    const int nch = (int)(c_end - c_begin);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wo = wave & 3, wk = wave >> 2;
    const unsigned lds0 = (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)lds);

    // ---- loads: LDS slot s = 512 j + tid of a stage (16 bytes) holds row s >> 2, piece (s & 3) ^ ((row >> 1) & 3); rows below
    // WG_TO are rows of g, the others rows of x.  A thread's four slots lie 128 rows apart: same piece, same permutation.
    constexpr int JG = WG_TO * (WG_PX / 8) / WG_THREADS;
    const int part = (tid & 3) ^ ((tid >> 3) & 3);
    const unsigned short* rowp[WG_PIECES];     // first pixel of the row in sample 0 (rows past the matrix: its last row, whose products are never stored)
    bool ones[WG_PIECES];                      // the bias column: all ones
#pragma unroll
    for (int j = 0; j < WG_PIECES; ++j) {
        const int row = (tid >> 2) + WG_RSTEP * j;
        if (j < JG) {
            rowp[j] = a.G + (int64_t)min(o0 + row, a.O - 1) * a.P;
            ones[j] = false;
        } else {
            const int k = k0 + row - WG_TO;
            rowp[j] = a.X + (int64_t)min(k, a.K - 1) * a.P;
            ones[j] = k == a.K && a.Kext > a.K;
        }
    }
    const unsigned short* zero16 = reinterpret_cast<const unsigned short*>(wg_zero16);
    const unsigned short* ones16 = reinterpret_cast<const unsigned short*>(wg_ones16);
    // next chunk to ask for: sample ib, chunk ic of the sample, and where its pieces lie (counted along: a chunk inside a
    // sample costs one addition per piece; the addresses are worked out afresh once per sample)
    int64_t ib = c_begin / a.cps;
    int64_t ic = c_begin - ib * a.cps;
    const unsigned short* cur[WG_PIECES];
    auto locate = [&]() {
        const int64_t p = ic * WG_PX + 8 * part;
        const int64_t og = ib * a.O * a.P + p, ox = ib * a.K * a.P + p;
#pragma unroll
        for (int j = 0; j < WG_PIECES; ++j) cur[j] = ones[j] ? ones16 : rowp[j] + (j < JG ? og : ox);
    };
    locate();
    auto issue = [&](int stage) {
        const unsigned dst = lds0 + stage * WG_STAGE + wave * 1024;
        if ((ic + 1) * WG_PX <= a.P) {         // (uniform) every piece of the chunk lies inside the sample
#pragma unroll
            for (int j = 0; j < WG_PIECES; ++j) wg_dma16(cur[j], dst + j * (WG_THREADS * 16));
        } else {
            // the last chunk of a sample: P is a multiple of 8, so a piece lies inside the row or outside
            const bool in = ic * WG_PX + 8 * part < a.P;
#pragma unroll
            for (int j = 0; j < WG_PIECES; ++j) wg_dma16(in ? cur[j] : zero16, dst + j * (WG_THREADS * 16));
        }
        if (++ic == a.cps) {
            ic = 0;
            ++ib;
            locate();
        } else {
#pragma unroll
            for (int j = 0; j < WG_PIECES; ++j) cur[j] += (j >= JG && ones[j]) ? 0 : WG_PX;
        }
    };

    f32x16 acc[2][4];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mt][nt][v] = 0.f;

    // fragments of this lane: row (lane & 31) of a 32-row block, pieces (lane >> 5) and 2 + (lane >> 5) of the row (pixels
    // 8 (lane >> 5) .. + 7 of the first and of the second 16-pixel step), at their permuted places
    const int sw = (lane >> 1) & 3, kg = lane >> 5;
    const unsigned fa = (wo * 64 + (lane & 31)) * 64, fb = (WG_TO + wk * 128 + (lane & 31)) * 64;
    const unsigned pk[2] = {(unsigned)((kg ^ sw) * 16), (unsigned)(((2 + kg) ^ sw) * 16)};

    const bool live = o0 + wo * 64 < a.O && k0 + wk * 128 < a.Kext;
    // Ring of four stages: chunk i is multiplied while chunks i + 1 .. i + 3 are on their way.  The only vector memory
    // operations of the loop are the four loads per wavefront and chunk, so "at most eight outstanding" means chunk i has
    // landed while two later ones may still be under way.
    static_assert(WG_STAGES == 4 && WG_PIECES == 4, "the wait counts below");
    for (int i = 0; i < WG_STAGES - 1; ++i)
        if (i < nch) issue(i);
    int stage = 0;
    for (int i = 0; i < nch; ++i) {
        __builtin_amdgcn_sched_barrier(0);
        if (i + 2 < nch)
            asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
        else if (i + 1 < nch)
            asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
        else
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // (every wavefront has read chunk i - 1: its stage takes chunk i + 3)
        if (i + 3 < nch) issue(stage == 0 ? WG_STAGES - 1 : stage - 1);
        const unsigned char* sb = lds + stage * WG_STAGE;
        // (a wavefront whose 64 x 128 part of the tile lies outside the matrix only moves data)
        if (live)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            bf16x8 af[2], bf[4];
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) af[mt] = *reinterpret_cast<const bf16x8*>(sb + fa + mt * 32 * 64 + pk[ks]);
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) bf[nt] = *reinterpret_cast<const bf16x8*>(sb + fb + nt * 32 * 64 + pk[ks]);
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mt], bf[nt], acc[mt][nt], 0, 0, 0);
        }
        stage = stage == WG_STAGES - 1 ? 0 : stage + 1;
    }

    // D layout of the 32x32 MFMA: register v of lane j holds D[8 (v / 4) + 4 (j / 32) + v % 4][j % 32]
    float* out = a.ws + (int64_t)split * a.O * a.Kext;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            const int kk = k0 + wk * 128 + nt * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int o = o0 + wo * 64 + mt * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (o < a.O && kk < a.Kext) out[(int64_t)o * a.Kext + kk] = acc[mt][nt][v];
            }
        }
}

// dW[o][k] = sum over the shares, in order; column K goes to db.  A thread sums four consecutive entries of the
// [O][Kext] matrices (16-byte loads, eight shares in flight) and stores them one by one: they may straddle a row.
__global__ __launch_bounds__(256) void pw_wgrad_reduce_kernel(const float* __restrict__ ws, float* __restrict__ dW, float* __restrict__ db, int O, int K,
                                                              int Kext, int splits) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const int64_t n = (int64_t)O * Kext;
    const int64_t idx = 4 * ((int64_t)blockIdx.x * blockDim.x + threadIdx.x);
    if (idx >= n) return;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    if (idx + 4 <= n && n % 4 == 0) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
        for (int i = 0; i < splits; ++i) acc += *reinterpret_cast<const f32x4*>(ws + (int64_t)i * n + idx);
#pragma unroll
        for (int e = 0; e < 4; ++e) s[e] = acc[e];
    } else {
        for (int i = 0; i < splits; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (idx + e < n) s[e] += ws[(int64_t)i * n + idx + e];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (idx + e >= n) break;
        const int o = (int)((idx + e) / Kext), k = (int)(idx + e - (int64_t)o * Kext);
        if (k < K)
            dW[(int64_t)o * K + k] = s[e];
        else if (db)
            db[o] = s[e];
    }
}

size_t pointwise_wgrad_workspace_bytes(int O, int K, int has_bias, int B, int64_t P) {
    const int Kext = K + (has_bias ? 1 : 0);
    const WgradShape s = wgrad_shape(O, Kext, B, P);
    return sizeof(float) * (size_t)s.splits * (size_t)O * (size_t)Kext;
}

int pointwise_wgrad_launch(const unsigned short* g, const unsigned short* x, float* dW, float* db, int B, int K, int O, int64_t P, float* ws,
                           size_t ws_bytes, hipStream_t s) {
    if (P < 8 || P % 8) return SFNO_EINVAL;
    const int Kext = K + (db ? 1 : 0);
    const WgradShape sh = wgrad_shape(O, Kext, B, P);
    if (ws_bytes < sizeof(float) * (size_t)sh.splits * (size_t)O * (size_t)Kext) return SFNO_EINVAL;
    WgradArgs a;
    a.G = g; a.X = x; a.ws = ws;
    a.O = O; a.K = K; a.Kext = Kext; a.B = B; a.P = P;
    a.n_ot = sh.n_ot; a.n_kt = sh.n_kt; a.splits = sh.splits; a.cps = sh.cps; a.chunks = sh.chunks;
    const int64_t nwg = 8 * (int64_t)((sh.splits + 7) / 8) * sh.n_ot * sh.n_kt;
    if (nwg > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(pw_wgrad_kernel, dim3((unsigned)nwg), dim3(WG_THREADS), 0, s, a);
    if (hipGetLastError() != hipSuccess) return SFNO_EHIP;
    const int64_t n = (int64_t)O * Kext;
    hipLaunchKernelGGL(pw_wgrad_reduce_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, s, ws, dW, db, O, K, Kext, sh.splits);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
