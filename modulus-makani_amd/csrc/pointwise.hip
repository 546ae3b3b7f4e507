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
// A wavefront owns 96 output rows x 64 pixels (3 x 2 tiles, 96 accumulator registers), eight wavefronts
// make a workgroup, two per SIMD.  Weights come from global memory (L2 resident) as A fragments, packed so
// that a fragment is 1 KiB of consecutive memory; the activation chunk (16 k rows) is shared through a
// triple-buffered LDS stage; both operand streams are prefetched several chunks ahead in registers: the
// loads in flight, not the arithmetic, bound this kernel (the activations stream from HBM).
#include "sfno_internal.h"

namespace sfno {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int PW_MT = 3;          // 32-row tiles per wavefront
constexpr int PW_NT = 2;          // pixels per lane = N tiles per wavefront
constexpr int PW_ROWS = 32 * PW_MT;
constexpr int PW_PX = 32 * PW_NT; // pixels per wavefront
constexpr int PW_KC = 16;         // k rows per MFMA K step
constexpr int PW_KS = 2;          // MFMA K steps per chunk (one LDS stage, one barrier)
constexpr int PW_KALIGN = 128;    // K is padded to whole unrolled loop bodies (PW_KC * prefetch distance)
constexpr int PW_THREADS = 512;

__device__ __forceinline__ float bf16_to_f(unsigned short h) { return __uint_as_float((unsigned int)h << 16); }
__device__ __forceinline__ unsigned short f_to_bf16(float f) { return __builtin_bit_cast(unsigned short, (__bf16)f); }

// exact (erf) GELU; erf by Abramowitz-Stegun 7.1.26 (|error| < 1.5e-7), written without cancellation in the
// negative tail: 1 + erf(z) = poly * exp(-z^2) for z < 0 (relative error there stays below 1e-2, at values
// under 1e-6 in magnitude)
__device__ __forceinline__ float gelu(float x) {
    const float z = fabsf(x) * 0.70710678118654752f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, z, 1.0f));
    float p = fmaf(t, 1.061405429f, -1.453152027f);
    p = fmaf(t, p, 1.421413741f);
    p = fmaf(t, p, -0.284496736f);
    p = fmaf(t, p, 0.254829592f);
    const float pe = p * t * __builtin_amdgcn_exp2f(-z * z * 1.44269504088896341f);
    return 0.5f * x * (x < 0.f ? pe : 2.0f - pe);
}

// WM = wavefronts along the output rows: 4 (x 2 along pixels: 384 rows x 128 pixels per workgroup) or
// 1 (x 8 along pixels: 96 rows x 512 pixels, for convolutions with few output channels)
template <int WM>
__global__ __launch_bounds__(PW_THREADS) void pw_gemm_kernel(PointwiseArgs a) {
    constexpr int WN = 8 / WM;
    constexpr int WPX = WN * PW_PX;               // pixels per workgroup
    constexpr int PITCH = WPX * 2 + 16;           // bytes per LDS row
    constexpr int CK = PW_KC * PW_KS;             // k rows per chunk = per loop step
    constexpr int STAGE = CK * PITCH;
    constexpr int D = (WM == 4) ? 4 : 2;          // prefetch distance in chunks
    constexpr int XW = (WM == 4) ? 1 : 4;         // 16-byte pieces of the activation chunk per thread
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
    const int o0 = ob * (PW_ROWS * WM) + (WM == 4 ? (wave >> 1) * PW_ROWS : 0);
    const int pxw = (WM == 4 ? (wave & 1) : wave) * PW_PX;                // wavefront's pixel offset inside the stage

    const unsigned short* __restrict__ X = a.X + (int64_t)b * a.K * a.P;
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
            dst[u] = *reinterpret_cast<const u32x4*>(X + (int64_t)k * a.P + xoff[u]);
        }
    };
    auto store_x = [&](int stage, const u32x4 (&src)[XW]) {
#pragma unroll
        for (int u = 0; u < XW; ++u) *reinterpret_cast<u32x4*>(&lds[stage * STAGE + loff[u]]) = src[u];
    };

    f32x16 acc[PW_MT][PW_NT];
#pragma unroll
    for (int mt = 0; mt < PW_MT; ++mt)
#pragma unroll
        for (int t = 0; t < PW_NT; ++t)
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

    // B fragments: lane = pixel pair q, k rows 8 ko .. 8 ko + 7 of a 16-row sub-step.  The raw words of the next
    // sub-step are read while the MFMAs of the current one run (hence three stages: chunk c + 1 is read during chunk c).
    const unsigned char* fragbase = &lds[0] + (8 * ko) * PITCH + (pxw + 2 * q) * 2;
    unsigned int rw[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) rw[r] = *reinterpret_cast<const unsigned int*>(fragbase + r * PITCH);
    int s0 = 0;                                    // stage of chunk c
    for (int c0 = 0; c0 < nchunks; c0 += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            const int c = c0 + u;
            const int s1 = (s0 == 2) ? 0 : s0 + 1; // stage of chunk c + 1
            const int s2 = (s1 == 2) ? 0 : s1 + 1; // stage of chunk c + 2
#pragma unroll
            for (int ks = 0; ks < PW_KS; ++ks) {
                u32x4 bf[PW_NT];
#pragma unroll
                for (int h = 0; h < 4; ++h) {
                    bf[0][h] = __builtin_amdgcn_perm(rw[2 * h + 1], rw[2 * h], 0x05040100u);
                    bf[1][h] = __builtin_amdgcn_perm(rw[2 * h + 1], rw[2 * h], 0x07060302u);
                }
                const unsigned char* fb = (ks + 1 < PW_KS) ? fragbase + s0 * STAGE + (ks + 1) * PW_KC * PITCH : fragbase + s1 * STAGE;
#pragma unroll
                for (int r = 0; r < 8; ++r) rw[r] = *reinterpret_cast<const unsigned int*>(fb + r * PITCH);
#pragma unroll
                for (int mt = 0; mt < PW_MT; ++mt) {
                    const bf16x8 av = __builtin_bit_cast(bf16x8, araw[u][ks][mt]);
#pragma unroll
                    for (int t = 0; t < PW_NT; ++t)
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

    // epilogue: lane holds rows 8 (v / 4) + 4 ko + v % 4 of each 32-row tile and pixels 2 q, 2 q + 1
    const int64_t px = pw0 + pxw + 2 * q;
    if (px >= a.P) return;
    unsigned short* __restrict__ Y = a.Y + (int64_t)b * a.O * a.P;
    const unsigned short* __restrict__ R = a.addend ? a.addend + (int64_t)b * a.O * a.P : nullptr;
#pragma unroll
    for (int mt = 0; mt < PW_MT; ++mt) {
        unsigned int rv[16];
        if (R) {
            // all addend loads of the tile first
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int o = min(o0 + 32 * mt + 8 * (v >> 2) + 4 * ko + (v & 3), a.O - 1);
                rv[v] = *reinterpret_cast<const unsigned int*>(R + (int64_t)o * a.P + px);
            }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int o = o0 + 32 * mt + 8 * (v >> 2) + 4 * ko + (v & 3);
            if (o >= a.O) continue;
            const float bs = a.bias ? a.bias[o] : 0.f;
            float y0 = acc[mt][0][v] + bs, y1 = acc[mt][1][v] + bs;
            if (a.act == SFNO_ACT_GELU) {
                y0 = gelu(y0);
                y1 = gelu(y1);
            }
            if (R) {
                const float sc = a.add_scale ? a.add_scale[(int64_t)b * a.O + o] : 1.f;
                const float sh = a.add_shift ? a.add_shift[(int64_t)b * a.O + o] : 0.f;
                y0 += fmaf(sc, __uint_as_float(rv[v] << 16), sh);
                y1 += fmaf(sc, __uint_as_float(rv[v] & 0xffff0000u), sh);
            }
            *reinterpret_cast<unsigned int*>(Y + (int64_t)o * a.P + px) = (unsigned int)f_to_bf16(y0) | ((unsigned int)f_to_bf16(y1) << 16);
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
        o[i] = (unsigned int)f_to_bf16(lo) | ((unsigned int)f_to_bf16(hi) << 16);
    }
    *reinterpret_cast<u32x4*>(y + i0) = o;
}

}  // namespace

int pointwise_kpad(int K) { return (K + PW_KALIGN - 1) / PW_KALIGN * PW_KALIGN; }
// rows are padded to whole workgroup tiles so that no fragment load needs a bound check
int pointwise_opad(int O) {
    const int tile = O > PW_ROWS ? 4 * PW_ROWS : PW_ROWS;
    return (O + tile - 1) / tile * tile;
}

int pointwise_pack_launch(const float* w, unsigned short* packed, int O, int K, hipStream_t s) {
    const int nc = pointwise_kpad(K) / PW_KC;
    const int64_t total = (int64_t)(pointwise_opad(O) / 32) * nc * 512;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(pointwise_pack_kernel, dim3((unsigned)blocks), dim3(256), 0, s, w, packed, O, K, nc, total);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int pointwise_gemm_launch(PointwiseArgs a, hipStream_t s) {
    a.Kpad = pointwise_kpad(a.K);
    if (a.P % 8 != 0 || a.K < 1 || a.O < 1 || a.B < 1 || a.P < 8) return SFNO_EUNSUPPORTED;
    const bool tall = a.O > PW_ROWS;              // several wavefronts share a pixel strip
    const int wm = tall ? 4 : 1;
    const int wpx = (8 / wm) * PW_PX;
    a.n_oblk = (a.O + PW_ROWS * wm - 1) / (PW_ROWS * wm);
    a.n_strips = (a.P + wpx - 1) / wpx;
    const int64_t strips = a.n_strips * a.B;
    const int64_t blocks = (strips + 7) / 8 * 8 * a.n_oblk;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    if (tall)
        hipLaunchKernelGGL((pw_gemm_kernel<4>), dim3((unsigned)blocks), dim3(PW_THREADS), 0, s, a);
    else
        hipLaunchKernelGGL((pw_gemm_kernel<1>), dim3((unsigned)blocks), dim3(PW_THREADS), 0, s, a);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int row_stats_segments(int64_t rows, int64_t P) {
    // enough workgroups to fill the chip, at least ~16 K elements each
    int64_t nseg = (2048 + rows - 1) / rows;
    nseg = std::min<int64_t>(nseg, std::max<int64_t>(1, P / 16384));
    return (int)std::max<int64_t>(1, std::min<int64_t>(nseg, 64));
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
