// dhconv on the matrix cores of gfx950:
//
//   y[b,o,l,m] = sum_i x[b,i,l,m] w[i,o,l]        (makani/models/common/contractions.py:130-136)
// as real GEMMs per degree l on the spectral layout.  Three kernels: dhconv_split_kernel (fp32 accuracy on the bf16
// matrix pipe, the default, further down), dhconv_bf16_kernel (bf16 operands) and, first in this file, dhconv_kernel
// on v_mfma_f32_32x32x2_f32, which serves odd channel counts.  In that one a complex product costs three real ones
// (Gauss):  k1 = wr (xr + xi),  k2 = xr (wi - wr),  k3 = xi (wr + wi),  yr = k1 - k3,  yi = k1 + k2,
// so each complex input channel feeds three MFMA operand pairs instead of the four of the 2x2 real
// embedding, and a wavefront keeps three accumulators (K1, K2, K3) per tile that are combined when the
// rows are stored.
//
// A workgroup owns (degree l, block of 64 output channels, group of 64 rows (m,b)): a small group, because a
// degree has at most mmax orders and the last group of a degree is rarely full.  Each of its four wavefronts
// owns 32 rows x 32 output channels: it reads its activation rows straight from HBM/L2 into MFMA A operands
// (rows are contiguous along i in the spectral layout) and keeps 32 rows x 32 channels x 3 sums.  The
// weight chunk (8 input channels x 64 output channels) is expanded from the packed complex weights into
// three LDS planes (wr, wi - wr, wr + wi) once per chunk and shared by the four wavefronts as the B
// operand.  Wavefronts whose rows lie beyond the orders present at this degree (m > l) do nothing, so the
// triangular structure costs no guarded matrix instructions.
#include <type_traits>

#include "sfno_internal.h"
#include "dhconv_map.h"

namespace sfno {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));

// grid = dh_blocks workgroups (see dh_map), row groups of DH_GROUP; VEC4: 2*I is a multiple of 4 so activation rows can be read as float4
constexpr int DH_GROUP = 64;                         // rows (m,b) per workgroup
template <bool VEC4>
__global__ __launch_bounds__(256, 4) void dhconv_kernel(DhconvArgs a) {
    constexpr int LDW = DH_COLS / 2 + 32;            // plane pitch = 32 mod 64: the two half-waves read different banks
    __shared__ __align__(16) float ws[2][3][8][LDW]; // [buffer][plane][input channel of the chunk][output channel]

    int l, ob, r0, ncols, rot;
    if (!dh_map(a, DH_GROUP, l, ob, r0, ncols, rot)) return;
    // Wavefront w of every workgroup runs on SIMD w, and low degrees fill only the first row blocks:
    // rotate the block a wavefront takes from workgroup to workgroup so that no SIMD gets all the work.
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = (__builtin_amdgcn_readfirstlane(tid >> 6) + rot) & 3;
    // wavefront = (row block of 32, column tile of 32 output channels)
    const int nrb = min(DH_GROUP / 32, (ncols - r0 + 31) / 32);
    const int rb = wave >> 1, t0 = wave & 1;
    const bool active = rb < nrb;
    const int nc = a.nc;                             // K chunks of 8 complex input channels
    const int kh = lane >> 5, cl = lane & 31;

    // my activation row (clamped: rows past the end repeat the last one and are not stored)
    const int n = min(r0 + 32 * rb + cl, ncols - 1);
    const int mm = n / a.B, bb = n - mm * a.B;
    const float* xrow = a.X + ((int64_t)mm * a.L + l) * a.ld_in + (int64_t)bb * a.I2;
    // packed weights of (l, ob): nc chunks of 8 x 64 complex, 16 bytes per thread and chunk
    const f4* wp = reinterpret_cast<const f4*>(a.W) + ((int64_t)l * a.nob + ob) * nc * 256 + tid;

    floatx16 acc[3];
#pragma unroll
    for (int p = 0; p < 3; ++p)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[p][v] = 0.0f;

    // A operands: lane (row, kh) holds the complex channels i = 8c + 4kh + s, s = 0..3, as (re, im) pairs; k-step s
    // of the chunk uses channel 4kh + s of the chunk on both operands.  Reads are clamped into the row; the weights
    // are zero beyond I.
    auto x_load = [&](int c, f4 (&xr)[2]) {
        if (VEC4) {
            // a group of two channels is either entirely inside the row or entirely in the zero-weight padding
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
    // thread t expands the complex pair (i = t/32, o = 2(t%32), 2(t%32)+1) of the chunk into the three planes
    auto w_store = [&](int buf, f4 w) {
        const int ii = tid >> 5, o2 = tid & 31;
        *reinterpret_cast<f2*>(&ws[buf][0][ii][2 * o2]) = f2{w[0], w[2]};
        *reinterpret_cast<f2*>(&ws[buf][1][ii][2 * o2]) = f2{w[1] - w[0], w[3] - w[2]};
        *reinterpret_cast<f2*>(&ws[buf][2][ii][2 * o2]) = f2{w[0] + w[1], w[2] + w[3]};
    };
    // one K-chunk of MFMAs; no branches inside
    auto compute = [&](int buf, const f4 (&xr)[2]) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const float re = xr[s >> 1][2 * (s & 1)], im = xr[s >> 1][2 * (s & 1) + 1];
            const float sum = re + im;
            const float* w0 = &ws[buf][0][4 * kh + s][32 * t0 + cl];
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(sum, w0[0], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(re, w0[8 * LDW], acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(im, w0[16 * LDW], acc[2], 0, 0, 0);
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
    // D rows = my 32 activation rows, D cols = output channels; (re, im) = (K1 - K3, K1 + K2)
    const int oc = DH_COLS * ob + 2 * (32 * t0 + cl);
    if (oc >= a.O2) return;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int nn = r0 + 32 * rb + 8 * (v >> 2) + 4 * kh + (v & 3);
        if (nn >= ncols) continue;
        const int m2 = nn / a.B, b2 = nn - m2 * a.B;
        float* orow = a.Y + ((int64_t)m2 * a.L + l) * a.ld_out + (int64_t)b2 * a.O2;
        *reinterpret_cast<f2*>(orow + oc) = f2{acc[0][v] - acc[2][v], acc[0][v] + acc[1][v]};
    }
}

// packed[l][ob][c][ii][o] (complex) = w[8c + ii][64 ob + o][l], zero outside the weight;
// adjoint: w is [O][I][L] and the packed element is conj(w[64 ob + o][8c + ii][l])
__global__ __launch_bounds__(256) void dhconv_pack_kernel(const float2* __restrict__ w, float2* __restrict__ packed, int I, int O, int L,
                                                          int nob, int nc, int adjoint) {
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
    if (i < I && oo < O) {
        if (adjoint) {
            v = w[((int64_t)oo * I + i) * L + l];
            v.y = -v.y;
        } else {
            v = w[((int64_t)i * O + oo) * L + l];
        }
    }
    packed[idx] = v;
}

int dhconv_pack_launch(const float2* w, float* packed, int I, int O, int L, int adjoint, hipStream_t s) {
    const int nob = (2 * O + DH_COLS - 1) / DH_COLS, nc = (2 * I + PG_KC - 1) / PG_KC;
    const int64_t total = (int64_t)L * nob * nc * 512;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(dhconv_pack_kernel, dim3((unsigned)blocks), dim3(256), 0, s, w, reinterpret_cast<float2*>(packed), I, O, L, nob, nc, adjoint);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

// ---- bf16 variant ---------------------------------------------------------------------------------------
// Same decomposition on v_mfma_f32_32x32x16_bf16 (fp32 accumulate): activations are rounded to bf16 (nearest
// even) in registers as they arrive, weights are stored as complex bf16 and expanded to the real embedding by
// two bit operations per word while they are copied to LDS.  K is walked in chunks of 32 i'; lane group kg of a
// wavefront takes i' = 32c + 16kg + 8s .. +7 in k-step s, on both operands, so that every lane reads 64
// contiguous bytes of its activation row and 16 contiguous bytes of a weight column per step.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));
typedef unsigned int u2 __attribute__((ext_vector_type(2)));
constexpr int DHB_COLS = 256;          // output columns o' per workgroup
constexpr int DHB_KC = 32;             // i' per chunk

__device__ __forceinline__ bf16x8 to_bf16x8(f4 a, f4 b) {
    bf16x8 v;
    v[0] = (__bf16)a[0]; v[1] = (__bf16)a[1]; v[2] = (__bf16)a[2]; v[3] = (__bf16)a[3];
    v[4] = (__bf16)b[0]; v[5] = (__bf16)b[1]; v[6] = (__bf16)b[2]; v[7] = (__bf16)b[3];
    return v;
}

// grid = dh_blocks workgroups (see dh_map), row groups of 128, nob = ceil(2*O / 256); requires 2*I % 8 == 0
__global__ __launch_bounds__(256, 2) void dhconv_bf16_kernel(DhconvArgs a) {
    constexpr int NT = DHB_COLS / 32;                // 8 column tiles per wavefront
    constexpr int PITCH = DHB_KC + 8;                // bf16 elements per LDS row (80 bytes: 16-byte reads of 16 lanes hit distinct banks)
    __shared__ __align__(16) unsigned short ws[2][DHB_COLS][PITCH];

    int l, ob, r0, ncols, rot;
    if (!dh_map(a, 128, l, ob, r0, ncols, rot)) return;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = (__builtin_amdgcn_readfirstlane(tid >> 6) + rot) & 3;
    const bool active = r0 + 32 * wave < ncols;
    const int nc = a.nc;                                           // chunks of 32 i'
    const int kg = lane >> 5, cl = lane & 31;

    const int n = min(r0 + 32 * wave + cl, ncols - 1);
    const int mm = n / a.B, bb = n - mm * a.B;
    const float* xrow = a.X + ((int64_t)mm * a.L + l) * a.ld_in + (int64_t)bb * a.I2;
    // packed weights of (l, ob): nc chunks of 128 (o) x 16 (i) complex bf16 = 8 KiB, two 16-byte pieces per thread
    const u4* wp = reinterpret_cast<const u4*>(a.W) + ((int64_t)l * a.nob + ob) * nc * 512 + tid;

    floatx16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.0f;

    // my 16 activations of the chunk: i' = 32c + 16kg .. +15 (clamped in groups of four; weights are zero past 2*I)
    auto x_load = [&](int c, f4 (&xr)[4]) {
        const int k = DHB_KC * c + 16 * kg;
#pragma unroll
        for (int j = 0; j < 4; ++j) xr[j] = *reinterpret_cast<const f4*>(xrow + min(k + 4 * j, a.I2 - 4));
    };
    // piece e (16 bytes = 4 complex = 8 i') of the chunk: o = e / 4, i-group g = e % 4; it becomes 16 bytes of row 2o
    // (re, -im, ...) and 16 bytes of row 2o+1 (im, re, ...)
    auto w_store = [&](int buf, const u4 (&w)[2]) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int e = tid + 256 * u, o = e >> 2, g = e & 3;
            const u4 even = w[u] ^ 0x80000000u;
            const u4 odd = (w[u] >> 16) | (w[u] << 16);
            *reinterpret_cast<u4*>(&ws[buf][2 * o][8 * g]) = even;
            *reinterpret_cast<u4*>(&ws[buf][2 * o + 1][8 * g]) = odd;
        }
    };
    auto compute = [&](int buf, const f4 (&xr)[4]) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const bf16x8 xa = to_bf16x8(xr[2 * s], xr[2 * s + 1]);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const bf16x8 wb = *reinterpret_cast<const bf16x8*>(&ws[buf][32 * t + cl][16 * kg + 8 * s]);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa, wb, acc[t], 0, 0, 0);
            }
        }
    };

    f4 xcur[4], xnext[4];
    u4 wnext[2];
    x_load(0, xcur);
    wnext[0] = wp[0];
    wnext[1] = wp[256];
    w_store(0, wnext);
    __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0)
    __syncthreads();
    for (int c = 0; c < nc; ++c) {
        const int buf = c & 1;
        const bool more = c + 1 < nc;
        if (more) {
            wnext[0] = wp[(int64_t)(c + 1) * 512];
            wnext[1] = wp[(int64_t)(c + 1) * 512 + 256];
            x_load(c + 1, xnext);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (active) compute(buf, xcur);
        __builtin_amdgcn_sched_barrier(0);
        if (more) w_store(buf ^ 1, wnext);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) xcur[j] = xnext[j];
    }

    if (!active) return;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int nn = r0 + 32 * wave + 8 * (v >> 2) + 4 * kg + (v & 3);
        if (nn >= ncols) continue;
        const int m2 = nn / a.B, b2 = nn - m2 * a.B;
        float* orow = a.Y + ((int64_t)m2 * a.L + l) * a.ld_out + (int64_t)b2 * a.O2;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int oc = DHB_COLS * ob + 32 * t + cl;
            if (oc < a.O2) orow[oc] = acc[t][v];
        }
    }
}

// packed[l][ob][c][o (128)][i (16)] = bf16(re) | bf16(im) << 16 of w[16c + i][128 ob + o][l], zero outside the weight
// (adjoint: of conj(w[128 ob + o][16c + i][l]), w being [O][I][L])
__global__ __launch_bounds__(256) void dhconv_pack_bf16_kernel(const float2* __restrict__ w, unsigned int* __restrict__ packed, int I, int O, int L,
                                                               int nob, int nc, int adjoint) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = (int64_t)L * nob * nc * 2048;
    if (idx >= total) return;
    const int ii = (int)(idx & 15), o = (int)((idx >> 4) & 127);
    int64_t rem = idx >> 11;
    const int c = (int)(rem % nc);
    rem /= nc;
    const int ob = (int)(rem % nob), l = (int)(rem / nob);
    const int i = 16 * c + ii, oo = 128 * ob + o;
    unsigned int v = 0;
    if (i < I && oo < O) {
        float2 z;
        if (adjoint) {
            z = w[((int64_t)oo * I + i) * L + l];
            z.y = -z.y;
        } else {
            z = w[((int64_t)i * O + oo) * L + l];
        }
        const __bf16 re = (__bf16)z.x, im = (__bf16)z.y;
        v = (unsigned int)__builtin_bit_cast(unsigned short, re) | ((unsigned int)__builtin_bit_cast(unsigned short, im) << 16);
    }
    packed[idx] = v;
}

int dhconv_pack_bf16_launch(const float2* w, void* packed, int I, int O, int L, int adjoint, hipStream_t s) {
    const int nob = (2 * O + DHB_COLS - 1) / DHB_COLS, nc = (2 * I + DHB_KC - 1) / DHB_KC;
    const int64_t total = (int64_t)L * nob * nc * 2048;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(dhconv_pack_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, s, w, reinterpret_cast<unsigned int*>(packed), I, O, L, nob, nc, adjoint);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int dhconv_bf16_launch(const DhconvArgs& a, hipStream_t s) {
    const int64_t rows_max = (int64_t)a.M * a.B;
    if (rows_max <= 0 || a.L <= 0) return SFNO_OK;
    if (a.I2 % 4 != 0 || a.ld_in % 4 != 0) return SFNO_EUNSUPPORTED;
    const int64_t blocks = dh_blocks(a, 128);
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(dhconv_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

// ---- fp32 on the bf16 matrix pipe -----------------------------------------------------------------------
// The decomposition of dhconv_bf16_kernel (2x2 real embedding, activation rows as A operands straight from the
// spectral layout, weights expanded into LDS) with fp32 accuracy: every operand is cut exactly into three bf16
// numbers (8 + 8 + 8 significant bits, by truncation) and the six partial products larger than 2^-23 of the result are
// accumulated in fp32, each of them exact.  One K = 16 step then costs 6 x 32 matrix-pipe cycles; the fp32 instruction
// needs 8 x 64 for the four real products of the embedding and 6 x 64 for Gauss's three.  The weights are stored as
// three planes of complex bf16 (12 bytes per complex weight), split when they are packed; the activations are split in
// registers, once per 16 values and wavefront, and reused for the four column tiles.
constexpr int DHS_COLS = 128;          // output columns o' per workgroup
constexpr int DHS_KC = 16;             // i' per chunk: one matrix K step, small enough for four workgroups per CU

// x = hi + mid + lo with 8 significant bits each; the pair (a, b) packed as two bf16 per plane
__device__ __forceinline__ void dh_split3(float a, float b, unsigned int& hi, unsigned int& mid, unsigned int& lo) {
    const unsigned int ab = __builtin_bit_cast(unsigned int, a), bb = __builtin_bit_cast(unsigned int, b);
    const float a1 = a - __builtin_bit_cast(float, ab & 0xffff0000u), b1 = b - __builtin_bit_cast(float, bb & 0xffff0000u);
    const unsigned int a1b = __builtin_bit_cast(unsigned int, a1), b1b = __builtin_bit_cast(unsigned int, b1);
    const float a2 = a1 - __builtin_bit_cast(float, a1b & 0xffff0000u), b2 = b1 - __builtin_bit_cast(float, b1b & 0xffff0000u);
    hi = __builtin_amdgcn_perm(bb, ab, 0x07060302u);
    mid = __builtin_amdgcn_perm(b1b, a1b, 0x07060302u);
    lo = __builtin_amdgcn_perm(__builtin_bit_cast(unsigned int, b2), __builtin_bit_cast(unsigned int, a2), 0x07060302u);
}

// Matrix and vector instructions of one wavefront overlap only where they alternate in its instruction stream (a
// wavefront queueing matrix instructions back to back also holds up the vector instructions of the other wavefronts of
// its SIMD), so the kernel is software-pipelined by hand: while the 24 matrix instructions of chunk c are issued, the
// activations of chunk c+1 are split and the weights of chunk c+1 are expanded into the other LDS buffer, a few vector
// instructions after each matrix instruction, behind scheduling fences; the loads run two chunks ahead.
// grid = dh_blocks workgroups (see dh_map), row groups of 128, nob = ceil(2*O / 128); requires 2*I % 4 == 0
__global__ __launch_bounds__(256, 3) void dhconv_split_kernel(DhconvArgs a) {
    constexpr int NT = DHS_COLS / 32;                // 4 column tiles per wavefront
    constexpr int PITCH = DHS_KC + 8;                // bf16 elements per LDS row (48 bytes: 16-byte reads of 8 lanes hit distinct banks)
    constexpr int PLANE = DHS_COLS * PITCH;
    __shared__ __align__(16) unsigned short ws[2][3][DHS_COLS][PITCH];

    int l, ob, r0, ncols, rot;
    if (!dh_map(a, 128, l, ob, r0, ncols, rot)) return;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = (__builtin_amdgcn_readfirstlane(tid >> 6) + rot) & 3;
    const bool active = r0 + 32 * wave < ncols;
    const int nc = a.nc;                                           // chunks of 16 i'
    const int kg = lane >> 5, cl = lane & 31;

    const int n = min(r0 + 32 * wave + cl, ncols - 1);
    const int mm = n / a.B, bb = n - mm * a.B;
    const float* xrow = a.X + ((int64_t)mm * a.L + l) * a.ld_in + (int64_t)bb * a.I2;
    // packed weights of (l, ob): nc chunks of 3 planes x 64 (o) x 8 (i) complex bf16 = 6 KiB, one 8-byte piece per thread and plane
    const u2* wp = reinterpret_cast<const u2*>(a.W) + ((int64_t)l * a.nob + ob) * nc * 768 + tid;

    floatx16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.0f;

    // my 8 activations of the chunk: i' = 16c + 8kg .. +7 (clamped in groups of four; weights are zero past 2*I)
    auto x_load = [&](int c, f4 (&xr)[2]) {
        const int k = DHS_KC * c + 8 * kg;
#pragma unroll
        for (int j = 0; j < 2; ++j) xr[j] = *reinterpret_cast<const f4*>(xrow + min(k + 4 * j, a.I2 - 4));
    };
    auto w_load = [&](int c, u2 (&w)[3]) {
#pragma unroll
        for (int p = 0; p < 3; ++p) w[p] = wp[(int64_t)c * 768 + 256 * p];
    };
    // piece tid (8 bytes = 2 complex = 4 i') of a plane: o = tid / 4, i-group g = tid % 4; it becomes 8 bytes of row 2o
    // (re, -im, ...) and 8 bytes of row 2o+1 (im, re, ...); negating a number negates each of its three parts
    const int wo_ = tid >> 2, wg_ = tid & 3;
    auto w_store_even = [&](int buf, int p, const u2 w) { *reinterpret_cast<u2*>(&ws[buf][p][2 * wo_][4 * wg_]) = w ^ 0x80000000u; };
    auto w_store_odd = [&](int buf, int p, const u2 w) { *reinterpret_cast<u2*>(&ws[buf][p][2 * wo_ + 1][4 * wg_]) = (w >> 16) | (w << 16); };
    // the three bf16 planes of my 8 activations: pl[0] = upper, pl[1] = middle, pl[2] = lower 8 significant bits
    auto split_pair = [&](const f4 (&xr)[2], int e, int stage, u4 (&pl)[3], float (&r)[2]) {
        const f4 src = xr[e >> 1];
        const float xa = src[2 * (e & 1)], xb = src[2 * (e & 1) + 1];
        if (stage == 0) {
            const unsigned int ab = __builtin_bit_cast(unsigned int, xa), bb2 = __builtin_bit_cast(unsigned int, xb);
            r[0] = xa - __builtin_bit_cast(float, ab & 0xffff0000u);
            r[1] = xb - __builtin_bit_cast(float, bb2 & 0xffff0000u);
            pl[0][e] = __builtin_amdgcn_perm(bb2, ab, 0x07060302u);
        } else {
            const unsigned int ab = __builtin_bit_cast(unsigned int, r[0]), bb2 = __builtin_bit_cast(unsigned int, r[1]);
            const float a2 = r[0] - __builtin_bit_cast(float, ab & 0xffff0000u), b2 = r[1] - __builtin_bit_cast(float, bb2 & 0xffff0000u);
            pl[1][e] = __builtin_amdgcn_perm(bb2, ab, 0x07060302u);
            pl[2][e] = __builtin_amdgcn_perm(__builtin_bit_cast(unsigned int, b2), __builtin_bit_cast(unsigned int, a2), 0x07060302u);
        }
    };
    auto split_all = [&](const f4 (&xr)[2], u4 (&pl)[3]) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float r[2];
            split_pair(xr, e, 0, pl, r);
            split_pair(xr, e, 1, pl, r);
        }
    };
    // Chunk `buf` contracted with planes pc; meanwhile xn (chunk c+1) is split into pn and wn (chunk c+1) goes to LDS.
    // 14 staging steps are dealt out behind the 24 matrix instructions.
    auto fused = [&](int buf, const u4 (&pc)[3], const f4 (&xn)[2], u4 (&pn)[3], const u2 (&wn)[3]) {
        const bf16x8 a0 = __builtin_bit_cast(bf16x8, pc[0]), a1 = __builtin_bit_cast(bf16x8, pc[1]), a2 = __builtin_bit_cast(bf16x8, pc[2]);
        const unsigned short* wb = &ws[buf][0][cl][8 * kg];
        float r[2];
        auto step = [&](int sidx) {
            if (sidx < 8) split_pair(xn, sidx >> 1, sidx & 1, pn, r);
            else if (sidx < 11) w_store_even(buf ^ 1, sidx - 8, wn[sidx - 8]);
            else w_store_odd(buf ^ 1, sidx - 11, wn[sidx - 11]);
        };
        constexpr int NM = 6 * NT, NS = 14;
        u4 bq[2][3];
#pragma unroll
        for (int p = 0; p < 3; ++p) bq[0][p] = *reinterpret_cast<const u4*>(wb + p * PLANE);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (t + 1 < NT) {
#pragma unroll
                for (int p = 0; p < 3; ++p) bq[(t + 1) & 1][p] = *reinterpret_cast<const u4*>(wb + p * PLANE + 32 * (t + 1) * PITCH);
            }
            const bf16x8 b0 = __builtin_bit_cast(bf16x8, bq[t & 1][0]), b1 = __builtin_bit_cast(bf16x8, bq[t & 1][1]),
                         b2 = __builtin_bit_cast(bf16x8, bq[t & 1][2]);
#pragma unroll
            for (int j = 0; j < 6; ++j) {
                // smallest terms first: a2 b0, a1 b1, a0 b2, a1 b0, a0 b1, a0 b0
                const bf16x8 av = (j == 0) ? a2 : (j == 1 || j == 3) ? a1 : a0;
                const bf16x8 bv = (j == 0 || j == 3 || j == 5) ? b0 : (j == 1 || j == 4) ? b1 : b2;
                __builtin_amdgcn_sched_barrier(0);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc[t], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                const int mi = 6 * t + j;
#pragma unroll
                for (int sidx = (mi * NS) / NM; sidx < ((mi + 1) * NS) / NM; ++sidx) step(sidx);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // a wavefront without rows still stages its share of the weights
    auto stage_only = [&](int buf, const u2 (&wn)[3]) {
#pragma unroll
        for (int p = 0; p < 3; ++p) {
            w_store_even(buf ^ 1, p, wn[p]);
            w_store_odd(buf ^ 1, p, wn[p]);
        }
    };

    // Register sets alternate between even and odd chunks (no copies: a copy would wait for the load it copies):
    // iteration c contracts planes P[c & 1], splits X[(c + 1) & 1] into P[(c + 1) & 1], stores W[(c + 1) & 1] to LDS and
    // then requests chunk c + 3 into those two sets; chunk c + 2 is already on its way into X[c & 1] and W[c & 1].
    f4 X0[2], X1[2];
    u2 W0[3], W1[3];
    u4 P0[3], P1[3];
    x_load(0, X0);
    w_load(0, W0);
    x_load(min(1, nc - 1), X1);
    w_load(min(1, nc - 1), W1);
    stage_only(1, W0);                            // chunk 0 into buffer 0
    split_all(X0, P0);
    __syncthreads();
    auto iter = [&](int c, const u4 (&pc)[3], u4 (&pn)[3], f4 (&xn)[2], u2 (&wn)[3]) {
        // chunk c+1 is staged even in the last iteration (a repeat of the last chunk, into the idle buffer)
        if (active) fused(c & 1, pc, xn, pn, wn);
        else stage_only(c & 1, wn);
        // xn and wn are consumed: chunk c+3 goes there (chunk c+2 is in flight or has landed in the other sets)
        x_load(min(c + 3, nc - 1), xn);
        w_load(min(c + 3, nc - 1), wn);
        __syncthreads();
    };
    // X0/W0 held chunk 0 (consumed by the prologue): chunk 2 goes there before the loop
    x_load(min(2, nc - 1), X0);
    w_load(min(2, nc - 1), W0);
    int c = 0;
    for (; c + 1 < nc; c += 2) {
        iter(c, P0, P1, X1, W1);
        iter(c + 1, P1, P0, X0, W0);
    }
    if (c < nc) iter(c, P0, P1, X1, W1);

    if (!active) return;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int nn = r0 + 32 * wave + 8 * (v >> 2) + 4 * kg + (v & 3);
        if (nn >= ncols) continue;
        const int m2 = nn / a.B, b2 = nn - m2 * a.B;
        float* orow = a.Y + ((int64_t)m2 * a.L + l) * a.ld_out + (int64_t)b2 * a.O2;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int oc = DHS_COLS * ob + 32 * t + cl;
            if (oc < a.O2) orow[oc] = acc[t][v];
        }
    }
}

// packed[l][ob][c][plane][o (64)][i (8)] = bf16(re part) | bf16(im part) << 16 of plane `plane` of w[8c + i][64 ob + o][l], zero
// outside the weight (adjoint: of conj(w[64 ob + o][8c + i][l]), w being [O][I][L]); plane p of a float is its p-th group of 8
// significant bits.  The parameter has l fastest, the stream has it slowest: a workgroup moves the 8 x 64 channel pairs of
// one (c, ob) for 8 degrees through LDS, reading 64 contiguous bytes per pair and writing 2 KiB contiguous per plane and degree.
// grid (nc * nob, ceil(L / 8)), block 256
__global__ __launch_bounds__(256) void dhconv_pack_split_kernel(const float2* __restrict__ w, unsigned int* __restrict__ packed, int I, int O, int L,
                                                                int nob, int nc, int adjoint) {
    __shared__ float2 tile[512][9];                  // [pair = ii * 64 + o][degree], padded
    const int c = blockIdx.x % nc, ob = blockIdx.x / nc;
    const int l0 = blockIdx.y * 8;
    const int tid = threadIdx.x, dl = tid & 7;
#pragma unroll 4
    for (int pass = 0; pass < 16; ++pass) {
        const int pr = pass * 32 + (tid >> 3);       // eight lanes per pair: one 64-byte segment
        const int ii = pr >> 6, o = pr & 63;
        const int i = 8 * c + ii, oo = 64 * ob + o, l = l0 + dl;
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
    for (int d = 0; d < 8; ++d) {
        const int l = l0 + d;
        if (l >= L) break;
        unsigned int* dst = packed + (((int64_t)l * nob + ob) * nc + c) * 1536;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int word = tid + 256 * u;          // o * 8 + ii
            const int o = word >> 3, ii = word & 7;
            float2 z = tile[ii * 64 + o][d];
#pragma unroll
            for (int plane = 0; plane < 3; ++plane) {
                const unsigned int xb = __builtin_bit_cast(unsigned int, z.x) & 0xffff0000u, yb = __builtin_bit_cast(unsigned int, z.y) & 0xffff0000u;
                dst[plane * 512 + word] = (xb >> 16) | yb;
                z.x -= __builtin_bit_cast(float, xb);
                z.y -= __builtin_bit_cast(float, yb);
            }
        }
    }
}

int dhconv_pack_split_launch(const float2* w, void* packed, int I, int O, int L, int adjoint, hipStream_t s) {
    const int nob = (2 * O + DHS_COLS - 1) / DHS_COLS, nc = (2 * I + DHS_KC - 1) / DHS_KC;
    if ((int64_t)nob * nc > 0x7fffffffLL || (L + 7) / 8 > 65535) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(dhconv_pack_split_kernel, dim3((unsigned)(nob * nc), (unsigned)((L + 7) / 8)), dim3(256), 0, s, w,
                       reinterpret_cast<unsigned int*>(packed), I, O, L, nob, nc, adjoint);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int dhconv_split_launch(const DhconvArgs& a, hipStream_t s) {
    const int64_t rows_max = (int64_t)a.M * a.B;
    if (rows_max <= 0 || a.L <= 0) return SFNO_OK;
    if (a.I2 % 4 != 0 || a.ld_in % 4 != 0) return SFNO_EUNSUPPORTED;
    const int64_t blocks = dh_blocks(a, 128);
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(dhconv_split_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int dhconv_launch(const DhconvArgs& a, hipStream_t s) {
    const int64_t rows_max = (int64_t)a.M * a.B;
    if (rows_max <= 0 || a.L <= 0) return SFNO_OK;
    const int64_t blocks = dh_blocks(a, DH_GROUP);
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    const dim3 grid((unsigned)blocks);
    const bool vec4 = a.I2 % 4 == 0 && a.ld_in % 4 == 0;
    if (vec4)
        hipLaunchKernelGGL((dhconv_kernel<true>), grid, dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL((dhconv_kernel<false>), grid, dim3(256), 0, s, a);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
