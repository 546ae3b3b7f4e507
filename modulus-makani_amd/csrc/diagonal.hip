// "diagonal" spectral operator: y[b,o,l,m] = sum_i x[b,i,l,m] w[i,o,l,m] on complex64 tensors in the
// reference layout (makani/models/common/contractions.py:121-127), its input gradient (the same sum over o
// with conj(w)) and its weight gradient.  One weight element is used once per batch entry, so the kernels
// are bound by the weight stream: a thread owns two consecutive (l, m) positions of one output channel
// (16-byte loads, consecutive threads on consecutive positions) and walks the contracted channel.
#include "sfno_internal.h"

namespace sfno {
namespace {

constexpr int DG_B = 4;   // batch entries accumulated per pass over the weights

__device__ __forceinline__ void cmac(float2& acc, const float2 a, const float2 w, const bool conj_w) {
    const float wi = conj_w ? -w.y : w.y;
    acc.x = fmaf(a.x, w.x, fmaf(-a.y, wi, acc.x));
    acc.y = fmaf(a.x, wi, fmaf(a.y, w.x, acc.y));
}

// y[b][r][p] = sum_a x[b][a][p] * W(a, r, p),  W(a, r, p) = w[(a * sa + r * sr) * P + p]  (conjugated if conj_w)
// forward: a = i, r = o, sa = O, sr = 1;   input gradient: a = o, r = i, sa = 1, sr = O, conj_w
__global__ __launch_bounds__(256) void diagonal_contract_kernel(const float2* __restrict__ x, const float2* __restrict__ w, float2* __restrict__ y,
                                                                int B, int A, int R, int64_t P, int64_t sa, int64_t sr, int conj_w, int vec) {
    const int64_t pair = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;      // pair of positions
    const int r = blockIdx.y;
    const int64_t p = 2 * pair;
    if (p >= P) return;
    const bool two = vec != 0;                    // even P and 16-byte aligned tensors: both positions in one load
    for (int b0 = 0; b0 < B; b0 += DG_B) {
        float2 acc[DG_B][2];
#pragma unroll
        for (int b = 0; b < DG_B; ++b) acc[b][0] = acc[b][1] = make_float2(0.f, 0.f);
        for (int a = 0; a < A; ++a) {
            const float2* wp = w + (a * sa + r * sr) * P + p;
            float2 w0, w1 = make_float2(0.f, 0.f);
            if (two) {
                const float4 t = *reinterpret_cast<const float4*>(wp);
                w0 = make_float2(t.x, t.y);
                w1 = make_float2(t.z, t.w);
            } else {
                w0 = wp[0];
                if (p + 1 < P) w1 = wp[1];
            }
#pragma unroll
            for (int b = 0; b < DG_B; ++b) {
                if (b0 + b < B) {
                    const float2* xp = x + ((int64_t)(b0 + b) * A + a) * P + p;
                    float2 x0, x1 = make_float2(0.f, 0.f);
                    if (two) {
                        const float4 t = *reinterpret_cast<const float4*>(xp);
                        x0 = make_float2(t.x, t.y);
                        x1 = make_float2(t.z, t.w);
                    } else {
                        x0 = xp[0];
                        if (p + 1 < P) x1 = xp[1];
                    }
                    cmac(acc[b][0], x0, w0, conj_w);
                    cmac(acc[b][1], x1, w1, conj_w);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < DG_B; ++b) {
            if (b0 + b < B) {
                float2* yp = y + ((int64_t)(b0 + b) * R + r) * P + p;
                yp[0] = acc[b][0];
                if (p + 1 < P) yp[1] = acc[b][1];
            }
        }
    }
}

// gw[i][o][p] = sum_b conj(x[b][i][p]) * g[b][o][p]
__global__ __launch_bounds__(256) void diagonal_wgrad_kernel(const float2* __restrict__ x, const float2* __restrict__ g, float2* __restrict__ gw,
                                                             int B, int I, int O, int64_t P) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= P) return;
    const int o = blockIdx.y, i = blockIdx.z;
    float2 acc = make_float2(0.f, 0.f);
    for (int b = 0; b < B; ++b) {
        const float2 xv = x[((int64_t)b * I + i) * P + p], gv = g[((int64_t)b * O + o) * P + p];
        acc.x = fmaf(xv.x, gv.x, fmaf(xv.y, gv.y, acc.x));
        acc.y = fmaf(xv.x, gv.y, fmaf(-xv.y, gv.x, acc.y));
    }
    gw[((int64_t)i * O + o) * P + p] = acc;
}

}  // namespace

int diagonal_contract_launch(const float2* x, const float2* w, float2* y, int B, int I, int O, int64_t P, int adjoint, hipStream_t s) {
    // adjoint: x is the output gradient [B][O][P], y the input gradient [B][I][P]
    const int A = adjoint ? O : I, R = adjoint ? I : O;
    if (B < 1 || I < 1 || O < 1 || P < 1 || R > 65535) return SFNO_EUNSUPPORTED;
    const int64_t pairs = (P + 1) / 2, blocks = (pairs + 255) / 256;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    const int vec = P % 2 == 0 && (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0;
    hipLaunchKernelGGL(diagonal_contract_kernel, dim3((unsigned)blocks, (unsigned)R), dim3(256), 0, s, x, w, y, B, A, R, P,
                       (int64_t)(adjoint ? 1 : O), (int64_t)(adjoint ? O : 1), adjoint, vec);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

int diagonal_wgrad_launch(const float2* x, const float2* g, float2* gw, int B, int I, int O, int64_t P, hipStream_t s) {
    if (B < 1 || I < 1 || O < 1 || P < 1 || O > 65535 || I > 65535) return SFNO_EUNSUPPORTED;
    const int64_t blocks = (P + 255) / 256;
    if (blocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    hipLaunchKernelGGL(diagonal_wgrad_kernel, dim3((unsigned)blocks, (unsigned)O, (unsigned)I), dim3(256), 0, s, x, g, gw, B, I, O, P);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

}  // namespace sfno
