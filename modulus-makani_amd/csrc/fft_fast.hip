// Specialised FFTs for the transform lengths the SFNO uses (1440 = 16*10*9, 480 = 10*16*3, ...),
// along longitude and, for the planar transform pair, along latitude: everything about the
// length is a compile-time constant.
//
// A workgroup transforms S complex sequences (2*S channels at one latitude) held in LDS.
// The length factors as N = R0*R1*R2 and every pass is one radix-R butterfly per thread,
// computed in registers by a compile-time Cooley-Tukey recursion over the base radices
// 2,3,4,5 with constant twiddles.  Passes work in place:
//   forward (rfft) : decimation in frequency, natural-order input, digit-reversed output,
//                    which the Hermitian split / order-major store gathers anyway;
//   inverse (irfft): decimation in time, the Hermitian extension scatters its input to
//                    digit-reversed positions, output is in natural order so rows leave
//                    LDS as contiguous float4 stores.
// Inter-pass twiddles come from two small per-plan tables (float64-computed, read through
// L1): tw0[j*R0 + k0] = w_N^(k0*j), tw1[n2*R1 + k1] = w_N^(R0*k1*n2) -- the factors of one
// butterfly are neighbours in memory (entry 0 of each group is 1 and never read), so a thread
// fetches them with 16-byte loads at constant offsets from one address.
#include "sfno_internal.h"

#include <algorithm>
#include <cmath>
#include <vector>

namespace sfno {

namespace {

constexpr double kTwoPi = 6.283185307179586476925286766559;

constexpr double ct_cos(double x) {
    double term = 1.0, sum = 1.0;
    for (int i = 1; i <= 24; ++i) {
        term *= -x * x / ((2.0 * i - 1.0) * (2.0 * i));
        sum += term;
    }
    return sum;
}
constexpr double ct_sin(double x) {
    double term = x, sum = x;
    for (int i = 1; i <= 24; ++i) {
        term *= -x * x / ((2.0 * i) * (2.0 * i + 1.0));
        sum += term;
    }
    return sum;
}

// forward twiddles w_R^i = exp(-2 pi i / R): c = cos, s = -sin
template <int R>
struct TwTab {
    float c[R];
    float s[R];
};
template <int R>
constexpr TwTab<R> make_tw() {
    TwTab<R> t{};
    for (int i = 0; i < R; ++i) {
        // reduce to (-pi, pi] for the series; quarter turns are exact
        int num = i % R;
        double c = 0.0, s = 0.0;
        if ((4 * num) % R == 0) {
            int q = (4 * num) / R;
            c = (q == 0) ? 1.0 : (q == 2) ? -1.0 : 0.0;
            s = (q == 1) ? 1.0 : (q == 3) ? -1.0 : 0.0;
        } else {
            double x = kTwoPi * (double)num / (double)R;
            if (x > kTwoPi / 2) x -= kTwoPi;
            c = ct_cos(x);
            s = ct_sin(x);
        }
        t.c[i] = (float)c;
        t.s[i] = (float)(-s);
    }
    return t;
}

__device__ __forceinline__ float2 cmul(float2 a, float2 b) { return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x); }
__device__ __forceinline__ float2 cadd(float2 a, float2 b) { return make_float2(a.x + b.x, a.y + b.y); }
__device__ __forceinline__ float2 csub(float2 a, float2 b) { return make_float2(a.x - b.x, a.y - b.y); }
template <int INV>
__device__ __forceinline__ float2 mul_mi(float2 a) { return INV ? make_float2(-a.y, a.x) : make_float2(a.y, -a.x); }
template <int INV>
__device__ __forceinline__ float2 cmul_tw(float2 a, float2 w) {
    if (INV) w.y = -w.y;
    return cmul(a, w);
}

constexpr int first_factor(int r) { return (r % 4 == 0 && r > 4) ? 4 : (r % 2 == 0) ? 2 : (r % 3 == 0) ? 3 : (r % 5 == 0) ? 5 : r; }

// In-register DFT of length R (natural order in and out), sign -1 (INV = 0) or +1 (INV = 1).
template <int R, int INV>
__device__ __forceinline__ void dft(float2 (&v)[R]) {
    if constexpr (R == 1) {
    } else if constexpr (R == 2) {
        float2 a = v[0], b = v[1];
        v[0] = cadd(a, b);
        v[1] = csub(a, b);
    } else if constexpr (R == 3) {
        const float s3 = 0.86602540378443864676f;
        float2 t1 = cadd(v[1], v[2]);
        float2 t2 = make_float2(v[0].x - 0.5f * t1.x, v[0].y - 0.5f * t1.y);
        float2 d = csub(v[1], v[2]);
        float2 t3 = mul_mi<INV>(make_float2(s3 * d.x, s3 * d.y));
        v[0] = cadd(v[0], t1);
        v[1] = cadd(t2, t3);
        v[2] = csub(t2, t3);
    } else if constexpr (R == 4) {
        float2 a0 = cadd(v[0], v[2]), a1 = csub(v[0], v[2]);
        float2 a2 = cadd(v[1], v[3]), a3 = mul_mi<INV>(csub(v[1], v[3]));
        v[0] = cadd(a0, a2);
        v[1] = cadd(a1, a3);
        v[2] = csub(a0, a2);
        v[3] = csub(a1, a3);
    } else if constexpr (R == 5) {
        const float c1 = 0.30901699437494742410f, c2 = -0.80901699437494742410f;
        const float s1 = 0.95105651629515357212f, s2 = 0.58778525229247312917f;
        float2 p1 = cadd(v[1], v[4]), m1 = csub(v[1], v[4]);
        float2 p2 = cadd(v[2], v[3]), m2 = csub(v[2], v[3]);
        float2 e1 = make_float2(v[0].x + c1 * p1.x + c2 * p2.x, v[0].y + c1 * p1.y + c2 * p2.y);
        float2 e2 = make_float2(v[0].x + c2 * p1.x + c1 * p2.x, v[0].y + c2 * p1.y + c1 * p2.y);
        float2 f1 = mul_mi<INV>(make_float2(s1 * m1.x + s2 * m2.x, s1 * m1.y + s2 * m2.y));
        float2 f2 = mul_mi<INV>(make_float2(s2 * m1.x - s1 * m2.x, s2 * m1.y - s1 * m2.y));
        v[0] = cadd(v[0], cadd(p1, p2));
        v[1] = cadd(e1, f1);
        v[2] = cadd(e2, f2);
        v[3] = csub(e2, f2);
        v[4] = csub(e1, f1);
    } else {
        // R = A*B, n = n1*B + n2, k = k1 + A*k2:
        //   X[k1 + A k2] = sum_n2 w_B^(n2 k2) w_R^(n2 k1) sum_n1 x[n1 B + n2] w_A^(n1 k1)
        constexpr int A = first_factor(R), B = R / A;
        static_assert(A > 1 && A < R, "radix must factor into 2, 3, 4, 5");
        constexpr TwTab<R> tw = make_tw<R>();
        float2 y[R];
#pragma unroll
        for (int n2 = 0; n2 < B; ++n2) {
            float2 t[A];
#pragma unroll
            for (int n1 = 0; n1 < A; ++n1) t[n1] = v[n1 * B + n2];
            dft<A, INV>(t);
#pragma unroll
            for (int k1 = 0; k1 < A; ++k1) {
                const int idx = (n2 * k1) % R;
                y[k1 * B + n2] = (idx == 0) ? t[k1] : cmul_tw<INV>(t[k1], make_float2(tw.c[idx], tw.s[idx]));
            }
        }
#pragma unroll
        for (int k1 = 0; k1 < A; ++k1) {
            float2 u[B];
#pragma unroll
            for (int n2 = 0; n2 < B; ++n2) u[n2] = y[k1 * B + n2];
            dft<B, INV>(u);
#pragma unroll
            for (int k2 = 0; k2 < B; ++k2) v[k1 + A * k2] = u[k2];
        }
    }
}


template <int N, int R0, int R1, int R2>
struct Geo {
    static_assert(R0 * R1 * R2 == N, "factorisation");
    static constexpr int PITCH = N + 2;          // complex elements between sequences (keeps 16 B alignment, spreads banks)
    // position of output bin m of the decimation-in-frequency passes (= input slot of bin m for decimation in time)
    static __device__ __forceinline__ int pos(int m) {
        const int k0 = m % R0, t = m / R0;
        const int k1 = t % R1, k2 = t / R1;
        return k0 * (R1 * R2) + k1 * R2 + k2;
    }
};

// Grid-side element type: float (BF16 = false) or bfloat16 (BF16 = true).  The bf16 variants fuse the
// up-cast before the forward transform and the round-to-nearest-even down-cast after the inverse
// (the `x.float()` / `x.to(dtype)` passes of makani/models/common/spectral_convolution.py:127,146).
template <bool BF16>
__device__ __forceinline__ float4 load4(const void* base, int64_t idx) {
    if (BF16) {
        const uint2 v = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned short*>(base) + idx);
        return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                           __uint_as_float(v.y & 0xffff0000u));
    }
    return *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(base) + idx);
}
// A tile's input as it sits in registers between its request and its use: four floats, or four bfloat16 in two words.
template <bool BF16>
struct Raw4 {
    using type = float4;
};
template <>
struct Raw4<true> {
    using type = uint2;
};
template <bool BF16>
__device__ __forceinline__ typename Raw4<BF16>::type load_raw4(const void* base, int64_t idx) {
    if constexpr (BF16)
        return *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned short*>(base) + idx);
    else
        return *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(base) + idx);
}
__device__ __forceinline__ float4 widen4(float4 v) { return v; }
__device__ __forceinline__ float4 widen4(uint2 v) {
    return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
}
// Marks the point up to which a requested value stays untouched in its registers: without it the compiler moves the
// register shuffles of the consumer up to the request and waits for the data there, before the work it should overlap.
__device__ __forceinline__ void use_here(float4& v) { asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w)); }
__device__ __forceinline__ void use_here(uint2& v) { asm volatile("" : "+v"(v.x), "+v"(v.y)); }

// two floats rounded to nearest-even bf16 in one word (the hardware conversion: one instruction per pair, NaN stays NaN)
__device__ __forceinline__ unsigned bf16_pair(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    const floatx2 f = {lo, hi};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f, bf16x2));
}
template <bool BF16>
__device__ __forceinline__ void store4(void* base, int64_t idx, float4 v) {
    if (BF16) {
        uint2 o;
        o.x = bf16_pair(v.x, v.y);
        o.y = bf16_pair(v.z, v.w);
        *reinterpret_cast<uint2*>(reinterpret_cast<unsigned short*>(base) + idx) = o;
    } else {
        *reinterpret_cast<float4*>(reinterpret_cast<float*>(base) + idx) = v;
    }
}

// Workgroups are handed to the 8 XCDs round-robin by linear id.  All channel groups of one
// latitude go to the same XCD, back to back, so that the 64-byte pieces they read or write
// of one order-major row meet in that XCD's L2 as whole cache lines.
__device__ __forceinline__ bool map_block(int nlat, int ngroups, int& lat, int& group) {
    const int id = blockIdx.x, xcd = id & 7, q = id >> 3;
    lat = (q / ngroups) * 8 + xcd;
    group = q % ngroups;
    return lat < nlat;
}

// Twiddle look-up of the passes.  TL = false: the per-plan tables in global memory, factors of one butterfly adjacent
// (tw0[j * R0 + r], tw1[n2 * R1 + r]).  TL = true: copies in LDS, one slab per factor index so that neighbouring lanes
// read neighbouring words (tw0[(r - 1) * NB + j], tw1[(r - 1) * R2 + n2]); see lds_tables.
template <bool TL, int R, int NJ>
__device__ __forceinline__ float2 twiddle(const float2* __restrict__ tw, int j, int r) {
    return TL ? tw[(r - 1) * NJ + j] : tw[j * R + r];
}

// Butterfly index of thread `tid` in round `it` of a pass with TOT butterflies.  A last, partial round is not given to the
// first wavefronts again but to those that idle in the pass with the fewest butterflies (1440 points, four sequences,
// eight wavefronts: 360 / 576 / 640 butterflies; the 64 + 128 left over go to wavefronts 6 and 7, whose SIMDs have no
// share in the first pass), which evens out the load of the four SIMDs.
template <int N, int R0, int R1, int R2, int S, int FT>
struct PassRounds {
    static constexpr int RL = (R2 > 1) ? R2 : R1;
    static constexpr int T0 = S * (N / R0), T1 = (R2 > 1) ? S * (N / R1) : T0, T2 = S * (N / RL);
    static constexpr int TMIN = T0 < T1 ? (T0 < T2 ? T0 : T2) : (T1 < T2 ? T1 : T2);
    static constexpr int ROT = TMIN < FT ? (((TMIN + 63) / 64) % (FT / 64)) * 64 : 0;
    template <int TOT>
    static __device__ __forceinline__ int index(int tid, int it) {
        if ((it + 1) * FT > TOT && it > 0 && ROT > 0) return it * FT + ((tid + FT - ROT) & (FT - 1));
        return it * FT + tid;
    }
};

// ---- forward: decimation in frequency ---------------------------------------------------------------
template <int N, int R0, int R1, int R2, int S, int FT, bool TL = false>
__device__ __forceinline__ void passes_dif(float2* z, const float2* __restrict__ tw0, const float2* __restrict__ tw1, int tid) {
    using G = Geo<N, R0, R1, R2>;
    {
        constexpr int NB = N / R0, TOT = S * NB;
#pragma unroll
        for (int it = 0; it < (TOT + FT - 1) / FT; ++it) {
            const int e = PassRounds<N, R0, R1, R2, S, FT>::template index<TOT>(tid, it);
            if (e < TOT) {
                const int p = e / NB, j = e - p * NB;
                float2* base = z + p * G::PITCH + j;
                float2 v[R0];
#pragma unroll
                for (int r = 0; r < R0; ++r) v[r] = base[r * NB];
                dft<R0, 0>(v);
                base[0] = v[0];
#pragma unroll
                for (int r = 1; r < R0; ++r) base[r * NB] = cmul(v[r], twiddle<TL, R0, NB>(tw0, j, r));
            }
        }
    }
    __syncthreads();
    if constexpr (R2 > 1) {
        constexpr int NB = N / R1, TOT = S * NB;
#pragma unroll
        for (int it = 0; it < (TOT + FT - 1) / FT; ++it) {
            const int e = PassRounds<N, R0, R1, R2, S, FT>::template index<TOT>(tid, it);
            if (e < TOT) {
                const int p = e / NB, j = e - p * NB;
                const int k0 = j / R2, n2 = j - k0 * R2;
                float2* base = z + p * G::PITCH + k0 * (R1 * R2) + n2;
                float2 v[R1];
#pragma unroll
                for (int r = 0; r < R1; ++r) v[r] = base[r * R2];
                dft<R1, 0>(v);
                base[0] = v[0];
#pragma unroll
                for (int r = 1; r < R1; ++r) base[r * R2] = cmul(v[r], twiddle<TL, R1, R2>(tw1, n2, r));
            }
        }
        __syncthreads();
    }
    {
        constexpr int RL = (R2 > 1) ? R2 : R1;     // last radix acts on contiguous groups
        constexpr int NB = N / RL, TOT = S * NB;
#pragma unroll
        for (int it = 0; it < (TOT + FT - 1) / FT; ++it) {
            const int e = PassRounds<N, R0, R1, R2, S, FT>::template index<TOT>(tid, it);
            if (e < TOT) {
                const int p = e / NB, j = e - p * NB;
                float2* base = z + p * G::PITCH + j * RL;
                float2 v[RL];
#pragma unroll
                for (int r = 0; r < RL; ++r) v[r] = base[r];
                dft<RL, 0>(v);
#pragma unroll
                for (int r = 0; r < RL; ++r) base[r] = v[r];
            }
        }
    }
    __syncthreads();
}

// ---- inverse: decimation in time -------------------------------------------------------------------------
template <int N, int R0, int R1, int R2, int S, int FT, bool TL = false>
__device__ __forceinline__ void passes_dit(float2* z, const float2* __restrict__ tw0, const float2* __restrict__ tw1, int tid) {
    using G = Geo<N, R0, R1, R2>;
    {
        constexpr int RL = (R2 > 1) ? R2 : R1;
        constexpr int NB = N / RL, TOT = S * NB;
#pragma unroll
        for (int it = 0; it < (TOT + FT - 1) / FT; ++it) {
            const int e = PassRounds<N, R0, R1, R2, S, FT>::template index<TOT>(tid, it);
            if (e < TOT) {
                const int p = e / NB, j = e - p * NB;
                float2* base = z + p * G::PITCH + j * RL;
                float2 v[RL];
#pragma unroll
                for (int r = 0; r < RL; ++r) v[r] = base[r];
                dft<RL, 1>(v);
#pragma unroll
                for (int r = 0; r < RL; ++r) base[r] = v[r];
            }
        }
    }
    __syncthreads();
    if constexpr (R2 > 1) {
        constexpr int NB = N / R1, TOT = S * NB;
#pragma unroll
        for (int it = 0; it < (TOT + FT - 1) / FT; ++it) {
            const int e = PassRounds<N, R0, R1, R2, S, FT>::template index<TOT>(tid, it);
            if (e < TOT) {
                const int p = e / NB, j = e - p * NB;
                const int k0 = j / R2, n2 = j - k0 * R2;
                float2* base = z + p * G::PITCH + k0 * (R1 * R2) + n2;
                float2 v[R1];
                v[0] = base[0];
#pragma unroll
                for (int r = 1; r < R1; ++r) v[r] = cmul_tw<1>(base[r * R2], twiddle<TL, R1, R2>(tw1, n2, r));
                dft<R1, 1>(v);
#pragma unroll
                for (int r = 0; r < R1; ++r) base[r * R2] = v[r];
            }
        }
        __syncthreads();
    }
    {
        constexpr int NB = N / R0, TOT = S * NB;
#pragma unroll
        for (int it = 0; it < (TOT + FT - 1) / FT; ++it) {
            const int e = PassRounds<N, R0, R1, R2, S, FT>::template index<TOT>(tid, it);
            if (e < TOT) {
                const int p = e / NB, j = e - p * NB;
                float2* base = z + p * G::PITCH + j;
                float2 v[R0];
                v[0] = base[0];
#pragma unroll
                for (int r = 1; r < R0; ++r) v[r] = cmul_tw<1>(base[r * NB], twiddle<TL, R0, NB>(tw0, j, r));
                dft<R0, 1>(v);
#pragma unroll
                for (int r = 0; r < R0; ++r) base[r * NB] = v[r];
            }
        }
    }
    __syncthreads();
}

// Order handled by thread group u (0 <= u < MP) of a sweep over MP consecutive orders.  With R0 = 16 and four channel
// pairs per workgroup a wavefront serves 16 orders; bits 3 and 4 of u are swapped so that these are two runs of eight
// consecutive orders 16 apart: their slots k0 * (N / 16) + k1 * R2 + k2 then fall on all LDS bank pairs evenly
// (eight consecutive k0 at two consecutive k1), where 16 consecutive orders would share half of them.
template <int R0, int S, int MP>
__device__ __forceinline__ int sweep_order(int u) {
    if constexpr (R0 == 16 && S == 4 && MP >= 32) return (u & ~0x18) | ((u & 8) << 1) | ((u & 16) >> 1);
    return u;
}

// ---- longitude kernels ---------------------------------------------------------------------------------------
// Persistent workgroups: the grid holds as many workgroups as the chip keeps resident (two per CU), and each walks the
// tiles (latitude, group of S channel pairs) of its XCD in steps of the XCD's workgroup count, so that workgroups
// running at the same time work on neighbouring groups of the same latitudes and the 64-byte pieces they exchange
// with the order-major buffer meet in that XCD's L2 as whole lines.  The input of the next tile is requested into
// registers as soon as the current one has been copied to LDS and arrives while the passes run.  Between that request
// and its use no other value may come from global memory (loads return in order: waiting for a later one waits for
// the tile as well), so the inter-pass twiddles and the slot table are copied to LDS once per workgroup.
template <int N, int R0, int R1, int R2>
struct LdsTables {
    static constexpr int NB = N / R0;
    static constexpr int NTW1 = (R2 > 1) ? (R1 - 1) * R2 : 1;
    float2 tw0[(R0 - 1) * NB];
    float2 tw1[NTW1];
    unsigned post[N / 2 + 1];
};

template <int N, int R0, int R1, int R2, int FT>
__device__ __forceinline__ void lds_tables(LdsTables<N, R0, R1, R2>& t, const float2* __restrict__ tw0, const float2* __restrict__ tw1,
                                           const unsigned* __restrict__ post, int tid) {
    constexpr int NB = N / R0;
    for (int i = tid; i < (R0 - 1) * NB; i += FT) {
        const int r = i / NB, j = i - r * NB;
        t.tw0[i] = tw0[j * R0 + r + 1];
    }
    if constexpr (R2 > 1)
        for (int i = tid; i < (R1 - 1) * R2; i += FT) {
            const int r = i / R2, n2 = i - r * R2;
            t.tw1[i] = tw1[n2 * R1 + r + 1];
        }
    for (int i = tid; i <= N / 2; i += FT) t.post[i] = post[i];
}

// tile -> (latitude, first channel pair); tiles of XCD x are the groups of latitudes x, x + 8, ... in that order
struct TileWalk {
    int xcd, step, ntiles, ngroups;
    __device__ __forceinline__ TileWalk(int nlat, int ngroups_) : ngroups(ngroups_) {
        xcd = blockIdx.x & 7;
        step = gridDim.x >> 3;
        ntiles = ((nlat - xcd + 7) >> 3) * ngroups_;
    }
    __device__ __forceinline__ int first() const { return blockIdx.x >> 3; }
    __device__ __forceinline__ void locate(int t, int& lat, int& group) const {
        const int q = t / ngroups;
        lat = q * 8 + xcd;
        group = t - q * ngroups;
    }
};

// A tile is one latitude and S * H channel pairs: H = 2 batches of S = 4 pairs for the long rows, one batch of 8 for the
// shorter ones, so that per order a tile owns one whole 128-byte line of the order-major buffer (8 pairs x 16 bytes).
// Lines written or read in halves by different workgroups cost a third of the achievable bandwidth here (the two halves
// reach memory as separate partial-line transactions), so the forward kernel keeps the first batch's results in
// registers and stores both halves together, and the inverse kernel requests both halves together.
//
// grid = 8 * (workgroups per XCD) workgroups, see go_fast
template <int N, int R0, int R1, int R2, int S, int H, int FT, bool BF16>
__global__ __launch_bounds__(FT, 4) void rfft_fast_kernel(const float2* __restrict__ tw0, const float2* __restrict__ tw1, const unsigned* __restrict__ post,
                                                          const void* __restrict__ x, float* __restrict__ xm, int64_t rows, int nlat, int mmax, int ld,
                                                          int ngroups, float scale) {
    using G = Geo<N, R0, R1, R2>;
    static_assert((S & (S - 1)) == 0 && FT % S == 0 && N % 4 == 0, "a power-of-two number of channel pairs shares the threads evenly");
    static_assert(H == 1 || H == 2, "one or two batches per tile");
    __shared__ __align__(16) float2 z[S * G::PITCH];
    __shared__ LdsTables<N, R0, R1, R2> tab;
    const int tid = threadIdx.x;
    const TileWalk walk(nlat, ngroups);
    int t = walk.first();
    if (t >= walk.ntiles) return;
    lds_tables<N, R0, R1, R2, FT>(tab, tw0, tw1, post, tid);
    constexpr int TP = FT / S;                          // threads per channel pair
    constexpr int Q = N / 4, IT = (Q + TP - 1) / TP;
    constexpr int NSW = (N / 2 + 1 + TP - 1) / TP;      // sweeps of TP orders that cover every order a plan can keep
    // TP threads walk the two rows of one channel pair in steps of TP groups of four longitudes: one address per thread and
    // batch, constant offsets after that.  Requests are unconditional (a load under a branch would be waited for at the end
    // of its branch): rows that do not exist and the groups of four beyond the row's end read a valid address instead and
    // are zeroed on their way to LDS.
    const int pl = tid / TP, q0 = tid - pl * TP;
    typename Raw4<BF16>::type a[IT], b[IT];
    bool ha = false, hb = false;
    auto request = [&](int tile, int half) {
        int lat, group;
        walk.locate(tile, lat, group);
        const int64_t r0 = 2 * (int64_t)((group * H + half) * S + pl);
        ha = r0 < rows;
        hb = r0 + 1 < rows;
        const int64_t ia = ((ha ? r0 : 0) * nlat + lat) * N, ib = ((hb ? r0 + 1 : 0) * nlat + lat) * N;
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            // (a row can be shorter than one step of the TP threads: the fall-back address is the row's start, not the thread's)
            const bool in = (it + 1) * TP <= Q || q0 + it * TP < Q;
            const int off = in ? 4 * (q0 + it * TP) : 0;
            a[it] = load_raw4<BF16>(x, ia + off);
            b[it] = load_raw4<BF16>(x, ib + off);
        }
    };
    // the requested batch goes to LDS as complex sequences a + i b
    auto fill = [&]() {
        float4* dst = reinterpret_cast<float4*>(z + pl * G::PITCH) + 2 * q0;
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            use_here(a[it]);
            use_here(b[it]);
        }
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            if ((it + 1) * TP <= Q || q0 + it * TP < Q) {
                float4 fa = widen4(a[it]), fb = widen4(b[it]);
                if (!ha) fa = make_float4(0.f, 0.f, 0.f, 0.f);
                if (!hb) fb = make_float4(0.f, 0.f, 0.f, 0.f);
                dst[2 * it * TP] = make_float4(fa.x, fb.x, fa.y, fb.y);
                dst[2 * it * TP + 1] = make_float4(fa.z, fb.z, fa.w, fb.w);
            }
        }
    };
    const float h = 0.5f * scale;
    const int pp_ = tid & (S - 1);
    const int mfirst = sweep_order<R0, S, TP>(tid / S);
    const float2* zz = z + pp_ * G::PITCH;
    // Hermitian split: the two channels of a pair from bins m and N - m
    auto split = [&](int m) {
        const unsigned pp = tab.post[m];
        const float2 zp = zz[pp & 0xffffu], zq = zz[pp >> 16];
        return make_float4(h * (zp.x + zq.x), h * (zp.y - zq.y), h * (zp.y + zq.y), h * (zq.x - zp.x));
    };
    const int64_t mstep = (int64_t)TP * nlat * ld;
    request(t, 0);
    for (;;) {
        int lat, group;
        walk.locate(t, lat, group);
        const int tn = t + walk.step;
        const int tq = tn < walk.ntiles ? tn : t;       // the last tile requests itself again: always a request, never a branch around one
        const int pair = group * H * S + pp_;
        float* o = xm + ((int64_t)mfirst * nlat + lat) * ld + 4 * (int64_t)pair;
        fill();
        if (H == 2)
            request(t, 1);
        else
            request(tq, 0);
        __syncthreads();
        passes_dif<N, R0, R1, R2, S, FT, true>(z, tab.tw0, tab.tw1, tid);
        if constexpr (H == 1) {
            if (pair < ld / 4) {
#pragma unroll
                for (int u = 0; u < NSW; ++u)
                    if (mfirst + u * TP < mmax) *reinterpret_cast<float4*>(o + u * mstep) = split(mfirst + u * TP);
            }
        } else {
            float4 first[NSW];
#pragma unroll
            for (int u = 0; u < NSW; ++u)
                if (mfirst + u * TP < mmax) first[u] = split(mfirst + u * TP);
            __syncthreads();
            fill();
            request(tq, 0);
            __syncthreads();
            passes_dif<N, R0, R1, R2, S, FT, true>(z, tab.tw0, tab.tw1, tid);
            const bool va = pair < ld / 4, vb = pair + S < ld / 4;
#pragma unroll
            for (int u = 0; u < NSW; ++u) {
                if (mfirst + u * TP < mmax) {
                    const float4 second = split(mfirst + u * TP);
                    if (va) *reinterpret_cast<float4*>(o + u * mstep) = first[u];
                    if (vb) *reinterpret_cast<float4*>(o + u * mstep + 4 * S) = second;
                }
            }
        }
        if (tn >= walk.ntiles) break;
        __syncthreads();
        t = tn;
    }
}

// Inverse.  NSWA = sweeps of TP orders that are read from memory (ceil(mmax / TP), chosen by the launcher among the
// instantiated values; the orders of the remaining sweeps enter as zeros), LS = the per-latitude moments are written.
// Every global store that follows a request in program order is unconditional: the wait for a requested value counts the
// memory operations issued after it, and a store under a branch cannot be counted -- the kernel would wait for its
// stores to be acknowledged before it touches the next tile's input.  So nothing is skipped, it is aliased instead:
// a pair slot beyond the last pair of the tensor does the work of the last pair once more (same loads, same sequence,
// same stores of the same values), the missing second channel of an odd row count is a copy of the first and is stored
// to the first one's row, and the lanes past the end of a row store its last four values again.
template <int N, int R0, int R1, int R2, int S, int H, int FT, bool BF16, int NSWA, bool LS>
__global__ __launch_bounds__(FT, 4) void irfft_fast_kernel(const float2* __restrict__ tw0, const float2* __restrict__ tw1, const unsigned* __restrict__ post,
                                                           const float* __restrict__ xm, void* __restrict__ x, int64_t rows, int nlat, int mmax, int ld,
                                                           int ngroups, float2* __restrict__ lat_stats) {
    using G = Geo<N, R0, R1, R2>;
    static_assert(N % 4 == 0, "even length");
    static_assert((S & (S - 1)) == 0 && FT % S == 0 && 64 % S == 0, "a thread serves one channel pair");
    static_assert(H == 1 || H == 2, "one or two batches per tile");
    __shared__ __align__(16) float2 z[S * G::PITCH];
    __shared__ LdsTables<N, R0, R1, R2> tab;
    __shared__ float4 red[FT / 64][S];
    const int tid = threadIdx.x;
    const TileWalk walk(nlat, ngroups);
    int t = walk.first();
    if (t >= walk.ntiles) return;
    lds_tables<N, R0, R1, R2, FT>(tab, tw0, tw1, post, tid);
    constexpr int HALF = N / 2, TP = FT / S;
    constexpr int NSW = (HALF + 1 + TP - 1) / TP;        // sweeps over the orders 0..N/2
    static_assert(NSWA >= 1 && NSWA <= NSW, "sweeps that are read");
    // With few sweeps the coefficients of both batches of a tile are requested together (the two 64-byte halves of each line
    // in neighbouring requests: whole-line reads); with many, registers only allow one batch ahead.
    constexpr bool BOTH = H == 2 && NSWA * H <= 6;
    constexpr int HV = BOTH ? H : 1;
    const int pp_ = tid & (S - 1);
    const int mfirst = sweep_order<R0, S, TP>(tid / S);
    const int pl = tid / TP, q0 = tid - pl * TP;
    const int last_pair = (int)((rows + 1) / 2) - 1;
    float2* zz = z + pp_ * G::PITCH;
    // A thread keeps its pair and walks the orders in sweeps of TP.  Requests are unconditional, see the forward kernel: an
    // order the plan does not keep reads order 0 instead and is zeroed when it is used.
    float4 v[HV][NSWA];
    auto request = [&](int tile, int half) {
        int lat, group;
        walk.locate(tile, lat, group);
        const float* src = xm + (int64_t)lat * ld;
#pragma unroll
        for (int u = 0; u < NSWA; ++u) {
            const int m = mfirst + u * TP;
            const float* row = src + (int64_t)(m < mmax ? m : 0) * nlat * ld;
#pragma unroll
            for (int hh = 0; hh < HV; ++hh) {
                const int pair = (group * H + half + hh) * S + pp_;
                v[hh][u] = *reinterpret_cast<const float4*>(row + 4 * (pair < last_pair ? pair : last_pair));
            }
        }
    };
    request(t, 0);
    __syncthreads();                                      // tables
    for (;;) {
        int lat, group;
        walk.locate(t, lat, group);
        const int tn = t + walk.step;
        const int tq = tn < walk.ntiles ? tn : t;         // the last tile requests itself again: always a request, never a branch around one
#pragma unroll
        for (int hh = 0; hh < H; ++hh) {
            const int pair0 = (group * H + hh) * S;
            // moments of the output row over longitude, from the coefficients on their way in (LS): the mean is
            // Re X_0, the mean squared deviation from it 2 sum_{0<m<N/2} |X_m|^2 + (Re X_{N/2})^2; (A, B) = the two channels of the pair
            float mean_a = 0.f, mean_b = 0.f, dev_a = 0.f, dev_b = 0.f;
            {
                // Hermitian extension into the slots the decimation-in-time passes expect
                const int pe = pair0 + pp_ < last_pair ? pair0 + pp_ : last_pair;
                const bool hb = 2 * (int64_t)pe + 1 < rows;       // odd row count: the second channel of the last pair is a copy of the first
                float4(&vv)[NSWA] = v[BOTH ? hh : 0];
#pragma unroll
                for (int u = 0; u < NSWA; ++u) use_here(vv[u]);
#pragma unroll
                for (int u = 0; u < NSW; ++u) {
                    const int m = mfirst + u * TP;
                    if (m <= HALF) {
                        const unsigned pp = tab.post[m];
                        float4 w = make_float4(0.f, 0.f, 0.f, 0.f);
                        if (u < NSWA) {
                            w = vv[u < NSWA ? u : 0];
                            if (m >= mmax) w = make_float4(0.f, 0.f, 0.f, 0.f);
                            if (!hb) {
                                w.z = w.x;
                                w.w = w.y;
                            }
                        }
                        if (m == 0 || m == HALF) {
                            zz[pp & 0xffffu] = make_float2(w.x, w.z);                  // C2R: Im of mean and Nyquist bins dropped
                            if (m == 0) {
                                mean_a = w.x;
                                mean_b = w.z;
                            } else {
                                dev_a = fmaf(w.x, w.x, dev_a);
                                dev_b = fmaf(w.z, w.z, dev_b);
                            }
                        } else {
                            zz[pp & 0xffffu] = make_float2(w.x - w.w, w.y + w.z);
                            zz[pp >> 16] = make_float2(w.x + w.w, w.z - w.y);
                            if (LS && u < NSWA) {
                                dev_a += 2.f * fmaf(w.x, w.x, w.y * w.y);
                                dev_b += 2.f * fmaf(w.z, w.z, w.w * w.w);
                            }
                        }
                    }
                }
            }
            if constexpr (LS) {
                // lanes S apart serve the same pair: fold them, one entry per wavefront and pair
#pragma unroll
                for (int off = S; off < 64; off <<= 1) {
                    mean_a += __shfl_xor(mean_a, off, 64);
                    mean_b += __shfl_xor(mean_b, off, 64);
                    dev_a += __shfl_xor(dev_a, off, 64);
                    dev_b += __shfl_xor(dev_b, off, 64);
                }
                if ((tid & 63) < S) red[tid >> 6][tid & 63] = make_float4(mean_a, mean_b, dev_a, dev_b);
            }
            __syncthreads();
            if constexpr (LS) {
                if (tid < S) {
                    float4 s4 = red[0][tid];
#pragma unroll
                    for (int w = 1; w < FT / 64; ++w) {
                        const float4 u = red[w][tid];
                        s4.x += u.x; s4.y += u.y; s4.z += u.z; s4.w += u.w;
                    }
                    const int pe = pair0 + tid < last_pair ? pair0 + tid : last_pair;
                    const int64_t ra = 2 * (int64_t)pe, rb = ra + 1 < rows ? ra + 1 : ra;
                    lat_stats[ra * nlat + lat] = make_float2(s4.x, s4.z);
                    lat_stats[rb * nlat + lat] = make_float2(s4.y, s4.w);
                }
            }
            // the next batch's coefficients (after the stores above, so that only unconditional stores follow the request)
            if constexpr (BOTH) {
                if (hh == H - 1) request(tq, 0);
            } else {
                if (hh < H - 1)
                    request(t, hh + 1);
                else
                    request(tq, 0);
            }
            passes_dit<N, R0, R1, R2, S, FT, true>(z, tab.tw0, tab.tw1, tid);
            {
                // rows leave LDS in natural order: TP threads walk the two rows of one channel pair, constant offsets from one address
                constexpr int Q = N / 4, ITS = (Q + TP - 1) / TP;
                const int pe = pair0 + pl < last_pair ? pair0 + pl : last_pair;
                const int64_t ra = 2 * (int64_t)pe, rb = ra + 1 < rows ? ra + 1 : ra;
                const float4* src = reinterpret_cast<const float4*>(z + pl * G::PITCH);
#pragma unroll
                for (int it = 0; it < ITS; ++it) {
                    int i4 = q0 + it * TP;
                    if ((it + 1) * TP > Q) i4 = i4 < Q ? i4 : Q - 1;
                    const float4 u0 = src[2 * i4], u1 = src[2 * i4 + 1];
                    store4<BF16>(x, (ra * nlat + lat) * N + 4 * i4, make_float4(u0.x, u0.z, u1.x, u1.z));
                    store4<BF16>(x, (rb * nlat + lat) * N + 4 * i4, make_float4(u0.y, u0.w, u1.y, u1.w));
                }
            }
            if (hh < H - 1) __syncthreads();
        }
        if (tn >= walk.ntiles) break;
        __syncthreads();
        t = tn;
    }
}

// ---- latitude FFT of the planar transform pair -------------------------------------------------------------
// in[m][k][ld] -> out[m][j][ld] on the order-major layout (see latfft_launch): a workgroup transforms the LS = 8
// complex channels of one 64-byte line of every row of one order.  Rows arrive channel-contiguous and are
// transposed on the way into LDS, where each channel is one sequence of the in-place passes above.
//   INV = 0: decimation in frequency; kept frequency f leaves from slot pos(f).
//   INV = 1: decimation in time; kept frequency f enters at slot pos(f), dropped frequencies enter as zeros.
// grid = 8 * ceil(mmax/8) * ceil(ld / 16) workgroups: all channel groups of one order run back to back on one XCD
// (map_block), so that the two 64-byte halves of a 128-byte line are fetched into that XCD's L2 once.
constexpr int LS = 8;

template <int N, int R0, int R1, int R2, int FT, int INV>
__global__ __launch_bounds__(FT) void latfft_fast_kernel(const float2* __restrict__ tw0, const float2* __restrict__ tw1, const float* __restrict__ in,
                                                         float* __restrict__ out, int mmax, int lmax, int ld, int ngroups,
                                                         const float* __restrict__ mscale) {
    using G = Geo<N, R0, R1, R2>;
    __shared__ __align__(16) float2 z[LS * G::PITCH];
    const int tid = threadIdx.x;
    int m, group;
    if (!map_block(mmax, ngroups, m, group)) return;
    const int c0 = group * LS;
    const int lhigh = (lmax + 1) / 2, gap = N - lmax;
    const int nin = INV ? lmax : N, nout = INV ? N : lmax;
    const int c = tid & (LS - 1);
    const bool live = 2 * (c0 + c) < ld;
    const float* src = in + (int64_t)m * nin * ld + 2 * (c0 + c);
    {
        // all global loads of the workgroup are issued before the first LDS store
        constexpr int TOT = LS * N, IT = (TOT + FT - 1) / FT;
        float2 v[IT];
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int i = (tid + it * FT) / LS;
            // row of the input that belongs to element i of the sequence (-1: a dropped frequency)
            const int k = !INV ? i : i < lhigh ? i : i >= lhigh + gap ? i - gap : -1;
            v[it] = make_float2(0.f, 0.f);
            if (i < N && k >= 0 && live) v[it] = *reinterpret_cast<const float2*>(src + (int64_t)k * ld);
        }
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int i = (tid + it * FT) / LS;
            if (i < N) z[c * G::PITCH + (INV ? G::pos(i) : i)] = v[it];
        }
    }
    __syncthreads();
    if (INV)
        passes_dit<N, R0, R1, R2, LS, FT>(z, tw0, tw1, tid);
    else
        passes_dif<N, R0, R1, R2, LS, FT>(z, tw0, tw1, tid);
    if (!live) return;
    const float sc = mscale[m];
    float* dst = out + (int64_t)m * nout * ld + 2 * (c0 + c);
    for (int j = tid / LS; j < nout; j += FT / LS) {
        const int i = INV ? j : G::pos(j < lhigh ? j : j + gap);
        const float2 v = z[c * G::PITCH + i];
        *reinterpret_cast<float2*>(dst + (int64_t)j * ld) = make_float2(sc * v.x, sc * v.y);
    }
}

// Latitude FFT of a length n with a large prime factor (721 = 7 * 103, the 0.25 degree grid with both poles), as a
// circular convolution of length M >= 2n - 1 on the specialised passes (Bluestein):
//     X[j] = c[j] sum_k (x[k] c[k]) conj(c)[j - k],   c[k] = exp(-i pi k^2 / n)          (forward; conjugate c for the inverse)
// u = x c zero-padded to M -> decimation-in-frequency passes -> times vhat (the transform of conj(c) wrapped around M, in
// the slot order those passes leave, 1/M folded in; conj(c) is even, so the inverse uses conj(vhat)) -> decimation-in-time
// passes -> times c.  Same layouts, truncation rule and workgroup order as latfft_fast_kernel; S channels per workgroup.
template <int M, int R0, int R1, int R2, int S, int FT, int INV>
__global__ __launch_bounds__(FT) void latfft_chirp_kernel(const float2* __restrict__ tw0, const float2* __restrict__ tw1, const float2* __restrict__ chirp,
                                                          const float2* __restrict__ vhat, const float* __restrict__ in, float* __restrict__ out, int n,
                                                          int mmax, int lmax, int ld, int ngroups, const float* __restrict__ mscale) {
    using G = Geo<M, R0, R1, R2>;
    __shared__ __align__(16) float2 z[S * G::PITCH];
    const int tid = threadIdx.x;
    int m, group;
    if (!map_block(mmax, ngroups, m, group)) return;
    const int c0 = group * S;
    const int lhigh = (lmax + 1) / 2, gap = n - lmax;
    const int nin = INV ? lmax : n, nout = INV ? n : lmax;
    const int c = tid & (S - 1);
    const bool live = 2 * (c0 + c) < ld;
    const float* src = in + (int64_t)m * nin * ld + 2 * (c0 + c);
    for (int i = tid / S; i < M; i += FT / S) {
        const int k = i >= n ? -1 : !INV ? i : i < lhigh ? i : i >= lhigh + gap ? i - gap : -1;
        float2 v = make_float2(0.f, 0.f);
        if (k >= 0 && live) v = cmul_tw<INV>(*reinterpret_cast<const float2*>(src + (int64_t)k * ld), chirp[i]);
        z[c * G::PITCH + i] = v;
    }
    __syncthreads();
    passes_dif<M, R0, R1, R2, S, FT>(z, tw0, tw1, tid);
    for (int i = tid / S; i < M; i += FT / S) z[c * G::PITCH + i] = cmul_tw<INV>(z[c * G::PITCH + i], vhat[i]);
    __syncthreads();
    passes_dit<M, R0, R1, R2, S, FT>(z, tw0, tw1, tid);
    if (!live) return;
    const float sc = mscale[m];
    float* dst = out + (int64_t)m * nout * ld + 2 * (c0 + c);
    for (int j = tid / S; j < nout; j += FT / S) {
        const int i = INV ? j : j < lhigh ? j : j + gap;
        const float2 v = cmul_tw<INV>(z[c * G::PITCH + i], chirp[i]);
        *reinterpret_cast<float2*>(dst + (int64_t)j * ld) = make_float2(sc * v.x, sc * v.y);
    }
}

struct FastEntry {
    int n, r0, r1, r2;
};
// lengths with a specialised kernel; the last radix acts on contiguous groups, an odd one keeps LDS banks apart
const FastEntry kFast[] = {{1536, 16, 12, 8}, {1440, 16, 10, 9}, {1024, 16, 8, 8}, {720, 16, 5, 9}, {512, 8, 8, 8}, {480, 4, 8, 15}, {360, 8, 5, 9},
                           {256, 16, 16, 1}, {240, 16, 5, 3}, {180, 4, 5, 9}, {128, 8, 16, 1}, {64, 8, 8, 1}};

const FastEntry* find_fast(int n) {
    for (const auto& e : kFast)
        if (e.n == n) return &e;
    return nullptr;
}

template <int N, int R0, int R1, int R2, bool BF16>
int go_fast(bool inverse, const FftPlan& p, const void* in, void* out, int64_t rows, int nlat, int mmax, int ld, float2* lat_stats, hipStream_t s) {
    constexpr int S = (N >= 1024) ? 4 : 8;              // channel pairs in LDS at a time
    constexpr int H = 8 / S;                            // batches per tile: a tile owns 8 pairs = one 128-byte line per order
    constexpr int FT = (S * N >= 4096) ? 512 : 256;     // threads per workgroup
    const int ngroups = (ld / 4 + S * H - 1) / (S * H);
    // as many workgroups as stay resident (four wavefronts per SIMD: two workgroups of 512 threads or four of 256 per CU), the
    // same number on every XCD; fewer when an XCD has fewer tiles than that
    constexpr int WG_PER_CU = 1024 / FT;
    const int64_t tiles_xcd = (int64_t)((nlat + 7) / 8) * ngroups;
    const int per_xcd = (int)std::min<int64_t>(tiles_xcd, std::max(1, WG_PER_CU * p.n_cu / 8));
    dim3 grid((unsigned)(8 * per_xcd));
    if (!inverse) {
        float scale = (float)(kTwoPi / (double)N);
        hipLaunchKernelGGL((rfft_fast_kernel<N, R0, R1, R2, S, H, FT, BF16>), grid, dim3(FT), 0, s, p.d_tw0, p.d_tw1, p.d_post, in,
                           reinterpret_cast<float*>(out), rows, nlat, mmax, ld, ngroups, scale);
    } else {
        // sweeps of FT / S orders the kernel reads: all of 0..N/2, or a third of them for truncated plans.  Only the truncated
        // plans afford the registers to request both batches of a tile at once (whole-line reads); the others walk tiles of one
        // batch, whose finer grain also leaves a shorter tail when the tiles do not divide evenly among the workgroups.
        constexpr int TP = FT / S, NSW = (N / 2 + 1 + TP - 1) / TP, NSMALL = (NSW + 2) / 3;
        const float* xm = reinterpret_cast<const float*>(in);
        const bool small = mmax <= NSMALL * TP;
        const int ng = small ? ngroups : (ld / 4 + S - 1) / S;
        const int per = (int)std::min<int64_t>((int64_t)((nlat + 7) / 8) * ng, std::max(1, WG_PER_CU * p.n_cu / 8));
#define IRFFT_GO(H_, NSWA_, LS_)                                                                                                            \
    hipLaunchKernelGGL((irfft_fast_kernel<N, R0, R1, R2, S, H_, FT, BF16, NSWA_, LS_>), dim3((unsigned)(8 * per)), dim3(FT), 0, s, p.d_tw0, \
                       p.d_tw1, p.d_post, xm, out, rows, nlat, mmax, ld, ng, lat_stats)
        if (lat_stats) {
            if (small) IRFFT_GO(H, NSMALL, true); else IRFFT_GO(1, NSW, true);
        } else {
            if (small) IRFFT_GO(H, NSMALL, false); else IRFFT_GO(1, NSW, false);
        }
#undef IRFFT_GO
    }
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

template <int N, int R0, int R1, int R2>
int go_lat(bool inverse, const FftPlan& p, const float* in, float* out, int mmax, int lmax, int ld, const float* mscale, hipStream_t s) {
    constexpr int FT = (LS * N >= 4096) ? 512 : 256;
    const int ngroups = (ld / 2 + LS - 1) / LS;
    const int64_t nblocks = (int64_t)((mmax + 7) / 8) * ngroups * 8;
    if (nblocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    dim3 grid((unsigned)nblocks);
    if (inverse)
        hipLaunchKernelGGL((latfft_fast_kernel<N, R0, R1, R2, FT, 1>), grid, dim3(FT), 0, s, p.d_tw0, p.d_tw1, in, out, mmax, lmax, ld, ngroups, mscale);
    else
        hipLaunchKernelGGL((latfft_fast_kernel<N, R0, R1, R2, FT, 0>), grid, dim3(FT), 0, s, p.d_tw0, p.d_tw1, in, out, mmax, lmax, ld, ngroups, mscale);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

template <int M, int R0, int R1, int R2>
int go_chirp(bool inverse, const FftPlan& p, const float* in, float* out, int mmax, int lmax, int ld, const float* mscale, hipStream_t s) {
    constexpr int S = (M >= 1024) ? 4 : 8;
    constexpr int FT = 256;
    const int ngroups = (ld / 2 + S - 1) / S;
    const int64_t nblocks = (int64_t)((mmax + 7) / 8) * ngroups * 8;
    if (nblocks > 0x7fffffffLL) return SFNO_EUNSUPPORTED;
    dim3 grid((unsigned)nblocks);
    if (inverse)
        hipLaunchKernelGGL((latfft_chirp_kernel<M, R0, R1, R2, S, FT, 1>), grid, dim3(FT), 0, s, p.d_tw0, p.d_tw1, p.d_chirp, p.d_vhat, in, out, p.n, mmax,
                           lmax, ld, ngroups, mscale);
    else
        hipLaunchKernelGGL((latfft_chirp_kernel<M, R0, R1, R2, S, FT, 0>), grid, dim3(FT), 0, s, p.d_tw0, p.d_tw1, p.d_chirp, p.d_vhat, in, out, p.n, mmax,
                           lmax, ld, ngroups, mscale);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

// inter-pass twiddles of the specialised passes of length f.n
int upload_pass_twiddles(const FastEntry& f, FftPlan& p) {
    const int N = f.n, nb = N / f.r0;
    std::vector<float2> tw0((size_t)f.r0 * nb, make_float2(1.f, 0.f)), tw1((size_t)std::max(1, f.r1 * f.r2), make_float2(1.f, 0.f));
    for (int k0 = 1; k0 < f.r0; ++k0)
        for (int j = 0; j < nb; ++j) {
            double a = -kTwoPi * (double)(((int64_t)k0 * j) % N) / (double)N;
            tw0[(size_t)j * f.r0 + k0] = make_float2((float)std::cos(a), (float)std::sin(a));
        }
    for (int k1 = 1; k1 < f.r1; ++k1)
        for (int n2 = 0; n2 < f.r2; ++n2) {
            double a = -kTwoPi * (double)(((int64_t)f.r0 * k1 * n2) % N) / (double)N;
            tw1[(size_t)n2 * f.r1 + k1] = make_float2((float)std::cos(a), (float)std::sin(a));
        }
    // slots of bin m and of bin N - m after the decimation-in-frequency passes (= before the decimation-in-time passes)
    std::vector<unsigned> post((size_t)N / 2 + 1);
    auto slot = [&](int m) {
        const int k0 = m % f.r0, t = m / f.r0, k1 = t % f.r1, k2 = t / f.r1;
        return (unsigned)(k0 * (f.r1 * f.r2) + k1 * f.r2 + k2);
    };
    for (int m = 0; m <= N / 2; ++m) post[m] = slot(m) | (slot((N - m) % N) << 16);
    if (hipMalloc(&p.d_post, sizeof(unsigned) * post.size()) != hipSuccess) return SFNO_ENOMEM;
    if (hipMemcpy(p.d_post, post.data(), sizeof(unsigned) * post.size(), hipMemcpyHostToDevice) != hipSuccess) return SFNO_EHIP;
    if (hipMalloc(&p.d_tw0, sizeof(float2) * tw0.size()) != hipSuccess) return SFNO_ENOMEM;
    if (hipMalloc(&p.d_tw1, sizeof(float2) * tw1.size()) != hipSuccess) return SFNO_ENOMEM;
    if (hipMemcpy(p.d_tw0, tw0.data(), sizeof(float2) * tw0.size(), hipMemcpyHostToDevice) != hipSuccess) return SFNO_EHIP;
    if (hipMemcpy(p.d_tw1, tw1.data(), sizeof(float2) * tw1.size(), hipMemcpyHostToDevice) != hipSuccess) return SFNO_EHIP;
    return SFNO_OK;
}

int largest_prime_factor(int n) {
    int best = 1;
    for (int q = 2; (int64_t)q * q <= n; ++q)
        while (n % q == 0) { best = q; n /= q; }
    return n > 1 ? n : best;
}

}  // namespace

bool fft_fast_supported(int n) { return find_fast(n) != nullptr; }

int fft_chirp_plan_init(FftPlan& p) {
    const int n = p.n;
    if (find_fast(n) || largest_prime_factor(n) <= 7) return SFNO_OK;      // the plain passes serve these lengths well
    const int M = 2 * n - 1 <= 512 ? 512 : 2 * n - 1 <= 1536 ? 1536 : 0;
    if (!M) return SFNO_OK;
    const FastEntry* f = find_fast(M);
    // chirp c[k] = exp(-i pi k^2 / n), the angle reduced exactly in integers
    std::vector<double> cr(n), ci(n);
    std::vector<float2> chirp(M, make_float2(0.f, 0.f));
    for (int k = 0; k < n; ++k) {
        const double a = -(kTwoPi / 2) * (double)(((int64_t)k * k) % (2 * (int64_t)n)) / (double)n;
        cr[k] = std::cos(a);
        ci[k] = std::sin(a);
        chirp[k] = make_float2((float)cr[k], (float)ci[k]);
    }
    // v = conj(c) wrapped around M (v[M - k] = v[k]); its transform, real-symmetric input pairs folded:
    // V[q] = v[0] + sum_{k=1}^{n-1} v[k] 2 cos(2 pi q k / M)
    std::vector<float2> vhat(M);
    std::vector<double> cosM(M);
    for (int j = 0; j < M; ++j) cosM[j] = std::cos(kTwoPi * (double)j / (double)M);
    const int r0 = f->r0, r1 = f->r1, r2 = f->r2;
    for (int q = 0; q < M; ++q) {
        double sr = cr[0], si = -ci[0];
        for (int k = 1; k < n; ++k) {
            const double w = 2.0 * cosM[(int)(((int64_t)q * k) % M)];
            sr += cr[k] * w;
            si -= ci[k] * w;
        }
        const int k0 = q % r0, t = q / r0, k1 = t % r1, k2 = t / r1;        // slot of bin q after the decimation-in-frequency passes
        vhat[k0 * (r1 * r2) + k1 * r2 + k2] = make_float2((float)(sr / M), (float)(si / M));
    }
    int rc = upload_pass_twiddles(*f, p);
    if (rc != SFNO_OK) return rc;
    if (hipMalloc(&p.d_chirp, sizeof(float2) * M) != hipSuccess || hipMalloc(&p.d_vhat, sizeof(float2) * M) != hipSuccess) return SFNO_ENOMEM;
    if (hipMemcpy(p.d_chirp, chirp.data(), sizeof(float2) * M, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(p.d_vhat, vhat.data(), sizeof(float2) * M, hipMemcpyHostToDevice) != hipSuccess)
        return SFNO_EHIP;
    p.chirp_m = M;
    return SFNO_OK;
}

int latfft_fast_launch(bool inverse, const FftPlan& p, const float* in, float* out, int mmax, int lmax, int ld, const float* mscale, hipStream_t s) {
    if (p.chirp_m == 1536) return go_chirp<1536, 16, 12, 8>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
    if (p.chirp_m == 512) return go_chirp<512, 8, 8, 8>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
    switch (p.n) {
        case 1024: return go_lat<1024, 16, 8, 8>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
        case 720: return go_lat<720, 16, 5, 9>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
        case 512: return go_lat<512, 8, 8, 8>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
        case 480: return go_lat<480, 4, 8, 15>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
        case 360: return go_lat<360, 8, 5, 9>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
        case 256: return go_lat<256, 16, 16, 1>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
        case 240: return go_lat<240, 16, 5, 3>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
        case 180: return go_lat<180, 4, 5, 9>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
        case 128: return go_lat<128, 8, 16, 1>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
        case 64: return go_lat<64, 8, 8, 1>(inverse, p, in, out, mmax, lmax, ld, mscale, s);
    }
    return SFNO_EUNSUPPORTED;
}

int fft_fast_plan_init(FftPlan& p) {
    const FastEntry* f = find_fast(p.n);
    return f ? upload_pass_twiddles(*f, p) : SFNO_OK;
}

int fft_fast_launch(bool inverse, const FftPlan& p, const void* in, void* out, int64_t rows, int nlat, int mmax, int ld, int grid_dtype,
                    hipStream_t s, float2* lat_stats) {
    const bool bf = grid_dtype == SFNO_DTYPE_BF16;
    if (!bf && grid_dtype != SFNO_DTYPE_F32) return SFNO_EUNSUPPORTED;
    if (lat_stats && !inverse) return SFNO_EINVAL;
#define FF_CASE(N_, A_, B_, C_)                                                                                     \
    case N_:                                                                                                        \
        return bf ? go_fast<N_, A_, B_, C_, true>(inverse, p, in, out, rows, nlat, mmax, ld, lat_stats, s)           \
                  : go_fast<N_, A_, B_, C_, false>(inverse, p, in, out, rows, nlat, mmax, ld, lat_stats, s);
    switch (p.n) {
        FF_CASE(1536, 16, 12, 8)
        FF_CASE(1440, 16, 10, 9)
        FF_CASE(1024, 16, 8, 8)
        FF_CASE(720, 16, 5, 9)
        FF_CASE(512, 8, 8, 8)
        FF_CASE(480, 4, 8, 15)
        FF_CASE(360, 8, 5, 9)
        FF_CASE(256, 16, 16, 1)
        FF_CASE(240, 16, 5, 3)
        FF_CASE(180, 4, 5, 9)
        FF_CASE(128, 8, 16, 1)
        FF_CASE(64, 8, 8, 1)
    }
#undef FF_CASE
    return SFNO_EUNSUPPORTED;
}

}  // namespace sfno
