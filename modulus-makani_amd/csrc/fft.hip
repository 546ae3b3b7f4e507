// Longitude real FFT / inverse real FFT for the SHT pair, gfx950.
//
// Replaces the torch.fft.rfft(norm="forward") * 2 pi (then [..., :mmax]) of
// RealSHT.forward and the torch.fft.irfft(n=nlon, norm="forward") of
// InverseRealSHT.forward (torch-harmonics; called from
// makani/models/common/spectral_convolution.py:131,133,141).
//
// Two real rows (two channels at the same latitude) are packed into one complex
// sequence z = a + i b, transformed with a mixed-radix Stockham FFT that lives entirely
// in LDS, and separated with the Hermitian identities
//     A[m] = (Z[m] + conj Z[N-m]) / 2,   B[m] = (Z[m] - conj Z[N-m]) / (2i).
// The spectral side uses the order-major layout xm[m][lat][ld] (channel axis contiguous,
// (re,im) of channel r at 2r,2r+1) so that the Legendre stage reads dense panels per m:
// one workgroup handles one latitude and PAIRS channel pairs, and writes/reads
// 16*PAIRS contiguous bytes per order.
#include "sfno_internal.h"

#include <cmath>
#include <vector>

namespace sfno {

__device__ __forceinline__ float2 cmul(float2 a, float2 b) { return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x); }
__device__ __forceinline__ float2 cadd(float2 a, float2 b) { return make_float2(a.x + b.x, a.y + b.y); }
__device__ __forceinline__ float2 csub(float2 a, float2 b) { return make_float2(a.x - b.x, a.y - b.y); }
// multiply by -i (forward) or +i (inverse)
template <int INV>
__device__ __forceinline__ float2 mul_mi(float2 a) { return INV ? make_float2(-a.y, a.x) : make_float2(a.y, -a.x); }
template <int INV>
__device__ __forceinline__ float2 twid(const float2* __restrict__ tw, int idx) {
    float2 w = tw[idx];
    if (INV) w.y = -w.y;
    return w;
}

// One Stockham pass of radix R over `nseq` sequences of length n held in LDS.
// For butterfly j (0 <= j < n/R), with ns = product of the radices already applied and
// k = j mod ns:  v[r] = in[j + r n/R] * w^(r k n/(ns R)),  out[(j-k) R + k + q ns] = DFT_R(v)[q].
// COL = false: sequence sq occupies [sq n, sq n + n) (longitude transforms: a sequence is a grid row);
// COL = true: element i of sequence sq sits at i nseq + sq (latitude transforms: the sequences are the
// channels of one order, contiguous in HBM and in LDS).  Either way neighbouring lanes touch neighbouring words.
template <int R, int INV, bool COL>
__device__ __forceinline__ void pass_fixed(const float2* __restrict__ in, float2* __restrict__ out, const float2* __restrict__ tw,
                                           int n, int ns, int nseq, int tid, int nthreads) {
    const int nb = n / R;
    const int tstep = n / (ns * R);
    const int es = COL ? nseq : 1;                    // distance between consecutive elements of a sequence
    for (int e = tid; e < nseq * nb; e += nthreads) {
        const int sq = COL ? e % nseq : e / nb, j = COL ? e / nseq : e - sq * nb;
        const int k = j % ns;
        const float2* src = in + (COL ? sq : sq * n) + j * es;
        float2 v[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            v[r] = src[r * nb * es];
            if (r > 0) v[r] = cmul(v[r], twid<INV>(tw, (r * k * tstep) % n));
        }
        float2* dst = out + (COL ? sq : sq * n) + ((j - k) * R + k) * es;
        const int os = ns * es;                        // distance between the outputs of the butterfly
        if (R == 2) {
            dst[0] = cadd(v[0], v[1]);
            dst[os] = csub(v[0], v[1]);
        } else if (R == 3) {
            const float s3 = 0.86602540378443864676f;
            float2 t1 = cadd(v[1], v[2]);
            float2 t2 = make_float2(v[0].x - 0.5f * t1.x, v[0].y - 0.5f * t1.y);
            float2 d = csub(v[1], v[2]);
            float2 t3 = mul_mi<INV>(make_float2(s3 * d.x, s3 * d.y));
            dst[0] = cadd(v[0], t1);
            dst[os] = cadd(t2, t3);
            dst[2 * os] = csub(t2, t3);
        } else if (R == 4) {
            float2 a0 = cadd(v[0], v[2]), a1 = csub(v[0], v[2]);
            float2 a2 = cadd(v[1], v[3]), a3 = mul_mi<INV>(csub(v[1], v[3]));
            dst[0] = cadd(a0, a2);
            dst[os] = cadd(a1, a3);
            dst[2 * os] = csub(a0, a2);
            dst[3 * os] = csub(a1, a3);
        } else if (R == 5) {
            const float c1 = 0.30901699437494742410f, c2 = -0.80901699437494742410f;
            const float s1 = 0.95105651629515357212f, s2 = 0.58778525229247312917f;
            float2 p1 = cadd(v[1], v[4]), m1 = csub(v[1], v[4]);
            float2 p2 = cadd(v[2], v[3]), m2 = csub(v[2], v[3]);
            float2 e1 = make_float2(v[0].x + c1 * p1.x + c2 * p2.x, v[0].y + c1 * p1.y + c2 * p2.y);
            float2 e2 = make_float2(v[0].x + c2 * p1.x + c1 * p2.x, v[0].y + c2 * p1.y + c1 * p2.y);
            float2 f1 = mul_mi<INV>(make_float2(s1 * m1.x + s2 * m2.x, s1 * m1.y + s2 * m2.y));
            float2 f2 = mul_mi<INV>(make_float2(s2 * m1.x - s1 * m2.x, s2 * m1.y - s1 * m2.y));
            dst[0] = cadd(v[0], cadd(p1, p2));
            dst[os] = cadd(e1, f1);
            dst[2 * os] = cadd(e2, f2);
            dst[3 * os] = csub(e2, f2);
            dst[4 * os] = csub(e1, f1);
        }
    }
}

// Any other (prime) radix: direct O(R^2) butterfly straight from LDS, no private arrays.
template <int INV, bool COL>
__device__ __forceinline__ void pass_generic(const float2* __restrict__ in, float2* __restrict__ out, const float2* __restrict__ tw,
                                             int n, int ns, int R, int nseq, int tid, int nthreads) {
    const int nb = n / R;
    const int tstep = n / (ns * R);
    const int rstep = n / R;
    const int es = COL ? nseq : 1;
    for (int e = tid; e < nseq * nb * R; e += nthreads) {
        int q, sq, j;
        if (COL) {
            sq = e % nseq;
            const int e2 = e / nseq;
            q = e2 % R;
            j = e2 / R;
        } else {
            q = e % R;
            const int e2 = e / R;
            sq = e2 / nb;
            j = e2 - sq * nb;
        }
        const int k = j % ns;
        const float2* src = in + (COL ? sq : sq * n) + j * es;
        float2 acc = make_float2(0.f, 0.f);
        for (int r = 0; r < R; ++r) {
            // input twiddle w^(r k tstep) and butterfly factor w^(r q n/R)
            int idx = (int)(((long long)r * k * tstep + (long long)((r * q) % R) * rstep) % n);
            acc = cadd(acc, cmul(src[r * nb * es], twid<INV>(tw, idx)));
        }
        out[(COL ? sq : sq * n) + ((j - k) * R + k + q * ns) * es] = acc;
    }
}

struct FftDev {
    const float2* tw;
    int n, npass;
    int radix[24];
};

template <int INV, bool COL = false>
__device__ __forceinline__ float2* run_passes(const FftDev& f, float2* buf0, float2* buf1, int nseq, int tid, int nthreads) {
    int ns = 1;
    float2* in = buf0;
    float2* out = buf1;
    for (int p = 0; p < f.npass; ++p) {
        const int R = f.radix[p];
        switch (R) {
            case 2: pass_fixed<2, INV, COL>(in, out, f.tw, f.n, ns, nseq, tid, nthreads); break;
            case 3: pass_fixed<3, INV, COL>(in, out, f.tw, f.n, ns, nseq, tid, nthreads); break;
            case 4: pass_fixed<4, INV, COL>(in, out, f.tw, f.n, ns, nseq, tid, nthreads); break;
            case 5: pass_fixed<5, INV, COL>(in, out, f.tw, f.n, ns, nseq, tid, nthreads); break;
            default: pass_generic<INV, COL>(in, out, f.tw, f.n, ns, R, nseq, tid, nthreads); break;
        }
        ns *= R;
        __syncthreads();
        float2* t = in;
        in = out;
        out = t;
    }
    return in;   // buffer holding the result
}

constexpr int FFT_THREADS = 256;

// grid = (nlat, ceil(npairs / PAIRS)); dynamic LDS = 2 * PAIRS * n * sizeof(float2)
template <int PAIRS>
__global__ __launch_bounds__(FFT_THREADS) void rfft_kernel(FftDev f, const float* __restrict__ x, float* __restrict__ xm, int64_t rows,
                                                           int nlat, int mmax, int ld, float scale) {
    extern __shared__ __align__(16) float2 lds[];
    const int n = f.n, tid = threadIdx.x;
    const int lat = blockIdx.x;
    const int pair0 = blockIdx.y * PAIRS;
    float2* buf0 = lds;
    float2* buf1 = lds + PAIRS * n;
    for (int e = tid; e < PAIRS * n; e += FFT_THREADS) {
        const int p = e / n, i = e - p * n;
        const int64_t r0 = 2 * (int64_t)(pair0 + p);
        float2 z = make_float2(0.f, 0.f);
        if (r0 < rows) z.x = x[(r0 * nlat + lat) * n + i];
        if (r0 + 1 < rows) z.y = x[((r0 + 1) * nlat + lat) * n + i];
        buf0[e] = z;
    }
    __syncthreads();
    const float2* z = run_passes<0>(f, buf0, buf1, PAIRS, tid, FFT_THREADS);
    const int npairs_ld = ld / 4;
    for (int e = tid; e < PAIRS * mmax; e += FFT_THREADS) {
        const int m = e / PAIRS, p = e - m * PAIRS;
        if (pair0 + p >= npairs_ld) continue;
        const float2 zp = z[p * n + m];
        const float2 zq = z[p * n + (m == 0 ? 0 : n - m)];
        // A = (Z[m] + conj Z[n-m]) / 2 ; B = -i (Z[m] - conj Z[n-m]) / 2
        const float h = 0.5f * scale;
        float4 o;
        o.x = h * (zp.x + zq.x);
        o.y = h * (zp.y - zq.y);
        o.z = h * (zp.y + zq.y);
        o.w = -h * (zp.x - zq.x);
        *reinterpret_cast<float4*>(xm + ((int64_t)m * nlat + lat) * ld + 4 * (int64_t)(pair0 + p)) = o;
    }
}

template <int PAIRS>
__global__ __launch_bounds__(FFT_THREADS) void irfft_kernel(FftDev f, const float* __restrict__ xm, float* __restrict__ x, int64_t rows,
                                                            int nlat, int mmax, int ld) {
    extern __shared__ __align__(16) float2 lds[];
    const int n = f.n, tid = threadIdx.x;
    const int lat = blockIdx.x;
    const int pair0 = blockIdx.y * PAIRS;
    float2* buf0 = lds;
    float2* buf1 = lds + PAIRS * n;
    const int npairs_ld = ld / 4;
    const int half = n / 2;                 // bins 0..half are independent
    const bool even = (n % 2) == 0;
    // Hermitian extension of A + i B:  z[m] = A[m] + i B[m],  z[n-m] = conj A[m] + i conj B[m]
    for (int e = tid; e < PAIRS * (half + 1); e += FFT_THREADS) {
        const int m = e / PAIRS, p = e - m * PAIRS;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (m < mmax && pair0 + p < npairs_ld) v = *reinterpret_cast<const float4*>(xm + ((int64_t)m * nlat + lat) * ld + 4 * (int64_t)(pair0 + p));
        // a channel slot past the last row is padding: whatever it holds must not leak into its partner
        if (2 * (int64_t)(pair0 + p) + 1 >= rows) v.z = v.w = 0.f;
        if (m == 0 || (even && m == half)) {
            // C2R semantics: the imaginary parts of the mean and Nyquist bins are dropped
            buf0[p * n + m] = make_float2(v.x, v.z);
        } else {
            buf0[p * n + m] = make_float2(v.x - v.w, v.y + v.z);
            buf0[p * n + n - m] = make_float2(v.x + v.w, v.z - v.y);
        }
    }
    __syncthreads();
    const float2* z = run_passes<1>(f, buf0, buf1, PAIRS, tid, FFT_THREADS);
    for (int e = tid; e < PAIRS * n; e += FFT_THREADS) {
        const int p = e / n, i = e - p * n;
        const int64_t r0 = 2 * (int64_t)(pair0 + p);
        const float2 v = z[e];
        if (r0 < rows) x[(r0 * nlat + lat) * n + i] = v.x;
        if (r0 + 1 < rows) x[((r0 + 1) * nlat + lat) * n + i] = v.y;
    }
}

int fft_plan_init(FftPlan& p, int n) {
    if (n < 1) return SFNO_EINVAL;
    p.n = n;
    p.npass = 0;
    {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0)
            p.n_cu = cus;
        else
            (void)hipGetLastError();
    }
    int rem = n;
    while (rem % 4 == 0) { p.radix[p.npass++] = 4; rem /= 4; }
    while (rem % 2 == 0) { p.radix[p.npass++] = 2; rem /= 2; }
    while (rem % 3 == 0) { p.radix[p.npass++] = 3; rem /= 3; }
    while (rem % 5 == 0) { p.radix[p.npass++] = 5; rem /= 5; }
    for (int q = 7; rem > 1; q += 2)
        while (rem % q == 0) {
            if (p.npass >= 24) return SFNO_EUNSUPPORTED;
            p.radix[p.npass++] = q;
            rem /= q;
        }
    std::vector<float2> tw(n);
    for (int j = 0; j < n; ++j) {
        double a = -2.0 * 3.14159265358979323846264338327950288 * (double)j / (double)n;
        tw[j] = make_float2((float)std::cos(a), (float)std::sin(a));
    }
    if (hipMalloc(&p.d_tw, sizeof(float2) * n) != hipSuccess) return SFNO_ENOMEM;
    if (hipMemcpy(p.d_tw, tw.data(), sizeof(float2) * n, hipMemcpyHostToDevice) != hipSuccess) return SFNO_EHIP;
    return fft_fast_plan_init(p);
}

void fft_plan_free(FftPlan& p) {
    if (p.d_tw) (void)hipFree(p.d_tw);
    if (p.d_tw0) (void)hipFree(p.d_tw0);
    if (p.d_tw1) (void)hipFree(p.d_tw1);
    if (p.d_chirp) (void)hipFree(p.d_chirp);
    if (p.d_vhat) (void)hipFree(p.d_vhat);
    if (p.d_post) (void)hipFree(p.d_post);
    p.d_tw = p.d_tw0 = p.d_tw1 = p.d_chirp = p.d_vhat = nullptr;
    p.d_post = nullptr;
    p.chirp_m = 0;
}

static FftDev make_dev(const FftPlan& p) {
    FftDev d;
    d.tw = p.d_tw;
    d.n = p.n;
    d.npass = p.npass;
    for (int i = 0; i < 24; ++i) d.radix[i] = i < p.npass ? p.radix[i] : 1;
    return d;
}

// LDS budget per workgroup (bytes) the FFT kernels may ask for
static const size_t kFftMaxLds = 160 * 1024;

// Latitude FFT of the planar transform pair (RealFFT2 / InverseRealFFT2, makani/models/common/layers.py:219-287):
// the second dimension of torch.fft.rfft2 / irfft2 with the reference's mode truncation.  Both sides use the
// order-major layout: in[m][k][ld] -> out[m][j][ld], channels contiguous.  A workgroup transforms 2^cshift complex
// channels of one order; the sequences stay channel-contiguous in LDS.
//   INV = 0: k = latitude (n rows), j = kept frequency (lmax rows): j < ceil(lmax/2) is frequency j, the rest are
//            the floor(lmax/2) highest (negative) frequencies n - lmax + j.
//   INV = 1: k = kept frequency, j = latitude; dropped frequencies are zero.
// Every output is multiplied by mscale[m] (normalisation, and the order weights of the adjoint transforms).
// grid = (ceil(ld / 2 / 2^cshift), mmax): the channel groups of one order are neighbours in dispatch order;
// dynamic LDS = 2 * n * 2^cshift * sizeof(float2)
constexpr int LATFFT_THREADS = 512;

template <int INV>
__global__ __launch_bounds__(LATFFT_THREADS) void latfft_kernel(FftDev f, const float* __restrict__ in, float* __restrict__ out, int lmax, int ld,
                                                                int cshift, const float* __restrict__ mscale) {
    extern __shared__ __align__(16) float2 lds[];
    const int n = f.n, tid = threadIdx.x, cw = 1 << cshift;
    const int m = blockIdx.y, c0 = blockIdx.x * cw;
    const int lhigh = (lmax + 1) / 2, gap = n - lmax;
    float2* buf0 = lds;
    float2* buf1 = lds + n * cw;
    const int nin = INV ? lmax : n, nout = INV ? n : lmax;
    for (int e = tid; e < n * cw; e += LATFFT_THREADS) {
        const int i = e >> cshift, c = e & (cw - 1);
        // row of the input that lands on element i of the sequence (-1: a dropped frequency)
        const int k = !INV ? i : i < lhigh ? i : i >= lhigh + gap ? i - gap : -1;
        float2 v = make_float2(0.f, 0.f);
        if (k >= 0 && 2 * (c0 + c) < ld) v = *reinterpret_cast<const float2*>(in + ((int64_t)m * nin + k) * ld + 2 * (c0 + c));
        buf0[e] = v;
    }
    __syncthreads();
    const float2* z = run_passes<INV, true>(f, buf0, buf1, cw, tid, LATFFT_THREADS);
    const float sc = mscale[m];
    for (int e = tid; e < nout * cw; e += LATFFT_THREADS) {
        const int j = e >> cshift, c = e & (cw - 1);
        const int i = INV ? j : j < lhigh ? j : j + gap;
        if (2 * (c0 + c) >= ld) continue;
        const float2 v = z[i * cw + c];
        *reinterpret_cast<float2*>(out + ((int64_t)m * nout + j) * ld + 2 * (c0 + c)) = make_float2(sc * v.x, sc * v.y);
    }
}

int latfft_launch(const FftPlan& p, bool inverse, const float* in, float* out, int mmax, int lmax, int ld, const float* mscale, hipStream_t s) {
    if (lmax < 1 || lmax > p.n || mmax < 1 || ld % 2 != 0 || !mscale) return SFNO_EINVAL;
    if (fft_fast_supported(p.n) || p.chirp_m) {
        const int rc = latfft_fast_launch(inverse, p, in, out, mmax, lmax, ld, mscale, s);
        if (rc != SFNO_EUNSUPPORTED) return rc;
    }
    // as many channels per workgroup as the two LDS buffers allow, at most 8 (one 64-byte line per row)
    int cshift = 3;
    while (cshift > 0 && (2 * sizeof(float2) * p.n << cshift) > kFftMaxLds) --cshift;
    const size_t lds = 2 * sizeof(float2) * p.n << cshift;
    if (lds > kFftMaxLds) return SFNO_EUNSUPPORTED;
    // the limit is a property of the function on the current device: set it on every launch that needs it (a host-side call)
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute(inverse ? (const void*)latfft_kernel<1> : (const void*)latfft_kernel<0>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)kFftMaxLds) != hipSuccess)
        return SFNO_EHIP;
    const int cw = 1 << cshift;
    if (mmax > 65535) return SFNO_EUNSUPPORTED;
    dim3 grid((unsigned)((ld / 2 + cw - 1) / cw), mmax);
    if (inverse)
        hipLaunchKernelGGL(latfft_kernel<1>, grid, dim3(LATFFT_THREADS), lds, s, make_dev(p), in, out, lmax, ld, cshift, mscale);
    else
        hipLaunchKernelGGL(latfft_kernel<0>, grid, dim3(LATFFT_THREADS), lds, s, make_dev(p), in, out, lmax, ld, cshift, mscale);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

template <int PAIRS>
static int rfft_go(const FftPlan& p, const float* x, float* xm, int64_t rows, int nlat, int mmax, int ld, hipStream_t s) {
    size_t lds = 2 * (size_t)PAIRS * p.n * sizeof(float2);
    // the limit is a property of the function on the current device: set it on every launch that needs it (a host-side call)
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute((const void*)rfft_kernel<PAIRS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kFftMaxLds) != hipSuccess)
        return SFNO_EHIP;
    dim3 grid(nlat, (unsigned)((ld / 4 + PAIRS - 1) / PAIRS));
    float scale = (float)(2.0 * 3.14159265358979323846264338327950288 / (double)p.n);
    hipLaunchKernelGGL((rfft_kernel<PAIRS>), grid, dim3(FFT_THREADS), lds, s, make_dev(p), x, xm, rows, nlat, mmax, ld, scale);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

template <int PAIRS>
static int irfft_go(const FftPlan& p, const float* xm, float* x, int64_t rows, int nlat, int mmax, int ld, hipStream_t s) {
    size_t lds = 2 * (size_t)PAIRS * p.n * sizeof(float2);
    // the limit is a property of the function on the current device: set it on every launch that needs it (a host-side call)
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute((const void*)irfft_kernel<PAIRS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kFftMaxLds) != hipSuccess)
        return SFNO_EHIP;
    dim3 grid(nlat, (unsigned)((ld / 4 + PAIRS - 1) / PAIRS));
    hipLaunchKernelGGL((irfft_kernel<PAIRS>), grid, dim3(FFT_THREADS), lds, s, make_dev(p), xm, x, rows, nlat, mmax, ld);
    return hipGetLastError() == hipSuccess ? SFNO_OK : SFNO_EHIP;
}

static int pick_pairs(int n) {
    // as many channel pairs per workgroup as fit ~48 KiB of LDS (3 workgroups per CU)
    size_t per_pair = 2 * (size_t)n * sizeof(float2);
    if (4 * per_pair <= 48 * 1024) return 4;
    if (2 * per_pair <= 48 * 1024) return 2;
    if (per_pair <= kFftMaxLds) return 1;
    return 0;
}

int rfft_launch(const FftPlan& p, const void* xv, int x_dtype, float* xm, int64_t rows, int nlat, int mmax, int ld, hipStream_t s) {
    if (mmax > p.n / 2 + 1 || ld % 4 != 0 || ld < 2 * rows) return SFNO_EINVAL;
    if (fft_fast_supported(p.n)) return fft_fast_launch(false, p, xv, xm, rows, nlat, mmax, ld, x_dtype, s);
    if (x_dtype != SFNO_DTYPE_F32) return SFNO_EUNSUPPORTED;     // the generic kernels read float only
    const float* x = reinterpret_cast<const float*>(xv);
    switch (pick_pairs(p.n)) {
        case 4: return rfft_go<4>(p, x, xm, rows, nlat, mmax, ld, s);
        case 2: return rfft_go<2>(p, x, xm, rows, nlat, mmax, ld, s);
        case 1: return rfft_go<1>(p, x, xm, rows, nlat, mmax, ld, s);
    }
    return SFNO_EUNSUPPORTED;
}

int irfft_launch(const FftPlan& p, const float* xm, void* xv, int x_dtype, int64_t rows, int nlat, int mmax, int ld, hipStream_t s, float2* lat_stats) {
    // orders above nlon/2 are dropped, as torch.fft.irfft(n=nlon) drops surplus input bins
    if (ld % 4 != 0 || ld < 2 * rows) return SFNO_EINVAL;
    if (fft_fast_supported(p.n)) return fft_fast_launch(true, p, xm, xv, rows, nlat, mmax, ld, x_dtype, s, lat_stats);
    if (lat_stats) return SFNO_EUNSUPPORTED;                      // only the specialised kernels produce the moments
    if (x_dtype != SFNO_DTYPE_F32) return SFNO_EUNSUPPORTED;
    float* x = reinterpret_cast<float*>(xv);
    switch (pick_pairs(p.n)) {
        case 4: return irfft_go<4>(p, xm, x, rows, nlat, mmax, ld, s);
        case 2: return irfft_go<2>(p, xm, x, rows, nlat, mmax, ld, s);
        case 1: return irfft_go<1>(p, xm, x, rows, nlat, mmax, ld, s);
    }
    return SFNO_EUNSUPPORTED;
}

}  // namespace sfno
