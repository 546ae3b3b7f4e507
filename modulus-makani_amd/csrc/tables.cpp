// Host-side construction of quadrature rules, Legendre tables and their packed MFMA
// operand streams.  Everything here is float64 until the final cast, like the tables the
// reference modules precompute in numpy before `.float()`
// (makani/models/networks/sfnonet.py:536-539).
#include <algorithm>
#include <cmath>
#include <cstring>
#include <numeric>
#include <thread>

#include "sfno_internal.h"

namespace sfno {

static const double kPi = 3.14159265358979323846264338327950288;

// Legendre polynomial P_n(x) and derivative by the three-term recurrence.
static void legendre_pn(int n, long double x, long double& p, long double& dp) {
    long double p0 = 1.0L, p1 = x;
    if (n == 0) { p = 1.0L; dp = 0.0L; return; }
    for (int k = 2; k <= n; ++k) {
        long double pk = ((2 * k - 1) * x * p1 - (k - 1) * p0) / k;
        p0 = p1;
        p1 = pk;
    }
    p = p1;
    dp = n * (x * p1 - p0) / (x * x - 1.0L);
}

static void gauss_legendre(int n, double* x, double* w) {
    for (int i = 0; i < n; ++i) {
        // ascending nodes: start from the Chebyshev-like guess for the i-th root from the left
        long double xi = -cosl((long double)kPi * (i + 0.75L) / (n + 0.5L));
        long double p, dp;
        for (int it = 0; it < 100; ++it) {
            legendre_pn(n, xi, p, dp);
            long double dx = p / dp;
            xi -= dx;
            if (fabsl(dx) < 1e-19L) break;
        }
        legendre_pn(n, xi, p, dp);
        x[i] = (double)xi;
        w[i] = (double)(2.0L / ((1.0L - xi * xi) * dp * dp));
    }
}

static void gauss_lobatto(int n, double* x, double* w) {
    const int N = n - 1;
    for (int i = 0; i < n; ++i) {
        long double xi = -cosl((long double)kPi * i / N);
        if (i == 0) xi = -1.0L;
        else if (i == N) xi = 1.0L;
        else {
            for (int it = 0; it < 100; ++it) {
                // Newton on q(x) = P'_N(x): q' from the Legendre ODE (1-x^2) P'' = 2x P' - N(N+1) P
                long double p, dp;
                legendre_pn(N, xi, p, dp);
                long double ddp = (2.0L * xi * dp - (long double)N * (N + 1) * p) / (1.0L - xi * xi);
                long double dx = dp / ddp;
                xi -= dx;
                if (fabsl(dx) < 1e-19L) break;
            }
        }
        long double p, dp;
        if (i == 0) p = (N % 2) ? -1.0L : 1.0L;
        else if (i == N) p = 1.0L;
        else legendre_pn(N, xi, p, dp);
        x[i] = (double)xi;
        w[i] = (double)(2.0L / ((long double)N * n * p * p));
    }
}

static void clenshaw_curtis(int n, double* x, double* w) {
    const int N = n - 1;
    for (int k = 0; k < n; ++k) {
        double theta = kPi - kPi * k / N;     // x ascending from -1
        x[k] = std::cos(theta);
        if (n == 2) { w[k] = 1.0; continue; }
        long double s = 0.0L;
        for (int j = 1; j <= N / 2; ++j) {
            long double b = (2 * j == N) ? 1.0L : 2.0L;
            s += b / (4.0L * j * j - 1.0L) * cosl(2.0L * j * (long double)theta);
        }
        double c = (k == 0 || k == N) ? 1.0 : 2.0;
        w[k] = (double)(c / N * (1.0L - s));
    }
    x[0] = -1.0;
    x[N] = 1.0;
}

int quadrature(int grid, int nlat, double* theta, double* w) {
    if (nlat < 2 || !theta || !w) return SFNO_EINVAL;
    std::vector<double> x(nlat), ww(nlat);
    switch (grid) {
        case SFNO_GRID_LEGENDRE_GAUSS: gauss_legendre(nlat, x.data(), ww.data()); break;
        case SFNO_GRID_LOBATTO: gauss_lobatto(nlat, x.data(), ww.data()); break;
        case SFNO_GRID_EQUIANGULAR: clenshaw_curtis(nlat, x.data(), ww.data()); break;
        default: return SFNO_EINVAL;
    }
    // x ascends from -1, so arccos descends from pi; flip to north-first (theta ascending)
    for (int k = 0; k < nlat; ++k) {
        double xv = std::min(1.0, std::max(-1.0, x[nlat - 1 - k]));
        theta[k] = std::acos(xv);
        w[k] = ww[nlat - 1 - k];
    }
    return SFNO_OK;
}

LegendreGen::LegendreGen(int mmax_, int lmax_, int nlat_, const double* theta, int norm_, int inverse_, int csphase_)
    : nlat(nlat_), lmax(lmax_), mmax(mmax_), norm(norm_), inverse(inverse_), csphase(csphase_) {
    cost.resize(nlat);
    for (int k = 0; k < nlat; ++k) cost[k] = std::cos(theta[k]);
    double nf = (norm == SFNO_NORM_ORTHO) ? 1.0 : std::sqrt(4.0 * kPi);
    if (inverse) nf = 1.0 / nf;
    diag.assign((size_t)mmax * nlat, 0.0);
    for (int k = 0; k < nlat; ++k) diag[k] = nf / std::sqrt(4.0 * kPi);
    for (int m = 1; m < mmax; ++m)
        for (int k = 0; k < nlat; ++k) {
            double c = cost[k];
            diag[(size_t)m * nlat + k] = std::sqrt((2.0 * m + 1.0) * (1.0 + c) * (1.0 - c) / 2.0 / m) * diag[(size_t)(m - 1) * nlat + k];
        }
}

void LegendreGen::rows_for_m(int m, double* out) const {
    const int nl = lmax - m;
    if (nl <= 0) return;
    const double* d = &diag[(size_t)m * nlat];
    for (int k = 0; k < nlat; ++k) out[k] = d[k];
    if (nl > 1) {
        const double f = std::sqrt(2.0 * (m + 1) + 1.0);
        for (int k = 0; k < nlat; ++k) out[nlat + k] = f * cost[k] * d[k];
    }
    for (int l = m + 2; l < lmax; ++l) {
        const double dl = l, dm = m;
        const double a = std::sqrt((2 * dl - 1) / (dl - dm) * (2 * dl + 1) / (dl + dm));
        const double b = std::sqrt((dl + dm - 1) / (dl - dm) * (2 * dl + 1) / (2 * dl - 3) * (dl - dm - 1) / (dl + dm));
        double* o = out + (size_t)(l - m) * nlat;
        const double* p1 = o - nlat;
        const double* p2 = o - 2 * (size_t)nlat;
        for (int k = 0; k < nlat; ++k) o[k] = cost[k] * a * p1[k] - b * p2[k];
    }
    const double sgn = (csphase && (m & 1)) ? -1.0 : 1.0;
    for (int l = m; l < lmax; ++l) {
        double f = sgn;
        if (norm == SFNO_NORM_SCHMIDT) f *= inverse ? std::sqrt(2.0 * l + 1.0) : 1.0 / std::sqrt(2.0 * l + 1.0);
        if (f != 1.0) {
            double* o = out + (size_t)(l - m) * nlat;
            for (int k = 0; k < nlat; ++k) o[k] *= f;
        }
    }
}

static int hw_threads() {
    unsigned n = std::thread::hardware_concurrency();
    if (n == 0) n = 4;
    return (int)std::min(16u, n);
}

template <class F>
static void parallel_for(int n, F f) {
    int nt = std::min(hw_threads(), std::max(1, n));
    std::vector<std::thread> th;
    for (int t = 0; t < nt; ++t)
        th.emplace_back([=]() {
            for (int i = t; i < n; i += nt) f(i);
        });
    for (auto& x : th) x.join();
}

// One 32 x 16 block (row block rb, K chunk c) of P (rows x K, accessed through get(row, k)) as the fragment stream
// described in sfno_internal.h wants it.
template <class G>
static void pack_block(float* blk, int rb, int c, int rows, int K, G get) {
    for (int h = 0; h < 2; ++h)
        for (int j = 0; j < 64; ++j)
            for (int s = 0; s < 4; ++s) {
                int row = PG_ROWS * rb + (j & 31);
                int k = PG_KC * c + 8 * h + 2 * s + (j >> 5);
                float v = (row < rows && k < K) ? (float)get(row, k) : 0.0f;
                blk[(h * 64 + j) * 4 + s] = v;
            }
}

// Folded tables: the grids are symmetric about the equator and Pbar_l^m(pi - theta) =
// (-1)^(l+m) Pbar_l^m(theta), so degrees of even and odd l+m only need the northern half of the
// latitudes, applied to the sum resp. difference of mirrored rows.  Per order m and parity p
// (l = m + p + 2 i) one packed stream:
//   analysis format : rows = i, K = latitude k < ceil(nlat/2) (the equator row counted once)
//   synthesis format: rows = latitude k < ceil(nlat/2), K = i (both parities padded to the chunk count of p = 0)
// Every value is P * lat_w[k] * order_scale[m] (either factor may be absent): the forward transform packs the
// quadrature weights into the analysis format, the inverse packs plain P into the synthesis format, and the
// adjoints of the two swap the formats.
// aoff[2*m + p] = first block of that stream.
static unsigned short bf16_rne(double v) {
    float f = (float)v;
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return (unsigned short)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// bf16 flavour: block = 64 lanes x 8 bf16; lane j holds P[32 rb + (j & 31)][16 c + 8 (j >> 5) + e], e = 0..7
template <class G>
static void pack_block_bf16(unsigned short* blk, int rb, int c, int rows, int K, G get) {
    for (int j = 0; j < 64; ++j)
        for (int e = 0; e < 8; ++e) {
            int row = PG_ROWS * rb + (j & 31);
            int k = PG_KC * c + 8 * (j >> 5) + e;
            blk[j * 8 + e] = (row < rows && k < K) ? bf16_rne(get(row, k)) : (unsigned short)0;
        }
}

// three-plane flavour: block = 3 planes x 64 lanes x 8 bf16, same (lane, e) -> (row, k) map as the bf16 flavour; the planes
// hold the fp32 value cut into its upper, middle and lower 8 significant bits (truncation, so the sum is exact)
template <class G>
static void pack_block_split(unsigned short* blk, int rb, int c, int rows, int K, G get) {
    for (int j = 0; j < 64; ++j)
        for (int e = 0; e < 8; ++e) {
            int row = PG_ROWS * rb + (j & 31);
            int k = PG_KC * c + 8 * (j >> 5) + e;
            float v = (row < rows && k < K) ? (float)get(row, k) : 0.0f;
            for (int pl = 0; pl < 3; ++pl) {
                uint32_t u;
                std::memcpy(&u, &v, 4);
                u &= 0xffff0000u;
                float t;
                std::memcpy(&t, &u, 4);
                blk[(pl * 64 + j) * 8 + e] = (unsigned short)(u >> 16);
                v -= t;
            }
        }
}

// fp16 with round-to-nearest-even from a double (|v| below 65520); returns the bits and the rounded value
static unsigned short f16_rne(double v, double* rounded) {
    const unsigned short sign = std::signbit(v) ? 0x8000u : 0u;
    const double av = std::fabs(v);
    int e = 0;
    if (av != 0.0) (void)std::frexp(av, &e);
    const int E = std::max(e - 1, -14);                       // binade of the value (subnormals share the lowest one)
    const double q = std::ldexp(1.0, E - 10);                 // spacing of fp16 numbers there
    const double r = std::nearbyint(av / q) * q;              // ties to even (default rounding mode)
    if (rounded) *rounded = sign ? -r : r;
    if (r == 0.0) return sign;
    int e2;
    const double f2 = std::frexp(r, &e2);                     // r = f2 * 2^e2, f2 in [0.5, 1)
    if (e2 - 1 < -14) return (unsigned short)(sign | (unsigned)std::lround(std::ldexp(r, 24)));
    return (unsigned short)(sign | ((unsigned)(e2 - 1 + 15) << 10) | ((unsigned)std::lround(std::ldexp(f2, 11)) - 1024u));
}

// two-part fp16 flavour: block = 2 planes x 64 lanes x 8 fp16, same (lane, e) -> (row, k) map as the bf16 flavour; plane 0
// holds the entry times 2^sh[row] rounded to fp16, plane 1 the rounded remainder (23 significant bits kept)
template <class G>
static void pack_block_f16x2(unsigned short* blk, int rb, int c, int rows, int K, G get, const int* sh) {
    for (int j = 0; j < 64; ++j)
        for (int e = 0; e < 8; ++e) {
            int row = PG_ROWS * rb + (j & 31);
            int k = PG_KC * c + 8 * (j >> 5) + e;
            const double v = (row < rows && k < K) ? std::ldexp((double)get(row, k), sh[j & 31]) : 0.0;
            double r0;
            blk[j * 8 + e] = f16_rne(v, &r0);
            blk[(64 + j) * 8 + e] = f16_rne(v - r0, nullptr);
        }
}

// Stream of one (order, parity): for every row block the chunks from its first non-negligible one on.  Towards the
// poles Pbar_l^m falls off like sin^m(theta) (and faster below the turning latitude sin(theta) = m / l): the leading
// chunks of a row block whose entries are all at most `thr` in magnitude are left out -- `skip[rb]` of them, the kernel
// starts that row block's K loop there.  With thr = 2^-64 of the largest entry of the order the omitted terms are 2^-40
// of one fp32 rounding of the result.
// PG_FORMAT_F16X2: rinv receives, per row block, the 32 factors 2^-sh that undo the row scales.
template <class G>
static void pack_stream(std::vector<float>& out, std::vector<int>& skip, std::vector<float>& rinv, int rows, int K, int format, double thr, G get) {
    const int nrb = (rows + PG_ROWS - 1) / PG_ROWS, nc = (K + PG_KC - 1) / PG_KC;
    const size_t bf = (size_t)pg_block_floats(format);
    for (int rb = 0; rb < nrb; ++rb) {
        int c0 = 0;
        for (; c0 < nc; ++c0) {
            bool negligible = true;
            for (int row = PG_ROWS * rb; row < std::min(rows, PG_ROWS * (rb + 1)) && negligible; ++row)
                for (int k = PG_KC * c0; k < std::min(K, PG_KC * (c0 + 1)); ++k)
                    if (std::fabs(get(row, k)) > thr) {
                        negligible = false;
                        break;
                    }
            if (!negligible) break;
        }
        skip.push_back(c0);
        int sh[PG_ROWS];
        if (format == PG_FORMAT_F16X2) {
            // the largest entry of a row lands in [2^14, 2^15)
            for (int r = 0; r < PG_ROWS; ++r) {
                const int row = PG_ROWS * rb + r;
                double mx = 0.0;
                if (row < rows)
                    for (int k = 0; k < K; ++k) mx = std::max(mx, std::fabs((double)get(row, k)));
                int e = 0;
                if (mx > 0.0) (void)std::frexp(mx, &e);           // mx in [2^(e-1), 2^e)
                sh[r] = mx > 0.0 ? 15 - e : 0;
                rinv.push_back((float)std::ldexp(1.0, -sh[r]));
            }
        }
        const size_t at = out.size();
        out.resize(at + (size_t)(nc - c0) * bf, 0.0f);
        for (int c = c0; c < nc; ++c) {
            float* blk = out.data() + at + (size_t)(c - c0) * bf;
            if (format == PG_FORMAT_F16X2) pack_block_f16x2(reinterpret_cast<unsigned short*>(blk), rb, c, rows, K, get, sh);
            else if (format == PG_FORMAT_BF16) pack_block_bf16(reinterpret_cast<unsigned short*>(blk), rb, c, rows, K, get);
            else if (format == PG_FORMAT_SPLIT) pack_block_split(reinterpret_cast<unsigned short*>(blk), rb, c, rows, K, get);
            else pack_block(blk, rb, c, rows, K, get);
        }
    }
}

void pack_legendre_fold(const LegendreGen& g, const double* lat_w, const double* order_scale, bool analysis, int format,
                        std::vector<float>& packed, std::vector<int64_t>& aoff, std::vector<double>* chunks_per_rb, std::vector<float>* rinv) {
    const int mmax = g.mmax, lmax = g.lmax, nlat = g.nlat;
    const int K2 = (nlat + 1) / 2;
    auto nl_p = [&](int m, int p) { return (lmax - m - p > 0) ? (lmax - m - p + 1) / 2 : 0; };
    // per (order, parity): the packed blocks and the number of skipped leading chunks of every row block
    std::vector<std::vector<float>> part((size_t)2 * mmax);
    std::vector<std::vector<int>> skip((size_t)2 * mmax);
    std::vector<std::vector<float>> rpart((size_t)2 * mmax);          // row factors of the two-part fp16 format, per row-block entry
    parallel_for(mmax, [&](int m) {
        int nl = lmax - m;
        if (nl <= 0) {
            // no degrees: the synthesis still has its row blocks (they produce zeros), each with an empty K loop
            if (!analysis)
                for (int p = 0; p < 2; ++p) {
                    skip[2 * m + p].assign((size_t)(K2 + PG_ROWS - 1) / PG_ROWS, 0);
                    if (format == PG_FORMAT_F16X2) rpart[2 * m + p].assign(skip[2 * m + p].size() * PG_ROWS, 1.0f);
                }
            return;
        }
        std::vector<double> rows((size_t)nl * nlat);
        g.rows_for_m(m, rows.data());
        const double* r = rows.data();
        const double sc = order_scale ? order_scale[m] : 1.0;
        auto lw = [=](int k) { return lat_w ? lat_w[k] * sc : sc; };
        double vmax = 0.0;
        for (int i = 0; i < nl; ++i)
            for (int k = 0; k < K2; ++k) vmax = std::max(vmax, std::fabs(r[(size_t)i * nlat + k] * lw(k)));
        const double thr = std::ldexp(vmax, -64);
        for (int p = 0; p < 2; ++p) {
            const int np = nl_p(m, p);
            // K extent of the synthesis padded to the even-parity chunk count so that both parities run the same loop
            const int kpad = nl_p(m, 0);
            auto wa = [=](int row, int k) { return r[(size_t)(p + 2 * row) * nlat + k] * lw(k); };
            auto ws = [=](int row, int k) { return k < np ? r[(size_t)(p + 2 * k) * nlat + row] * lw(row) : 0.0; };
            if (analysis) pack_stream(part[2 * m + p], skip[2 * m + p], rpart[2 * m + p], np, K2, format, thr, wa);
            else pack_stream(part[2 * m + p], skip[2 * m + p], rpart[2 * m + p], K2, kpad, format, thr, ws);
        }
    });
    // index: aoff[2 m + p] = position (in aoff) of the first row-block entry of that stream; an entry is
    // (first block of the row block in the stream) | (skipped chunks << 48)
    const size_t blk_floats = (size_t)pg_block_floats(format);
    size_t nent = 0, nfl = 0;
    for (size_t b = 0; b < part.size(); ++b) {
        nent += skip[b].size();
        nfl += part[b].size();
    }
    aoff.assign((size_t)2 * mmax + nent, 0);
    packed.resize(nfl);
    if (chunks_per_rb) chunks_per_rb->assign(mmax, 0.0);
    if (rinv) {
        // one group of 32 factors per row-block entry, in the order of the entries
        rinv->clear();
        for (size_t b = 0; b < rpart.size(); ++b) rinv->insert(rinv->end(), rpart[b].begin(), rpart[b].end());
    }
    size_t ent = (size_t)2 * mmax, blk = 0, fl = 0;
    for (int m = 0; m < mmax; ++m) {
        double kept = 0.0;
        size_t nrb_m = 0;
        for (int p = 0; p < 2; ++p) {
            const size_t b = (size_t)2 * m + p;
            aoff[b] = (int64_t)ent;
            const int64_t nc = analysis ? (K2 + PG_KC - 1) / PG_KC : (nl_p(m, 0) + PG_KC - 1) / PG_KC;
            for (int c0 : skip[b]) {
                aoff[ent++] = (int64_t)blk | ((int64_t)c0 << 48);
                blk += (size_t)(nc - c0);
                kept += (double)(nc - c0);
                ++nrb_m;
            }
            if (!part[b].empty()) std::memcpy(packed.data() + fl, part[b].data(), sizeof(float) * part[b].size());
            fl += part[b].size();
            std::vector<float>().swap(part[b]);
        }
        if (chunks_per_rb && nrb_m) (*chunks_per_rb)[m] = kept / (double)nrb_m;
    }
    // the kernel's wavefronts without a row block read (and discard) the head of the stream: keep it at least one block long
    if (packed.size() < blk_floats) packed.resize(blk_floats, 0.0f);
}

void build_worklist(const std::vector<int>& nrb, const std::vector<double>& cost, std::vector<int2>& work, int rb_step) {
    // Workgroups are handed to the 8 XCDs round-robin by linear id, so entry 8*i + x of the
    // list runs on XCD x.  All workgroups of one batch share their Q panel through that XCD's
    // L2, so a batch is never split across queues; batches are assigned longest-first to the
    // least loaded queue and each queue runs its batches in decreasing cost order.
    const int nb = (int)nrb.size();
    std::vector<int> order(nb);
    std::iota(order.begin(), order.end(), 0);
    auto total = [&](int b) { return cost[b] * ((nrb[b] + rb_step - 1) / rb_step); };
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return total(a) > total(b); });
    std::vector<std::vector<int2>> q(8);
    double load[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int b : order) {
        if (nrb[b] <= 0) continue;
        int best = 0;
        for (int x = 1; x < 8; ++x)
            if (load[x] < load[best]) best = x;
        for (int rb = 0; rb < nrb[b]; rb += rb_step) q[best].push_back(make_int2(b, rb));
        load[best] += total(b);
    }
    size_t len = 0;
    for (auto& v : q) len = std::max(len, v.size());
    work.assign(len * 8, make_int2(-1, 0));
    for (int x = 0; x < 8; ++x)
        for (size_t i = 0; i < q[x].size(); ++i) work[i * 8 + x] = q[x][i];
}

}  // namespace sfno

extern "C" int sfno_quadrature(int grid, int nlat, double* theta, double* w) {
    return sfno::quadrature(grid, nlat, theta, w);
}

extern "C" int sfno_legendre_table(int mmax, int lmax, int nlat, const double* theta, int norm, int inverse,
                                   int csphase, double* out) {
    if (mmax < 1 || lmax < 1 || nlat < 1 || !theta || !out) return SFNO_EINVAL;
    if (norm < 0 || norm > 2) return SFNO_EINVAL;
    sfno::LegendreGen g(mmax, lmax, nlat, theta, norm, inverse, csphase);
    std::memset(out, 0, sizeof(double) * (size_t)mmax * lmax * nlat);
    std::vector<double> rows((size_t)lmax * nlat);
    for (int m = 0; m < mmax && m < lmax; ++m) {
        g.rows_for_m(m, rows.data());
        std::memcpy(out + ((size_t)m * lmax + m) * nlat, rows.data(), sizeof(double) * (size_t)(lmax - m) * nlat);
    }
    return SFNO_OK;
}

extern "C" int64_t sfno_legendre_stream_skips(int mmax, int lmax, int nlat, const double* theta, const double* lat_w, int norm, int inverse,
                                              int csphase, int analysis, int32_t* skips, int64_t capacity) {
    if (mmax < 1 || lmax < 1 || nlat < 1 || !theta || capacity < 0 || (capacity > 0 && !skips)) return SFNO_EINVAL;
    if (norm < 0 || norm > 2) return SFNO_EINVAL;
    sfno::LegendreGen g(mmax, lmax, nlat, theta, norm, inverse, csphase);
    std::vector<float> packed;
    std::vector<int64_t> aoff;
    sfno::pack_legendre_fold(g, lat_w, nullptr, analysis != 0, sfno::PG_FORMAT_BF16, packed, aoff);
    const int64_t n = (int64_t)aoff.size() - 2 * (int64_t)mmax;
    for (int64_t i = 0; i < n && i < capacity; ++i) skips[i] = (int32_t)(aoff[(size_t)(2 * mmax + i)] >> 48);
    return n;
}
