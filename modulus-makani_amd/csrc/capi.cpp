// C ABI of libsfno_spectral: plan management and the enqueue-only compute entry points.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <new>

#include "sfno_internal.h"

using namespace sfno;

namespace {

const int kVersion = 1;

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

template <class T>
int upload(T** dst, const std::vector<T>& src) {
    *dst = nullptr;
    size_t bytes = sizeof(T) * std::max<size_t>(src.size(), 1);
    if (hipMalloc((void**)dst, bytes) != hipSuccess) return SFNO_ENOMEM;
    if (!src.empty() && hipMemcpy(*dst, src.data(), sizeof(T) * src.size(), hipMemcpyHostToDevice) != hipSuccess) return SFNO_EHIP;
    return SFNO_OK;
}

void free_table(PgemmTable& t) {
    if (t.d_A) (void)hipFree(t.d_A);
    if (t.d_rinv) (void)hipFree(t.d_rinv);
    if (t.d_aoff) (void)hipFree(t.d_aoff);
    if (t.d_work) (void)hipFree(t.d_work);
    if (t.d_wrec) (void)hipFree(t.d_wrec);
    t = PgemmTable();
}

// inverse: which of the two Legendre normalisations (they differ for norm = schmidt); analysis: stream format
int build_legendre_table(const sfno_sht_plan& p, const double* theta, const double* lat_w, const double* order_scale, bool inverse,
                         bool analysis, PgemmTable& t) {
    LegendreGen gen(p.mmax, p.lmax, p.nlat, theta, p.norm, inverse ? 1 : 0, p.csphase);
    std::vector<float> packed;
    std::vector<int64_t> aoff;
    std::vector<double> kept;          // mean number of K chunks a row block of order m runs through
    std::vector<float> rinv;
    pack_legendre_fold(gen, lat_w, order_scale, analysis, p.format, packed, aoff, &kept, &rinv);
    // a workgroup covers two 32-row blocks of each parity
    const int K2 = (p.nlat + 1) / 2;
    std::vector<int> nrb(p.mmax);
    std::vector<double> cost(p.mmax);
    for (int m = 0; m < p.mmax; ++m) {
        int nl0 = (p.lmax - m > 0) ? (p.lmax - m + 1) / 2 : 0;
        if (analysis) {
            nrb[m] = (nl0 + PG_ROWS - 1) / PG_ROWS;
        } else {
            nrb[m] = (K2 + PG_ROWS - 1) / PG_ROWS;       // orders without any degree still zero-fill their rows
        }
        cost[m] = 1.0 + kept[m];
    }
    std::vector<int2> work;
    build_worklist(nrb, cost, work, 2);
    t.n_work = (int)work.size();
    t.n_blocks = (int64_t)(packed.size() / pg_block_floats(p.format));
    int rc;
    if ((rc = upload(&t.d_A, packed)) != SFNO_OK) return rc;
    if (p.format == PG_FORMAT_F16X2 && (rc = upload(&t.d_rinv, rinv)) != SFNO_OK) return rc;
    if ((rc = upload(&t.d_aoff, aoff)) != SFNO_OK) return rc;
    if ((rc = upload(&t.d_work, work)) != SFNO_OK) return rc;
    if (p.format == PG_FORMAT_F16X2) {
        std::vector<int64_t> wrec(work.size() * PG_WREC, 0);
        for (size_t w = 0; w < work.size(); ++w) {
            int64_t* r = &wrec[w * PG_WREC];
            const int m = work[w].x, rb0 = work[w].y;
            r[PG_WREC_M] = m;
            r[PG_WREC_RB] = rb0;
            if (m < 0) continue;
            const int nl0 = (p.lmax - m > 0) ? (p.lmax - m + 1) / 2 : 0;
            const int nl1 = (p.lmax - m - 1 > 0) ? (p.lmax - m) / 2 : 0;
            const int nc = analysis ? (K2 + PG_KC - 1) / PG_KC : (nl0 + PG_KC - 1) / PG_KC;
            for (int par = 0; par < 2; ++par) {
                const int nr = analysis ? (par ? nl1 : nl0) : K2;
                r[PG_WREC_POS + par] = aoff[2 * m + par];
                for (int j = 0; j < 2; ++j) {
                    const int rb = rb0 + j;
                    // (an order without degrees has no entries: nc = 0; a row block past the stream's rows has none either)
                    r[PG_WREC_ENTRY + 2 * par + j] = (nc > 0 && rb * PG_ROWS < nr) ? aoff[(size_t)(aoff[2 * m + par] + rb)] : (int64_t)nc << 48;
                }
            }
        }
        if ((rc = upload(&t.d_wrec, wrec)) != SFNO_OK) return rc;
    }
    return SFNO_OK;
}

struct Ws {
    float* xm;
    float* spec;
    size_t bytes;
};

Ws carve(const sfno_sht_plan* p, int64_t rows, void* base) {
    const int64_t ld = sfno_spectral_ld(rows);
    Ws w;
    size_t xm_bytes = align_up(sizeof(float) * (size_t)p->mmax * p->nlat * ld, 256);
    size_t spec_bytes = align_up(sizeof(float) * (size_t)p->mmax * p->lmax * ld, 256);
    w.xm = reinterpret_cast<float*>(base);
    w.spec = reinterpret_cast<float*>(reinterpret_cast<char*>(base) + xm_bytes);
    w.bytes = xm_bytes + spec_bytes;
    return w;
}

PgemmArgs legendre_args(const sfno_sht_plan* p, const PgemmTable& t, const float* q, float* out, int64_t ld) {
    PgemmArgs a;
    std::memset(&a, 0, sizeof(a));
    a.A = t.d_A;
    a.a_off = t.d_aoff;
    a.work = t.d_work;
    a.wrec = t.d_wrec;
    a.Q = q;
    a.Out = out;
    a.rinv = t.d_rinv;
    a.lmax = p->lmax;
    a.nlat = p->nlat;
    a.mmax = p->mmax;
    a.ld = (int)ld;
    return a;
}

bool rows_ok(int64_t rows) { return rows > 0 && sfno_spectral_ld(rows) < (int64_t)1 << 30; }

// Planar plans (SFNO_GRID_PLANAR).  The longitude kernels are those of the spherical transforms,
//   F: x -> s * sum_n x_n e^{-i m phi_n} (s = 2 pi / nlon)   and   C: the unnormalised complex-to-real transform,
// so torch.fft.rfft2(norm="ortho") is  a * (latitude DFT) o F  with a = 1 / (s sqrt(nlat nlon)), and
// torch.fft.irfft2(norm="ortho") is  C o b * (inverse latitude DFT)  with b = 1 / sqrt(nlat nlon).  The unnormalised
// latitude DFT pair are each other's conjugate transposes; with F^T = s C o diag(1, 1/2, ..., 1/2, 1) and
// C^T = diag(1, 2, ..., 2, 1) o F / s the adjoint of either transform is the other one with order weights.
enum { MS_FWD = 0, MS_INV = 1, MS_FWD_ADJ = 2, MS_INV_ADJ = 3 };

int planar_init(sfno_sht_plan* p) {
    int rc = fft_plan_init(p->fft, p->nlon);
    if (rc == SFNO_OK) rc = fft_plan_init(p->fft_lat, p->nlat);
    if (rc == SFNO_OK) rc = fft_chirp_plan_init(p->fft_lat);
    if (rc != SFNO_OK) return rc;
    const double s = 2.0 * 3.14159265358979323846264338327950288 / p->nlon;
    const double b = 1.0 / std::sqrt((double)p->nlat * (double)p->nlon), a = b / s;
    const bool even = p->nlon % 2 == 0;
    const int bits[4] = {SFNO_DIR_FORWARD, SFNO_DIR_INVERSE, SFNO_DIR_FORWARD_ADJOINT, SFNO_DIR_INVERSE_ADJOINT};
    for (int d = 0; d < 4; ++d) {
        if (!(p->directions & bits[d])) continue;
        std::vector<float> ms(p->mmax);
        for (int m = 0; m < p->mmax; ++m) {
            const bool edge = m == 0 || (even && m == p->nlon / 2);
            ms[m] = (float)(d == MS_FWD ? a : d == MS_INV ? b : d == MS_FWD_ADJ ? b * (edge ? 1.0 : 0.5) : a * (edge ? 1.0 : 2.0));
        }
        if ((rc = upload(&p->d_mscale[d], ms)) != SFNO_OK) return rc;
    }
    return SFNO_OK;
}

// latitude stage of a planar plan: `which` selects the order factors, `inverse` the direction of the latitude FFT
int planar_stage(const sfno_sht_plan* p, int which, bool inverse, const float* in, float* out, int64_t rows, void* stream) {
    if (!p->d_mscale[which]) return SFNO_EINVAL;
    return latfft_launch(p->fft_lat, inverse, in, out, p->mmax, p->lmax, (int)sfno_spectral_ld(rows), p->d_mscale[which], (hipStream_t)stream);
}

bool planar(const sfno_sht_plan* p) { return p->grid == SFNO_GRID_PLANAR; }

}  // namespace

extern "C" const char* sfno_strerror(int code) {
    switch (code) {
        case SFNO_OK: return "ok";
        case SFNO_EINVAL: return "invalid argument";
        case SFNO_ENOMEM: return "out of memory";
        case SFNO_EHIP: return "HIP runtime error";
        case SFNO_EWORKSPACE: return "workspace too small";
        case SFNO_EUNSUPPORTED: return "unsupported configuration";
    }
    return "unknown error";
}

extern "C" int sfno_version(void) { return kVersion; }

// 16 floats = 64 bytes: the pieces of a row that FFT workgroups exchange with HBM stay cache-line aligned
extern "C" int64_t sfno_spectral_ld(int64_t rows) { return (2 * rows + 15) / 16 * 16; }

extern "C" int64_t sfno_spectral_elems(const sfno_sht_plan* p, int64_t rows) {
    if (!p || rows <= 0) return 0;
    return (int64_t)p->mmax * p->lmax * sfno_spectral_ld(rows);
}

extern "C" int sfno_sht_plan_create(int nlat, int nlon, int lmax, int mmax, int grid, int norm, int csphase, int directions,
                                    int compute, sfno_sht_plan** out) {
    if (!out) return SFNO_EINVAL;
    *out = nullptr;
    if (nlat < 2 || nlon < 1 || lmax < 1 || mmax < 1) return SFNO_EINVAL;
    // the forward transform keeps the first mmax of nlon/2+1 Fourier bins; the inverse zero-pads or
    // drops orders like a C2R transform, so only the forward direction bounds mmax
    const int all_dirs = SFNO_DIR_FORWARD | SFNO_DIR_INVERSE | SFNO_DIR_FORWARD_ADJOINT | SFNO_DIR_INVERSE_ADJOINT;
    if ((directions & (SFNO_DIR_FORWARD | SFNO_DIR_FORWARD_ADJOINT)) && mmax > nlon / 2 + 1) return SFNO_EINVAL;
    // the adjoint of the zero-padding inverse would need Fourier bins the real FFT does not produce
    if ((directions & SFNO_DIR_INVERSE_ADJOINT) && mmax > nlon / 2 + 1) return SFNO_EUNSUPPORTED;
    if (grid < 0 || grid > SFNO_GRID_PLANAR || norm < 0 || norm > 2) return SFNO_EINVAL;
    if (grid == SFNO_GRID_PLANAR && (lmax > nlat || mmax > nlon / 2 + 1)) return SFNO_EINVAL;
    if (!(directions & all_dirs) || (directions & ~all_dirs)) return SFNO_EINVAL;
    if (compute != SFNO_COMPUTE_FP32 && compute != SFNO_COMPUTE_BF16 && compute != SFNO_COMPUTE_FP32_MFMA && compute != SFNO_COMPUTE_FP32_BF16X3)
        return SFNO_EUNSUPPORTED;
    sfno_sht_plan* p = new (std::nothrow) sfno_sht_plan();
    if (!p) return SFNO_ENOMEM;
    p->nlat = nlat; p->nlon = nlon; p->lmax = lmax; p->mmax = mmax;
    p->grid = grid; p->norm = norm; p->csphase = csphase ? 1 : 0;
    p->directions = directions;
    p->compute = compute == SFNO_COMPUTE_BF16 ? SFNO_COMPUTE_BF16 : SFNO_COMPUTE_FP32;
    p->format = compute == SFNO_COMPUTE_BF16 ? PG_FORMAT_BF16 : compute == SFNO_COMPUTE_FP32_MFMA ? PG_FORMAT_FP32
                : compute == SFNO_COMPUTE_FP32_BF16X3 ? PG_FORMAT_SPLIT : PG_FORMAT_F16X2;
    if (hipGetDevice(&p->device) != hipSuccess) { delete p; return SFNO_EHIP; }
    // set-up of sfno_sht_forward_static on this device; a failure is reported by that entry point, not here
    (void)static_scratch_prepare();
    if (grid == SFNO_GRID_PLANAR) {
        int rc = planar_init(p);
        if (rc != SFNO_OK) { sfno_sht_plan_destroy(p); return rc; }
        *out = p;
        return SFNO_OK;
    }
    std::vector<double> theta(nlat), w(nlat);
    int rc = quadrature(grid, nlat, theta.data(), w.data());
    if (rc == SFNO_OK) rc = fft_plan_init(p->fft, nlon);
    if (rc == SFNO_OK && (directions & SFNO_DIR_FORWARD))
        rc = build_legendre_table(*p, theta.data(), w.data(), nullptr, false, true, p->fwd);
    if (rc == SFNO_OK && (directions & SFNO_DIR_INVERSE))
        rc = build_legendre_table(*p, theta.data(), nullptr, nullptr, true, false, p->inv);
    // Adjoints.  The real FFT pair of this library is  F: x -> s * sum_n x_n e^{-i m phi_n}  (s = 2 pi / nlon)  and
    // C: Y -> Re Y_0 + 2 sum_{0<m<nlon/2} Re(Y_m e^{i m phi_n}) + Re Y_{nlon/2} (-1)^n.  As real-linear maps,
    // F^T = s * C o diag(1, 1/2, ..., 1/2, 1)  and  C^T = diag(1, 2, ..., 2, 1) o F / s, so each adjoint transform is
    // the other FFT kernel around a Legendre stream whose orders carry those factors.
    const bool even = nlon % 2 == 0;
    const double s = 2.0 * 3.14159265358979323846264338327950288 / nlon;
    if (rc == SFNO_OK && (directions & SFNO_DIR_FORWARD_ADJOINT)) {
        std::vector<double> sc(mmax);
        for (int m = 0; m < mmax; ++m) sc[m] = s * ((m == 0 || (even && m == nlon / 2)) ? 1.0 : 0.5);
        rc = build_legendre_table(*p, theta.data(), w.data(), sc.data(), false, false, p->fwd_adj);
    }
    if (rc == SFNO_OK && (directions & SFNO_DIR_INVERSE_ADJOINT)) {
        std::vector<double> sc(mmax);
        for (int m = 0; m < mmax; ++m) sc[m] = ((m == 0 || (even && m == nlon / 2)) ? 1.0 : 2.0) / s;
        rc = build_legendre_table(*p, theta.data(), nullptr, sc.data(), true, true, p->inv_adj);
    }
    if (rc != SFNO_OK) { sfno_sht_plan_destroy(p); return rc; }
    *out = p;
    return SFNO_OK;
}

extern "C" int sfno_sht_plan_destroy(sfno_sht_plan* p) {
    if (!p) return SFNO_OK;
    free_table(p->fwd);
    free_table(p->inv);
    free_table(p->fwd_adj);
    free_table(p->inv_adj);
    fft_plan_free(p->fft);
    fft_plan_free(p->fft_lat);
    for (float*& d : p->d_mscale)
        if (d) { (void)hipFree(d); d = nullptr; }
    delete p;
    return SFNO_OK;
}

extern "C" size_t sfno_sht_workspace_bytes(const sfno_sht_plan* p, int64_t rows) {
    if (!p || !rows_ok(rows)) return 0;
    return carve(p, rows, nullptr).bytes;
}

extern "C" int64_t sfno_fourier_elems(const sfno_sht_plan* p, int64_t rows) {
    if (!p || rows <= 0) return 0;
    return (int64_t)p->mmax * p->nlat * sfno_spectral_ld(rows);
}

extern "C" int sfno_sht_io_dtype_supported(const sfno_sht_plan* p, int x_dtype) {
    if (!p) return 0;
    if (x_dtype == SFNO_DTYPE_F32) return 1;
    return x_dtype == SFNO_DTYPE_BF16 && fft_fast_supported(p->nlon) ? 1 : 0;
}

extern "C" int sfno_rfft(const sfno_sht_plan* p, const void* x, int x_dtype, float* xm, int64_t rows, void* stream) {
    if (!p || !x || !xm || !rows_ok(rows)) return SFNO_EINVAL;
    return rfft_launch(p->fft, x, x_dtype, xm, rows, p->nlat, p->mmax, (int)sfno_spectral_ld(rows), (hipStream_t)stream);
}

extern "C" int sfno_irfft(const sfno_sht_plan* p, const float* xm, void* x, int x_dtype, int64_t rows, void* stream) {
    if (!p || !x || !xm || !rows_ok(rows)) return SFNO_EINVAL;
    return irfft_launch(p->fft, xm, x, x_dtype, rows, p->nlat, p->mmax, (int)sfno_spectral_ld(rows), (hipStream_t)stream);
}

extern "C" int sfno_legendre_analysis(const sfno_sht_plan* p, const float* xm, float* spec, int64_t rows, void* stream) {
    if (!p || !xm || !spec || !rows_ok(rows)) return SFNO_EINVAL;
    if (!(p->directions & SFNO_DIR_FORWARD)) return SFNO_EINVAL;
    if (planar(p)) return planar_stage(p, MS_FWD, false, xm, spec, rows, stream);
    const int64_t ld = sfno_spectral_ld(rows);
    PgemmArgs a = legendre_args(p, p->fwd, xm, spec, ld);
    return legendre_fold_launch(true, p->format, a, p->fwd.n_work, (hipStream_t)stream);
}

extern "C" int sfno_legendre_synthesis(const sfno_sht_plan* p, const float* spec, float* xm, int64_t rows, void* stream) {
    if (!p || !xm || !spec || !rows_ok(rows)) return SFNO_EINVAL;
    if (!(p->directions & SFNO_DIR_INVERSE)) return SFNO_EINVAL;
    if (planar(p)) return planar_stage(p, MS_INV, true, spec, xm, rows, stream);
    const int64_t ld = sfno_spectral_ld(rows);
    PgemmArgs a = legendre_args(p, p->inv, spec, xm, ld);
    return legendre_fold_launch(false, p->format, a, p->inv.n_work, (hipStream_t)stream);
}

extern "C" int sfno_sht_analysis(const sfno_sht_plan* p, const void* x, int x_dtype, float* spec, int64_t rows, void* workspace,
                                 size_t workspace_bytes, void* stream) {
    if (!p || !x || !spec || !rows_ok(rows)) return SFNO_EINVAL;
    if (!(p->directions & SFNO_DIR_FORWARD)) return SFNO_EINVAL;
    Ws w = carve(p, rows, workspace);
    if (!workspace || workspace_bytes < w.bytes) return SFNO_EWORKSPACE;
    int rc = sfno_rfft(p, x, x_dtype, w.xm, rows, stream);
    if (rc != SFNO_OK) return rc;
    return sfno_legendre_analysis(p, w.xm, spec, rows, stream);
}

extern "C" int sfno_sht_synthesis(const sfno_sht_plan* p, const float* spec, void* x, int x_dtype, int64_t rows, void* workspace,
                                  size_t workspace_bytes, void* stream) {
    if (!p || !x || !spec || !rows_ok(rows)) return SFNO_EINVAL;
    if (!(p->directions & SFNO_DIR_INVERSE)) return SFNO_EINVAL;
    Ws w = carve(p, rows, workspace);
    if (!workspace || workspace_bytes < w.bytes) return SFNO_EWORKSPACE;
    int rc = sfno_legendre_synthesis(p, spec, w.xm, rows, stream);
    if (rc != SFNO_OK) return rc;
    return sfno_irfft(p, w.xm, x, x_dtype, rows, stream);
}

extern "C" int sfno_sht_lat_stats_supported(const sfno_sht_plan* p) { return p && fft_fast_supported(p->nlon) ? 1 : 0; }

extern "C" int sfno_sht_synthesis_lat_stats(const sfno_sht_plan* p, const float* spec, void* x, int x_dtype, int64_t rows, void* workspace,
                                            size_t workspace_bytes, float* lat_stats, void* stream) {
    if (!p || !x || !spec || !lat_stats || !rows_ok(rows)) return SFNO_EINVAL;
    if (!(p->directions & SFNO_DIR_INVERSE)) return SFNO_EINVAL;
    if (!sfno_sht_lat_stats_supported(p)) return SFNO_EUNSUPPORTED;
    Ws w = carve(p, rows, workspace);
    if (!workspace || workspace_bytes < w.bytes) return SFNO_EWORKSPACE;
    int rc = sfno_legendre_synthesis(p, spec, w.xm, rows, stream);
    if (rc != SFNO_OK) return rc;
    return irfft_launch(p->fft, w.xm, x, x_dtype, rows, p->nlat, p->mmax, (int)sfno_spectral_ld(rows), (hipStream_t)stream,
                        reinterpret_cast<float2*>(lat_stats));
}

extern "C" int sfno_sht_forward(const sfno_sht_plan* p, const float* x, void* coeffs, int64_t rows, void* workspace,
                                size_t workspace_bytes, void* stream) {
    if (!p || !coeffs || !rows_ok(rows)) return SFNO_EINVAL;
    Ws w = carve(p, rows, workspace);
    if (!workspace || workspace_bytes < w.bytes) return SFNO_EWORKSPACE;
    int rc = sfno_sht_analysis(p, x, SFNO_DTYPE_F32, w.spec, rows, workspace, workspace_bytes, stream);
    if (rc != SFNO_OK) return rc;
    return spectral_to_coeffs_launch(w.spec, reinterpret_cast<float2*>(coeffs), rows, p->lmax, p->mmax,
                                     (int)sfno_spectral_ld(rows), planar(p) ? 0 : 1, (hipStream_t)stream);
}

extern "C" int sfno_sht_inverse(const sfno_sht_plan* p, const void* coeffs, float* x, int64_t rows, void* workspace,
                                size_t workspace_bytes, void* stream) {
    if (!p || !coeffs || !rows_ok(rows)) return SFNO_EINVAL;
    Ws w = carve(p, rows, workspace);
    if (!workspace || workspace_bytes < w.bytes) return SFNO_EWORKSPACE;
    int rc = coeffs_to_spectral_launch(reinterpret_cast<const float2*>(coeffs), w.spec, rows, p->lmax, p->mmax,
                                       (int)sfno_spectral_ld(rows), planar(p) ? 0 : 1, (hipStream_t)stream);
    if (rc != SFNO_OK) return rc;
    return sfno_sht_synthesis(p, w.spec, x, SFNO_DTYPE_F32, rows, workspace, workspace_bytes, stream);
}

// ---- adjoints (vector-Jacobian products of the transforms) -----------------------------------------

extern "C" int sfno_sht_analysis_adjoint(const sfno_sht_plan* p, const float* gspec, void* gx, int x_dtype, int64_t rows, void* workspace,
                                         size_t workspace_bytes, void* stream) {
    if (!p || !gspec || !gx || !rows_ok(rows)) return SFNO_EINVAL;
    if (!(p->directions & SFNO_DIR_FORWARD_ADJOINT)) return SFNO_EINVAL;
    Ws w = carve(p, rows, workspace);
    if (!workspace || workspace_bytes < w.bytes) return SFNO_EWORKSPACE;
    const int64_t ld = sfno_spectral_ld(rows);
    int rc;
    if (planar(p)) {
        rc = planar_stage(p, MS_FWD_ADJ, true, gspec, w.xm, rows, stream);
    } else {
        PgemmArgs a = legendre_args(p, p->fwd_adj, gspec, w.xm, ld);
        rc = legendre_fold_launch(false, p->format, a, p->fwd_adj.n_work, (hipStream_t)stream);
    }
    if (rc != SFNO_OK) return rc;
    return sfno_irfft(p, w.xm, gx, x_dtype, rows, stream);
}

extern "C" int sfno_sht_synthesis_adjoint(const sfno_sht_plan* p, const void* gx, int x_dtype, float* gspec, int64_t rows, void* workspace,
                                          size_t workspace_bytes, void* stream) {
    if (!p || !gspec || !gx || !rows_ok(rows)) return SFNO_EINVAL;
    if (!(p->directions & SFNO_DIR_INVERSE_ADJOINT)) return SFNO_EINVAL;
    Ws w = carve(p, rows, workspace);
    if (!workspace || workspace_bytes < w.bytes) return SFNO_EWORKSPACE;
    int rc = sfno_rfft(p, gx, x_dtype, w.xm, rows, stream);
    if (rc != SFNO_OK) return rc;
    if (planar(p)) return planar_stage(p, MS_INV_ADJ, false, w.xm, gspec, rows, stream);
    const int64_t ld = sfno_spectral_ld(rows);
    PgemmArgs a = legendre_args(p, p->inv_adj, w.xm, gspec, ld);
    return legendre_fold_launch(true, p->format, a, p->inv_adj.n_work, (hipStream_t)stream);
}

extern "C" int sfno_sht_forward_adjoint(const sfno_sht_plan* p, const void* gcoeffs, float* gx, int64_t rows, void* workspace,
                                        size_t workspace_bytes, void* stream) {
    if (!p || !gcoeffs || !gx || !rows_ok(rows)) return SFNO_EINVAL;
    Ws w = carve(p, rows, workspace);
    if (!workspace || workspace_bytes < w.bytes) return SFNO_EWORKSPACE;
    int rc = coeffs_to_spectral_launch(reinterpret_cast<const float2*>(gcoeffs), w.spec, rows, p->lmax, p->mmax,
                                       (int)sfno_spectral_ld(rows), planar(p) ? 0 : 1, (hipStream_t)stream);
    if (rc != SFNO_OK) return rc;
    return sfno_sht_analysis_adjoint(p, w.spec, gx, SFNO_DTYPE_F32, rows, workspace, workspace_bytes, stream);
}

extern "C" int sfno_sht_inverse_adjoint(const sfno_sht_plan* p, const float* gx, void* gcoeffs, int64_t rows, void* workspace,
                                        size_t workspace_bytes, void* stream) {
    if (!p || !gcoeffs || !gx || !rows_ok(rows)) return SFNO_EINVAL;
    Ws w = carve(p, rows, workspace);
    if (!workspace || workspace_bytes < w.bytes) return SFNO_EWORKSPACE;
    int rc = sfno_sht_synthesis_adjoint(p, gx, SFNO_DTYPE_F32, w.spec, rows, workspace, workspace_bytes, stream);
    if (rc != SFNO_OK) return rc;
    return spectral_to_coeffs_launch(w.spec, reinterpret_cast<float2*>(gcoeffs), rows, p->lmax, p->mmax,
                                     (int)sfno_spectral_ld(rows), planar(p) ? 0 : 1, (hipStream_t)stream);
}

extern "C" int sfno_coeffs_to_spectral(const void* coeffs, float* spec, int64_t rows, int lmax, int mmax, int triangular,
                                       void* stream) {
    if (!coeffs || !spec || !rows_ok(rows)) return SFNO_EINVAL;
    return coeffs_to_spectral_launch(reinterpret_cast<const float2*>(coeffs), spec, rows, lmax, mmax, (int)sfno_spectral_ld(rows),
                                     triangular, (hipStream_t)stream);
}

extern "C" int sfno_spectral_to_coeffs(const float* spec, void* coeffs, int64_t rows, int lmax, int mmax, int triangular,
                                       void* stream) {
    if (!coeffs || !spec || !rows_ok(rows)) return SFNO_EINVAL;
    return spectral_to_coeffs_launch(spec, reinterpret_cast<float2*>(coeffs), rows, lmax, mmax, (int)sfno_spectral_ld(rows),
                                     triangular, (hipStream_t)stream);
}

// ---- dhconv -------------------------------------------------------------------------------------

extern "C" int sfno_dhconv_weights_create(int I, int O, int L, int compute, sfno_dhconv_weights** out) {
    if (!out) return SFNO_EINVAL;
    *out = nullptr;
    if (I < 1 || O < 1 || L < 1) return SFNO_EINVAL;
    if (compute != SFNO_COMPUTE_FP32 && compute != SFNO_COMPUTE_BF16 && compute != SFNO_COMPUTE_FP32_BF16X3) return SFNO_EUNSUPPORTED;
    // the bf16 kernel reads activation rows in groups of four floats
    if (compute == SFNO_COMPUTE_BF16 && (2 * I) % 4 != 0) return SFNO_EUNSUPPORTED;
    sfno_dhconv_weights* w = new (std::nothrow) sfno_dhconv_weights();
    if (!w) return SFNO_ENOMEM;
    w->I = I; w->O = O; w->L = L; w->compute = compute;
    // fp32 on the bf16 matrix pipe reads activation rows in groups of four floats; odd channel counts stay on fp32 MFMA
    w->split = compute == SFNO_COMPUTE_FP32_BF16X3 && (2 * I) % 4 == 0;
    w->f16 = compute == SFNO_COMPUTE_FP32 && (2 * I) % 4 == 0;
    if (hipGetDevice(&w->device) != hipSuccess) { delete w; return SFNO_EHIP; }
    size_t bytes;
    if (w->f16) {
        const int co = 32 * dhconv_f16_ntc(O);              // output channels per column block
        w->nob = (O + co - 1) / co;
        w->nc = (I + 15) / 16;
        bytes = (size_t)128 * co * L * w->nob * w->nc;      // (Re, Im) x 2 planes x co x 16 complex fp16 per (degree, column block, chunk)
        if (hipMalloc((void**)&w->d_cinv, sizeof(float) * co * (size_t)L * w->nob) != hipSuccess ||
            hipMalloc((void**)&w->d_cmax, sizeof(float) * (size_t)L * O) != hipSuccess) {
            sfno_dhconv_weights_destroy(w);
            return SFNO_ENOMEM;
        }
    } else if (w->split) {
        w->nob = (2 * O + 127) / 128;
        w->nc = (2 * I + 15) / 16;
        bytes = 6144 * (size_t)L * w->nob * w->nc;          // 3 planes x 64 x 8 complex bf16 per (degree, column block, chunk)
    } else if (compute == SFNO_COMPUTE_BF16) {
        w->nob = (2 * O + 255) / 256;
        w->nc = (2 * I + 31) / 32;
        bytes = 8192 * (size_t)L * w->nob * w->nc;          // 128 x 16 complex bf16 per (degree, column block, chunk)
    } else {
        w->nob = (2 * O + DH_COLS - 1) / DH_COLS;
        w->nc = (2 * I + PG_KC - 1) / PG_KC;
        bytes = sizeof(float) * 1024 * (size_t)L * w->nob * w->nc;   // 8 x 64 complex fp32
    }
    if (hipMalloc((void**)&w->d_W, bytes) != hipSuccess) { sfno_dhconv_weights_destroy(w); return SFNO_ENOMEM; }
    *out = w;
    return SFNO_OK;
}

static int pack_weights(sfno_dhconv_weights* w, const void* weight, int adjoint, void* stream) {
    if (!w || !weight) return SFNO_EINVAL;
    if (w->f16)
        return dhconv_pack_f16_launch(reinterpret_cast<const float2*>(weight), w->d_W, w->d_cinv, w->d_cmax, w->I, w->O, w->L, adjoint,
                                      (hipStream_t)stream);
    if (w->split)
        return dhconv_pack_split_launch(reinterpret_cast<const float2*>(weight), w->d_W, w->I, w->O, w->L, adjoint, (hipStream_t)stream);
    if (w->compute == SFNO_COMPUTE_BF16)
        return dhconv_pack_bf16_launch(reinterpret_cast<const float2*>(weight), w->d_W, w->I, w->O, w->L, adjoint, (hipStream_t)stream);
    return dhconv_pack_launch(reinterpret_cast<const float2*>(weight), w->d_W, w->I, w->O, w->L, adjoint, (hipStream_t)stream);
}

extern "C" int sfno_dhconv_weights_update(sfno_dhconv_weights* w, const void* weight, void* stream) {
    return pack_weights(w, weight, 0, stream);
}

extern "C" int sfno_dhconv_weights_update_adjoint(sfno_dhconv_weights* w, const void* weight, void* stream) {
    return pack_weights(w, weight, 1, stream);
}

extern "C" int sfno_dhconv_weight_grad(int I, int O, int L, const float* spec_in, const float* gspec_out, void* gweight, int batch,
                                       int mmax, int triangular, void* stream) {
    if (I < 1 || O < 1 || L < 1 || !spec_in || !gspec_out || !gweight || batch < 1 || mmax < 1) return SFNO_EINVAL;
    DhconvWgradArgs a;
    a.X = spec_in;
    a.G = gspec_out;
    a.GW = reinterpret_cast<float*>(gweight);
    a.B = batch; a.I = I; a.O = O; a.L = L; a.M = mmax;
    a.tri = triangular ? 1 : 0;
    a.ld_in = (int)sfno_spectral_ld((int64_t)batch * I);
    a.ld_out = (int)sfno_spectral_ld((int64_t)batch * O);
    return dhconv_wgrad_launch(a, (hipStream_t)stream);
}

extern "C" int sfno_dhconv_weights_destroy(sfno_dhconv_weights* w) {
    if (!w) return SFNO_OK;
    if (w->d_W) (void)hipFree(w->d_W);
    if (w->d_cinv) (void)hipFree(w->d_cinv);
    if (w->d_cmax) (void)hipFree(w->d_cmax);
    delete w;
    return SFNO_OK;
}

extern "C" int sfno_dhconv_spectral(const sfno_dhconv_weights* w, const float* spec_in, float* spec_out, int batch, int mmax,
                                    int triangular, void* stream) {
    if (!w || !spec_in || !spec_out || batch < 1 || mmax < 1) return SFNO_EINVAL;
    DhconvArgs a;
    a.X = spec_in;
    a.W = w->d_W;
    a.Y = spec_out;
    a.B = batch;
    a.I2 = 2 * w->I;
    a.O2 = 2 * w->O;
    a.L = w->L;
    a.M = mmax;
    a.tri = triangular ? 1 : 0;
    a.ld_in = (int)sfno_spectral_ld((int64_t)batch * w->I);
    a.ld_out = (int)sfno_spectral_ld((int64_t)batch * w->O);
    a.nob = w->nob;
    a.nc = w->nc;
    a.cinv = w->d_cinv;
    if (w->f16) return dhconv_f16_launch(a, (hipStream_t)stream);
    if (w->split) return dhconv_split_launch(a, (hipStream_t)stream);
    if (w->compute == SFNO_COMPUTE_BF16) return dhconv_bf16_launch(a, (hipStream_t)stream);
    return dhconv_launch(a, (hipStream_t)stream);
}

extern "C" size_t sfno_dhconv_workspace_bytes(const sfno_dhconv_weights* w, int batch, int mmax) {
    if (!w || batch < 1 || mmax < 1) return 0;
    size_t in_b = align_up(sizeof(float) * (size_t)mmax * w->L * sfno_spectral_ld((int64_t)batch * w->I), 256);
    size_t out_b = align_up(sizeof(float) * (size_t)mmax * w->L * sfno_spectral_ld((int64_t)batch * w->O), 256);
    return in_b + out_b;
}

extern "C" int sfno_dhconv(const sfno_dhconv_weights* w, const void* x, void* y, int batch, int mmax, int triangular,
                           void* workspace, size_t workspace_bytes, void* stream) {
    if (!w || !x || !y || batch < 1 || mmax < 1) return SFNO_EINVAL;
    if (!workspace || workspace_bytes < sfno_dhconv_workspace_bytes(w, batch, mmax)) return SFNO_EWORKSPACE;
    size_t in_b = align_up(sizeof(float) * (size_t)mmax * w->L * sfno_spectral_ld((int64_t)batch * w->I), 256);
    float* sin = reinterpret_cast<float*>(workspace);
    float* sout = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + in_b);
    int rc = sfno_coeffs_to_spectral(x, sin, (int64_t)batch * w->I, w->L, mmax, triangular, stream);
    if (rc != SFNO_OK) return rc;
    rc = sfno_dhconv_spectral(w, sin, sout, batch, mmax, triangular, stream);
    if (rc != SFNO_OK) return rc;
    return sfno_spectral_to_coeffs(sout, y, (int64_t)batch * w->O, w->L, mmax, triangular, stream);
}

// ---- per-degree power (spectral losses) ----------------------------------------------------------------

extern "C" int sfno_degree_power(const float* spec, float* power, int64_t rows, int lmax, int mmax, void* stream) {
    if (!spec || !power || !rows_ok(rows)) return SFNO_EINVAL;
    return degree_power_launch(spec, power, rows, lmax, mmax, (int)sfno_spectral_ld(rows), (hipStream_t)stream);
}

extern "C" int sfno_degree_power_grad(const float* spec, const float* gpower, float* gspec, int64_t rows, int lmax, int mmax, void* stream) {
    if (!spec || !gpower || !gspec || !rows_ok(rows)) return SFNO_EINVAL;
    return degree_power_grad_launch(spec, gpower, gspec, rows, lmax, mmax, (int)sfno_spectral_ld(rows), (hipStream_t)stream);
}

// ---- diagonal operator -----------------------------------------------------------------------------

extern "C" int sfno_diagonal_contract(const void* x, const void* weight, void* y, int batch, int in_channels, int out_channels,
                                      int64_t positions, int adjoint, void* stream) {
    if (!x || !weight || !y || batch < 1 || in_channels < 1 || out_channels < 1 || positions < 1) return SFNO_EINVAL;
    return diagonal_contract_launch(reinterpret_cast<const float2*>(x), reinterpret_cast<const float2*>(weight), reinterpret_cast<float2*>(y),
                                    batch, in_channels, out_channels, positions, adjoint ? 1 : 0, (hipStream_t)stream);
}

extern "C" int sfno_diagonal_weight_grad(const void* x, const void* gy, void* gweight, int batch, int in_channels, int out_channels,
                                         int64_t positions, void* stream) {
    if (!x || !gy || !gweight || batch < 1 || in_channels < 1 || out_channels < 1 || positions < 1) return SFNO_EINVAL;
    return diagonal_wgrad_launch(reinterpret_cast<const float2*>(x), reinterpret_cast<const float2*>(gy), reinterpret_cast<float2*>(gweight), batch,
                                 in_channels, out_channels, positions, (hipStream_t)stream);
}

// ---- pointwise tail -----------------------------------------------------------------------------

extern "C" int64_t sfno_pointwise_weight_elems(int O, int K) {
    if (O < 1 || K < 1) return 0;
    return (int64_t)pointwise_opad(O) * pointwise_kpad(K, O);
}

extern "C" int sfno_pointwise_pack_weight(const float* w, void* packed, int O, int K, void* stream) {
    if (!w || !packed || O < 1 || K < 1) return SFNO_EINVAL;
    return pointwise_pack_launch(w, reinterpret_cast<unsigned short*>(packed), O, K, (hipStream_t)stream);
}

extern "C" int sfno_pointwise_conv(const void* x, const void* w, const float* bias, void* y, int batch, int K, int O, int64_t P,
                                   int act, const void* addend, const float* add_scale, const float* add_shift, void* stream) {
    if (!x || !w || !y || batch < 1 || K < 1 || O < 1 || P < 1) return SFNO_EINVAL;
    if (act != SFNO_ACT_NONE && act != SFNO_ACT_GELU) return SFNO_EINVAL;
    PointwiseArgs a;
    std::memset(&a, 0, sizeof(a));
    a.X = reinterpret_cast<const unsigned short*>(x);
    a.W = reinterpret_cast<const unsigned short*>(w);
    a.bias = bias;
    a.Y = reinterpret_cast<unsigned short*>(y);
    a.addend = reinterpret_cast<const unsigned short*>(addend);
    a.add_scale = add_scale;
    a.add_shift = add_shift;
    a.K = K; a.O = O; a.B = batch; a.act = act; a.P = P;
    return pointwise_gemm_launch(a, (hipStream_t)stream);
}

extern "C" int sfno_pointwise_conv_cat(const void* x1, int K1, const void* x2, int K2, const void* w, const float* bias, void* y, int batch,
                                       int O, int64_t P, int act, void* stream) {
    if (!x1 || !x2 || !w || !y || batch < 1 || K1 < 1 || K2 < 1 || O < 1 || P < 1) return SFNO_EINVAL;
    if (act != SFNO_ACT_NONE && act != SFNO_ACT_GELU) return SFNO_EINVAL;
    PointwiseArgs a;
    std::memset(&a, 0, sizeof(a));
    a.X = reinterpret_cast<const unsigned short*>(x1);
    a.X2 = reinterpret_cast<const unsigned short*>(x2);
    a.K1 = K1;
    a.W = reinterpret_cast<const unsigned short*>(w);
    a.bias = bias;
    a.Y = reinterpret_cast<unsigned short*>(y);
    a.K = K1 + K2; a.O = O; a.B = batch; a.act = act; a.P = P;
    return pointwise_gemm_launch(a, (hipStream_t)stream);
}

extern "C" size_t sfno_pointwise_weight_grad_workspace_bytes(int batch, int K, int O, int64_t P, int has_bias) {
    if (batch < 1 || K < 1 || O < 1 || P < 8 || P % 8) return 0;
    return pointwise_wgrad_workspace_bytes(O, K, has_bias, batch, P);
}

extern "C" int sfno_pointwise_weight_grad(const void* gy, const void* x, float* gweight, float* gbias, int batch, int K, int O, int64_t P,
                                          void* workspace, size_t workspace_bytes, void* stream) {
    if (!gy || !x || !gweight || !workspace || batch < 1 || K < 1 || O < 1 || P < 8 || P % 8) return SFNO_EINVAL;
    // 16-byte loads of eight bf16 values
    if ((reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(workspace)) & 15) return SFNO_EINVAL;
    return pointwise_wgrad_launch(reinterpret_cast<const unsigned short*>(gy), reinterpret_cast<const unsigned short*>(x), gweight, gbias, batch, K, O, P,
                                  reinterpret_cast<float*>(workspace), workspace_bytes, (hipStream_t)stream);
}

extern "C" size_t sfno_instance_norm_workspace_bytes(int64_t rows, int64_t P) {
    if (rows < 1 || P < 1) return 0;
    return sizeof(float2) * (size_t)rows * row_stats_segments(rows, P);
}

extern "C" int sfno_instance_norm_coeffs(const void* x, const float* gamma, const float* beta, float* scale, float* shift, int64_t rows,
                                         int channels, int64_t P, float eps, void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !scale || !shift || rows < 1 || channels < 1 || P < 1) return SFNO_EINVAL;
    if (!workspace || workspace_bytes < sfno_instance_norm_workspace_bytes(rows, P)) return SFNO_EWORKSPACE;
    return instance_norm_coeffs_launch(reinterpret_cast<const unsigned short*>(x), gamma, beta, scale, shift, reinterpret_cast<float2*>(workspace),
                                       rows, channels, P, eps, (hipStream_t)stream);
}

extern "C" int sfno_instance_norm_coeffs_lat(const float* lat_stats, const float* gamma, const float* beta, float* scale, float* shift, int64_t rows,
                                             int channels, int nlat, float eps, void* stream) {
    if (!lat_stats || !scale || !shift) return SFNO_EINVAL;
    return instance_norm_coeffs_lat_launch(reinterpret_cast<const float2*>(lat_stats), gamma, beta, scale, shift, rows, channels, nlat, eps,
                                           (hipStream_t)stream);
}

extern "C" int sfno_scale_shift_act(const void* x, const float* scale, const float* shift, void* y, int64_t rows, int64_t P, int act,
                                    void* stream) {
    if (!x || !scale || !shift || !y || rows < 1 || P < 1) return SFNO_EINVAL;
    if (act != SFNO_ACT_NONE && act != SFNO_ACT_GELU) return SFNO_EINVAL;
    return scale_shift_act_launch(reinterpret_cast<const unsigned short*>(x), scale, shift, reinterpret_cast<unsigned short*>(y), rows, P, act,
                                  (hipStream_t)stream);
}
