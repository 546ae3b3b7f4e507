// Internal declarations shared by the host code and the HIP kernels of libsfno_spectral.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <vector>

#include "sfno_spectral.h"

namespace sfno {

// ---- packed operands -------------------------------------------------------------------
// One operand of every contraction on this path is constant between calls (Legendre
// table, SpectralConv weight).  It is stored as a stream of 32x16 blocks, each laid out
// exactly as the MFMA fragments of one wavefront consume it: block = 2 halves x 64 lanes
// x float4; lane j of half h holds, for s = 0..3,
//     P[row = 32*rb + (j & 31)][k = 16*c + 8*h + 2*s + (j >> 5)].
// A wavefront owns one 32-row block `rb` of one batch (order m and parity, or degree l) and
// walks its K-chunks c = 0..nc-1, which are contiguous in memory.
constexpr int PG_ROWS = 32;        // rows per block (MFMA 32x32x2)
constexpr int PG_KC = 16;          // K per block
constexpr int PG_BLOCK_FLOATS = PG_ROWS * PG_KC;   // 512 floats = 2 KiB
constexpr int PG_WAVES = 4;        // wavefronts (= row blocks) per workgroup

// Work record of the two-part fp16 kernels, 8 x int64 per work-list entry: the order and first row block, the index
// entries of the workgroup's four (parity, row block) streams (an absent one reads nc << 48: nothing to do) and the
// positions of the two parities' first entries -- one 64-byte read instead of a chain of dependent look-ups.
constexpr int PG_WREC = 8;
constexpr int PG_WREC_M = 0, PG_WREC_RB = 1, PG_WREC_ENTRY = 2, PG_WREC_POS = 6;

struct PgemmTable {
    float* d_A = nullptr;          // packed stream
    float* d_rinv = nullptr;       // two-part fp16 format: 32 factors per row-block entry that undo the row scales
    int64_t* d_aoff = nullptr;     // index of the stream, see pack_legendre_fold
    int2* d_work = nullptr;        // [n_work] {batch, first row block} per workgroup, -1 = idle
    int64_t* d_wrec = nullptr;     // two-part fp16 format: [n_work][8] everything a workgroup needs of the index, see PG_WREC_*
    int n_work = 0;                // multiple of 8 (one queue per XCD, interleaved)
    int64_t n_blocks = 0;
};

struct PgemmArgs {
    const float* A;
    const int64_t* a_off;
    const int2* work;
    const int64_t* wrec;           // two-part fp16 format: work records (PG_WREC_*)
    const float* Q;
    float* Out;
    const float* rinv;             // two-part fp16 format: row factors, [entry position - 2 mmax][32]
    int lmax, nlat, mmax;          // Legendre modes
    int ld;                        // channel leading dimension of Q and Out (Legendre modes)
};

// dhconv: output columns o' per workgroup, and the kernel arguments
constexpr int DH_COLS = 128;
struct DhconvArgs {
    const float* X;                // spectral layout, rows (m, l, b) of 2*I floats
    const float* W;                // packed complex weights [L][nob][nc][8][64]
    float* Y;                      // spectral layout, rows of 2*O floats
    int B, I2, O2, L, M, tri, ld_in, ld_out;
    int nob, nc;                   // column blocks of DH_COLS over 2*O, K chunks of 16 over 2*I
    const float* cinv;             // fp16-pair kernel: [L][nob * channels per block] factors that undo the column scales of the packed weights
};
int dhconv_launch(const DhconvArgs& a, hipStream_t s);
// bf16 MFMA variant: 256 output columns per workgroup, K chunks of 32, weights packed as complex bf16
int dhconv_bf16_launch(const DhconvArgs& a, hipStream_t s);
// fp32 operands on the bf16 matrix pipe: 128 output columns per workgroup, K chunks of 32, weights packed as three planes of
// complex bf16 whose sum is the fp32 weight
int dhconv_split_launch(const DhconvArgs& a, hipStream_t s);
int dhconv_pack_split_launch(const float2* w, void* packed, int I, int O, int L, int adjoint, hipStream_t s);
// fp32 operands on the fp16 matrix pipe (two fp16 planes per operand, power-of-two scales per weight column and per activation
// row): 32 dhconv_f16_ntc(O) output channels per workgroup (a.nob blocks of them), a.nc chunks of 16 input channels; cinv
// receives [L][nob * 32 ntc] inverse column scales, cmax is [L][O] scratch
int dhconv_f16_ntc(int O);
int dhconv_f16_launch(const DhconvArgs& a, hipStream_t s);
int dhconv_pack_f16_launch(const float2* w, void* packed, float* cinv, float* cmax, int I, int O, int L, int adjoint, hipStream_t s);
// adjoint = 1 packs the conjugate transpose: w then has shape [O][I][L] and element (i, o) is conj(w[o][i])
int dhconv_pack_bf16_launch(const float2* w, void* packed, int I, int O, int L, int adjoint, hipStream_t s);
// gradient of the contraction with respect to its weight:
// gw[i][o][l] = sum over rows (m, b) of conj(X[(m, l, b)][i]) * G[(m, l, b)][o]
struct DhconvWgradArgs {
    const float* X;                // spectral layout, rows of 2*I floats
    const float* G;                // spectral layout, rows of 2*O floats
    float* GW;                     // complex [I][O][L]
    int B, I, O, L, M, tri, ld_in, ld_out;
};
int dhconv_wgrad_launch(const DhconvWgradArgs& a, hipStream_t s);

// ---- "diagonal" operator on the reference layout (diagonal.hip): x [B][I][P], w [I][O][P], y [B][O][P], P = L*M ----
int diagonal_contract_launch(const float2* x, const float2* w, float2* y, int B, int I, int O, int64_t P, int adjoint, hipStream_t s);
int diagonal_wgrad_launch(const float2* x, const float2* g, float2* gw, int B, int I, int O, int64_t P, hipStream_t s);

// ---- pointwise tail (pointwise.hip): bf16 NCHW activations, 1x1 convolutions on bf16 MFMA ------------
struct PointwiseArgs {
    const unsigned short* X;       // bf16 [B][K][P]; with X2: [B][K1][P], the first K1 input channels
    const unsigned short* X2;      // null, or bf16 [B][K - K1][P]: the remaining input channels come from a second tensor
    int K1;
    const unsigned short* W;       // packed by pointwise_pack_launch
    const float* bias;             // [O] or null
    unsigned short* Y;             // bf16 [B][O][P]
    const unsigned short* addend;  // bf16 [B][O][P] or null: y += add_scale[b][o] * addend + add_shift[b][o]
    const float* add_scale;        // [B][O] or null (1)
    const float* add_shift;        // [B][O] or null (0)
    int K, Kpad, O, B, act;
    int64_t P;
    int n_oblk;                    // filled by the launcher
    int64_t n_strips;
};
int pointwise_gemm_launch(PointwiseArgs a, hipStream_t s);
int pointwise_kpad(int K, int O);
int pointwise_opad(int O);
int pointwise_pack_launch(const float* w, unsigned short* packed, int O, int K, hipStream_t s);
// weight and bias gradient of the 1x1 convolution (pointwise_wgrad.hip); db null: no bias column
size_t pointwise_wgrad_workspace_bytes(int O, int K, int has_bias, int B, int64_t P);
int pointwise_wgrad_launch(const unsigned short* g, const unsigned short* x, float* dW, float* db, int B, int K, int O, int64_t P, float* ws,
                           size_t ws_bytes, hipStream_t s);
int row_stats_segments(int64_t rows, int64_t P);
int instance_norm_coeffs_launch(const unsigned short* x, const float* gamma, const float* beta, float* scale, float* shift, float2* partial,
                                int64_t rows, int channels, int64_t P, float eps, hipStream_t s);
int instance_norm_coeffs_lat_launch(const float2* stats, const float* gamma, const float* beta, float* scale, float* shift, int64_t rows, int channels,
                                    int nlat, float eps, hipStream_t s);
int scale_shift_act_launch(const unsigned short* x, const float* scale, const float* shift, unsigned short* y, int64_t rows, int64_t P, int act,
                           hipStream_t s);

// ---- host-side table construction (tables.cpp) -----------------------------------------
int quadrature(int grid, int nlat, double* theta, double* w);
// rows l = m..lmax-1 of order m at all latitudes: out[(l-m)*nlat + k]
struct LegendreGen {
    int nlat, lmax, mmax, norm, inverse, csphase;
    std::vector<double> cost;
    std::vector<double> diag;      // [mmax][nlat]  Pbar_m^m
    LegendreGen(int mmax, int lmax, int nlat, const double* theta, int norm, int inverse, int csphase);
    void rows_for_m(int m, double* out) const;
};
// XCD-aware work list: cost[b] = relative time of one workgroup of batch b, nrb[b] = row blocks
void build_worklist(const std::vector<int>& nrb, const std::vector<double>& cost, std::vector<int2>& work,
                    int rb_step = PG_WAVES);
// equator-folded Legendre streams (two per order: even and odd l+m), see tables.cpp
// format of one 32 x 16 block of the stream:
//   PG_FORMAT_FP32 : 512 floats, fragments of v_mfma_f32_32x32x2_f32
//   PG_FORMAT_BF16 : 8 bf16 per lane (rounded to nearest even), 256 floats = 1 KiB
//   PG_FORMAT_SPLIT: three planes of 8 bf16 per lane whose sum is the fp32 value exactly, 768 floats = 3 KiB
//   PG_FORMAT_F16X2: two planes of 8 fp16 per lane, the entry times a power of two per row (rounded, and the rounded remainder),
//                    512 floats = 2 KiB; the factors that undo the row scales go to a separate array
enum { PG_FORMAT_FP32 = 0, PG_FORMAT_BF16 = 1, PG_FORMAT_SPLIT = 2, PG_FORMAT_F16X2 = 3 };
inline int pg_block_floats(int format) { return format == PG_FORMAT_BF16 ? 256 : format == PG_FORMAT_SPLIT ? 768 : 512; }
// value = P * lat_w[k] * order_scale[m]; a null pointer stands for all ones
// aoff: [2 m + p] -> position in aoff of the stream's first row-block entry; entry of row block rb (at that position + rb) =
// first block of the row block | (number of leading K chunks left out as negligible << 48); chunks_per_rb (optional): mean
// number of kept chunks per row block of every order (work-list cost)
// rinv (PG_FORMAT_F16X2): 32 row factors per row-block entry, in the order of the entries
void pack_legendre_fold(const LegendreGen& g, const double* lat_w, const double* order_scale, bool analysis, int format,
                        std::vector<float>& packed, std::vector<int64_t>& aoff, std::vector<double>* chunks_per_rb = nullptr,
                        std::vector<float>* rinv = nullptr);
int legendre_fold_launch(bool analysis, int format, const PgemmArgs& a, int n_work, hipStream_t s);
int legendre_f16_launch(bool analysis, const PgemmArgs& a, int n_work, hipStream_t s);

// ---- FFT (fft.hip) -----------------------------------------------------------------------
struct FftPlan {
    int n = 0;                     // transform length (nlon)
    int n_cu = 256;                // compute units of the plan's device (sizes the persistent grids of fft_fast.hip)
    int npass = 0;
    int radix[24];
    float2* d_tw = nullptr;        // [n] exp(-2 pi i j / n)
    float2* d_tw0 = nullptr;       // inter-pass twiddles of the specialised kernels (fft_fast.hip)
    float2* d_tw1 = nullptr;
    unsigned* d_post = nullptr;    // [n/2+1] LDS slot of bin m (low half) and of bin n - m (high half) around the specialised passes
    // latitude plans of lengths with a large prime factor (fft_chirp_plan_init): the DFT as a circular convolution of
    // length chirp_m with a chirp; d_tw0 / d_tw1 then belong to the specialised passes of length chirp_m
    int chirp_m = 0;
    float2* d_chirp = nullptr;     // [n] exp(-i pi k^2 / n)
    float2* d_vhat = nullptr;      // [chirp_m] transform of the conjugate chirp, in the slot order of the passes, divided by chirp_m
};
bool fft_fast_supported(int n);
int fft_fast_plan_init(FftPlan& p);
// grid_dtype: element type of the grid-side tensor (SFNO_DTYPE_*); the Fourier side is always float
// lat_stats (inverse only, may be null): float2 [rows][nlat] = mean over longitude of the output row and of its squared deviation from that mean
int fft_fast_launch(bool inverse, const FftPlan& p, const void* in, void* out, int64_t rows, int nlat, int mmax, int ld, int grid_dtype,
                    hipStream_t s, float2* lat_stats = nullptr);
// latitude FFT on the specialised passes; SFNO_EUNSUPPORTED for a length without them
int latfft_fast_launch(bool inverse, const FftPlan& p, const float* in, float* out, int mmax, int lmax, int ld, const float* mscale, hipStream_t s);
int fft_plan_init(FftPlan& p, int n);
// adds the chirp tables to a latitude plan whose length has no specialised passes and a prime factor above 7 (no-op otherwise)
int fft_chirp_plan_init(FftPlan& p);
void fft_plan_free(FftPlan& p);
// x [rows][nlat][nlon] -> xm [mmax][nlat][ld] (re,im of row r at 2r,2r+1), scaled by 2 pi / nlon
int rfft_launch(const FftPlan& p, const void* x, int x_dtype, float* xm, int64_t rows, int nlat, int mmax, int ld, hipStream_t s);
// xm [mmax][nlat][ld] -> x [rows][nlat][nlon]
int irfft_launch(const FftPlan& p, const float* xm, void* x, int x_dtype, int64_t rows, int nlat, int mmax, int ld, hipStream_t s, float2* lat_stats = nullptr);
// latitude FFT of the planar transforms on the order-major layout: in[m][nlat | lmax][ld] -> out[m][lmax | nlat][ld]
// (forward keeps lmax frequencies, inverse zero-fills the dropped ones); outputs are multiplied by mscale[m] (device array)
int latfft_launch(const FftPlan& p, bool inverse, const float* in, float* out, int mmax, int lmax, int ld, const float* mscale, hipStream_t s);

// ---- per-degree power of spectral-layout coefficients and its gradient (degree_power.hip) ------------
int degree_power_launch(const float* spec, float* power, int64_t rows, int lmax, int mmax, int ld, hipStream_t s);
int degree_power_grad_launch(const float* spec, const float* gpower, float* gspec, int64_t rows, int lmax, int mmax, int ld, hipStream_t s);

// ---- file-scope scratch array of sfno_sht_forward_static (static_scratch.hip) ----------------
// looks up, once per device, the device address of the array on the current device; called at plan creation
int static_scratch_prepare();

// ---- layout passes (layout.hip) ----------------------------------------------------------
int coeffs_to_spectral_launch(const float2* coeffs, float* spec, int64_t rows, int lmax, int mmax, int ld, int tri,
                              hipStream_t s);
int spectral_to_coeffs_launch(const float* spec, float2* coeffs, int64_t rows, int lmax, int mmax, int ld, int tri,
                              hipStream_t s);
int dhconv_pack_launch(const float2* w, float* packed, int I, int O, int L, int adjoint, hipStream_t s);

}  // namespace sfno

struct sfno_sht_plan {
    int nlat, nlon, lmax, mmax, grid, norm, csphase, directions, compute, device;
    int format;                         // PG_FORMAT_* of the Legendre streams
    sfno::PgemmTable fwd, inv;          // analysis (forward) and synthesis (inverse) streams
    sfno::PgemmTable fwd_adj, inv_adj;  // their adjoints: synthesis-format stream of the analysis table and vice versa
    sfno::FftPlan fft;
    // grid == SFNO_GRID_PLANAR: the latitude stage is an FFT of length nlat instead of a Legendre stream
    sfno::FftPlan fft_lat;
    float* d_mscale[4] = {nullptr, nullptr, nullptr, nullptr};   // per-order output factors: forward, inverse, forward adjoint, inverse adjoint
};

struct sfno_dhconv_weights {
    int I, O, L, compute, device;
    int split;                     // fp32 compute with the weights stored as three bf16 planes (even in_channels)
    int f16;                       // fp32 compute with the weights stored as two scaled fp16 planes (even in_channels)
    int nob, nc;                   // column blocks (over 2*O) and K chunks (over 2*I) per degree
    float* d_W = nullptr;          // packed complex weights
    float* d_cinv = nullptr;       // f16: [L][nob * channels per block] inverse column scales
    float* d_cmax = nullptr;       // f16: [L][O] scratch of the pack kernels
};
