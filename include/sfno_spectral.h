/*
 * sfno_spectral.h -- C ABI of the MI355X (gfx950) SFNO spectral hot path.
 *
 * The library replaces, for one GPU, the device work that Makani's SFNO issues
 * through torch-harmonics and torch.einsum:
 *   - RealSHT.forward / InverseRealSHT.forward (torch-harmonics; constructed at
 *     makani/models/networks/sfnonet.py:536-539, called at
 *     makani/models/common/spectral_convolution.py:131,133,141 and
 *     makani/models/networks/sfnonet.py:596,598,616),
 *   - the "dhconv" contraction, makani/models/common/contractions.py:130-136
 *     (selected by makani/models/common/factorizations.py:212-232).
 *
 * Conventions
 *   - every function returns 0 on success or a negative SFNO_E* code; nothing throws.
 *   - all device pointers are plain HIP device addresses owned by the caller;
 *     `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *   - the compute entry points only enqueue kernels on `stream`: they do not
 *     allocate, free, synchronise or create streams.  Scratch memory is passed in by
 *     the caller (`workspace`), sized by the matching *_workspace_bytes query.
 *   - "rows" is the product of all leading dimensions (batch x channels).
 *   - real fields are float32 [rows][nlat][nlon]; coefficients are complex64
 *     (interleaved re,im) [rows][lmax][mmax], m fastest -- the memory layout the
 *     reference modules produce.
 *   - the "spectral" layout is the library's internal, order-major coefficient
 *     layout float32 [mmax][lmax][ld] with ld = sfno_spectral_ld(rows) and the
 *     channel axis holding (re,im) of row r at 2r, 2r+1.  Entries with l < m are
 *     never read and never written.
 */
#ifndef SFNO_SPECTRAL_H
#define SFNO_SPECTRAL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* error codes */
#define SFNO_OK 0
#define SFNO_EINVAL (-1)    /* bad argument (shape, enum, null pointer) */
#define SFNO_ENOMEM (-2)    /* device or host allocation failed at plan creation */
#define SFNO_EHIP (-3)      /* a HIP runtime call failed */
#define SFNO_EWORKSPACE (-4) /* workspace too small */
#define SFNO_EUNSUPPORTED (-5)

/* grid = quadrature rule in latitude (torch-harmonics `grid=` strings) */
#define SFNO_GRID_LEGENDRE_GAUSS 0
#define SFNO_GRID_LOBATTO 1
#define SFNO_GRID_EQUIANGULAR 2
/* Not a quadrature rule: the planar pair RealFFT2 / InverseRealFFT2 of makani/models/common/layers.py:219-287
 * (torch.fft.rfft2 / irfft2 with norm="ortho") behind the same plan and entry points.  The latitude stage is an
 * FFT of length nlat; `lmax` <= nlat counts the kept latitude frequencies (the ceil(lmax/2) lowest non-negative
 * and the floor(lmax/2) highest, in that order, as the reference concatenates them), `mmax` <= nlon/2+1 the
 * kept longitude frequencies.  `norm` and `csphase` are ignored, the spectral layout is full (no l < m rule). */
#define SFNO_GRID_PLANAR 3

/* norm = normalisation of the harmonics (torch-harmonics `norm=` strings) */
#define SFNO_NORM_ORTHO 0
#define SFNO_NORM_FOUR_PI 1
#define SFNO_NORM_SCHMIDT 2

/* which tables a plan holds */
#define SFNO_DIR_FORWARD 1
#define SFNO_DIR_INVERSE 2
#define SFNO_DIR_FORWARD_ADJOINT 4   /* tables of sfno_sht_forward_adjoint / sfno_sht_analysis_adjoint */
#define SFNO_DIR_INVERSE_ADJOINT 8   /* tables of sfno_sht_inverse_adjoint / sfno_sht_synthesis_adjoint */

/* element type of a grid-side (real field) tensor */
#define SFNO_DTYPE_F32 0
#define SFNO_DTYPE_BF16 1

/* arithmetic of the Legendre / channel-mix contractions */
#define SFNO_COMPUTE_FP32 0      /* fp32 operands, fp32 accumulate.  Both contractions (Legendre stage and channel mix) run on
                                  * the fp16 matrix pipe: each operand is scaled by a power of two (tables and weights per
                                  * row or column when they are packed, activations per row or per panel column as they are
                                  * staged) and cut into two fp16 numbers (22 of its 24 significant bits), three of the four
                                  * partial products are accumulated in fp32 and the scales are undone on output: error of
                                  * the size of fp32 rounding, relative to the sum of |x||t| over the contracted index.
                                  * Channel mixes with an odd number of input channels run on fp32 MFMA. */
#define SFNO_COMPUTE_BF16 1      /* bf16 MFMA inputs (tables and activations rounded to bf16), fp32 accumulate */
#define SFNO_COMPUTE_FP32_MFMA 2 /* transform plans only: as SFNO_COMPUTE_FP32 with the Legendre stage on the fp32 MFMA
                                  * instruction (fp32 tables, no operand splitting) */
#define SFNO_COMPUTE_FP32_BF16X3 3 /* as SFNO_COMPUTE_FP32 with every operand cut exactly into three bf16 numbers and the six
                                  * products larger than 2^-23 of the result accumulated in fp32 (no scales) */

/* activation fused into the pointwise kernels */
#define SFNO_ACT_NONE 0
#define SFNO_ACT_GELU 1          /* exact (erf) GELU, torch.nn.GELU() */

typedef struct sfno_sht_plan sfno_sht_plan;
typedef struct sfno_dhconv_weights sfno_dhconv_weights;

const char* sfno_strerror(int code);
/* library ABI version, bumped on any signature change */
int sfno_version(void);

/* ---- host-only helpers (no GPU needed) ------------------------------------------- */

/* Colatitudes theta[nlat] (ascending: row 0 is the northernmost) and quadrature
 * weights w[nlat] of a grid.  Replaces torch_harmonics.quadrature.{legendre_gauss,
 * lobatto,clenshaw_curtiss}_weights as called by the transform constructors and by
 * makani/utils/grids.py:32,77,83. */
int sfno_quadrature(int grid, int nlat, double* theta, double* w);

/* Dense float64 table out[m][l][k] = Pbar_l^m(cos theta[k]) (zero for l < m), the
 * tensor the reference modules keep as the buffers `weights` (after multiplication by
 * w[k]) and `pct`.  `inverse` selects the synthesis normalisation. */
int sfno_legendre_table(int mmax, int lmax, int nlat, const double* theta, int norm,
                        int inverse, int csphase, double* out);

/* Which part of that table a plan streams.  Towards the poles Pbar_l^m falls off like
 * sin^m(theta), so the device streams (32-row blocks x K chunks of 16 over the northern
 * latitudes, per order m and parity p of l + m) leave out the leading chunks of a row block
 * whose entries are all at most 2^-64 of the largest entry of the order.  Writes the number
 * of omitted chunks of every row block, in stream order (m, p, row block), to skips (at most
 * `capacity` values) and returns the number of row blocks, or a negative error code.
 * analysis != 0: rows are the degrees l = m + p + 2 i, K runs over the latitudes and the
 * entries carry lat_w[k] (may be null); otherwise rows are the latitudes and K runs over i.
 * No counterpart in the reference (its tables are dense); host-only, for tests and sizing. */
int64_t sfno_legendre_stream_skips(int mmax, int lmax, int nlat, const double* theta, const double* lat_w,
                                   int norm, int inverse, int csphase, int analysis, int32_t* skips,
                                   int64_t capacity);

/* ---- transform plans --------------------------------------------------------------- */

/* Builds the packed Legendre tables and FFT twiddles on the current HIP device.
 * Mirrors RealSHT.__init__ / InverseRealSHT.__init__(nlat, nlon, lmax, mmax, grid, norm,
 * csphase); `directions` is a mask of SFNO_DIR_*; `compute` one of SFNO_COMPUTE_*. */
int sfno_sht_plan_create(int nlat, int nlon, int lmax, int mmax, int grid, int norm,
                         int csphase, int directions, int compute, sfno_sht_plan** out);
int sfno_sht_plan_destroy(sfno_sht_plan* plan);

/* leading dimension (floats) of the channel axis of the spectral layout */
int64_t sfno_spectral_ld(int64_t rows);
/* floats in one spectral-layout buffer: mmax * lmax * ld */
int64_t sfno_spectral_elems(const sfno_sht_plan* plan, int64_t rows);

/* bytes of scratch the calls below need for `rows` rows */
size_t sfno_sht_workspace_bytes(const sfno_sht_plan* plan, int64_t rows);

/* sfno_sht_synthesis that also returns, for every channel row and latitude, two moments of the field it writes:
 * lat_stats float32 [rows][nlat][2] = (mean over longitude, mean over longitude of the squared deviation from that
 * mean).  They come from the Fourier coefficients the longitude kernel has in hand (mean = Re X_0, deviation =
 * 2 sum_{0<m<nlon/2} |X_m|^2 + (Re X_{nlon/2})^2) and save the statistics pass of the nn.InstanceNorm2d that
 * follows SpectralConv in the SFNO block (makani/models/networks/sfnonet.py:246-250); they describe the field before
 * any rounding to x_dtype.  Only plans whose nlon has specialised kernels (sfno_sht_lat_stats_supported). */
int sfno_sht_lat_stats_supported(const sfno_sht_plan* plan);
int sfno_sht_synthesis_lat_stats(const sfno_sht_plan* plan, const float* spec, void* x, int x_dtype, int64_t rows, void* workspace,
                                 size_t workspace_bytes, float* lat_stats, void* stream);

/* RealSHT.forward: x float32 [rows][nlat][nlon] -> coeffs complex64 [rows][lmax][mmax] */
int sfno_sht_forward(const sfno_sht_plan* plan, const float* x, void* coeffs, int64_t rows,
                     void* workspace, size_t workspace_bytes, void* stream);
/* InverseRealSHT.forward: coeffs complex64 [rows][lmax][mmax] -> x float32 [rows][nlat][nlon] */
int sfno_sht_inverse(const sfno_sht_plan* plan, const void* coeffs, float* x, int64_t rows,
                     void* workspace, size_t workspace_bytes, void* stream);

/* sfno_sht_forward without a workspace argument and without any allocation, for callers that cannot allocate device memory:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (PyTorch allocates the intermediates of RealSHT.forward on every call).  The Fourier and spectral-layout
 * buffers live in one array of SFNO_STATIC_SCRATCH_BYTES that the library holds on every GPU it runs on until the process
 * ends; sfno_sht_plan_create looks up its address for the plan's device.  Returns SFNO_EWORKSPACE when
 * sfno_sht_workspace_bytes(plan, rows) exceeds the array (64 MiB: e.g. 8 rows of 721 x 1440 with lmax = mmax = 721, or
 * 64 rows of 241 x 480), SFNO_EHIP when the look-up failed.  Results equal sfno_sht_forward's bit for bit.  All calls on
 * one GPU share the array: calls that overlap in time on one GPU (different streams or threads) race. */
#define SFNO_STATIC_SCRATCH_BYTES (64u << 20)
int sfno_sht_forward_static(const sfno_sht_plan* plan, const float* x, void* coeffs, int64_t rows, void* stream);

/* Same transforms with coefficients kept in the spectral layout (no layout pass).  The grid-side
 * tensor x may be float32 or bfloat16 (`x_dtype`, SFNO_DTYPE_*): a bf16 field is widened on load /
 * rounded to nearest even on store inside the FFT kernels, which is what the reference's
 * `x.float()` before and `x.to(dtype)` after the transforms compute
 * (makani/models/common/spectral_convolution.py:127,146).  sfno_sht_io_dtype_supported tells
 * whether the plan's longitude length has such kernels (otherwise SFNO_EUNSUPPORTED). */
int sfno_sht_io_dtype_supported(const sfno_sht_plan* plan, int x_dtype);
int sfno_sht_analysis(const sfno_sht_plan* plan, const void* x, int x_dtype, float* spec, int64_t rows,
                      void* workspace, size_t workspace_bytes, void* stream);
int sfno_sht_synthesis(const sfno_sht_plan* plan, const float* spec, void* x, int x_dtype, int64_t rows,
                       void* workspace, size_t workspace_bytes, void* stream);

/* The four stages of the transform pair on their own (what sfno_sht_analysis and
 * sfno_sht_synthesis chain).  xm is the order-major Fourier buffer float32
 * [mmax][nlat][ld]: (re,im) of 2 pi/nlon * sum_n x[r][k][n] e^{-i m phi_n} at
 * xm[m][k][2r], xm[m][k][2r+1]. */
int sfno_rfft(const sfno_sht_plan* plan, const void* x, int x_dtype, float* xm, int64_t rows, void* stream);
int sfno_irfft(const sfno_sht_plan* plan, const float* xm, void* x, int x_dtype, int64_t rows, void* stream);
int sfno_legendre_analysis(const sfno_sht_plan* plan, const float* xm, float* spec, int64_t rows,
                           void* stream);
int sfno_legendre_synthesis(const sfno_sht_plan* plan, const float* spec, float* xm, int64_t rows,
                            void* stream);
/* floats in one xm buffer: mmax * nlat * ld */
int64_t sfno_fourier_elems(const sfno_sht_plan* plan, int64_t rows);

/* Vector-Jacobian products of the transforms, i.e. what autograd runs as the backward of
 * RealSHT.forward / InverseRealSHT.forward (the reference differentiates its einsum + FFT graph;
 * tests/test_models.py:149-157 checks that the input receives a gradient).  Gradients of complex
 * tensors follow the PyTorch convention dL/dRe + i dL/dIm.  The plan must have been created with
 * the matching SFNO_DIR_*_ADJOINT bit; workspace size as for the transforms themselves.
 *   forward_adjoint : gcoeffs complex64 [rows][lmax][mmax] -> gx float32 [rows][nlat][nlon]
 *   inverse_adjoint : gx float32 [rows][nlat][nlon] -> gcoeffs complex64 [rows][lmax][mmax]
 *                     (zero for m > l, which the inverse transform never reads)
 * and the same on the spectral layout, with the grid-side tensor float32 or bfloat16. */
int sfno_sht_forward_adjoint(const sfno_sht_plan* plan, const void* gcoeffs, float* gx, int64_t rows,
                             void* workspace, size_t workspace_bytes, void* stream);
int sfno_sht_inverse_adjoint(const sfno_sht_plan* plan, const float* gx, void* gcoeffs, int64_t rows,
                             void* workspace, size_t workspace_bytes, void* stream);
int sfno_sht_analysis_adjoint(const sfno_sht_plan* plan, const float* gspec, void* gx, int x_dtype, int64_t rows,
                              void* workspace, size_t workspace_bytes, void* stream);
int sfno_sht_synthesis_adjoint(const sfno_sht_plan* plan, const void* gx, int x_dtype, float* gspec, int64_t rows,
                               void* workspace, size_t workspace_bytes, void* stream);

/* layout passes between the reference coefficient layout and the spectral layout */
/* `triangular` != 0: only entries with m <= l are moved (to_coeffs writes zeros for
 * m > l); 0: the whole lmax x mmax rectangle is moved. */
int sfno_coeffs_to_spectral(const void* coeffs, float* spec, int64_t rows, int lmax, int mmax,
                            int triangular, void* stream);
int sfno_spectral_to_coeffs(const float* spec, void* coeffs, int64_t rows, int lmax, int mmax,
                            int triangular, void* stream);

/* ---- dhconv ------------------------------------------------------------------------ */

/* Packs a SpectralConv weight (complex64 [I][O][L], l fastest: the parameter layout of
 * makani/models/common/spectral_convolution.py:73-102) into the per-degree MFMA operand
 * stream.  Allocates device memory owned by the handle. */
int sfno_dhconv_weights_create(int in_channels, int out_channels, int lmax, int compute,
                               sfno_dhconv_weights** out);
/* (re)fill the packed stream from the current value of the parameter; enqueue only */
int sfno_dhconv_weights_update(sfno_dhconv_weights* w, const void* weight, void* stream);
int sfno_dhconv_weights_destroy(sfno_dhconv_weights* w);
/* Fills a handle created as (out_channels, in_channels, lmax) with the conjugate transpose of the
 * parameter `weight` (complex64 [I][O][L]).  sfno_dhconv_spectral / sfno_dhconv on that handle then
 * map the gradient of the output to the gradient of the input: gx[b,i,l,m] = sum_o gy[b,o,l,m]
 * conj(w[i,o,l]) -- the backward of the einsum at contractions.py:130-136 with respect to `ac`. */
int sfno_dhconv_weights_update_adjoint(sfno_dhconv_weights* w, const void* weight, void* stream);

/* y[b,o,l,m] = sum_i x[b,i,l,m] w[i,o,l] on spectral-layout buffers:
 * spec_in rows = batch*in_channels, spec_out rows = batch*out_channels.  With
 * `triangular` != 0 only m <= l is read and written (coefficients of a forward
 * transform are zero elsewhere).  Replaces _contract_dhconv (contractions.py:130-136). */
int sfno_dhconv_spectral(const sfno_dhconv_weights* w, const float* spec_in, float* spec_out,
                         int batch, int mmax, int triangular, void* stream);

/* Gradient of the contraction with respect to the weight (the einsum's backward with respect to
 * `bc`): gweight[i,o,l] = sum_{b,m} conj(x[b,i,l,m]) gy[b,o,l,m], complex64 [I][O][L] overwritten.
 * spec_in and gspec_out are spectral-layout buffers of batch*I and batch*O rows; `triangular` != 0
 * sums over m <= l only. */
int sfno_dhconv_weight_grad(int in_channels, int out_channels, int lmax, const float* spec_in,
                            const float* gspec_out, void* gweight, int batch, int mmax, int triangular,
                            void* stream);

/* Same contraction on the reference layout: x complex64 [B][I][L][M] -> y complex64
 * [B][O][L][M] (contiguous), as the callable returned by get_contract_fun
 * (factorizations.py:229-232) computes it.  `triangular` as above (then y is zero for
 * m > l, which equals the reference result whenever x is zero there). */
size_t sfno_dhconv_workspace_bytes(const sfno_dhconv_weights* w, int batch, int mmax);
int sfno_dhconv(const sfno_dhconv_weights* w, const void* x, void* y, int batch, int mmax,
                int triangular, void* workspace, size_t workspace_bytes, void* stream);

/* ---- per-degree power (spectral losses) ------------------------------------------------ */

/* power[r][l] = |c[r,l,0]|^2 + 2 sum_{0<m<mmax} |c[r,l,m]|^2 from coefficients in the spectral layout (the output of
 * sfno_sht_analysis): the reduction GeometricH1Loss applies to RealSHT output before it weights the degrees with
 * l(l+1) (makani/utils/losses.py:301-305, 320-331), without the pass to the reference coefficient layout.
 * spec: float [mmax][lmax][sfno_spectral_ld(rows)], power: float [rows][lmax]. */
int sfno_degree_power(const float* spec, float* power, int64_t rows, int lmax, int mmax, void* stream);
/* cotangent of the above in the spectral layout, ready for sfno_sht_analysis_adjoint:
 * gspec[r,l,m] = 2 w_m gpower[r][l] c[r,l,m], w_0 = 1, w_m = 2 otherwise */
int sfno_degree_power_grad(const float* spec, const float* gpower, float* gspec, int64_t rows, int lmax, int mmax,
                           void* stream);

/* ---- "diagonal" operator ------------------------------------------------------------- */

/* y[b,o,l,m] = sum_i x[b,i,l,m] w[i,o,l,m] (makani/models/common/contractions.py:121-127, operator_type
 * "diagonal"): x complex64 [B][I][P], weight complex64 [I][O][P], y complex64 [B][O][P], P = lmax*mmax
 * contiguous.  `adjoint` != 0 computes the input gradient instead: x is then the output gradient
 * [B][O][P] and y[b,i,p] = sum_o x[b,o,p] conj(w[i,o,p]). */
int sfno_diagonal_contract(const void* x, const void* weight, void* y, int batch, int in_channels,
                           int out_channels, int64_t positions, int adjoint, void* stream);
/* gweight[i,o,p] = sum_b conj(x[b,i,p]) gy[b,o,p] */
int sfno_diagonal_weight_grad(const void* x, const void* gy, void* gweight, int batch, int in_channels,
                              int out_channels, int64_t positions, void* stream);

/* ---- pointwise tail of the SFNO block (bf16 activations) -------------------------------- */

/* 1x1 convolution on NCHW bfloat16 activations with a fused epilogue:
 *   y[b][o][p] = act( sum_k w[o][k] x[b][k][p] + bias[o] ) + add_scale[b][o] * addend[b][o][p] + add_shift[b][o]
 * x bf16 [B][K][P], y bf16 [B][O][P] (P = H*W, a multiple of 8); w is the weight packed by
 * sfno_pointwise_pack_weight; bias, addend, add_scale, add_shift may be null.  fp32 accumulation, one
 * rounding at the store.  Replaces nn.Conv2d(kernel_size=1) followed by the activation of EncoderDecoder / MLP
 * (makani/models/common/layers.py:95-116,160-216) and, with `addend`, the "norm1(x) + outer_skip(residual)"
 * and "decoder(x) + residual_transform(residual)" sums (makani/models/networks/sfnonet.py:258-262,636-638). */
int sfno_pointwise_conv(const void* x, const void* w, const float* bias, void* y, int batch, int K, int O,
                        int64_t P, int act, const void* addend, const float* add_scale, const float* add_shift,
                        void* stream);

/* The same convolution over the channel-wise concatenation of two tensors, without building it:
 *   y[b][o][p] = act( sum_{k<K1} w[o][k] x1[b][k][p] + sum_{k<K2} w[o][K1+k] x2[b][k][p] + bias[o] )
 * x1 bf16 [B][K1][P], x2 bf16 [B][K2][P], w packed from a float32 [O][K1+K2] matrix.  No counterpart in the reference, which would run torch.cat and a Conv2d; used where two
 * consecutive linear layers around a sum are merged into one (makani/models/networks/sfnonet.py:258-262 followed by
 * makani/models/common/layers.py:95-116) and where two convolutions feed one sum (decoder output + residual_transform
 * of the input, sfnonet.py:636-638). */
int sfno_pointwise_conv_cat(const void* x1, int K1, const void* x2, int K2, const void* w, const float* bias, void* y,
                            int batch, int O, int64_t P, int act, void* stream);

/* Gradients of that convolution with respect to its parameters, for training through it (what autograd derives for
 * nn.Conv2d(kernel_size=1), makani/models/common/layers.py:95-116,160-216; the reference trains the whole block,
 * makani/models/networks/sfnonet.py:239-267):
 *   gweight[o][k] = sum_{b,p} gy[b][o][p] x[b][k][p],      gbias[o] = sum_{b,p} gy[b][o][p]
 * gy bf16 [B][O][P], x bf16 [B][K][P] (both, and the workspace, 16-byte aligned; P a multiple of 8); gweight float32 [O][K]; gbias float32 [O]
 * or null.  fp32 accumulation in a fixed order (bit-identical from call to call).  `workspace` holds
 * sfno_pointwise_weight_grad_workspace_bytes(batch, K, O, P, gbias != null) bytes.  The gradient with respect to the
 * input is sfno_pointwise_conv itself on gy with the transposed weight ([K][O]) packed. */
size_t sfno_pointwise_weight_grad_workspace_bytes(int batch, int K, int O, int64_t P, int has_bias);
int sfno_pointwise_weight_grad(const void* gy, const void* x, float* gweight, float* gbias, int batch, int K, int O,
                               int64_t P, void* workspace, size_t workspace_bytes, void* stream);

/* Packs a 1x1 convolution weight (float32 [O][K], the nn.Conv2d parameter viewed as a matrix) into the bf16
 * MFMA operand stream sfno_pointwise_conv reads; `packed` holds sfno_pointwise_weight_elems(O, K) bf16 values. */
int64_t sfno_pointwise_weight_elems(int O, int K);
int sfno_pointwise_pack_weight(const float* w, void* packed, int O, int K, void* stream);

/* Instance norm as a per-(b, c) affine: scale = gamma[c] / sqrt(var + eps), shift = beta[c] - mean * scale over
 * the P pixels of each of the `rows` = B*C rows of x (bf16), statistics in fp32 with the biased variance
 * (nn.InstanceNorm2d(affine=True, track_running_stats=False), sfnonet.py:379-386).  gamma/beta may be null. */
size_t sfno_instance_norm_workspace_bytes(int64_t rows, int64_t P);
int sfno_instance_norm_coeffs(const void* x, const float* gamma, const float* beta, float* scale, float* shift,
                              int64_t rows, int channels, int64_t P, float eps, void* workspace,
                              size_t workspace_bytes, void* stream);
/* The coefficients of sfno_instance_norm_coeffs from the per-latitude moments of sfno_sht_synthesis_lat_stats:
 * mean = avg_k a_k, biased variance = avg_k ((a_k - mean)^2 + d_k) over the nlat rows (every row has nlon points). */
int sfno_instance_norm_coeffs_lat(const float* lat_stats, const float* gamma, const float* beta, float* scale, float* shift, int64_t rows,
                                  int channels, int nlat, float eps, void* stream);

/* y = act(scale[row] * x + shift[row]) on bf16 rows of P pixels: the norm0 -> activation step of
 * sfnonet.py:246-251 once the coefficients above are known. */
int sfno_scale_shift_act(const void* x, const float* scale, const float* shift, void* y, int64_t rows, int64_t P,
                         int act, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SFNO_SPECTRAL_H */
