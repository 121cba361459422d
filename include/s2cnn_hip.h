/*
 * C ABI of libs2cnn_hip.so - the MI355X (gfx950) kernels behind the spectral path
 * of spherical CNNs.  Plain pointers and sizes only; every pointer is DEVICE memory
 * unless stated, every tensor is dense fp32, complex numbers are (re, im) pairs.
 *
 * The reference has no C interface: its boundary is Python, and each entry point
 * below replaces one of the run-time compiled CUDA strings (or cuFFT/cuBLAS calls)
 * behind a reference function, cited per entry as file:line under s2cnn/.
 *
 * Conventions
 *   - return value: 0 on success, a negative S2CNN_E* code for rejected arguments,
 *     or a positive hipError_t reported by the launch;
 *   - launches are asynchronous on `stream` (a hipStream_t passed as void*;
 *     NULL = the default stream); nothing synchronises, nothing allocates;
 *   - inputs are never written; outputs are fully overwritten;
 *   - spectral index order is degree-major, then m, then n, with m, n in -l..l:
 *       SO(3): lmn = l(4l^2-1)/3 + (l+m)(2l+1) + (l+n),  nspec(b) = b(4b^2-1)/3
 *       S^2  : lm  = l^2 + l + m,                         nspec(b) = b^2
 *   - grids are [batch, beta, alpha, gamma] (SO(3)) or [batch, beta, alpha] (S^2),
 *     2b samples per axis.
 */
#ifndef S2CNN_HIP_H
#define S2CNN_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define S2CNN_OK 0
#define S2CNN_EINVAL (-1)      /* a size is out of range or inconsistent              */
#define S2CNN_EWORKSPACE (-2)  /* workspace pointer NULL or smaller than required     */
#define S2CNN_EALIGN (-3)      /* a pointer misses the alignment its entry documents   */
                               /* (4, 8 or 16 bytes)                                   */
#define S2CNN_ETOOBIG (-4)     /* needs more scratch than the library's own buffer     */

/* ABI version of this header; bumped when a signature changes. */
int s2cnn_abi_version(void);

/* Human-readable text for a return code of this library (static storage). */
const char *s2cnn_strerror(int code);

/* ---- block-diagonal spectral products on SO(3) ------------------------------------
 * x  [nspec(nl), nbatch, f_in , 2]
 * y  [nspec(nl), f_in  , f_out, 2]
 * z  [nspec(nl), nbatch, f_out, 2]
 *
 * fwd   : z [l,m,n,i,j] = sum_{p,k} x[l,m,p,i,k] * conj(y[l,n,p,k,j])
 *         replaces the forward launch of so3_mm.py:66-93 (kernel so3_mm.py:125-261
 *         with conj_y, trans_y_spec); CPU statement so3_mm.py:31-61.
 * gradx : gx[l,m,p,i,k] = sum_{n,j} gz[l,m,n,i,j] * y[l,n,p,k,j]
 *         replaces so3_mm.py:108-113 (trans_y_feature).
 * grady : gy[l,n,p,k,j] = sum_{m,i} conj(gz[l,m,n,i,j]) * x[l,m,p,i,k]
 *         replaces so3_mm.py:115-120 (trans_out_feature, conj_x, trans_x_spec,
 *         trans_x_feature).
 */
int s2cnn_so3_mm_fwd(const float *x, const float *y, float *z,
                     int nl, int nbatch, int f_in, int f_out, void *stream);
int s2cnn_so3_mm_gradx(const float *gz, const float *y, float *gx,
                       int nl, int nbatch, int f_in, int f_out, void *stream);
int s2cnn_so3_mm_grady(const float *gz, const float *x, float *gy,
                       int nl, int nbatch, int f_in, int f_out, void *stream);

/* ---- the same products for spectra of REAL signals, in the real basis -----------------
 * The spectrum of a real signal on SO(3) obeys X[l,-m,-n] = (-1)^(m-n) conj(X[l,m,n]), and so do the
 * kernel spectrum of so3_ft.py:4-25 (real kernel) and every product and gradient the convolution
 * layer soft/so3_conv.py:36-56 forms from them.  A fixed unitary U_l per degree,
 *     U[0,0] = 1,  U[+m,m] = 1/sqrt2,  U[+m,-m] = (-1)^m/sqrt2,  U[-m,m] = -i/sqrt2,  U[-m,-m] = i(-1)^m/sqrt2
 * (rows r = -l..l stored at l + r), makes every block R = U X U^H real, and  U (X Y^H) U^H = R_x R_y^T:
 * the complex products above become real ones with a quarter of the multiply-adds.  The reference
 * does not exploit this; the entries below have no counterpart there and are used by the convolution
 * layer only, where the symmetry is guaranteed.
 *
 * to_real    : x [nspec(nl), ncols, 2] -> r [nspec(nl), ncols],  r = Re(U x U^H) per column (any x)
 * to_complex : r [nspec(nl), ncols] -> x [nspec(nl), ncols, 2],  x = U^H r U  (inverse on real-signal
 *              spectra, and the adjoint of to_real)
 * mm_real    : x [nspec, nbatch, f_in], y [nspec, f_in, f_out], z [nspec, nbatch, f_out]
 *   fwd   : z [l,m,n,i,j] = sum_{p,k} x [l,m,p,i,k] * y[l,n,p,k,j]
 *   gradx : gx[l,m,p,i,k] = sum_{n,j} gz[l,m,n,i,j] * y[l,n,p,k,j]
 *   grady : gy[l,n,p,k,j] = sum_{m,i} gz[l,m,n,i,j] * x[l,m,p,i,k]
 * Pointers of mm_real need 4-byte alignment only (16-byte and feature counts divisible by 4 for the
 * fast path).
 */
int s2cnn_so3_spectrum_to_real(const float *x, float *r, int nl, long ncols, void *stream);
int s2cnn_so3_spectrum_to_complex(const float *r, float *x, int nl, long ncols, void *stream);
int s2cnn_so3_mm_real_fwd(const float *x, const float *y, float *z,
                          int nl, int nbatch, int f_in, int f_out, void *stream);
int s2cnn_so3_mm_real_gradx(const float *gz, const float *y, float *gx,
                            int nl, int nbatch, int f_in, int f_out, void *stream);
int s2cnn_so3_mm_real_grady(const float *gz, const float *x, float *gy,
                            int nl, int nbatch, int f_in, int f_out, void *stream);

/* ---- kernel spectrum of the SO(3) layer for grids with few distinct beta values ------------
 * The reference computes y[l,m,n] = sum_a x_a conj(D^l_{mn}(alpha_a, beta_a, gamma_a)) as one dense product with a
 * [len(grid), nspec] matrix (so3_ft.py:8-24).  For the grid points A_i that share beta_i,
 * conj D^l_{mn} = d^l_{mn}(beta_i) exp(-i(m alpha_a + n gamma_a)), hence
 *     y[l,m,n] = sum_i d^l_{mn}(beta_i) G_i[m,n],    G_i[m,n] = sum_{a in A_i} x_a exp(-i(m alpha_a + n gamma_a)):
 * a small GEMM (caller's library) for G, then the pass below, linear in the size of y.  Real x only.
 *   G    [nbeta, (2b-1) * b, 2, ncols]   row (m + b-1) * b + n, m in -(b-1)..b-1, n in 0..b-1; (re, im) planes
 *   dtab [nbeta, nspec(b)]               d^l_{mn}(beta_i), degree-major then m then n
 *   y    [nspec(b), ncols]               in the real basis of s2cnn_so3_spectrum_to_real
 * expand_real      : y from G              expand_real_grad : gG from gy (the adjoint)
 * expand           : the same spectrum as complex pairs, y [nspec(b), ncols, 2]: the output of so3_rft (so3_ft.py:24);
 *                    its adjoint is s2cnn_so3_spectrum_to_real followed by expand_real_grad
 * nbeta <= 4, ncols a multiple of 4, G / y / gy / gG 16-byte aligned.
 */
int s2cnn_so3_rft_expand_real(const float *G, const float *dtab, float *y, int b, int nbeta, long ncols, void *stream);
int s2cnn_so3_rft_expand(const float *G, const float *dtab, float *y, int b, int nbeta, long ncols, void *stream);
int s2cnn_so3_rft_expand_real_grad(const float *gy, const float *dtab, float *gG, int b, int nbeta, long ncols, void *stream);

/* ---- S^2 x S^2 -> SO(3) spectral outer products -------------------------------------
 * x  [nl^2, nbatch, f_in , 2]
 * y  [nl^2, f_in  , f_out, 2]
 * z  [nspec_so3(nl), nbatch, f_out, 2]
 *
 * fwd   : z [l,m,n,i,j] = sum_k x[l,m,i,k] * conj(y[l,n,k,j])        s2_mm.py:104-198
 * gradx : gx[l,m,i,k]   = sum_{n,j} gz[l,m,n,i,j] * y[l,n,k,j]       s2_mm.py:201-255
 * grady : gy[l,n,k,j]   = sum_{m,i} conj(gz[l,m,n,i,j]) * x[l,m,i,k] s2_mm.py:258-312
 */
int s2cnn_s2_mm_fwd(const float *x, const float *y, float *z,
                    int nl, int nbatch, int f_in, int f_out, void *stream);
int s2cnn_s2_mm_gradx(const float *gz, const float *y, float *gx,
                      int nl, int nbatch, int f_in, int f_out, void *stream);
int s2cnn_s2_mm_grady(const float *gz, const float *x, float *gy,
                      int nl, int nbatch, int f_in, int f_out, void *stream);

/* ---- the same products for spectra of REAL signals, in the real basis --------------------
 * The S^2 spectrum of a real signal (and of the real kernel of soft/s2_conv.py:47) obeys
 * x[l,-m] = (-1)^m conj(x[l,m]); in the basis of s2cnn_so3_spectrum_to_real it is the real vector
 * (row +m: sqrt2 Re x[l,m], row -m: sqrt2 Im x[l,m], row 0: x[l,0]) and the product above becomes
 *   fwd   : z [l,r,s,i,j] = sum_k x[l,r,i,k] * y[l,s,k,j]
 *   gradx : gx[l,r,i,k]   = sum_{s,j} gz[l,r,s,i,j] * y[l,s,k,j]
 *   grady : gy[l,s,k,j]   = sum_{r,i} gz[l,r,s,i,j] * x[l,r,i,k]
 * with x [nl^2, nbatch, f_in], y [nl^2, f_in, f_out], z [nspec_so3(nl), nbatch, f_out] (one float per entry):
 * z is the real-basis SO(3) spectrum that s2cnn_so3_synthesis_real_basis takes.  Replaces s2_mm inside
 * S2Convolution (soft/s2_conv.py:45-53) at half the bytes; the reference has no such step.
 */
int s2cnn_s2_mm_real_fwd(const float *x, const float *y, float *z,
                         int nl, int nbatch, int f_in, int f_out, void *stream);
int s2cnn_s2_mm_real_gradx(const float *gz, const float *y, float *gx,
                           int nl, int nbatch, int f_in, int f_out, void *stream);
int s2cnn_s2_mm_real_grady(const float *gz, const float *x, float *gy,
                           int nl, int nbatch, int f_in, int f_out, void *stream);

/* ---- SO(3) Fourier analysis: grid -> spectrum --------------------------------------
 * x     [nbatch, 2b_in, 2b_in, 2b_in]      (complex_in = 0)
 *       [nbatch, 2b_in, 2b_in, 2b_in, 2]   (complex_in = 1)
 * table [2b_in, nspec(b_out)]  row beta_j, entries scale * d^l_{mn}(beta_j); must satisfy
 *       table[j, l,-m,-n] = (-1)^(m-n) table[j, l,m,n] (true of Wigner small-d)
 *       and, for real input on the 64^3 grid (b_in = 32), table[2b-1-j, l,m,n] = (-1)^(l-n) table[j, l,-m,n]
 *       (true of Wigner small-d on the SOFT grid, whose weights are symmetric in j); x then needs
 *       16-byte alignment
 * packed_table  NULL, or the same table repacked once by s2cnn_so3_pack_table(..., synthesis = 0)
 *       (skips a per-call repack on the fast path; ignored where the fast path does not apply)
 * out   [nspec(b_out), nbatch, 2]
 *       out[l,m,n,z] = sum_beta table[beta,lmn] sum_{alpha,gamma} x[z,beta,alpha,gamma]
 *                      exp(-i(m alpha + n gamma)),   0 where |m| or |n| >= b_in
 * Replaces cuFFT + the kernel at soft/so3_fft.py:247-350 behind so3_rfft (so3_fft.py:64-112)
 * and so3_fft (so3_fft.py:12-61).
 * workspace: s2cnn_so3_analysis_workspace(...) bytes of device scratch, 256-byte aligned.
 */
size_t s2cnn_so3_analysis_workspace(int b_in, int b_out, long nbatch, int complex_in);
int s2cnn_so3_analysis(const float *x, const float *table, const float *packed_table, float *out,
                       void *workspace, size_t workspace_bytes,
                       int b_in, int b_out, long nbatch, int complex_in, void *stream);

/* ---- the analysis above without a workspace argument ---------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the same transform as s2cnn_so3_analysis
 * with its scratch in a buffer that the library itself holds, S2CNN_STATIC_SCRATCH_BYTES per GPU from the
 * moment the library is loaded until the process ends.  Calls nothing that allocates.
 *   - sizes whose s2cnn_so3_analysis_workspace(...) exceeds S2CNN_STATIC_SCRATCH_BYTES are rejected with
 *     S2CNN_ETOOBIG (real signals on the 64^3 grid: up to 276 volumes per call);
 *   - all calls on one GPU share that GPU's buffer: calls that overlap in time on one GPU (different
 *     streams or threads) race; calls on one stream are ordered and safe;
 *   - the first call on a GPU resolves the buffer's address for it (no allocation; make it outside a graph capture);
 *   - results are those of s2cnn_so3_analysis bit for bit.
 */
#define S2CNN_STATIC_SCRATCH_BYTES (64u << 20)
int s2cnn_so3_analysis_static(const float *x, const float *table, const float *packed_table, float *out,
                              int b_in, int b_out, long nbatch, int complex_in, void *stream);

/* ---- SO(3) Fourier synthesis: spectrum -> grid -------------------------------------
 * xhat  [nspec(b_in), nbatch, 2]
 * table [2b_out, nspec(b_in)]   (same symmetry requirement as above)
 * packed_table  NULL, or s2cnn_so3_pack_table(table, ..., synthesis = 1) of the same table
 * out   [nbatch, 2b_out, 2b_out, 2b_out]     (complex_out = 0): the REAL PART of
 *       [nbatch, 2b_out, 2b_out, 2b_out, 2]  (complex_out = 1):
 *       y[z,beta,alpha,gamma] = sum_{l < min(b_in,b_out)} sum_{m,n} xhat[l,m,n,z]
 *                               table[beta,lmn] exp(+i(m alpha + n gamma))
 * (no symmetry of xhat is assumed in either mode).
 * Replaces the kernel at soft/so3_fft.py:353-443 + cuFFT behind so3_rifft
 * (so3_fft.py:158-202, CPU-branch semantics) and so3_ifft (so3_fft.py:115-155).
 */
size_t s2cnn_so3_synthesis_workspace(int b_in, int b_out, long nbatch, int complex_out);
int s2cnn_so3_synthesis(const float *xhat, const float *table, const float *packed_table, float *out,
                        void *workspace, size_t workspace_bytes,
                        int b_in, int b_out, long nbatch, int complex_out, void *stream);
/* The same with complex_out = 0 and a bias in the epilogue: bias has nfeature values and, with the batch laid
 * out [..., nfeature] (nbatch a multiple of nfeature), bias[z % nfeature] is added to every sample of volume z.
 * Replaces SO3_ifft_real followed by "z + self.bias" (soft/s2_conv.py:50-53, soft/so3_conv.py:54-56) without
 * the extra pass over the output.  bias = NULL gives s2cnn_so3_synthesis(..., complex_out = 0, ...).
 */
int s2cnn_so3_synthesis_real_bias(const float *xhat, const float *table, const float *packed_table, float *out,
                                  void *workspace, size_t workspace_bytes,
                                  int b_in, int b_out, long nbatch,
                                  const float *bias, int nfeature, void *stream);
/* Bias (may be NULL) and max(., 0) in the epilogue: out = relu(synthesis(xhat) + bias).  real_basis = 0: xhat as
 * above; 1: the spectrum in the real basis, one float per entry (only where
 * s2cnn_so3_real_basis_transform_available(b_in, b_out, 1)).  Replaces F.relu applied to the output of a
 * convolution layer (examples/mnist/run.py:88-92) without its pass over the
 * activations.
 */
int s2cnn_so3_synthesis_real_relu(const float *xhat, const float *table, const float *packed_table, float *out,
                                  void *workspace, size_t workspace_bytes,
                                  int b_in, int b_out, long nbatch,
                                  const float *bias, int nfeature, int real_basis, void *stream);
/* The adjoint side of it: analysis of the real signal that equals x where mask > 0 and 0 elsewhere (mask: a
 * tensor of the shape of x, here the OUTPUT of the relu above, so that x * [mask > 0] is the gradient that
 * autograd would pass through it).  Workspace and tables as for s2cnn_so3_analysis with complex_in = 0;
 * real_basis = 1 writes the real-basis spectrum [nspec(b_out), nbatch] (only where
 * s2cnn_so3_real_basis_transform_available(b_in, b_out, 0)).
 */
int s2cnn_so3_analysis_real_masked(const float *x, const float *mask, const float *table, const float *packed_table,
                                   float *out, void *workspace, size_t workspace_bytes,
                                   int b_in, int b_out, long nbatch, int real_basis, void *stream);

/* The same pair with the mask as ONE BIT per sample (real signals on the 64^3 grid only: where
 * s2cnn_so3_relu_bits_bytes(b_grid, nbatch) is not 0).  The synthesis writes, beside `out`, bit = "out is not <= 0" for
 * every sample ([nbatch][beta][alpha % 8][alpha / 8] 64-bit words, bit = gamma; 32 KiB per volume, 16-byte aligned); the
 * masked analysis reads those bits instead of a tensor of the shape of x: a thirty-second of the mask traffic of the
 * backward pass, and the saved state of the activation shrinks by the same factor.  Results are those of the pair above
 * bit for bit.  No counterpart in the reference (its models call F.relu on the layer's output, examples/mnist/run.py:88-92).
 */
size_t s2cnn_so3_relu_bits_bytes(int b_grid, long nbatch);
int s2cnn_so3_synthesis_real_relu_bits(const float *xhat, const float *table, const float *packed_table, float *out,
                                       void *bits, void *workspace, size_t workspace_bytes,
                                       int b_in, int b_out, long nbatch,
                                       const float *bias, int nfeature, int real_basis, void *stream);
int s2cnn_so3_analysis_real_masked_bits(const float *x, const void *bits, const float *table, const float *packed_table,
                                        float *out, void *workspace, size_t workspace_bytes,
                                        int b_in, int b_out, long nbatch, int real_basis, void *stream);

/* ---- batch normalisation and max(., 0) between two layers, inside the transforms --------
 * The reference's shape networks put nn.BatchNorm3d and nn.ReLU between their layers (examples/shrec17/model.py:28-35,
 * model_original.py:28-35): three passes over the activations forward and five backward.  Here the next layer's analysis
 * applies the normalisation and the activation as it loads the previous layer's output y, and the backward analysis of
 * the previous layer forms the gradient with respect to y as it loads the incoming gradient:
 *   s2cnn_volume_moments            out[z] = (sum y, sum (y - mean_z)^2), mean_z the mean of the volume, for each of the nvol
 *                                   volumes of n samples (squares summed around a pivot and moved to the mean in float64: a
 *                                   mean far above the spread costs no digits); s2cnn_bn_forward_from_moments merges the
 *                                   volumes of a feature into its batch statistics
 *   s2cnn_so3_analysis_real_affine_relu     the analysis of max(a y + b, 0), a = params[z % nfeature],
 *                                   b = params[nfeature + z % nfeature]  (a = weight / sqrt(var + eps), b = bias - mean a)
 *   s2cnn_bn_relu_grad_moments      out[z] = (sum g m, sum g m y), m = (a y + b > 0): the two reductions of the backward
 *                                   pass of the normalisation (g: gradient with respect to the activation)
 *   s2cnn_so3_analysis_real_bn_relu_grad    the analysis of a (m ? g : 0) + p + q y, params [4][nfeature] = a, b, p, q:
 *                                   the gradient with respect to y (p, q from the reductions; p = q = 0 with fixed statistics)
 * x / g / y: [nbatch, 2b_in, 2b_in, 2b_in], 16-byte aligned on the 64^3 grid; other arguments as s2cnn_so3_analysis
 * (real_basis = 1 only where s2cnn_so3_real_basis_transform_available says so).  Available where
 * s2cnn_so3_analysis_prologue_available(b_in, b_out) returns 1: the 64^3 grid with b_out <= 32 and every other grid whose
 * planes fit the LDS; elsewhere S2CNN_EINVAL (apply the function with a pass of its own, then s2cnn_so3_analysis).
 * nbatch must be a multiple of nfeature.  No counterpart in the reference.
 */
int s2cnn_so3_analysis_prologue_available(int b_in, int b_out);
/* the same function in the loads of the integral that ends the reference's networks (examples/shrec17/model.py:44-45 after
 * the last BatchNorm3d + ReLU): out[z] = s2cnn_so3_integrate of max(a x + b, 0), params [2][nfeature] as above, any grid */
int s2cnn_so3_integrate_affine_relu(const float *x, const float *params, int nfeature, const float *w, float *out,
                                    int b, long n, void *stream);
int s2cnn_volume_moments(const float *x, float *out, long nvol, long n, void *stream);
int s2cnn_bn_relu_grad_moments(const float *g, const float *y, const float *params, int nfeature, float *out,
                               long nvol, long n, void *stream);
/* Where the synthesis that produces y (or the gradient g) stages whole planes in LDS it can form those sums itself, one
 * pair per plane, and the separate read is not needed; the per-volume kernels of the 44^3, 32^3 and 20^3 grids (b_out = 22,
 * 16, 10) form one pair per volume.  s2cnn_so3_synthesis_moment_parts(b_in, b_out) = pairs per volume (2 b_out, or 1 on those grids) where
 * s2cnn_so3_synthesis_real_moments can do that (real signals, complex spectrum; other arguments as
 * s2cnn_so3_synthesis_real_bias; with yref: no bias on those three grids), else 0.  moments [nbatch][pairs][2]; yref = NULL:
 * (sum y, sum (y - mean of the part)^2) of the output; yref = the tensor y and params = ab: (sum g m, sum g m y) with the
 * output as g. */
int s2cnn_so3_synthesis_moment_parts(int b_in, int b_out);
int s2cnn_so3_synthesis_real_moments(const float *xhat, const float *table, const float *packed_table, float *out,
                                     void *workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch,
                                     const float *bias, int nfeature, float *moments, const float *yref,
                                     const float *params, void *stream);
/* The same with the spectrum in the real basis (other arguments as s2cnn_so3_synthesis_real_basis), and also on the 64^3
 * grid, whose per-volume kernel forms the sums over the volume it writes: one pair per volume (with yref: no bias, and
 * on the 64^3 grid spectra of at most 28 degrees, for which the kernel has registers to spare).
 * s2cnn_so3_synthesis_real_basis_moment_parts(b_in, b_out, grad = whether yref is given) = pairs per volume (1 on the
 * 64^3, 44^3, 32^3 and 20^3 grids, 2 b_out elsewhere) where it can, else 0 (and the entry point returns -1); moments [nbatch][pairs][2]. */
int s2cnn_so3_synthesis_real_basis_moment_parts(int b_in, int b_out, int grad);
int s2cnn_so3_synthesis_real_basis_moments(const float *r, const float *table, const float *packed_table, float *out,
                                           void *workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch,
                                           const float *bias, int nfeature, float *moments, const float *yref,
                                           const float *params, void *stream);
/* the arithmetic between those calls, one small launch each instead of a chain of tensor operations (float64 inside):
 * forward : moments [batch][nfeature][parts][2] (parts = 1 from s2cnn_volume_moments, 2 b from the synthesis above; per
 *           part the sum and the squared deviations from the part's own mean, all parts of equal size),
 *           count = samples per feature -> ab [2][nfeature] for the
 *           analysis, stats [4][nfeature] = batch mean, biased batch variance, mean in use, 1/sqrt(var in use + eps)
 *           (in use: the batch's when training != 0, else running_mean / running_var); when training and the running
 *           buffers are given they move by `momentum` (unbiased variance), as nn.BatchNorm3d does; weight, bias: NULL = 1, 0
 * backward: moments of s2cnn_bn_relu_grad_moments -> params [4][nfeature] for s2cnn_so3_analysis_real_bn_relu_grad and
 *           gwb [2][nfeature] = the gradients of weight and bias */
int s2cnn_bn_forward_from_moments(const float *moments, int batch, int nfeature, int parts, double count, const float *weight,
                                  const float *bias, float *running_mean, float *running_var, double eps, double momentum,
                                  int training, float *ab, float *stats, void *stream);
int s2cnn_bn_backward_from_moments(const float *moments, int batch, int nfeature, int parts, double count, const float *ab,
                                   const float *stats, int training, float *params, float *gwb, void *stream);
int s2cnn_so3_analysis_real_affine_relu(const float *x, const float *params, int nfeature,
                                        const float *table, const float *packed_table, float *out,
                                        void *workspace, size_t workspace_bytes,
                                        int b_in, int b_out, long nbatch, int real_basis, void *stream);
int s2cnn_so3_analysis_real_bn_relu_grad(const float *g, const float *y, const float *params, int nfeature,
                                         const float *table, const float *packed_table, float *out,
                                         void *workspace, size_t workspace_bytes,
                                         int b_in, int b_out, long nbatch, int real_basis, void *stream);

/* ---- table repacking for the real-signal fast path of the two transforms above ------
 * The reference uploads its Wigner table once per (b, nl, weighted, device) and reuses it
 * (soft/so3_fft.py:205-209); a caller of this library does the same with the packed copy:
 *   bytes = s2cnn_so3_packed_table_bytes(b_in, b_out, synthesis)   (0: no fast path for these sizes)
 *   s2cnn_so3_pack_table(table, packed, b_in, b_out, synthesis, stream)
 * b_in / b_out have the meaning they have in the transform the table is for; `packed` must be
 * 16-byte aligned.  Passing packed_table = NULL to a transform is always valid (it repacks into
 * its workspace on every call).
 */
size_t s2cnn_so3_packed_table_bytes(int b_in, int b_out, int synthesis);
int s2cnn_so3_pack_table(const float *table, float *packed, int b_in, int b_out, int synthesis, void *stream);

/* ---- the two transforms with the spectrum in the real basis ------------------------------
 * For real signals the spectrum side of the transforms above can be read or written directly in the
 * real basis of s2cnn_so3_spectrum_to_real (one float per entry):
 *   analysis_real_basis (x)  = spectrum_to_real(analysis(x))          out [nspec(b_out), nbatch]
 *   synthesis_real_basis(r)  = synthesis(spectrum_to_complex(r))      r   [nspec(b_in),  nbatch]
 * which saves the conversion pass and half of the spectrum traffic inside the convolution layer
 * (soft/so3_conv.py:36-56 has no such step: the reference keeps complex spectra throughout).
 * Available where s2cnn_so3_real_basis_transform_available(b_in, b_out, synthesis) returns 1
 * (wherever s2cnn_so3_packed_table_bytes is not 0, for the analysis with b_out <= 32 as well;
 * S2CNN_EINVAL otherwise: compose the two calls instead).
 * Tables, packed tables and workspace exactly as for s2cnn_so3_analysis / s2cnn_so3_synthesis with
 * complex_in / complex_out = 0.
 * bias: NULL, or nfeature values; with the batch laid out [..., nfeature] (nbatch a multiple of nfeature),
 *       bias[z % nfeature] is added to every sample of volume z: the "+ self.bias" of soft/so3_conv.py:56
 *       in the epilogue of the transform instead of a pass of its own.
 */
int s2cnn_so3_real_basis_transform_available(int b_in, int b_out, int synthesis);
int s2cnn_so3_analysis_real_basis(const float *x, const float *table, const float *packed_table, float *out,
                                  void *workspace, size_t workspace_bytes,
                                  int b_in, int b_out, long nbatch, void *stream);
int s2cnn_so3_synthesis_real_basis(const float *r, const float *table, const float *packed_table, float *out,
                                   void *workspace, size_t workspace_bytes,
                                   int b_in, int b_out, long nbatch,
                                   const float *bias, int nfeature, void *stream);

/* ---- S^2 Fourier analysis / synthesis ----------------------------------------------
 * analysis : x [nbatch, 2b_in, 2b_in] (complex_in = 0) or [..., 2] (complex_in = 1),
 *            table [2b_in, b_out^2] (entries scale * d^l_{m0}), b_out <= b_in,
 *            out [b_out^2, nbatch, 2]:
 *            out[l,m,z] = sum_beta table[beta,lm] sum_alpha x[z,beta,alpha] exp(-i m alpha)
 *            replaces cuFFT + soft/s2_fft.py:150-185 behind s2_fft (s2_fft.py:13-58).
 * synthesis: xhat [b_in^2, nbatch, 2], table [2b_out, b_in^2], b_out >= b_in,
 *            out [nbatch, 2b_out, 2b_out] (real part, complex_out = 0) or [..., 2]:
 *            y[z,beta,alpha] = sum_{l,m} xhat[l,m,z] table[beta,lm] exp(+i m alpha)
 *            replaces soft/s2_fft.py:188-223 + cuFFT behind s2_ifft (s2_fft.py:61-106).
 */
size_t s2cnn_s2_analysis_workspace(int b_in, int b_out, long nbatch, int complex_in);
int s2cnn_s2_analysis(const float *x, const float *table, float *out,
                      void *workspace, size_t workspace_bytes,
                      int b_in, int b_out, long nbatch, int complex_in, void *stream);
size_t s2cnn_s2_synthesis_workspace(int b_in, int b_out, long nbatch, int complex_out);
int s2cnn_s2_synthesis(const float *xhat, const float *table, float *out,
                       void *workspace, size_t workspace_bytes,
                       int b_in, int b_out, long nbatch, int complex_out, void *stream);

/* ---- Haar integral over SO(3) -------------------------------------------------------
 * x [n, 2b, 2b, 2b], w [2b] -> out [n]:  out[z] = sum_beta w[beta] sum_{alpha,gamma} x[z,...]
 * replaces the two torch.sum + torch.mm of soft/so3_integrate.py:21-27.
 * grad : gx[z,beta,alpha,gamma] = g[z] * w[beta]   (its adjoint)
 */
int s2cnn_so3_integrate(const float *x, const float *w, float *out, int b, long n, void *stream);
int s2cnn_so3_integrate_grad(const float *g, const float *w, float *gx, int b, long n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* S2CNN_HIP_H */
