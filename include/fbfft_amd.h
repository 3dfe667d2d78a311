/*
 * fbfft_amd.h - C ABI of the MI355X (gfx950) implementation of fbcuda's fbfft path.
 *
 * Every entry point takes plain pointers, sizes and strides; no C++ or torch
 * types cross this boundary.  All work is enqueued on the caller's HIP stream
 * and nothing is synchronised.  Buffers (including scratch for the two-call
 * 64/128 forms and the device arrays of tile descriptors) are owned by the
 * caller.  The library keeps no mutable global state.
 *
 * File:line citations name the reference interface each declaration replaces
 * (paths relative to the fbcuda source tree).
 */
#ifndef FBFFT_AMD_H
#define FBFFT_AMD_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* hipStream_t is "struct ihipStream_t*"; declared here so that C callers do not
 * need the HIP headers. */
struct ihipStream_t;
typedef struct ihipStream_t* fbfft_stream_t;

/* FBFFTParameters::ErrorCode (fbfft/FBFFTParameters.h:9-14).  HipError takes the
 * place of CudaError.  Invariant violations that abort in the reference (glog
 * CHECK / assert) are reported as UnsupportedDimension or UnsupportedSize. */
enum fbfft_error {
  FBFFT_SUCCESS = 0,
  FBFFT_UNSUPPORTED_SIZE = 1,
  FBFFT_UNSUPPORTED_DIMENSION = 2,
  FBFFT_HIP_ERROR = 3
};

/* A non-owning strided view: the contents of DeviceTensor<float, dim>
 * (DeviceTensor.cuh:237-245: data pointer, then strides, then sizes), strides
 * in units of float.  Complex tensors are float tensors whose innermost
 * dimension has size 2 and stride 1. */
#define FBFFT_MAX_DIM 5
typedef struct fbfft_tensor {
  float* data;
  int stride[FBFFT_MAX_DIM];
  int size[FBFFT_MAX_DIM];
  int dim;
} fbfft_tensor;

/* TiledDeviceTensor<float, 4> (fbfft/FFTIteratedConvolution.cuh:71-88): 48 bytes,
 * layout-compatible with the reference so existing host code that builds and
 * uploads the descriptor arrays keeps working. */
typedef struct fbfft_tile {
  int padL;
  int padU;
  float* data;
  int stride[4];
  int size[4];
} fbfft_tile;

/* FFTConvolutionPassFFI (fbfft/FFTIteratedConvolution.cuh:616-622) */
enum fbfft_conv_pass {
  FBFFT_UPDATE_OUTPUT = 0,
  FBFFT_UPDATE_GRAD_INPUT = 1,
  FBFFT_ACC_GRAD_PARAMETERS = 2
};

/* fbfft1D<1> (fbfft/FBFFT.cuh:11-16, fbfft/FBFFT-inl.cuh:19-87).
 * real [B][N] -> cplx [B][N/2+1][2], N = real->size[1], a power of two in
 * [2, 256].  padL shifts the row right and drops its last padL samples. */
int fbfft_r2c_1d(const fbfft_tensor* real, const fbfft_tensor* cplx, int padL,
                 fbfft_stream_t stream);

/* fbifft1D<1> (fbfft/FBFFT.cuh:18-23, fbfft/FBFFT-inl.cuh:89-150).
 * cplx [B][N/2+1][2] -> real [B][N], unnormalised (gain N). */
int fbfft_c2r_1d(const fbfft_tensor* real, const fbfft_tensor* cplx, int padL,
                 fbfft_stream_t stream);

/* fbfft2D<1>(real, complexAsFloat, padL, padU) (fbfft/FBFFT.cuh:30-36,
 * fbfft/FBFFT2D-inl.cuh:450-623).
 * real [B][h][w] is placed at (padU, padL) of a zero N x N plane (h = 0 or w = 0
 * with B > 0: the spectra are written as zeros).
 *   cplx [B][N/2+1][N][2], N in {8,16,32}:  cplx[b][ky][kx]  (one kernel)
 *   cplx [B][N/2+1][N][2], N in {64,128}:   cplx[b][kx][ky]  (one kernel; an
 *       extension: the reference needs two calls and a scratch buffer)
 *   cplx [B][N][N/2+1][2], N in {64,128}:   the reference's first pass: row
 *       transforms into the caller's scratch, cplx[b][y][kx].
 *   cplx [B][N/2][N][2],   N in {8,16,32}:  the packed format (Unpack = false,
 *       fbfft/FFT2D32.cuh:421-427): rows 1 .. N/2-1 as above, row 0 holds
 *       F[0][kx] + i F[N/2][kx] (both spectra are those of real rows). */
int fbfft_r2c_2d(const fbfft_tensor* real, const fbfft_tensor* cplx, int padL, int padU,
                 fbfft_stream_t stream);

/* fbfft2D<1>(Complex src, Complex dst) (fbfft/FBFFT.cuh:39-43,
 * fbfft/FBFFT2D-inl.cuh:627-669): second pass for N in {64,128}.
 * src [B][N][N/2+1][2] (scratch) -> dst [B][N/2+1][N][2], dst[b][kx][ky]. */
int fbfft_c2c_2d_pass2(const fbfft_tensor* src, const fbfft_tensor* dst, fbfft_stream_t stream);

/* fbifft2D<1>(Complex src, real dst, padL, padU) (fbfft/FBFFT.cuh:50-56,
 * fbfft/FBIFFT2D-inl.cuh:567-742).  Unnormalised (gain N*N); only the window of
 * the N x N result that real covers at (padU, padL) is written.
 *   cplx [B][N/2+1][N][2], N in {8,16,32}:  one kernel
 *   cplx [B][N/2+1][N][2], N in {64,128}:   one kernel (extension, as above)
 *   cplx [B][N][N][2],     N in {64,128}:   the reference's second inverse pass
 *       over the scratch produced by fbfft_c2c_2d_inverse_pass1.
 *   cplx [B][N/2][N][2],   N in {8,16,32}:  packed input (PackedInput = true,
 *       fbfft/FFT2D32.cuh:302-316). */
int fbfft_c2r_2d(const fbfft_tensor* cplx, const fbfft_tensor* real, int padL, int padU,
                 fbfft_stream_t stream);

/* fbifft2D<1>(float src, float dst) (fbfft/FBFFT.cuh:45-49,
 * fbfft/FBIFFT2D-inl.cuh:529-563): first inverse pass for N in {64,128}.
 * src [B][N/2+1][N][2] -> dst [B][N][N][2] scratch; planes b and b + ceil(B/2)
 * share one complex transform, so only the first ceil(B/2) planes of dst are
 * written. */
int fbfft_c2c_2d_inverse_pass1(const fbfft_tensor* src, const fbfft_tensor* dst,
                               fbfft_stream_t stream);

/* transposeMM<Dim, ConjugateTransposeA, ConjugateTransposeB, Accumulate>
 * (MM.cuh:11-17, MM-inl.cuh:515-814).  Operands are float tensors of rank 3..5
 * whose last dimension is the (re, im) pair and whose dimensions between the
 * first two and the last are contiguous and collapse to xy:
 *   A [I][K][xy][2] (conjA: [K][I][xy][2]),  B [K][J][xy][2] (conjB: [J][K][xy][2])
 *   C[i][j][xy] = invNorm * ((accumulate ? C[i][j][xy] : 0) + sum_k opA * opB)
 * where opX conjugates when conjX is set.  Returns an fbfft_error (the
 * reference returns void and aborts on bad shapes). */
int fbfft_transpose_mm(const fbfft_tensor* A, const fbfft_tensor* B, const fbfft_tensor* C,
                       int conjA, int conjB, int accumulate, float invNorm,
                       fbfft_stream_t stream);

/* The same contraction on PACKED spectra: A, B, C are rank-5 tensors
 * [d0][d1][N/2][N][2], N in {8,16,32}, as fbfft_r2c_2d stores them when cplx has
 * N/2 rows (the Unpack = false format of fbfft/FFT2D32.cuh:421-427): rows
 * 1 .. N/2-1 are plain bins; row 0 holds P[x] = F[0][x] + i F[N/2][x] and follows
 * the product rule of the fused kernels (fbfft/FFTIteratedConvolution.cuh:161-186,
 * :485-504): both operands are unpacked, rows 0 and N/2 are multiplied
 * separately, and the result is packed again, so that C can go straight into
 * fbfft_c2r_2d in its packed form (fbfft2DVerticalCoreInverse<N, true>,
 * fbfft/FFT2D32.cuh:302-316).  The reference declares the format but ships no
 * contraction for it ("If a specialized gemm kernel is available, no need to
 * unpack", FFT2D32.cuh:422). */
int fbfft_transpose_mm_packed(const fbfft_tensor* A, const fbfft_tensor* B, const fbfft_tensor* C,
                              int conjA, int conjB, int accumulate, float invNorm,
                              fbfft_stream_t stream);

/* detail::FFTIteratedConvolution<FFTSize> (fbfft/FFTIteratedConvolution.cuh:624-755).
 * ins / outs are DEVICE pointers to numTiles descriptors each.  weight is
 * [Cout][Cin][kH][kW].  Returns 1 if a kernel was launched, 0 if the pass code or
 * FFT size matched nothing (the reference's bool) or the filter is larger than
 * the transform (kH or kW > fftSize), and a negative fbfft_error
 * (-FBFFT_HIP_ERROR ...) on launch failure.  FBFFT_ACC_GRAD_PARAMETERS overwrites
 * weight with scale * gradient; partial sums of several workgroups meet in atomic
 * adds, so its last bits can differ from run to run. */
int fbfft_iterated_conv(int fftSize, const fbfft_tile* ins, const fbfft_tile* outs,
                        const fbfft_tensor* weight, int pass, float scale, int batchSize,
                        size_t numTiles, fbfft_stream_t stream);

/* The same with flags.  FBFFT_DETERMINISTIC: FBFFT_ACC_GRAD_PARAMETERS runs the
 * reference's schedule - one workgroup per group of weight planes walks the whole
 * (tile, image) reduction in a fixed order (fbfft/FFTIteratedConvolution.cuh:
 * 600-613), no atomic adds - so the result is bit-for-bit reproducible from run to
 * run, at the price of leaving most of the chip idle (configs[4]: 10.5 ms instead of
 * 0.63 ms).  fbfft_conv_accgrad on the whole image is both reproducible and fast; it
 * needs a workspace.  The other passes are reproducible either way.  Unknown flag
 * bits return 0. */
#define FBFFT_DETERMINISTIC 1u
int fbfft_iterated_conv_ex(int fftSize, const fbfft_tile* ins, const fbfft_tile* outs,
                           const fbfft_tensor* weight, int pass, float scale, int batchSize,
                           size_t numTiles, unsigned flags, fbfft_stream_t stream);

/* detail::FFTIteratedConvolution<FFTSize> (fbfft/FFTIteratedConvolution.cuh:624-755) for
 * callers that can lend a workspace: the same operands - device arrays of tile
 * descriptors, any tiling - and the same results as fbfft_iterated_conv (to rounding;
 * the three passes of its table: outs[t] = sum_c ins[t] (*) weight, ins[t] = sum_f
 * outs[t] (*) weight, weight = scale * sum_(t, n) ins[t] (*) outs[t]), computed by the
 * three kernels of the convolution layer entry points instead of the fused kernel: each
 * filter plane is transformed once per call rather than once per tile and image group,
 * and the per-frequency products run on the matrix cores (configs[4]: 0.29 ms against
 * 0.62 ms).  The weight gradient is reproducible bit for bit from run to run.
 * workspace: device memory of fbfft_iterated_conv_workspace(fftSize, pass, batchSize,
 * numTiles, cin, cout) bytes, 256-byte aligned; contents need not survive.  Returns as
 * fbfft_iterated_conv: 1 launched, 0 nothing matched (pass, fftSize in {8, 16, 32},
 * filter larger than the transform), a negative fbfft_error on a workspace that is
 * missing, misaligned or too small (-FBFFT_UNSUPPORTED_DIMENSION) or a launch failure.
 * Tiles are read on the device only; a tile whose view does not hold an image or plane
 * (size[0] < batchSize, fewer planes than the filter) contributes zeros, as in the
 * fused kernel. */
size_t fbfft_iterated_conv_workspace(int fftSize, int pass, int batchSize, size_t numTiles,
                                     int cin, int cout);
int fbfft_iterated_conv_ws(int fftSize, const fbfft_tile* ins, const fbfft_tile* outs,
                           const fbfft_tensor* weight, int pass, float scale, int batchSize,
                           size_t numTiles, void* workspace, size_t workspaceBytes,
                           fbfft_stream_t stream);

/* Host-side builder of the tile descriptors FFTIteratedConvolution consumes; the
 * reference leaves this to its external caller (fbfft/FFTIteratedConvolution.cuh:
 * 71-88 declares the descriptor, :113-114 consumes ins[tile] / outs[tile]).
 * input is [B][Cin][H][W] and output [B][Cout][H-kH+1][W-kW+1] (device tensors;
 * only their addresses and strides are used).  Tile t covers the output window
 * whose origin advances by fftSize-kH+1 rows / fftSize-kW+1 columns, clipped at
 * the edges, and the fftSize x fftSize (clipped) input window at the same
 * origin; padL = padU = 0.  Row-major over (tileY, tileX).  Writes at most
 * capacity descriptors into the HOST arrays ins / outs, which the caller then
 * copies to the device, and returns the number of tiles of the grid; with
 * ins == NULL or outs == NULL it only returns that number.  0 = unsupported
 * arguments.  This grid serves FBFFT_UPDATE_OUTPUT and FBFFT_ACC_GRAD_PARAMETERS.
 * It does NOT serve FBFFT_UPDATE_GRAD_INPUT: that pass stores (does not add)
 * each tile's result into ins[tile], and these input windows overlap by kH-1
 * rows and kW-1 columns. */
size_t fbfft_make_tiles(const fbfft_tensor* input, const fbfft_tensor* output, int kH, int kW,
                        int fftSize, fbfft_tile* ins, fbfft_tile* outs, size_t capacity);

/* The same builder for a named pass.  pass = FBFFT_UPDATE_OUTPUT or
 * FBFFT_ACC_GRAD_PARAMETERS gives the grid of fbfft_make_tiles.
 * pass = FBFFT_UPDATE_GRAD_INPUT (input = gradInput, output = gradOutput) cuts
 * gradInput into DISJOINT windows of (fftSize-kH+1) x (fftSize-kW+1), clipped at
 * the edges, with padU = kH-1 and padL = kW-1, each paired with the gradOutput
 * window of up to fftSize x fftSize that starts kH-1 rows above and kW-1 columns
 * left of it (clipped at the tensor's edges; the clipped-off rows and columns
 * become its padU / padL), so that every gradInput element is written by exactly
 * one tile.  The tile count can differ from the other passes' count. */
size_t fbfft_make_tiles_for_pass(int pass, const fbfft_tensor* input, const fbfft_tensor* output,
                                 int kH, int kW, int fftSize, fbfft_tile* ins, fbfft_tile* outs,
                                 size_t capacity);

/* FFT convolution layer on the split path: the FFT -> transposeMM -> IFFT
 * sequences that the reference's external callers compose from the primitives
 * above, one entry point per pass of the role table at MM-inl.cuh:188-196.
 * Shapes throughout: input / gradInput [B][Cin][H][W], weight / gradWeight
 * [Cout][Cin][kH][kW], output / gradOutput [B][Cout][H-kH+1][W-kW+1], fftSize in
 * {8,16,32,64,128}, kH, kW <= fftSize.  Valid cross-correlation, no kernel flip.
 * Sizes up to 32 hand bin-major spectra between three fused kernels; 64 and 128
 * run fbfft2D -> transposeMM -> fbifft2D on plane-major spectra in the workspace
 * and need H, W <= fftSize.  With fftSize <= 32 the image may be larger than the
 * transform: it is then cut into overlapping fftSize x fftSize windows whose
 * origins advance by fftSize-kH+1 rows / fftSize-kW+1 columns (the tiling of
 * FFTIteratedConvolution, fbfft/FFTIteratedConvolution.cuh:71-88), and the
 * windows ride through the same three kernels as extra images (forward pass,
 * input gradient) or extra reduction steps (weight gradient).
 * workspace: device memory of at least fbfft_conv_workspace_image() bytes for
 * that pass and image size (fbfft_conv_workspace() when H, W <= fftSize),
 * 256-byte aligned; its contents need not survive between calls. */

/* fftSize = 0 in fbfft_conv_workspace_image, fbfft_conv_fprop / bprop / accgrad and
 * fbfft_conv_fprop_static stands for fbfft_conv_choose_fft_size(pass, ...): the size in
 * {8, 16, 32} (at least kH and kW) that is expected to run the pass fastest - the one
 * that moves the fewest spectrum values over its windows and filter planes, weighted by
 * the measured rate of each size; 0 if the filter is larger than the image or than 32.
 * The passes of one layer may get different sizes (configs[3]: 16 for the forward pass,
 * 91 us against 102 us at 32; 32 for both gradients); every size computes the same
 * convolution.  The reference leaves the choice to its caller (the FFTSize template
 * parameter of fbfft/FFTIteratedConvolution.cuh:624); 64 and 128 are only taken when asked
 * for - on this hardware 32-point windows measure faster than a 64- or 128-point
 * transform of the whole image (60 x 60 images, 5 x 5 filters: 36 us against 74 us and
 * 229 us). */
int fbfft_conv_choose_fft_size(int pass, int batch, int cin, int cout, int H, int W, int kH,
                               int kW);

/* Bytes of workspace for pass 0 (fprop), 1 (bprop) or 2 (accgrad): the values of
 * FFTConvolutionPassFFI (fbfft/FFTIteratedConvolution.cuh:616-622).  0 when the
 * arguments are not supported. */
size_t fbfft_conv_workspace(int pass, int batch, int cin, int cout, int fftSize);

/* The same for a layer with input extents H x W and a kH x kW filter; equal to
 * fbfft_conv_workspace when H, W <= fftSize. */
size_t fbfft_conv_workspace_image(int pass, int batch, int cin, int cout, int H, int W, int kH,
                                  int kW, int fftSize);

/* Same as fbfft_conv_workspace(0, ...). */
size_t fbfft_conv_fprop_workspace(int batch, int cin, int cout, int fftSize);

/* updateOutput: transposeMM<false, true> role (MM-inl.cuh:194).
 * output[b][f] = sum_c corr(input[b][c], weight[f][c]). */
int fbfft_conv_fprop(const fbfft_tensor* input, const fbfft_tensor* weight,
                     const fbfft_tensor* output, int fftSize, void* workspace,
                     size_t workspaceBytes, fbfft_stream_t stream);

/* updateGradInput: transposeMM<false, false> role (MM-inl.cuh:196).
 * gradInput[b][c] = sum_f fullconv(gradOutput[b][f], weight[f][c]). */
int fbfft_conv_bprop(const fbfft_tensor* gradOutput, const fbfft_tensor* weight,
                     const fbfft_tensor* gradInput, int fftSize, void* workspace,
                     size_t workspaceBytes, fbfft_stream_t stream);

/* accGradParameters: transposeMM<true, false> role (MM-inl.cuh:195).
 * gradWeight[f][c] = (accumulate ? gradWeight[f][c] : 0)
 *                    + scale * sum_b corr(input[b][c], gradOutput[b][f]). */
int fbfft_conv_accgrad(const fbfft_tensor* input, const fbfft_tensor* gradOutput,
                       const fbfft_tensor* gradWeight, int fftSize, float scale,
                       int accumulate, void* workspace, size_t workspaceBytes,
                       fbfft_stream_t stream);

/* fbfft_conv_fprop without a workspace argument and without any allocation.  It
 * has no counterpart in the reference; it is for callers that cannot allocate
 * device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  The spectra pass through a fixed array of
 * FBFFT_STATIC_SCRATCH_BYTES in the library's device image (each GPU the library
 * runs on holds its own copy until the process ends).  Layers whose
 * fbfft_conv_workspace(0, ...) exceeds that size return UnsupportedSize.  All
 * calls on one GPU share that GPU's array: calls on one stream are ordered, calls
 * that overlap in time on one GPU race.  Results are those of fbfft_conv_fprop.
 * The first call on a device looks the array's address up (and may make the runtime
 * load the library's device image); any call does, one with an empty batch included,
 * which launches nothing.  Make that call before stream capture begins or before the
 * loop that must not allocate; every later call only enqueues kernels. */
#define FBFFT_STATIC_SCRATCH_BYTES (32u << 20)
int fbfft_conv_fprop_static(const fbfft_tensor* input, const fbfft_tensor* weight,
                            const fbfft_tensor* output, int fftSize, fbfft_stream_t stream);

/* Measurement aid with no counterpart in the reference: a plain device-to-device copy
 * of `bytes` (a multiple of 16, both pointers 16-byte aligned) on `stream`, in the
 * shape that moves a batch the size of a transform's operands fastest from HBM to HBM.
 * Benchmarks time it beside the transforms as the price of moving the same bytes with
 * no arithmetic. */
int fbfft_bench_copy(const void* src, void* dst, size_t bytes, fbfft_stream_t stream);

/* Human-readable name of an fbfft_error. */
const char* fbfft_error_string(int code);

/* The 128-entry (cos, sin)(k*pi/128) table the kernels are built with
 * (fbfft/Twiddles.cuh:322-453); copies 256 floats to out. */
void fbfft_twiddle_table(float* out);

#ifdef __cplusplus
}
#endif
#endif /* FBFFT_AMD_H */
