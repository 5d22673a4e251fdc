/*
 * i8f.h -- C ABI of the MI355X (gfx950) INT8 linear-layer engine.
 *
 * One shared library, libi8f_gfx950.so, built by hipcc for gfx950 only.  It is
 * the drop-in replacement for the device side of ComfyUI-INT8-Fast's W8A8
 * linear path: the three Triton kernels of int8_fused_kernel.py, the online
 * QuaRot rotation of quarot.py and the elementwise torch chain that merges a
 * LoRA into int8 weights.  The reference has no foreign-function interface of
 * its own (it launches Triton from Python); each entry point therefore names
 * the Python function whose device work it replaces.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer owned by the caller.  The library never
 *     allocates, frees or keeps device memory.
 *   - Matrices are row-major.  Weights are int8 [N,K] with K contiguous and are
 *     consumed transposed ("NT" product), exactly the reference's layout
 *     (int8_fused_kernel.py:211-214,228).  Activation scales are [M] float
 *     (the reference's [M,1]); per-row weight scales are [N] float ([N,1]).
 *   - `stream` is a hipStream_t passed as void*; NULL is the default stream.
 *     Work is enqueued asynchronously; no entry point synchronises.
 *   - Return value: I8F_OK (0) or a negative i8f_status.  No C++ exception
 *     crosses this boundary.  Arguments are validated on the host BEFORE any
 *     launch; a failing call launches nothing.
 *   - The library keeps no mutable global state: calls are re-entrant and may
 *     be issued from several host threads on different streams.
 *   - Non-finite inputs (NaN/Inf) give unspecified int8 values, as in the
 *     reference (a float NaN cast to int8 is undefined there too).
 */
#ifndef I8F_H
#define I8F_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define I8F_VERSION 101 /* major*10000 + minor*100 + patch */

typedef enum i8f_status {
    I8F_OK = 0,
    I8F_ERR_INVALID = -1,     /* NULL pointer, negative size, bad enum, misaligned or aliased argument */
    I8F_ERR_UNSUPPORTED = -2, /* a shape this build has no kernel for (documented per entry point) */
    I8F_ERR_HIP = -3,         /* the HIP runtime refused the launch; see i8f_last_hip_error() */
    I8F_ERR_DEVICE = -4       /* the current device is not gfx950 */
} i8f_status;

typedef enum i8f_dtype { I8F_BF16 = 0, I8F_F16 = 1, I8F_F32 = 2 } i8f_dtype;

/* one weight scale for the whole matrix, or one per output row (weight row) */
typedef enum i8f_scale_mode { I8F_SCALE_TENSOR = 0, I8F_SCALE_ROW = 1 } i8f_scale_mode;

/*
 * Order of the floating-point operations of the dequantisation epilogue.
 *   I8F_EPI_TORCH  the reference's torch path (int8_quant.py:84-87, 115-118):
 *                  round the scaled accumulator to the output dtype, then add
 *                  the bias (itself rounded to the output dtype) and round again.
 *                  Bit-identical to that path on the CPU.  The default of the
 *                  Python host layer.
 *   I8F_EPI_FUSED  the operation order of the reference's fused kernels
 *                  (int8_fused_kernel.py:156-173, 310-324): acc * (xs * ws),
 *                  then + bias, each a rounded binary32 operation, then one
 *                  rounding to the output dtype.  The reference's compiler may
 *                  contract the multiply and the add into one fused multiply-add
 *                  on its device; this library never does, so bit-for-bit parity
 *                  with those kernels is unpinned (the two differ by at most one
 *                  binary32 rounding before the final rounding).
 */
typedef enum i8f_epilogue { I8F_EPI_TORCH = 0, I8F_EPI_FUSED = 1 } i8f_epilogue;

/*
 * Elementwise operation applied to the activations while the quantiser reads them
 * (i8f_quant_rowwise_prologue).
 *   I8F_PRO_NONE       none
 *   I8F_PRO_MODULATE   (1 + s[k]) * x + t[k], the adaLN modulation in front of a DiT
 *                      block's qkv and MLP projections; the three tensor operations
 *                      are each rounded to x's dtype, as torch's eager kernels do
 *   I8F_PRO_GELU_TANH  gelu(x, approximate="tanh") in binary32, rounded once to x's dtype
 *   I8F_PRO_SILU_GATE  silu(x) * g[k], the gated activation in front of the down projection of a
 *                      SwiGLU feed-forward (w2(silu(w1 x) * w3 x)): silu in binary32 rounded to x's
 *                      dtype, then the product rounded to x's dtype, as torch's two eager kernels do
 *   I8F_PRO_NORM_MODULATE  (1 + s[k]) * layer_norm(x) + t[k] (no affine parameters); taken by
 *                      i8f_quant_rowwise_norm_modulate only, which carries the epsilon
 *   I8F_PRO_CONCAT_GELU  cat(a, gelu(b, approximate="tanh")) along the row; taken by
 *                      i8f_quant_rowwise_concat_gelu only, which carries the second tensor
 *   I8F_PRO_GELU_ERF   gelu(x) in its exact form, 0.5 x (1 + erf(x / sqrt 2)), in binary32, rounded once to x's dtype
 *   I8F_PRO_MODULATE_FUSED  the same modulation as torch.addcmul(t, x, 1 + s) computes it: the gain 1 + s rounded to x's
 *                      dtype, its product with x (exact in binary32) added to t and rounded ONCE; 16-bit dtypes only.
 *                      The norm entry points below take the same choice as their modulate_fused argument.
 *   I8F_PRO_RMS_NORM   rms_norm(x, weight, eps), optionally followed by (1 + s[k]) * y and + t[k]; taken by
 *                      i8f_quant_rowwise_rms_norm only, which carries the epsilon and the weight
 */
typedef enum i8f_prologue {
    I8F_PRO_NONE = 0, I8F_PRO_MODULATE = 1, I8F_PRO_GELU_TANH = 2, I8F_PRO_SILU_GATE = 3, I8F_PRO_NORM_MODULATE = 4,
    I8F_PRO_CONCAT_GELU = 5, I8F_PRO_GELU_ERF = 6, I8F_PRO_RMS_NORM = 7, I8F_PRO_MODULATE_FUSED = 8
} i8f_prologue;

/* Library version (I8F_VERSION of the build). */
int i8f_version(void);

/* Static, human-readable text for a status code. */
const char *i8f_status_string(int status);

/* hipError_t of the most recent I8F_ERR_HIP on the calling thread (0 if none). */
int i8f_last_hip_error(void);

/*
 * Fused (optional block rotation +) dynamic per-row absmax int8 quantisation.
 * Replaces triton_quantize_rowwise / _quantize_rowwise_kernel
 * (int8_fused_kernel.py:10-73), with the arithmetic of the torch path
 * quantize_int8_axiswise (int8_quant.py:28-31, 20-21), and, when
 * rotate_block == 128, the preceding rotate_activation (quarot.py:73-102 called
 * at int8_quant.py:741-744) or rotate_weight (quarot.py:42-70 called at
 * int8_quant.py:602-607) in the same pass over memory.
 *
 *   x        [M,K] of x_dtype, row stride ldx elements (ldx >= K)
 *   rotate_block   0 (no rotation) or 128 (K must then be a multiple of 128)
 *   q        [M,K] int8, contiguous            scale   [M] float
 *
 * Any M >= 0 and K >= 0.  I8F_ERR_UNSUPPORTED for another rotate_block.
 */
int i8f_quant_rowwise(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                      int rotate_block, int8_t *q, float *scale, void *stream);

/*
 * i8f_quant_rowwise for several row blocks of one width K and one dtype in ONE launch: group i is an
 * independent i8f_quant_rowwise(x, x_dtype, M, K, ldx, rotate_block, q, scale).  No counterpart in the reference,
 * whose operator quantises one layer's input at a time (int8_fused_kernel.py:55-73); it is for callers that hold
 * the inputs of two layers at once -- the image and the text tokens of a double-stream transformer block, which
 * have their own weights and therefore their own linear layers -- where kernels of a few microseconds cost as
 * much in the gaps between launches as in themselves.  Results are those of the separate calls bit for bit.
 * The array of groups is read on the host during the call.  Up to 8 groups of 16-bit activations with 16-byte
 * aligned rows and K % 16 == 0 (K <= 16384) take one launch; anything else is launched group by group.
 */
typedef struct i8f_quant_group {
    const void *x;   /* [M,K] of x_dtype, row stride ldx elements */
    int64_t M, ldx;
    int8_t *q;       /* [M,K] int8, contiguous */
    float *scale;    /* [M] */
} i8f_quant_group;
int i8f_quant_rowwise_grouped(const i8f_quant_group *groups, int n_groups, int x_dtype, int64_t K,
                              int rotate_block, void *stream);

/*
 * i8f_quant_rowwise with the elementwise operation in front of the linear layer
 * applied on the fly.  The reference gets this fusion from torch.compile, which
 * fuses the producer of the activations into its traceable Triton quantiser
 * (README.md:4,56; int8_fused_kernel.py:10-53); here it is an explicit variant of
 * the quantiser, so the modulated / activated tensor is never written to memory.
 *   prologue      i8f_prologue
 *   mod_scale, mod_shift   I8F_PRO_MODULATE: [ceil(M / rows_per_vec), K] of x_dtype,
 *                 contiguous; row m uses vector m / rows_per_vec (one pair of vectors
 *                 per image of a batch).  I8F_PRO_SILU_GATE: mod_scale is the gate operand g,
 *                 same layout (rows_per_vec = 1 for a gate tensor of x's shape), mod_shift
 *                 is ignored.  Both ignored otherwise.
 * I8F_PRO_MODULATE is bit-identical to torch's three eager operations followed by
 * i8f_quant_rowwise; I8F_PRO_GELU_TANH, I8F_PRO_GELU_ERF and I8F_PRO_SILU_GATE agree with torch's gelu / silu
 * to the last bits of binary32 before the rounding to x_dtype (tests state the tolerance).
 */
int i8f_quant_rowwise_prologue(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                               int prologue, const void *mod_scale, const void *mod_shift,
                               int64_t rows_per_vec, int rotate_block, int8_t *q, float *scale,
                               void *stream);

/*
 * The quantiser with the whole adaLN producer of a DiT block in front of it:
 *   y = layer_norm(x, eps) without affine parameters, rounded to x's dtype
 *       (mean and variance of the row in binary32: mean = sum / K, var = sum (x - mean)^2 / K,
 *        y = (x - mean) * (1 / sqrt(var + eps)))
 *   z = (1 + s[k]) * y + t[k], three operations each rounded to x's dtype (I8F_PRO_MODULATE)
 *   then rotation, absmax and int8 as i8f_quant_rowwise.
 * No counterpart in the reference's files: there the LayerNorm and the modulation are the model's
 * own torch operations in front of Linear.forward (int8_quant.py:703), fused by torch.compile into
 * the quantiser's producer (README.md:4,56); here neither y nor z is ever written to memory.
 * torch's LayerNorm takes its sums in another order and its reciprocal square root from the
 * hardware, so y agrees with it to the last place of the dtype (tests state the tolerance).
 *   mod_scale, mod_shift, rows_per_vec: as for I8F_PRO_MODULATE.
 *   modulate_fused   0: three rounded operations; 1: z = round((1 + s[k]) * y + t[k]) with the gain rounded and the
 *                    product and sum rounded once, as torch.addcmul(shift, y, 1 + scale) (I8F_PRO_MODULATE_FUSED)
 * I8F_ERR_UNSUPPORTED unless x_dtype is I8F_BF16 or I8F_F16, K % 16 == 0, K <= 16384 and x, q and
 * the vectors are 16-byte aligned (the row stays in the registers of one to four wavefronts): other callers
 * normalise with their own kernel and use I8F_PRO_MODULATE.
 */
int i8f_quant_rowwise_norm_modulate(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                    float eps, const void *mod_scale, const void *mod_shift,
                                    int64_t rows_per_vec, int modulate_fused, int rotate_block, int8_t *q,
                                    float *scale, void *stream);

/*
 * The quantiser with an RMSNorm, and optionally the modulation behind it, in front of it:
 *   y = x * (1 / sqrt(sum x^2 / K + eps)) * weight[k]      in binary32, rounded once to x's dtype (torch's rms_norm;
 *                                                          weight NULL: no weight)
 *   z = (1 + s[k]) * y    if mod_scale is given: 1 + s rounded, the product rounded
 *   z = z + t[k]          if mod_shift is given: rounded
 *   then rotation, absmax and int8 as i8f_quant_rowwise.
 * The producer of the attention and feed-forward projections of blocks that normalise with an RMSNorm
 * (modulate(norm(x), scale) = norm(x) * (1 + scale) in the z-image family, rms_norm(x) * (1 + scale) + shift in the
 * ltx family; the loader names both, int8_unet_loader.py:60-93).  No counterpart in the reference's files: there
 * these are the model's own torch operations in front of Linear.forward (int8_quant.py:703), fused by torch.compile
 * into the quantiser's producer (README.md:4,56); here none of the intermediate tensors is written to memory.
 * The row's sum is taken in this kernel's order, torch's in its own: y agrees with torch's to the last place of the
 * dtype (tests state the tolerance).
 *   weight [K] of x_dtype or NULL; mod_scale, mod_shift [ceil(M / rows_per_vec), K] of x_dtype or NULL each;
 *   rows_per_vec as for I8F_PRO_MODULATE (ignored when both are NULL); modulate_fused as for
 *   i8f_quant_rowwise_norm_modulate (it matters only when both scale and shift are given).
 * I8F_ERR_UNSUPPORTED unless x_dtype is I8F_BF16 or I8F_F16, K % 16 == 0, K <= 16384 and x, q and the vectors are
 * 16-byte aligned (the row stays in the registers of one to four wavefronts): other callers normalise with their own kernel.
 */
int i8f_quant_rowwise_rms_norm(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx, float eps,
                               const void *weight, const void *mod_scale, const void *mod_shift,
                               int64_t rows_per_vec, int modulate_fused, int rotate_block, int8_t *q, float *scale,
                               void *stream);

/*
 * The quantiser on the concatenation of two tensors along the row, the second through tanh-GELU:
 *   z[m] = ( a[m, 0..Ka) , gelu(b[m, 0..Kb), approximate="tanh") )        then rotation, absmax and int8 over Ka + Kb
 * the input of the second projection of a single-stream transformer block, linear2(cat(attn, gelu(mlp))): neither
 * the activated tensor nor the concatenation is ever written to memory.  No counterpart in the reference's files:
 * there both are the model's own torch operations in front of Linear.forward (int8_quant.py:703), fused by
 * torch.compile into the quantiser's producer (README.md:4,56).  GELU as I8F_PRO_GELU_TANH (same tolerance); the
 * a part is taken as it is, so with Kb == 0 the result is i8f_quant_rowwise's bit for bit.
 *   a [M,Ka] (row stride lda), b [M,Kb] (row stride ldb) of dtype; q [M, Ka+Kb] contiguous; scale [M]
 * I8F_ERR_UNSUPPORTED unless dtype is I8F_BF16 or I8F_F16, Ka % 16 == 0, Kb % 16 == 0, Ka + Kb <= 16384 and rows
 * are 16-byte aligned: other callers concatenate themselves and use i8f_quant_rowwise.
 */
int i8f_quant_rowwise_concat_gelu(const void *a, int dtype, int64_t M, int64_t Ka, int64_t lda, const void *b,
                                  int64_t Kb, int64_t ldb, int rotate_block, int8_t *q, float *scale,
                                  void *stream);

/*
 * One absmax scale for a whole tensor, then int8 quantisation with it.
 * Replaces quantize_int8_tensorwise (int8_quant.py:23-26), the load-time
 * quantiser of tensorwise checkpoints and of BASELINE config 0's weight:
 *   scale = max(float(max|x|) / 127, 1e-30),  q = sat8(rne(float(x) * (1 / scale)))
 * in two launches that use the whole GPU (the partial maxima of the first launch
 * are what the workspace holds).
 *   x        n elements of x_dtype, contiguous      q   n int8      scale   1 float
 *   workspace        device memory of at least i8f_quant_tensorwise_workspace_bytes(n)
 *                    bytes, 4-byte aligned, owned by the caller; contents need no
 *                    initialisation and are garbage afterwards
 * n == 0 writes scale = 1e-30.
 */
int64_t i8f_quant_tensorwise_workspace_bytes(int64_t n);
int i8f_quant_tensorwise(const void *x, int x_dtype, int64_t n, int8_t *q, float *scale,
                         void *workspace, int64_t workspace_bytes, void *stream);

/*
 * i8f_quant_tensorwise without a workspace argument and without any allocation.
 * No counterpart in the reference: it exists for callers that cannot allocate
 * device memory (code under HIP graph capture, serving loops and harnesses that
 * forbid hipMalloc).  The partial maxima live in a 4 KB file-scope device array of
 * the library, one copy per GPU, held until the process ends.  Same results as
 * i8f_quant_tensorwise bit for bit.
 * I8F_ERR_UNSUPPORTED for n > 2^32 elements.  Calls that overlap in time on one
 * GPU (different streams or threads) race on that array: serialise them.  The first
 * call on a device looks the array's address up (hipGetSymbolAddress): make it outside
 * a stream capture; later calls only launch kernels.
 */
int i8f_quant_tensorwise_static(const void *x, int x_dtype, int64_t n, int8_t *q, float *scale,
                                void *stream);

/*
 * Block rotation alone (no quantisation): every aligned block of 128 elements of
 * each row is multiplied by the normalised Hadamard matrix, result in x's dtype.
 * Replaces rotate_weight / rotate_activation (quarot.py:42-102) where the rotated
 * tensor itself is wanted: the LoRA delta of a rotated layer
 * (int8_quant.py:300-306, 387-393).  Same butterfly as i8f_quant_rowwise.
 *   x [M,K] of dtype (row stride ldx), out [M,K] contiguous, K % 128 == 0.
 *   out may equal x when ldx == K.
 */
int i8f_rotate128(const void *x, int dtype, int64_t M, int64_t K, int64_t ldx, void *out,
                  void *stream);

/*
 * int8 x int8 -> int32 product, acc[m,n] = sum_k a[m,k] * w[n,k].
 * Replaces torch._int_mm(x8, weight.T) (int8_quant.py:80,110); it is the
 * accumulator of the fused kernels (int8_fused_kernel.py:132-144) made visible,
 * so that parity of the integer part can be checked bit for bit.
 *   a [M,K] int8   w [N,K] int8   acc [M,N] int32, all contiguous.
 */
int i8f_gemm_i32(const int8_t *a, const int8_t *w, int64_t M, int64_t N, int64_t K,
                 int32_t *acc, void *stream);

/*
 * The tile configuration i8f_gemm_i32 / i8f_linear_w8a8 use for an aligned M x N x K
 * problem: rows and columns of the output tile one workgroup computes and the number
 * of K-tile stages it keeps in LDS (1 x 1, 0 stages for shapes that take the
 * one-thread-per-output kernel).  No counterpart in the reference; for benchmarks
 * and profiles that have to name the kernel variant they measured.
 */
int i8f_gemm_tile(int64_t M, int64_t N, int64_t K, int *bm, int *bn, int *stages);

/*
 * INT8 GEMM with the dequantisation epilogue fused in registers.
 * Replaces _int8_matmul_dequant_kernel and _int8_matmul_dequant_per_row_kernel
 * (int8_fused_kernel.py:91-173, 253-324) and the torch epilogue
 * (int8_quant.py:84-87, 115-118):
 *   out[m,n] = epilogue( sum_k a[m,k]*w[n,k], a_scale[m], w_scale[n or 0], bias[n] )
 *
 *   a [M,K] int8, a_scale [M] float          (outputs of i8f_quant_rowwise)
 *   w [N,K] int8
 *   w_scale   device pointer to 1 (TENSOR) or N (ROW) floats; with TENSOR it may
 *             be NULL, and then the host value w_scale_host is used
 *   bias      NULL or [N] of bias_dtype
 *   out       [M,N] of out_dtype (I8F_BF16 or I8F_F16; I8F_F32 for debugging)
 *   order     i8f_epilogue
 */
int i8f_linear_w8a8(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                    float w_scale_host, int scale_mode, const void *bias, int bias_dtype,
                    void *out, int out_dtype, int64_t M, int64_t N, int64_t K, int order,
                    void *stream);

/*
 * The same, with a second matrix added to the result inside the epilogue:
 *   out[m,n] = round( i8f_linear_w8a8(...)[m,n] + addend[m,n] )
 * Replaces the addition of the dynamic (unmerged) LoRA side branch at the end of
 * Linear.forward (int8_quant.py:762-774: y = y + lora_out.to(y.dtype)), which in
 * the reference is a separate elementwise pass over [M,N].  The sum is rounded once
 * more to out_dtype, as the reference's tensor addition does.
 *   addend    [M,N] of out_dtype, contiguous; NULL gives i8f_linear_w8a8 exactly
 */
int i8f_linear_w8a8_add(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                        float w_scale_host, int scale_mode, const void *bias, int bias_dtype,
                        const void *addend, void *out, int out_dtype, int64_t M, int64_t N, int64_t K,
                        int order, void *stream);

/*
 * i8f_linear_w8a8_add with a workspace, which lets outputs of few tiles and a long K (K >= 10240: a text
 * stream's down-projection, a decode-sized batch) deal the K range of a tile over several workgroups that
 * exchange their integer sums through the workspace.  Same arguments, same results bit for bit (integer
 * sums do not depend on their order); the same Triton launches as i8f_linear_w8a8 (int8_fused_kernel.py:216,
 * 357), whose grids cover the output only.  512 x 3072 x 12288 with weights from HBM: 42 -> 34 us.
 *   workspace        device memory of i8f_linear_w8a8_workspace_bytes() bytes (16 MB + 4 KB), 16-byte aligned,
 *                    whose first 4096 bytes (one arrival word per output tile) are ZERO before the first call;
 *                    every call that completes leaves them zero again.  Each launch stamps its arrival words
 *                    with a tag of its own and treats a word with another tag as "nobody has arrived", so the
 *                    words a launch that never finished (killed, aborted) left behind do not poison the next
 *                    one.  A captured launch is replayed with the tag it was captured with: a graph whose
 *                    replays may be aborted should clear the 4096 bytes with a fill kernel in front of the call.
 *                    One workspace serves any number of calls that do NOT OVERLAP IN TIME (one per stream, and
 *                    not an eager call next to the replay of a graph that captured the same workspace): calls
 *                    that overlap race on the partial sums.  NULL gives i8f_linear_w8a8_add exactly.
 * I8F_ERR_INVALID for a workspace that is too small or misaligned.
 */
int64_t i8f_linear_w8a8_workspace_bytes(void);
int i8f_linear_w8a8_splitk(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                           float w_scale_host, int scale_mode, const void *bias, int bias_dtype,
                           const void *addend, void *out, int out_dtype, int64_t M, int64_t N, int64_t K,
                           int order, void *workspace, int64_t workspace_bytes, void *stream);

/*
 * i8f_linear_w8a8_splitk with the gated residual of an adaLN-Zero transformer block in the epilogue:
 *   out[m,n] = round( residual[m,n] + round( gate[m / rows_per_gate, n] * y[m,n] ) ),   y = i8f_linear_w8a8(...)
 * i.e. `x + gate * linear(h)` as torch's two tensor operations compute it on tensors of out_dtype (each rounded
 * to out_dtype), bit for bit.  No counterpart in the reference's files: there the multiplication by the gate and
 * the residual addition are the model's own torch operations behind Linear.forward (int8_quant.py:703-778), two
 * more passes over [M,N] that torch.compile fuses into one; here neither exists.
 *   gate       [ceil(M / rows_per_gate), N] of out_dtype, contiguous: one vector per group of rows_per_gate
 *              consecutive rows (one per image of a batch); NULL: no gate (i8f_linear_w8a8_splitk exactly)
 *   residual   [M,N] of out_dtype, contiguous, or NULL (then out = round(gate * y)); may equal out
 * Other arguments and the workspace as for i8f_linear_w8a8_splitk.
 */
int i8f_linear_w8a8_gated(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                          float w_scale_host, int scale_mode, const void *bias, int bias_dtype,
                          const void *gate, int64_t rows_per_gate, const void *residual, void *out,
                          int out_dtype, int64_t M, int64_t N, int64_t K, int order, void *workspace,
                          int64_t workspace_bytes, void *stream);

/*
 * i8f_linear_w8a8_splitk for several layers of one shape at once: group i is a problem of its own
 * (activations, weights, scales, bias, gate, addend, output, row count M) and the groups share N, K, the
 * scale mode, the dtypes and the operation order.  No counterpart in the reference, whose operator
 * (int8_forward_dynamic*, int8_quant.py:65-118; Int8TensorwiseOps.Linear.forward, :703-778) takes one
 * layer: a double-stream transformer block runs every projection twice, for its image and for its
 * text tokens, and the few tiles of the text stream fit into the compute units that the image
 * stream's last round of tiles leaves idle (4096 and 512 tokens into 3072 columns: 192 + 24 tiles of
 * 256 x 256 on 256 units), so in one launch the smaller problem costs nothing.  Where the groups'
 * tiles together need a round more than the largest group alone, or a group has a shape the tiled
 * kernel does not take, the call launches group by group exactly as i8f_linear_w8a8_splitk would
 * (workspace: as there, may be NULL).  Results are those of the separate calls bit for bit.
 * The array of groups is read on the host during the call; at most I8F_MAX_LINEAR_GROUPS groups.
 */
#define I8F_MAX_LINEAR_GROUPS 4
typedef struct i8f_linear_group {
    const int8_t *a;        /* [M,K] int8 */
    const float *a_scale;   /* [M] */
    const int8_t *w;        /* [N,K] int8 */
    const float *w_scale;   /* [N] (I8F_SCALE_ROW), [1] or NULL (then w_scale_host) */
    float w_scale_host;
    const void *bias;       /* [N] of bias_dtype or NULL */
    const void *addend;     /* [M,N] of out_dtype or NULL */
    void *out;              /* [M,N] of out_dtype */
    int64_t M;
    const void *gate;       /* [ceil(M / rows_per_gate), N] of out_dtype or NULL: as for i8f_linear_w8a8_gated */
    int64_t rows_per_gate;
} i8f_linear_group;
int i8f_linear_w8a8_grouped(const i8f_linear_group *groups, int n_groups, int scale_mode,
                            int bias_dtype, int out_dtype, int64_t N, int64_t K, int order,
                            void *workspace, int64_t workspace_bytes, void *stream);

/*
 * i8f_linear_w8a8 with the second product of the dynamic (unmerged) LoRA side branch
 * computed inside the epilogue on the matrix cores:
 *   out[m,n] = round( i8f_linear_w8a8(...)[m,n] + side[m,n] )
 *   side     = round( round( sum_j side_t[m,j] * side_b[n,j] ) * alpha )   (the multiplication
 *              by alpha and its rounding only if has_alpha)
 * Replaces lora_y = F.linear(lora_x, lB); lora_y * alpha; y + lora_y.to(y.dtype) of Linear.forward
 * (int8_quant.py:768-774): no [M,N] side tensor is written or read.  side_t = lora_x [M,rank]
 * (the caller's first product F.linear(x, lA)), side_b = lB [N,rank], both of out_dtype and
 * contiguous; all roundings are to out_dtype.  The sum over j is accumulated in binary32 by the
 * matrix core; the reference's order is its BLAS library's, so results agree to the rounding of
 * that sum (tests state the tolerance).
 * I8F_ERR_UNSUPPORTED unless out_dtype is I8F_BF16 or I8F_F16, rank is a multiple of 16 up to 64,
 * K is a multiple of 128 and the operands are 16-byte aligned (N % 8 == 0, K % 16 == 0): such
 * callers use i8f_linear_w8a8_add with a side tensor instead.
 */
int i8f_linear_w8a8_lora(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                         float w_scale_host, int scale_mode, const void *bias, int bias_dtype,
                         const void *side_t, const void *side_b, int64_t rank, int has_alpha, float alpha,
                         void *out, int out_dtype, int64_t M, int64_t N, int64_t K, int order,
                         void *stream);

/*
 * Small-batch W8A16 path, M <= 16: activations stay in their dtype, the int8
 * weight is dequantised on the fly.  Replaces the "small batch fallback" of
 * Linear.forward (int8_quant.py:756-760):
 *   out = F.linear(x, (float(w) * w_scale).to(x.dtype), bias.to(x.dtype))
 * without materialising the dequantised weight.  Products are accumulated in
 * binary32; the result is within the tolerance the tests state of the
 * reference, whose BLAS summation order is unspecified.
 *   x [M,K] of x_dtype (row stride ldx), out [M,N] of x_dtype.
 * I8F_ERR_UNSUPPORTED for M > 16.
 */
int i8f_linear_w8a16_small_m(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                             const int8_t *w, const float *w_scale, float w_scale_host,
                             int scale_mode, const void *bias, int bias_dtype, void *out,
                             int64_t N, void *stream);

/*
 * i8f_linear_w8a16_small_m for several layers in one launch: the modulation projections of the image and of the
 * text stream of a double-stream block, each Linear.forward(vec) with M <= 16 on its own weight (int8_quant.py:756-760
 * called once per layer).  No counterpart in the reference, whose operator takes one layer; results are those of the
 * separate calls bit for bit.  Why: a weight stream of tens of megabytes lasts little longer than the memory system
 * takes to ramp up and drain, and two of them in one grid keep it busy through the seam.
 *   groups[i]: a [M,K] of x_dtype (row stride ldx), w int8 [N,K], w_scale / w_scale_host as above, bias [N] of
 *   bias_dtype or NULL, out [M,N] of x_dtype.  x_dtype, scale_mode and bias_dtype are shared.
 * Up to 4 layers with 16-bit activations, K % 16 == 0 and 16-byte aligned operands take one launch; anything else is
 * launched layer by layer.  The array is read on the host during the call.
 */
typedef struct i8f_small_m_group {
    const void *a;
    int64_t M, K, ldx;
    const int8_t *w;
    const float *w_scale;
    float w_scale_host;
    const void *bias;
    void *out;
    int64_t N;
} i8f_small_m_group;
int i8f_linear_w8a16_small_m_grouped(const i8f_small_m_group *groups, int n_groups, int x_dtype, int scale_mode,
                                     int bias_dtype, void *stream);

/*
 * Stochastic rounding of a float delta to int8 with SUPPLIED uniform noise.
 * Replaces stochastic_round_int8_delta (int8_quant.py:36-62); the reference
 * draws the noise from a device generator (:41,55), which no other device can
 * reproduce, so the caller passes the [N,K] float noise in [0,1).
 *   dq[n,k] = int8(clamp(noise < frac(x/scale) ? floor(x/scale)+1 : floor(x/scale)))
 *   x, noise [N,K] float; scale as w_scale above; dq [N,K] int8.
 * x / scale is a correctly rounded binary32 division, which is what torch computes for a tensor
 * scale on any device and for a Python-float scale on the CPU; for a Python-float scale on a GPU
 * torch multiplies by the rounded reciprocal instead, which can differ in the last bit: bit-for-bit
 * parity is with the CPU chain.  (The kernels obtain the same quotient from a correctly rounded
 * reciprocal and two fma corrections where that is exact, and divide elsewhere.)  A NaN quotient
 * (NaN input, 0/0, inf/inf) gives -128 here; the reference converts a NaN to int8, which is undefined.
 */
int i8f_sr_quant_delta(const float *x, const float *scale, float scale_host, int scale_mode,
                       const float *noise, int64_t N, int64_t K, int8_t *dq, void *stream);

/*
 * LoRA merge in int8 space.  Replaces the int8 branch of
 * INT8LoRAPatchAdapter.calculate_weight / INT8MergedLoRAPatchAdapter
 * (int8_quant.py:293-318, 382-404): stochastic rounding of the scaled delta with
 * the layer's weight scale, saturating int8 add, in ONE pass over memory.
 *
 *   w_out[n,k] = sat8( w[n,k] + SR(delta_f[n,k] / w_scale[n or 0], noise[n,k]) )
 *
 * delta_f is either supplied (delta != NULL: [N,K] float, already multiplied by
 * the LoRA scale; up/down/rank ignored) or rebuilt in the kernel from the
 * low-rank factors (delta == NULL): up [N,rank], down [rank,K] float,
 *   delta_f[n,k] = (sum_j up[n,j]*down[j,k]) * lora_scale
 * with the sum taken as a chain of fused multiply-adds in increasing j
 * (reconstruct_lora_diff case 1, int8_quant.py:143-157, and :295).
 * w_out may equal w (in-place).  rank <= 256 for the fused form.
 */
int i8f_lora_merge_sr(const int8_t *w, const float *w_scale, float w_scale_host, int scale_mode,
                      const float *delta, const float *up, const float *down, int64_t rank,
                      float lora_scale, const float *noise, int64_t N, int64_t K, int8_t *w_out,
                      void *stream);

#ifdef __cplusplus
}
#endif
#endif /* I8F_H */
