/*
 * int4linear.h -- host API of the MI355X (gfx950) signed-int4 linear-layer GEMM.
 *
 *   C[M x N] (int32, row-major, ld = N)  =  A[M x K] (s4)  *  B[N x K]^T (s4)
 *
 * A and B are K-contiguous and packed two signed 4-bit values per byte, element e of
 * a row in byte e/2, even e in the low nibble (the layout written by the reference's
 * utils/packer.cpp:3-18).  Row stride is K/2 bytes.  Accumulation is exact int32.
 *
 * Two layers are exported by libint4linear.so:
 *   1. a C ABI (extern "C", plain pointers and sizes, status codes, asynchronous on a
 *      caller-supplied HIP stream) -- the drop-in boundary other languages bind to;
 *   2. the reference's own C++-linkage entry points (linear_vN_launch, pack, unpack)
 *      with the reference's signatures and blocking behaviour, implemented on top of 1.
 *
 * All pointers named *_d are device pointers owned by the caller.  The only device
 * memory the library itself allocates is one workspace per device (see
 * int4linear_workspace_bytes), which holds the FP6 kernel's converted operands and the
 * partial sums of the split-K forms: created on first need, grown when a larger problem
 * arrives, never larger than the workspace limit, freed by int4linear_release_workspace;
 * a process that never calls that keeps it until it ends (the library installs no exit
 * handler).  With the limit set to 0 no entry point allocates anything.  Besides that the
 * library's device image holds the fixed scratch array of int4linear_gemm_s4s4s32_static
 * (INT4LINEAR_STATIC_SCRATCH_BYTES, 128 MiB of device memory on every device a process
 * initialises the library on, whether or not that entry point is ever called) and 32 KiB
 * of arrival counters.
 *
 * HIP graphs: the first call on a device sets the library up (device queries, kernel
 * attributes, the address of the scratch array), which must not happen inside a capture:
 * call int4linear_init(), or any other entry point, on the device before the capture
 * begins; a first call that arrives while its stream is capturing returns
 * INT4LINEAR_ERR_NOT_INITIALISED.  A call whose stream is being captured into a HIP graph never
 * touches that workspace either: under automatic dispatch it runs the kernels that need
 * none, and an explicit INT4LINEAR_KERNEL_FP6 request returns INT4LINEAR_ERR_UNSUPPORTED
 * (graphs that want the FP6 kernel use int4linear_gemm_fp6_converted on their own buffers,
 * or int4linear_gemm_s4s4s32_static).
 */
#ifndef INT4LINEAR_H
#define INT4LINEAR_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes returned by every C-ABI entry point. */
enum {
    INT4LINEAR_OK = 0,
    INT4LINEAR_ERR_SHAPE = 1,       /* negative dimension, or K not a multiple of 8      */
    INT4LINEAR_ERR_NULL = 2,        /* null pointer with a non-empty operand             */
    INT4LINEAR_ERR_ALIGN = 3,       /* operand base not 16-byte aligned                  */
    INT4LINEAR_ERR_HIP = 4,         /* a HIP runtime call failed (see last_hip_error)    */
    INT4LINEAR_ERR_UNSUPPORTED = 5, /* the requested kernel cannot run this shape        */
    INT4LINEAR_ERR_NO_DEVICE = 6,   /* no gfx950 device is visible                       */
    INT4LINEAR_ERR_SCRATCH = 7,     /* int4linear_gemm_s4s4s32_static: the only fast kernel
                                       for the shape needs more scratch memory than
                                       INT4LINEAR_STATIC_SCRATCH_BYTES                   */
    INT4LINEAR_ERR_NOT_INITIALISED = 8 /* first call on this device while its stream is being
                                       captured: call int4linear_init() before capturing */
};

/* Element type of the output of int4linear_linear_fp6_converted. */
enum {
    INT4LINEAR_OUT_S32 = 0,  /* int32: sum + bias                                         */
    INT4LINEAR_OUT_F32 = 1,  /* float: ((float)(sum + bias) * row_scale) * col_scale      */
    INT4LINEAR_OUT_F16 = 2,  /* the float value rounded to IEEE half                      */
    INT4LINEAR_OUT_BF16 = 3  /* the float value rounded to bfloat16                       */
};

/* Kernel selector for int4linear_gemm_s4s4s32_ex. */
enum {
    INT4LINEAR_KERNEL_AUTO = 0,   /* shape-based dispatch (what the plain entry uses)    */
    INT4LINEAR_KERNEL_SIMPLE = 1, /* one thread per output, scalar nibble decode; any K%8==0 */
    INT4LINEAR_KERNEL_MFMA = 2,   /* LDS-pipelined v_mfma_i32_32x32x32_i8 kernel (tile and form
                                     chosen from the grid); K%128==0 */
    INT4LINEAR_KERNEL_SKINNY = 3, /* weight-streaming kernel: M <= 64 and K%128==0, or more
                                     rows (in runs of 64) when K splits into 128-byte tiles */
    INT4LINEAR_KERNEL_FP6 = 4,    /* operands converted to FP6 (E2M3) in a workspace, then
                                     v_mfma_f32_32x32x64_f8f6f4; exact; any K%8==0
                                     below 2^18 (the converter pads K to 128 with zeros) */
    INT4LINEAR_KERNEL_MFMA_128 = 5, /* the int8 kernel's pipelined form, 128x128 workgroup tile */
    INT4LINEAR_KERNEL_MFMA_256 = 6  /* the int8 kernel with its 256x256 workgroup tile   */
};

/* One-time set-up for the current HIP device (queries the CU count, raises the
 * dynamic-LDS limit of the kernels, takes the addresses of the scratch arrays).  Called
 * implicitly by the other entry points, except while their stream is being captured (see
 * above); idempotent and thread-safe; a failed set-up is tried again by the next call.
 * Replaces the per-call cudaFuncSetAttribute of kernels/linear_v21.cu:14-18. */
int int4linear_init(void);

/* The GEMM.  Asynchronous: work is enqueued on `stream` (a hipStream_t, NULL = the
 * default stream) and the call returns without synchronising.  C is fully overwritten.
 * M == 0 or N == 0 is a no-op; K == 0 zero-fills C.
 * Replaces kernels/linear_v21.cu:9-49 (linear_v21_launch) minus its device-wide
 * synchronisation, and the direct kernel launch of test/benchmark.cu:46-72. */
int int4linear_gemm_s4s4s32(const void *a_packed_d, const void *b_packed_d, void *c_d,
                            int m, int n, int k, void *stream);

/* int4linear_gemm_s4s4s32 for callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart
 * in the reference (whose launcher needs no scratch memory, kernels/linear_v21.cu:9-49).
 * Same arguments, same result, same choice of kernel as int4linear_gemm_s4s4s32 makes with
 * a workspace limit of the array's size, but where that entry point would use its allocated workspace (the
 * FP6 kernel's converted operands, the partial sums of the split-K forms) this one uses a
 * fixed array of INT4LINEAR_STATIC_SCRATCH_BYTES that is part of the library's device image:
 * every device the library is initialised on holds one copy until the process ends.  The
 * call allocates and frees nothing, records no events and takes no locks.  A shape whose
 * kernel would need more scratch than the array holds (at M = N = K the FP6 form fits up to
 * 9216) runs on the kernels that need none, as it does under graph capture through the
 * ordinary entry point; only when that would leave a large problem to the scalar kernel (K
 * not a multiple of 128, which among the fast kernels only the FP6 one takes) is the call
 * refused with INT4LINEAR_ERR_SCRATCH before anything is enqueued.  Set the device up
 * (int4linear_init) before capturing.  All calls on one device share the one array and nothing orders
 * them: calls whose execution may overlap on a device (different streams, graphs replayed
 * concurrently) race on it; calls on one stream are ordered by the stream. */
#define INT4LINEAR_STATIC_SCRATCH_BYTES (128u << 20)
int int4linear_gemm_s4s4s32_static(const void *a_packed_d, const void *b_packed_d, void *c_d,
                                   int m, int n, int k, void *stream);

/* Same as int4linear_gemm_s4s4s32 with an explicit kernel choice (INT4LINEAR_KERNEL_*).  Returns
 * INT4LINEAR_ERR_UNSUPPORTED when that kernel cannot run the shape. */
int int4linear_gemm_s4s4s32_ex(const void *a_packed_d, const void *b_packed_d, void *c_d,
                               int m, int n, int k, int kernel, void *stream);

/* The linear layer with an epilogue fused into the GEMM's store.  The reference has no
 * such entry point; its README lists the bias add as future work (README.md:72).
 *   int4linear_linear_s32:  Y[i][j] = sum_l X[i][l] W[j][l] + bias[j]          (int32, wraps)
 *   int4linear_linear_f32:  Y[i][j] = ((float)(sum + bias[j]) * row_scale[i]) * col_scale[j]
 *   int4linear_linear_f16:  the same value rounded once more, to IEEE half (nearest even;
 *                           beyond 65504 it becomes infinity)
 *   int4linear_linear_bf16: the same value rounded once more, to bfloat16 (nearest even)
 *                           (both: denormals are kept; a NaN, which only a scale can bring
 *                           in, keeps its sign and upper payload bits and becomes quiet)
 * bias_d (n int32), row_scale_d (m floats: per-token activation scale) and col_scale_d
 * (n floats: per-output-channel weight scale) may each be NULL (0 / 1).  The integer part is
 * exact; the conversion to float rounds to nearest once and each multiplication once, in
 * the order written (the README's natural next step after the bias: dequantised output in
 * the type the next layer takes).  y_d of the two half-width forms is m x n 16-bit elements,
 * row-major, base 16-byte aligned like the others.  `kernel` is an INT4LINEAR_KERNEL_*
 * value; other arguments as for int4linear_gemm_s4s4s32. */
int int4linear_linear_s32(const void *x_packed_d, const void *w_packed_d, const int *bias_d, void *y_d,
                          int m, int n, int k, int kernel, void *stream);
int int4linear_linear_f32(const void *x_packed_d, const void *w_packed_d, const int *bias_d,
                          const float *row_scale_d, const float *col_scale_d, float *y_d,
                          int m, int n, int k, int kernel, void *stream);
int int4linear_linear_f16(const void *x_packed_d, const void *w_packed_d, const int *bias_d,
                          const float *row_scale_d, const float *col_scale_d, void *y_d,
                          int m, int n, int k, int kernel, void *stream);
int int4linear_linear_bf16(const void *x_packed_d, const void *w_packed_d, const int *bias_d,
                           const float *row_scale_d, const float *col_scale_d, void *y_d,
                           int m, int n, int k, int kernel, void *stream);

/* Device-side counterparts of utils/packer.cpp:3-18 (pack) and :20-31 (unpack):
 * src_d / dst_d are device arrays with the reference's host layouts (m x n ints
 * unpacked, m x ceil(n/8) 32-bit words packed).  Asynchronous on `stream`. */
int int4linear_pack_s32_to_s4(const int *src_d, int *dst_d, int m, int n, void *stream);
int int4linear_unpack_s4_to_s32(const int *src_d, int *dst_d, int m, int n, void *stream);

/* The two halves of INT4LINEAR_KERNEL_FP6 on caller-owned memory, for callers whose
 * weights are static (a linear layer converts W once when it is loaded and X per call)
 * or who may not let the library allocate.  The reference has no counterpart: it
 * consumes the packed layout directly (kernels/linear_v21.cu:121-172).
 *   int4linear_fp6_operand_bytes  size of the converted form of a rows x k operand
 *                                 (0 if the FP6 kernel cannot take this k);
 *   int4linear_fp6_convert        packed s4 (rows x k/2 bytes) -> converted form;
 *                                 converted_d must be 256-byte aligned;
 *   int4linear_gemm_fp6_converted C = A * B^T from two converted operands.
 *   int4linear_linear_fp6_converted the same product with the epilogue of the
 *                                 int4linear_linear_* entry points fused into the store
 *                                 (bias_d, row_scale_d, col_scale_d may each be NULL; out_type
 *                                 is an INT4LINEAR_OUT_* value and y_d an m x n array of that
 *                                 type; INT4LINEAR_OUT_S32 takes a bias only).  The
 *                                 README's bias add (README.md:72) on the path a layer
 *                                 with static weights uses.
 * The converted form is opaque and specific to this library version.  Neither GEMM entry
 * point allocates or touches the library's workspace: both may be captured into a graph. */
size_t int4linear_fp6_operand_bytes(int rows, int k);
int int4linear_fp6_convert(const void *packed_d, void *converted_d, int rows, int k, void *stream);
int int4linear_gemm_fp6_converted(const void *a_conv_d, const void *b_conv_d, void *c_d,
                                  int m, int n, int k, void *stream);
int int4linear_linear_fp6_converted(const void *x_conv_d, const void *w_conv_d, const int *bias_d,
                                    const float *row_scale_d, const float *col_scale_d, void *y_d,
                                    int out_type, int m, int n, int k, void *stream);

/* Bytes of internal workspace INT4LINEAR_KERNEL_AUTO would use for a shape on the current
 * device (0 when the chosen kernel needs none).  Sets the device up if that has not
 * happened yet, so the answer does not depend on what was called before. */
size_t int4linear_workspace_bytes(int m, int n, int k);

/* Upper bound for the internal workspace (default 1 GiB).  Shapes that would need more,
 * and every shape when the limit is 0, run on the kernels that need no workspace. */
void int4linear_set_workspace_limit(size_t bytes);

/* Frees the current device's internal workspace (it is re-created on next need). */
int int4linear_release_workspace(void);

/* Name of the kernel INT4LINEAR_KERNEL_AUTO would pick for a shape on the current device
 * ("simple", "mfma", "fp6", "skinny"); never NULL.  Sets the device up like a compute call
 * does; without a usable device the answer is the one that depends on the shape alone. */
const char *int4linear_kernel_for_shape(int m, int n, int k);

/* Human-readable text for a status code; never NULL. */
const char *int4linear_status_string(int status);

/* hipError_t value of the most recent failing HIP call on this thread (0 if none). */
int int4linear_last_hip_error(void);

/* Number of compute units the library saw on the current device (0 before init). */
int int4linear_device_cu_count(void);

#ifdef __cplusplus
} /* extern "C" */

/*
 * The reference's entry points, C++ linkage, same signatures and semantics:
 * blocking (the call returns after the device has finished), default stream, void
 * return, silent on success.  As in the reference, each name is one step of the
 * optimisation history, here the one of this library's kernels:
 *   v0   scalar kernel, no matrix cores (also the independent on-device cross-check)
 *   v1   int8 MFMA kernel, 128x128 workgroup tile
 *   v2   int8 MFMA kernel, 256x256 workgroup tile
 *   v10  int8 MFMA kernel, tile chosen from the grid size
 *   v11  v10 plus the weight-streaming kernel for skinny M
 *   v20  v11 plus the FP6 kernel wherever it can run
 *   v21  the full automatic dispatch (what int4linear_gemm_s4s4s32 does)
 * A version whose kernel cannot take a shape falls back to the one before it, so every
 * name accepts every valid shape.
 *   kernels/linear_v0.h:168   kernels/linear_v1.h:208   kernels/linear_v2.h:284
 *   kernels/linear_v10.h:492  kernels/linear_v11.h:658  kernels/linear_v20.h:738
 *   kernels/linear_v21.h:760
 * A failing call prints one line to stderr (the reference prints only under __DEBUG,
 * kernels/linear_v21.cu:41-47).
 */
void linear_v0_launch(void *x_packed_d, void *w_packed_d, void *y_d, int m, int n, int k);
void linear_v1_launch(void *x_packed_d, void *w_packed_d, void *y_d, int m, int n, int k);
void linear_v2_launch(void *x_packed_d, void *w_packed_d, void *y_d, int m, int n, int k);
void linear_v10_launch(void *x_packed_d, void *w_packed_d, void *y_d, int m, int n, int k);
void linear_v11_launch(void *x_packed_d, void *w_packed_d, void *y_d, int m, int n, int k);
void linear_v20_launch(void *x_packed_d, void *w_packed_d, void *y_d, int m, int n, int k);
void linear_v21_launch(void *x_packed_d, void *w_packed_d, void *y_d, int m, int n, int k);

/* Host packer with the reference's signatures (utils/packer.h:5-6): host arrays in,
 * host arrays out. */
void pack(const int *src, int *dst, const int m, const int n);
void unpack(const int *src, int *dst, const int m, const int n);
#endif

#endif /* INT4LINEAR_H */
