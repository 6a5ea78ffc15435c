/*
 * C-ABI of the MI355X runtime for onnx-mlir's int8 quantized-inference path.
 *
 * Each op entry point is the target of one `krnl.call` emitted by the MI355X
 * accelerator's ONNX->Krnl patterns.  The calling convention is the one
 * KrnlCallOpLowering generates (src/Conversion/KrnlToLLVM/KrnlCall.cpp:34-102):
 * a plain C call returning void whose parameters are, in order, the op's
 * OUTPUT tensors, then its INPUT tensors (src/Dialect/Krnl/Krnl.td:59-66),
 * then its attributes in name-sorted order (KrnlCall.cpp:61-69); memrefs
 * arrive as non-owning `OMTensor *` wrappers (KrnlCall.cpp:121-138), an
 * absent optional operand as NULL (KrnlCall.cpp:139-145), integer attributes
 * as int64_t (KrnlCall.cpp:164-226).  Outputs are pre-allocated by the caller
 * and the callee never allocates, frees or retains a tensor
 * (src/Dialect/Krnl/Krnl.td:62).
 *
 * A tensor's data pointer may be ordinary host memory (what a compiled model
 * passes) or GPU memory (what a caller that keeps tensors resident passes,
 * e.g. memory from om_mi355x_malloc); GPU memory is used in place without a
 * copy.
 *
 * No entry point reports failure through a return value (a krnl.call target
 * has none).  On a HIP error or an unsupported argument the entry point prints
 * a message to stderr, sets errno (EIO / EINVAL) and records the message for
 * om_mi355x_last_error(); the outputs are then unspecified.
 */
#ifndef OM_MI355X_H
#define OM_MI355X_H

#include <stddef.h>
#include <stdint.h>

#include "om_tensor_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- accelerator life cycle -------------------------------------------- */
/* Names and semantics fixed by the generated entry point
 * (src/Conversion/KrnlToLLVM/KrnlEntryPoint.cpp:149-186,409-428); pattern of
 * src/Accelerators/NNPA/Runtime/OMRuntimeNNPA.c:91,105-118,159-228,241-250. */
extern long OMIsInitAccelMI355X;
void OMInitAccelMI355X(void);
/* Returns non-zero when a model compiled for `versionNum` can run on this
 * runtime and device; otherwise sets errno = EPERM and returns 0. */
uint64_t OMInitCompatibleAccelMI355X(uint64_t versionNum);
void OMShutdownAccelMI355X(void);

/* Version of this runtime, encoded 0x00MMmmpp.  The major number changes with
 * every change of an existing signature (1: the fused entry points gained
 * `activation`), the minor number with every entry point added that
 * generated code may call (1: om_mi355x_SetQuantMode, activation = 2). */
#define OM_MI355X_VERSION 0x00010100ULL

/* ---- compiler options that change this path's arithmetic ------------------ */
/* The reference compiles QuantizeLinear / DynamicQuantizeLinear differently
 * under two of its options, and DequantizeLinear under one:
 *   OM_MI355X_QUANT_RECIPROCAL     --enable-fast-math at -O3
 *     (src/Compiler/CompilerPasses.cpp:298-301): the quotient x / scale
 *     becomes x * (1 / scale), one f32 divide per scale
 *     (src/Conversion/ONNXToKrnl/Quantization/QuantizeLinear.cpp:43-44,119-132);
 *   OM_MI355X_QUANT_NO_ZERO_POINT  --disable-quantization-zero-point
 *     (src/Compiler/CompilerOptions.cpp:255-262): QuantizeLinear and
 *     DequantizeLinear ignore the zero point they are given (it still fixes
 *     the 8-bit type; QuantizeLinear.cpp:231-237, Elementwise.cpp:1453), and
 *     DynamicQuantizeLinear returns a zero point of 0 and adds none
 *     (DynamicQuantizeLinear.cpp:75-84,142-152).
 * The form is a property of the compiled model in the reference, so here it
 * is a property of each op, never a lasting state of the thread:
 * om_mi355x_SetQuantMode(anchor, mode) applies to the NEXT call of
 * om_mi355x_QuantizeLinear, om_mi355x_DequantizeLinear,
 * om_mi355x_DynamicQuantizeLinear[NoAlloc] or om_mi355x_DynQuantMatMulDequant
 * that the calling thread makes.  That call takes the mode (mode: 0, the
 * default, or a combination of the two bits) when it is entered -- also when
 * it then fails -- and leaves 0 behind, so an op that no SetQuantMode call
 * precedes always computes the default form, whatever model ran on the thread
 * before.  Code compiled with either option calls it in front of each of these
 * ops ("krnl.call"(%y) {funcName = "om_mi355x_SetQuantMode", mode = 3 : si64,
 * numOfOutput = 1 : si64}); code compiled without them calls nothing.  The
 * other entry points neither read nor change the pending mode.  `anchor` is
 * not used: generated code names the op's result buffer there, as an output,
 * because a krnl.call without an operand it writes counts as dead and is
 * removed (and writing the same buffer keeps the pair in order); other callers
 * pass NULL.  om_mi355x_GetQuantMode returns the mode the thread's next such
 * op would take.  Any value outside 0..3 is refused (EINVAL) and leaves the
 * pending mode as it was. */
#define OM_MI355X_QUANT_RECIPROCAL 1
#define OM_MI355X_QUANT_NO_ZERO_POINT 2
void om_mi355x_SetQuantMode(OMTensor *anchor, int64_t mode);
int64_t om_mi355x_GetQuantMode(void);

/* ---- ops ---------------------------------------------------------------- */

/* onnx.QuantizeLinear.  Replaces the loop nest generated by
 * ONNXQuantizeLinearOpLowering
 * (src/Conversion/ONNXToKrnl/Quantization/QuantizeLinear.cpp:155-246).
 * y: ui8/i8 (type follows y_zp, ui8 when absent), x: f32, y_scale: f32 scalar
 * or 1-D [x.shape[axis]], y_zp: NULL or same shape as y_scale.
 * `saturate` only matters for float8 outputs and is ignored. */
void om_mi355x_QuantizeLinear(OMTensor *y, const OMTensor *x,
    const OMTensor *y_scale, const OMTensor *y_zp, int64_t axis,
    int64_t saturate);

/* onnx.DequantizeLinear.  Replaces emitScalarOpFor<ONNXDequantizeLinearOp>
 * (src/Conversion/ONNXToKrnl/Math/Elementwise.cpp:1439-1461).
 * x: ui8/i8/i32, x_scale: f32 scalar or 1-D, x_zp: NULL or like x_scale with
 * x's element type, y: f32. */
void om_mi355x_DequantizeLinear(OMTensor *y, const OMTensor *x,
    const OMTensor *x_scale, const OMTensor *x_zp, int64_t axis);

/* onnx.DynamicQuantizeLinear.  Replaces ONNXDynamicQuantizeLinearOpLowering
 * (src/Conversion/ONNXToKrnl/Quantization/DynamicQuantizeLinear.cpp:86-158).
 * Three outputs: y ui8 (x's shape), y_scale f32 scalar, y_zp ui8 scalar. */
void om_mi355x_DynamicQuantizeLinear(
    OMTensor *y, OMTensor *y_scale, OMTensor *y_zp, const OMTensor *x);

/* DynamicQuantizeLinear for callers that cannot allocate.  This entry point
 * has no counterpart in the reference; it exists for callers that must not
 * reach hipMalloc / hipFree while they run: tight serving loops, harnesses
 * that forbid allocation, a thread that has a HIP graph capture open on a
 * stream of its own.  (The call's kernels run on the runtime's stream of the
 * calling thread, which is private: they are not recorded into the caller's
 * graph.  Should that stream itself be under capture, the entry point records
 * its two-launch form, which replays correctly; the one-launch kernel carries
 * a launch number and would not.)  Same operands and results as
 * om_mi355x_DynamicQuantizeLinear, with these conditions:
 *  - every tensor's data pointer is GPU memory (om_mi355x_malloc, or a host
 *    buffer declared with om_mi355x_KeepOnDevice); a host tensor is refused
 *    (EINVAL), because staging it could allocate;
 *  - the calling thread has used the runtime before (any entry point, e.g.
 *    om_mi355x_synchronize()), so that its stream exists; otherwise EINVAL;
 *  - x has at most OM_MI355X_NOALLOC_MAX_ELEMENTS elements; more is refused
 *    (EINVAL).
 * The kernels' scratch (per-block minima / maxima, arrival counter, exchange
 * slots: 12,544 bytes) is a fixed array in the library's GPU image, one copy
 * per GPU, shared by every call on that GPU: calls that overlap in time on one
 * GPU (from different threads) race on it and must be serialised by the
 * caller.  The call returns once its kernels are queued on the calling
 * thread's stream; failures of the kernels are reported by the next
 * om_mi355x_synchronize(). */
#define OM_MI355X_NOALLOC_MAX_ELEMENTS ((int64_t)1 << 31)
void om_mi355x_DynamicQuantizeLinearNoAlloc(
    OMTensor *y, OMTensor *y_scale, OMTensor *y_zp, const OMTensor *x);

/* onnx.MatMulInteger.  Replaces ONNXMatMulIntegerOpLowering
 * (src/Conversion/ONNXToKrnl/Math/MatMulInteger.cpp:26-93) and the int32
 * MatMul under it (src/Conversion/ONNXToKrnl/Math/MatMul.cpp:278-327).
 * y: i32 [M,N]; a: ui8/i8 [M,K]; b: ui8/i8 [K,N]; a_zp: NULL, scalar/[1] or
 * [M]; b_zp: NULL, scalar/[1] or [N].  Leading batch dimensions of `a` are
 * folded into M when b is 2-D.  With a batched b ([.., K, N]) the batch
 * dimensions of a and b are paired as in
 * src/Dialect/ONNX/ONNXOps/Math/MatMul.cpp:200-292 (right-aligned, a
 * dimension of 1 broadcasts), one GEMM per pair; a_zp may then also be
 * [.., M, 1] and b_zp [.., 1, N], one row / column vector per matrix of the
 * operand it belongs to.  A 1-D a is a row ([K] -> [1,K]) and a 1-D b a column
 * ([K] -> [K,1]), and that dimension is dropped from y. */
void om_mi355x_MatMulInteger(OMTensor *y, const OMTensor *a,
    const OMTensor *b, const OMTensor *a_zp, const OMTensor *b_zp);

/* onnx.QLinearMatMul.  Replaces ONNXQLinearMatMulOpLowering
 * (src/Conversion/ONNXToKrnl/Math/QLinearMatMul.cpp:26-143).
 * narrow_mode 0 = wrap (what the reference computes: trunci, :134-138),
 *             1 = saturate (what the ONNX specification says).
 * Operand ranks and batch pairing as for om_mi355x_MatMulInteger; a_scale,
 * y_scale and y_zp are scalars; b_scale is a scalar or, beyond what the
 * reference's lowering takes (:53-68 refuses it), one value per column of b
 * ([N]): column j is then scaled by (a_scale * b_scale[j]) / y_scale, the
 * reference's expression (:127) with that column's scale. */
void om_mi355x_QLinearMatMul(OMTensor *y, const OMTensor *a,
    const OMTensor *a_scale, const OMTensor *a_zp, const OMTensor *b,
    const OMTensor *b_scale, const OMTensor *b_zp, const OMTensor *y_scale,
    const OMTensor *y_zp, int64_t narrow_mode);

/* Fused MatMulInteger -> Cast(f32) -> Mul(a_scale * b_scale) [-> Add(bias)]:
 * the graph shape documented at
 * src/Accelerators/NNPA/Conversion/ONNXToZHigh/ONNXToZHigh.cpp:1021-1060, with
 * the bias C of a linear layer `A*B+C` (which that accelerator folds into its
 * matmul's bias operand, :440-470).  y: f32 [M,N]; a_scale: f32 scalar;
 * b_scale: f32 scalar or [N]; bias: NULL, f32 scalar or [N], added to the
 * rounded product as onnx.Add would.  activation: 0 = none, 1 = a following
 * onnx.Relu, max(0, x) with NaN -> 0 as the reference's lowering computes it
 * (src/Conversion/ONNXToKrnl/Math/Elementwise.cpp:746-754); 2 = a following
 * onnx.Gelu with approximate = "none", (0.5 * x) * (1 + erf(x * f32(1/sqrt 2)))
 * in the operation order of the reference's lowering (Elementwise.cpp:374-388).
 * The reference's erf is a polynomial approximation that its compiler expands
 * (src/Conversion/KrnlToLLVM/ConvertKrnlToLLVM.cpp:223-225); the one used here
 * is within 2^-22 of erf everywhere, so the result agrees with the
 * reference's to that times |0.5 x|, not bit for bit.  Any other value is
 * refused. */
#define OM_MI355X_ACTIVATION_NONE 0
#define OM_MI355X_ACTIVATION_RELU 1
#define OM_MI355X_ACTIVATION_GELU 2
void om_mi355x_MatMulIntegerDequant(OMTensor *y, const OMTensor *a,
    const OMTensor *b, const OMTensor *a_zp, const OMTensor *b_zp,
    const OMTensor *a_scale, const OMTensor *b_scale, const OMTensor *bias,
    int64_t activation);

/* Fused DynamicQuantizeLinear(x) -> MatMulInteger(., b) -> Cast -> Mul
 * [-> Add(bias)]: the whole dynamically quantized linear layer of the
 * reference's graphs (ONNXToZHigh.cpp:895-912).  y: f32 [M,N]; x: f32 [M,K];
 * b: i8/ui8 [K,N]; b_zp: NULL, scalar or [N]; b_scale: f32 scalar or [N];
 * bias: NULL, f32 scalar or [N]; activation as for
 * om_mi355x_MatMulIntegerDequant.  The quantized activations never leave the
 * GPU. */
void om_mi355x_DynQuantMatMulDequant(OMTensor *y, const OMTensor *x,
    const OMTensor *b, const OMTensor *b_zp, const OMTensor *b_scale,
    const OMTensor *bias, int64_t activation);

/* The same layer in a chain of such layers (FFN-up -> Gelu -> FFN-down).
 * DynamicQuantizeLinear starts with two reductions over its whole input,
 * ReduceMin and ReduceMax
 * (src/Conversion/ONNXToKrnl/Quantization/DynamicQuantizeLinear.cpp:100-110),
 * before it can quantize any of it; when the input is the result of the layer
 * before, that layer's kernel can take them over what it stores.
 *   y_limits: NULL, or f32[2] that receives min(y) and max(y) over all
 *             elements of y, NaN ignored (what those reductions give; zero
 *             is not included yet);
 *   x_limits: NULL, or f32[2] holding min(x) and max(x) in that sense, as an
 *             earlier call's y_limits received them for this very tensor: the
 *             call then quantizes x in one pass without looking for them.
 *             Values that are not x's minimum and maximum give a different
 *             scale and zero point than DynamicQuantizeLinear(x) would.
 * Everything else, and every bit of y, as om_mi355x_DynQuantMatMulDequant. */
void om_mi355x_DynQuantMatMulDequantLimits(OMTensor *y, OMTensor *y_limits,
    const OMTensor *x, const OMTensor *x_limits, const OMTensor *b,
    const OMTensor *b_zp, const OMTensor *b_scale, const OMTensor *bias,
    int64_t activation);

/* ---- residency ---------------------------------------------------------- */
/* Declares that the host buffer behind `t` never changes for the life of the
 * process (a krnl.global constant: src/Conversion/KrnlToLLVM/KrnlGlobal.cpp
 * :74-200).  Its GPU copy, and for a matmul right-hand side its packed form
 * and column sums, are then made once and reused. */
void om_mi355x_MarkConstant(const OMTensor *t);
/* Takes the declaration back before the buffer is freed or changed: the GPU
 * copy and the packed form made for it are dropped (after the work that may
 * still read them). */
void om_mi355x_UnmarkConstant(const OMTensor *t);
/* Drops every cached GPU copy and packed weight. */
void om_mi355x_ClearCache(void);
/* Declares that, until om_mi355x_Release, the host buffer behind `t` is read
 * and written only through entry points of this library (an intermediate
 * result that a compiled model allocated with memref.alloc and that feeds
 * nothing but other offloaded ops).  The runtime backs it with GPU memory of
 * the same size: entry points given that buffer, or a part of it, use the GPU
 * memory in place -- no staging, no copy back, no synchronisation -- and the
 * host buffer itself is never touched.  This is how tensors stay on the device
 * between the quantized ops of a compiled model; it has no counterpart in the
 * reference, whose accelerators describe device layouts in the type system
 * instead (src/Accelerators/NNPA/Dialect/ZLow).  Release must come before the
 * buffer is freed or reused (the accelerator pass puts it after the last
 * offloaded user, which keeps the memref.dealloc behind it).  The GPU memory
 * comes from the calling thread's pool and returns to it, so repeated
 * inferences do not allocate; a release from the declaring thread does not
 * wait (later users of the memory are ordered behind it on that thread's
 * stream), one from another thread waits for the declaring thread's work. */
void om_mi355x_KeepOnDevice(const OMTensor *t);
void om_mi355x_Release(const OMTensor *t);

/* ---- GPU memory for callers that keep tensors resident ------------------ */
void *om_mi355x_malloc(size_t bytes);
void om_mi355x_free(void *dev_ptr);
int om_mi355x_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes);
int om_mi355x_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes);
/* Waits for all work the calling thread has issued; 0, or -1 with the error
 * kept for om_mi355x_last_error(). */
int om_mi355x_synchronize(void);
/* The same for generated code, which reaches the runtime through krnl.call
 * and passes every operand as an OMTensor*: "krnl.call"(%y) {funcName =
 * "om_mi355x_Synchronize", numOfOutput = 1 : si64}.  `anchor` is not read
 * (naming one buffer as an output keeps the call from being removed as
 * dead); a failure is kept for om_mi355x_last_error() and shows at the next
 * entry point. */
void om_mi355x_Synchronize(OMTensor *anchor);

/* ---- measurement --------------------------------------------------------- */
/* Brackets subsequent entry-point calls of this thread with HIP events on the
 * runtime's own stream.  om_mi355x_timer_stop waits and returns the elapsed
 * milliseconds, or a negative value on error. */
int om_mi355x_timer_start(void);
float om_mi355x_timer_stop(void);

/* Last error message of the calling thread ("" if none); clears it. */
const char *om_mi355x_last_error(void);
/* Name of the GEMM kernel that the calling thread's last matmul entry point
 * launched ("" before the first). */
const char *om_mi355x_last_gemm_kernel(void);
/* Fills `buf` with "name|arch|CUs|clockMHz|memGiB" of device 0. */
int om_mi355x_device_info(char *buf, size_t len);

#ifdef __cplusplus
}
#endif
#endif
