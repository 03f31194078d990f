/*
 * kten_hip.h — C ABI of libkten_hip.so, the MI355X (gfx950) device side of a kten
 * backend. The Kotlin `HipRawTensor` / `HipTensorOperations` classes (or any FFI host:
 * Panama FFM, JNI, ctypes) bind exactly these entry points; each one names the member of
 * the reference's backend contract it serves. Reference paths are relative to the
 * reference root:
 *
 *   RAW = kten-api/src/main/kotlin/eu/redbean/kten/api/tensor/store/AbstractRawTensor.kt
 *   OPS = kten-api/src/main/kotlin/eu/redbean/kten/api/tensor/operations/TensorOperations.kt
 *   JVM = backend/kten-jvm/src/main/kotlin/eu/redbean/kten/jvm/tensor/store/JVMRawTensor.kt
 *   OCL = backend/kten-opencl/src/main/kotlin/eu/redbean/kten/opencl/tensor
 *
 * Conventions
 *   - Every call returns 0 (KTH_OK) or a negative KTH_E_* code; kth_last_error() gives
 *     the calling thread's message for the last failure. No exception crosses the ABI.
 *   - A buffer handle is an opaque uint64_t naming a device-resident fp32 store. All
 *     data is fp32, row-major contiguous; shapes are int32 with at most KTH_MAX_DIMS
 *     dims (OCL/platform/kernels/OCLKernelConstant.kt:4) and fewer than 2^31 elements
 *     (kten-api/.../autograd/utils/ShapeFunctions.kt:344).
 *   - Shapes travel by value inside the kernel arguments; nothing is uploaded per launch.
 *   - All launches are asynchronous on one internal in-order stream. The only blocking
 *     calls are kth_upload (above 1 MiB), kth_download, kth_read_scalar, kth_contains_nan, kth_sync,
 *     kth_gather / kth_scatter / kth_scatter_fill (they report bad index values) and
 *     kth_shutdown.
 *   - Shape / argument errors are reported before anything is launched, as the
 *     reference throws IllegalArgumentException host-side before computing
 *     (JVM:89-93, ShapeFunctions.kt:187-201).
 *   - Calls are serialised by one internal mutex; the reference is single-threaded by
 *     convention (kten-api/.../tensor/platform/PlatformProvider.kt:42-46).
 */
#ifndef KTEN_HIP_H
#define KTEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KTH_MAX_DIMS 10

/* status codes */
#define KTH_OK            0
#define KTH_E_NOT_INIT   -1   /* kth_init has not succeeded */
#define KTH_E_HANDLE     -2   /* unknown, stale or released handle */
#define KTH_E_ARGUMENT   -3   /* bad op code, size, range, dims > KTH_MAX_DIMS, null pointer */
#define KTH_E_SHAPE      -4   /* shapes do not broadcast / do not match */
#define KTH_E_MEMORY     -5   /* device allocation failed or pool cap exceeded */
#define KTH_E_DEVICE     -6   /* a HIP runtime call failed */

/* Operation codes. Numbering follows OCL/platform/kernels/OCLKernelConstant.kt:5-43 so a
 * Kotlin host can reuse that enum; KTH_NEG (unaryMinus, RAW:51) has no OpenCL code. */
enum kth_op {
    KTH_PLUS = 0, KTH_MINUS = 1, KTH_TIMES = 2, KTH_DIV = 3, KTH_POW = 4,
    KTH_RECIPROCAL = 5, KTH_LOG = 6,
    KTH_SUM = 7, KTH_MEAN = 8, KTH_MAX = 9, KTH_MIN = 10, KTH_ARG_MAX = 11, KTH_ARG_MIN = 12,
    KTH_LT = 13, KTH_LTE = 14, KTH_GT = 15, KTH_GTE = 16, KTH_EQ = 17, KTH_NEQ = 18,
    KTH_EXP = 19, KTH_TANH = 20, KTH_SIGMOID = 21, KTH_SINH = 22, KTH_COSH = 23, KTH_ABS = 24,
    KTH_SIGN = 25, KTH_SQRT = 26, KTH_SIN = 27, KTH_COS = 28, KTH_TAN = 29, KTH_ASIN = 30,
    KTH_ACOS = 31, KTH_ATAN = 32, KTH_FLOOR = 33, KTH_CEIL = 34, KTH_ROUND = 35, KTH_TRUNC = 36,
    KTH_RSQRT = 37,
    KTH_NEG = 40
};

/* ------------------------------------------------------------------ platform bring-up */

/* Select the device, create the stream and the buffer pool. Idempotent for the same
 * device. Serves the PlatformInitializer of a backend
 * (OCL/platform/OCLPlatformInitializer.kt:20-41, OCL/platform/OCLEnvironment.kt:203-300). */
int kth_init(int device);

/* Drain the stream and free every device buffer, live or pooled. */
int kth_shutdown(void);

/* Message for the calling thread's last failed call ("" if none). */
const char* kth_last_error(void);

/* Device name, total memory, compute-unit count and wavefront width: the fields a
 * backend puts into PlatformInfo (kten-api/.../tensor/platform/PlatformInfo.kt:3-9). */
int kth_device_info(char* name, size_t cap, uint64_t* total_mem, int* compute_units, int* wave_size);

/* PlatformProvider.epsilon (PlatformProvider.kt:12), used by EQ/NEQ as |a-b| < eps
 * (JVM:371-377,387-393). Default 1e-7f. */
int kth_set_epsilon(float eps);

/* How the transcendental maps (log exp tanh sinh cosh sin cos tan asin acos atan, and pow with a general exponent)
 * are evaluated. kotlin.math's Float overloads return the f64 libm value rounded once to fp32 (JVM:138-144,395-425).
 *   KTH_MATH_EXACT         f64 routines that return that float bit for bit (0 of 2^32 inputs differ for 10 of the
 *                          11 maps, 3 for log; pow a few per 10^8, by 1 ulp); the maps are then bound by f64
 *                          arithmetic, 1.1 to 1.6 times the time of a copy;
 *   KTH_MATH_WITHIN_2_ULP  fp32 routines (pow: a shorter f64 one) that stay within 2 units in the last place of that
 *                          float (measured over all 2^32 inputs: at most 1) at the time of a copy. The default.
 * Everything else is unaffected: + - x / sqrt abs neg floor ceil trunc round sign reciprocal rsqrt clamp, the
 * comparisons, pow with the exponents 2, 1, 3, 4, -1, -2, 0.5 and sigmoid (whose float expression, JVM:399, amplifies an
 * ulp of its exp) are the same bits in both modes. The mode is a property of the library, not of a store; it applies
 * to the calls made after it is set. */
#define KTH_MATH_EXACT        0
#define KTH_MATH_WITHIN_2_ULP 1
int kth_set_math_mode(int mode);
int kth_get_math_mode(int* mode);

/* PlatformProvider.memoryUsageScaleHint (PlatformProvider.kt:23-29): fraction of device
 * memory that live + pooled buffers may occupy; pooled buffers are freed first, then
 * kth_alloc fails with KTH_E_MEMORY. Default 0.85. */
int kth_set_memory_scale_hint(double fraction);

/* ------------------------------------------------------------------ stores */

/* A store of n_floats fp32 values (contents undefined), reference count 1. Buffers
 * come from a size-keyed reuse pool, the role of OCLEnvironment's reuse pool
 * (OCL/platform/OCLEnvironment.kt:36-200). Serves createRaw(shape) (OPS:16). */
int kth_alloc(uint64_t n_floats, uint64_t* handle);

/* incrementRef (OPS:28) and the store-sharing of copy(shallow=true) / view
 * (OCL/store/OCLRawTensor.kt:252-263). */
int kth_retain(uint64_t handle);

/* release (OPS:22): at zero the buffer returns to the pool (OCL/store/OCLRawTensor.kt:37-48). */
int kth_release(uint64_t handle);

/* Host -> device. Serves createRaw(shape, init) (OPS:11), fromCommonSerializable
 * (OPS:135) and the JVM -> device platform transformer. `src` may be reused as soon as
 * the call returns. Uploads of up to 1 MiB do not wait for the stream (they are staged
 * through pinned memory or, for a few values, carried in kernel arguments); larger ones
 * block until the copy is done. */
int kth_upload(uint64_t handle, uint64_t offset, const float* src, uint64_t n);

/* Device -> host after draining the stream. Serves toSerializableData (OPS:133) and
 * the device -> JVM platform transformer. */
int kth_download(float* dst, uint64_t handle, uint64_t offset, uint64_t n);

/* getSingleValue (RAW:166) / Tensor.item(). Blocking. */
int kth_read_scalar(uint64_t handle, uint64_t index, float* out);

/* copy(shallow=false) (RAW:168, JVM:257-262) and contiguous slice moves. A copy of the head of
 * `src` that fills the whole of `dst` (what copy() asks for) is put off: dst holds src's values
 * from this call on, but reads them from src's memory until either store is written, when the
 * copy is made first; if src is released before that, dst takes over its buffer. Nothing of this
 * shows in results; kth_metrics counts neither a launch nor bytes for a copy that was never made. */
int kth_copy(uint64_t dst, uint64_t dst_offset, uint64_t src, uint64_t src_offset, uint64_t n);

/* inplaceFill (RAW:244), zerosLike / zeroOut (OPS:24-26), createRawFill (OPS:18-20),
 * set(range, Float) on a contiguous range (RAW:35-37).
 * A fill that starts at offset 0 (and the upload of a single value at offset 0) is noted on the
 * store and launched only when some call reads the store as memory; every entry point sees the
 * filled values. Calls that can use the constant directly do so and produce the bits of the plain
 * sequence: kth_binary / kth_binary_inplace with + - x / take it as the scalar operand,
 * kth_scalar of such a store with + - x / yields another noted constant, kth_broadcast_to and a
 * whole-range kth_copy pass it on, kth_scatter / kth_scatter_fill (row form) and kth_index_add
 * (sorted form) start the target's rows from it, a result that overwrites the store drops it,
 * kth_release forgets it. */
int kth_fill(uint64_t handle, uint64_t offset, uint64_t n, float value);

/* containsNan (RAW:240, JVM:520-522). Blocking. */
int kth_contains_nan(uint64_t handle, uint64_t n, int* out);

/* ------------------------------------------------------------------ elementwise */

/* plus/minus/times/div/pow(tensor) (RAW:39,47,53,61,67; JVM:81-87,110-138) with the
 * broadcast fused into the kernel, and lt..neq(tensor) (RAW:194-199; JVM:355-377).
 * oshape must be the common shape of RAW:170-192; each operand must broadcast to it by
 * the rule of ShapeFunctions.kt:187-201 (else KTH_E_SHAPE). `out` must not alias an
 * operand unless all three shapes are equal. op: KTH_PLUS..KTH_POW, KTH_LT..KTH_NEQ. */
int kth_binary(int op,
               uint64_t a, const int32_t* ashape, int adims,
               uint64_t b, const int32_t* bshape, int bdims,
               uint64_t out, const int32_t* oshape, int odims);

/* plusAssign / timesAssign(tensor) (RAW:43,55; JVM:89-97,114,126): a[i] = a[i] op b[i]
 * on equal shapes (the host checks shape equality and throws, JVM:90-93). */
int kth_binary_inplace(int op, uint64_t a, uint64_t b, uint64_t n);

/* plus/minus/times/div/pow(Float) (RAW:41,49,57,63,69; JVM:99-103,112-140) and
 * lt..neq(Float) (RAW:201-206; JVM:379-393): out[i] = a[i] op c. reverse != 0 computes
 * c op a[i]; the contract needs it for TensorOperations.pow(constant, raw) (OPS:39).
 * out == a is allowed and gives plusAssign/timesAssign/divAssign(Float)
 * (RAW:45,59,65; JVM:105-108,116,130,136). pow with c == 1 into a store of its own (the backward
 * pass of pow(2) asks for it, `input pow constant - 1f`: kten-api/.../autograd/functions/
 * BasicFunctions.kt:193-198) is a copy of a and
 * is put off like the whole-store kth_copy. */
int kth_scalar(int op, uint64_t a, float c, int reverse, uint64_t out, uint64_t n);

/* unaryMinus, reciprocal, log (RAW:51,71,73; JVM:122,142,144) and exp..rsqrt
 * (RAW:208-227; JVM:395-435). op: KTH_NEG, KTH_RECIPROCAL, KTH_LOG, KTH_EXP..KTH_RSQRT.
 * out == a is allowed. */
int kth_unary(int op, uint64_t a, uint64_t out, uint64_t n);

/* clamp (RAW:215; JVM:409-411): min(max(x, lo), hi) with java.lang.Math NaN rules. */
int kth_clamp(uint64_t a, uint64_t out, uint64_t n, float lo, float hi);

/* broadcastTo (RAW:25; JVM:51-73): materialise src at dshape. The host returns `this`
 * without calling when the shapes are equal (JVM:52-53). */
int kth_broadcast_to(uint64_t src, const int32_t* sshape, int sdims,
                     uint64_t dst, const int32_t* dshape, int ddims);

/* ------------------------------------------------------------------ reductions */

/* aggregateOverAxis (RAW:75,92-119; JVM:154-225) on a tensor seen as
 * [outer, axis, inner] -> [outer, 1, inner]. op: KTH_SUM, KTH_MEAN, KTH_MAX, KTH_MIN,
 * KTH_ARG_MAX, KTH_ARG_MIN (indices stored as float, JVM:180; axis must be <= 2^24).
 * Deterministic: the same input gives the same bits on every call.
 * A small SUM / MEAN may return before anything is launched: `out` is then owed the reduction,
 * which runs when `out` is next read or `in` next written, or, when the next call sums `out`
 * over what was the inner dim (the next step of the autograd reduce-to-shape, mayUnexpand, kten-api/.../
 * autograd/functions/Utils.kt:14-41), as part of that call's one launch over `in`. The
 * values every call sees are those of the calls made in order; `in` may be released first. */
int kth_reduce_axis(int op, uint64_t in, uint64_t out, uint64_t outer, uint64_t axis, uint64_t inner);

/* sum() / mean() (RAW:121-122; JVM:146-152) of n values into out[0]. op: KTH_SUM, KTH_MEAN. */
int kth_reduce_all(int op, uint64_t in, uint64_t n, uint64_t out);

/* kth_reduce_axis for callers that cannot allocate: tight serving loops, harnesses that forbid
 * hipMalloc, hosts that keep device memory fixed while a HIP graph is being captured elsewhere in
 * the process. It has no counterpart in the reference. (The library launches on its own internal
 * stream, which a caller cannot put under capture: this entry point does not by itself make the
 * reduction part of a caller's graph; it only guarantees that the call creates nothing.)
 * Same arguments, checks and results (bit for bit: the same kernels and the same plan) as
 * kth_reduce_axis, but the partials of a two-pass reduction go to a fixed array of
 * kth_reduce_scratch_bytes() = 4 MiB in the library's device code instead of a pool
 * workspace, and the call creates nothing: no hipMalloc / hipFree, no pool traffic, no
 * events (its launches are counted by kth_metrics but left out of a kth_profile recording).
 * A shape whose plan needs more partial bytes than the array holds (outputs x axis segments
 * x 8 bytes; only reductions whose outputs alone cannot fill the device are cut into
 * segments) returns KTH_E_ARGUMENT before anything is launched, the fill an operand may still
 * be owed included (see kth_fill); single-pass shapes of any size are accepted. In an accepted
 * call an input that is a noted constant has its fill launched first: a kernel launch into the
 * store's own memory, nothing is allocated for it. Every call on a device shares that device's
 * array, which keeps the last call's partials; nothing in it needs clearing because every
 * partial is written before it is read. The library's mutex and its one in-order stream keep
 * calls of one process apart; anything that made two such calls overlap on one GPU would race
 * on the array. */
int kth_reduce_axis_static(int op, uint64_t in, uint64_t out, uint64_t outer, uint64_t axis, uint64_t inner);

/* Size of that array in bytes. */
int kth_reduce_scratch_bytes(uint64_t* bytes);

/* ------------------------------------------------------------------ indexed moves along an axis */

/* When the indexed moves below report an index value outside its axis. immediate != 0 (the default): every such
 * call waits for its own kernels and returns KTH_E_ARGUMENT itself, as the reference throws IllegalArgumentException
 * at the operation (JVM:238-239,345-346,494-496). immediate == 0: the calls do not wait; an out-of-range index sets a
 * flag on the device and the next blocking call (kth_sync, kth_download, kth_read_scalar, kth_contains_nan) returns
 * KTH_E_ARGUMENT in its place, once; what that call was asked for (the downloaded floats, the NaN answer) has been
 * delivered all the same. Either way the kernels skip the offending entry and the in-place target of a scatter or indexAdd has
 * been updated by the entries before it (the JVM, too, has assigned those when it throws).
 * In immediate mode a call does not wait when its index store is known to hold only valid values: an earlier indexed
 * move checked it against an axis no longer than this one (or kth_reduce_axis wrote it as ARG_MAX / ARG_MIN positions
 * of such an axis) and no call has taken the store since. Any call that takes the store other than as the index of
 * an indexed move forgets that, so a changed index is checked again and reported at its next use. */
int kth_set_index_check(int immediate);

/* gather (RAW:164; JVM:334-353). in and index have `dims` dims; out has index's shape:
 * out[p, i] = in[p, (int) index[p, i]] for every position p of index's shape without the
 * axis. index dims other than the axis must not exceed in's. Blocking: an index value
 * outside [0, in_shape[axis]) returns KTH_E_ARGUMENT, as the reference throws
 * IllegalArgumentException (JVM:345-346). */
int kth_gather(uint64_t in, const int32_t* in_shape, uint64_t index, const int32_t* index_shape,
               int dims, int axis, uint64_t out);

/* inplaceScatter / inplaceScatterAdd(axis, index, src) (RAW:146-148; JVM:227-255):
 * target[p, (int) index[p, i]] = (or +=, when add != 0) src[p, i], i ascending, so
 * duplicate indices inside one position resolve as on the JVM. Shape rule of
 * kten-api/.../autograd/utils/ShapeFunctions.kt:346-371 (else KTH_E_SHAPE). Blocking:
 * an out-of-range index returns KTH_E_ARGUMENT (JVM:238-239). */
int kth_scatter(int add, uint64_t target, const int32_t* target_shape, uint64_t index, const int32_t* index_shape,
                uint64_t src, const int32_t* src_shape, int dims, int axis);

/* inplaceScatter(axis, index, Float) (RAW:150; JVM:317-332). */
int kth_scatter_fill(uint64_t target, const int32_t* target_shape, uint64_t index, const int32_t* index_shape,
                     int dims, int axis, float value);

/* indexSelect (RAW:236; JVM:484-501): index holds k floats; out has `shape` with the axis
 * resized to k: out[p, i] = in[p, (int) index[i]]. Blocking: an index outside
 * [0, shape[axis]) returns KTH_E_ARGUMENT (JVM:494-496). */
int kth_index_select(uint64_t in, const int32_t* shape, int dims, int axis, uint64_t index, uint64_t k, uint64_t out);

/* indexAdd (RAW:238; JVM:503-516): target[p, (int) index[i]] += src[p, i] * alpha, i
 * ascending, so repeated indices accumulate in index order. src has `shape` with the axis
 * resized to k (checked on the host by ShapeFunctions.kt:280-293). Blocking, as above. */
int kth_index_add(uint64_t target, const int32_t* shape, int dims, int axis, uint64_t index, uint64_t k, uint64_t src, float alpha);

/* ------------------------------------------------------------------ layout movers */

/* get(Array<IntRange>) (RAW:29; JVM:276-280) and narrow (RAW:232; JVM:468-473): copies the
 * box first[d]..last[d] (inclusive, already normalised by the host as
 * kten-api/.../autograd/utils/ShapeFunctions.kt:240-259 does, one range per dim, unindexed
 * trailing dims given as 0..shape[d]-1) of `in` into `out` in row-major order, which is the
 * order in which the reference concatenates its sparse store ranges
 * (kten-api/.../tensor/store/AbstractIndexing.kt:65-88). A range outside its dim returns
 * KTH_E_ARGUMENT. get(IntArray) (RAW:27; JVM:270-274) selects one contiguous store range:
 * the host uses kth_copy for it. */
int kth_get_range(uint64_t in, const int32_t* shape, int dims, const int32_t* first, const int32_t* last, uint64_t out);

/* set(Array<IntRange>, tensor) (RAW:33; JVM:291-304): the first value_n
 * floats of `value` fill the box in row-major order. As in the reference only the element
 * count is compared (JVM:295-296): a different count returns KTH_E_SHAPE. set(IntArray,
 * tensor) (RAW:31; JVM:282-289) is one contiguous range: the host uses kth_copy. */
int kth_set_range(uint64_t target, const int32_t* shape, int dims, const int32_t* first, const int32_t* last,
                  uint64_t value, uint64_t value_n);

/* TensorOperations.concat(axis, inputs) (kten-api/.../tensor/operations/TensorOperations.kt:41), which every
 * backend of the reference builds from one range set per input at its offset along the axis
 * (backend/kten-jvm/.../operations/AbstractJVMTensorOperations.kt:106-120;
 * backend/kten-opencl/.../operations/OCLTensorOperations.kt:138-152). Here it is one launch that writes every
 * element of `out` once: out has `out_shape`; input i has the same shape except axis_lens[i] along `axis`
 * (already normalised), the lengths adding up to out_shape[axis] (else KTH_E_SHAPE; the host has checked the
 * other dims as ShapeFunctions.kt:85-104 does). Inputs of length 0 are allowed. `out` must not be one of the
 * inputs. */
int kth_concat(const uint64_t* inputs, const int32_t* axis_lens, int n_inputs, const int32_t* out_shape, int dims, int axis,
               uint64_t out);

/* set(Array<IntRange>, Float) (RAW:37; JVM:311-315). set(IntArray, Float) (RAW:35;
 * JVM:306-309) is one contiguous range: the host uses kth_fill. */
int kth_fill_range(uint64_t target, const int32_t* shape, int dims, const int32_t* first, const int32_t* last, float value);

/* transpose (RAW:228; JVM:437-451): out has `shape` with dims axis1 and axis2 (already
 * normalised, different) exchanged, out[.., i at axis1, .., j at axis2, ..] =
 * in[.., j at axis1, .., i at axis2, ..]: the axis swap the contract documents
 * (kten-api/.../tensor/Tensor.kt:1028-1058) and the reference's OpenCL backend computes
 * (backend/kten-opencl/src/main/resources/kernels.cl:263-287). kten-jvm's slab copy gives
 * the same result when the axes are adjacent or every dim between them has size 1, and a
 * different element order otherwise. */
int kth_transpose(uint64_t in, const int32_t* shape, int dims, int axis1, int axis2, uint64_t out);

/* permute (RAW:230; JVM:453-466): out.shape[d] = shape[axes[d]] and the element at
 * multi-index t of `in` lands at (t[axes[0]], t[axes[1]], ..) of out. axes must name every
 * dim once (ShapeFunctions.kt:106-113), else KTH_E_ARGUMENT. */
int kth_permute(uint64_t in, const int32_t* shape, int dims, const int32_t* axes, uint64_t out);

/* maskedFill (RAW:246; JVM:537-540): out[i] = mask'[i] == 1f ? value : a[i] where mask' is
 * the mask broadcast to a's shape inside the kernel (JVM:538 materialises it). A mask that
 * does not broadcast to a's shape returns KTH_E_SHAPE. out may be a. */
int kth_masked_fill(uint64_t a, const int32_t* ashape, int adims, uint64_t mask, const int32_t* mshape, int mdims,
                    float value, uint64_t out);

/* ------------------------------------------------------------------ fused batch normalisation */

/* BatchNormOperation.calculateOutput (kten-api/.../tensor/operations/nn/BatchNormOperation.kt:7-13,
 * obtained from TensorOperations.batchNorm(axis, momentum, epsilon, training),
 * kten-api/.../tensor/operations/TensorOperations.kt:129; arithmetic of
 * backend/kten-jvm/.../operations/nn/JVMBatchNorm.kt:33-99). `in` has `shape`; every
 * per-channel tensor holds shape[axis] floats. running_mean and running_var are both given
 * or both 0 (a handle is never 0); they are required when training == 0 and are updated in
 * place when training != 0. gamma and beta may be 0 (1 and 0). Outputs: out (same shape),
 * current_mean and current_std = 1 / sqrt(var + epsilon) per channel (zeros in inference
 * mode, as the reference leaves them). */
int kth_batch_norm_forward(uint64_t in, const int32_t* shape, int dims, int axis, int training, float momentum, float epsilon,
                           uint64_t running_mean, uint64_t running_var, uint64_t gamma, uint64_t beta,
                           uint64_t out, uint64_t current_mean, uint64_t current_std);

/* BatchNormOperation.calculateGrads (BatchNormOperation.kt:15-26; JVMBatchNorm.kt:101-183).
 * grad_in, grad_gamma, grad_beta are outputs; 0 means "not required" (the reference's
 * inRequiresGrad / gammaRequiresGrad / betaRequiresGrad flags). Training mode reads
 * current_mean / current_std as returned by the forward call, inference mode reads
 * running_mean / running_var. */
int kth_batch_norm_backward(uint64_t in, const int32_t* shape, int dims, int axis, int training, float epsilon,
                            uint64_t running_mean, uint64_t running_var, uint64_t current_mean, uint64_t current_std,
                            uint64_t gamma, uint64_t grad_out, uint64_t grad_in, uint64_t grad_gamma, uint64_t grad_beta);

/* ------------------------------------------------------------------ control and metrics */

/* Wait for everything launched so far. */
int kth_sync(void);

/* PlatformMetricsProvider.getMetrics (kten-api/.../operations/PlatformMetricsProvider.kt:3-6,
 * OCL/platform/OCLEnvironment.kt:89-96): bytes in live stores, bytes parked in the pool,
 * kernel launches so far, and the algorithmic bytes those launches moved (operands at
 * their un-broadcast size plus the output, 4 bytes each). Any pointer may be NULL. */
int kth_metrics(uint64_t* live_bytes, uint64_t* pool_bytes, uint64_t* launches, uint64_t* bytes_moved);

#ifdef __cplusplus
}
#endif
#endif /* KTEN_HIP_H */
