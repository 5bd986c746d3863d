/* maidenx_hip — C ABI of the MI355X (gfx950) compute backend for MaidenX.
 *
 * Every entry point is what maidenx_core::be::* would bind for a `Device::HIP` arm: the symbol
 * family `hip_<op>_<dtype>` mirrors `cuda_<op>_<dtype>` of crates/maidenx_cuda (same argument
 * order and meaning), with the numerical semantics of crates/maidenx_cpu.
 *
 * Conventions
 *  - Data pointers are device pointers obtained from hip_malloc.  `metadata` pointers are HOST
 *    pointers (as on the reference's CPU arm, crates/maidenx_core/src/be/ops/binary.rs:113-116);
 *    their contents are consumed before the call returns.
 *  - dtype suffixes: f32 = float, bf16 = the upper 16 bits of an IEEE binary32 (uint16_t storage),
 *    bool = one byte holding 0 or 1.
 *  - Kernels are queued on one in-order stream (hip_set_stream, default: the device's default
 *    stream) and return without waiting.  hip_memcpy_d2h / hip_memcpy_h2d wait for completion.
 *  - Kernel wrappers return void like the reference's; the first error since the last query is
 *    kept and read with hip_get_last_status() / hip_status_string().
 *  - Outputs are fully overwritten; no entry point relies on the incoming contents of an output.
 *  - Strided operands must have fewer than 2^31 logical elements (contiguous ones have no limit).
 */
#ifndef MAIDENX_HIP_H
#define MAIDENX_HIP_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t mx_bf16;   /* bf16 bit pattern */
typedef uint16_t mx_f16;    /* IEEE binary16 bit pattern (the `half` crate's f16) */
typedef uint8_t mx_bool;    /* 0 or 1 */

/* ---- status ------------------------------------------------------------------------------------ */
#define MX_HIP_OK 0
#define MX_HIP_ERR_INVALID 1
#define MX_HIP_ERR_OOM 2          /* crates/maidenx_core/src/error.rs:144-150 maps code 2 to OutOfMemory */
#define MX_HIP_ERR_TOO_LARGE 3
#define MX_HIP_ERR_LAUNCH 4
#define MX_HIP_ERR_UNSUPPORTED 5
int hip_get_last_status(void);          /* first error since the previous call; clears it */
const char* hip_status_string(void);    /* text for the status last returned */

/* ---- device / memory / stream: replaces crates/maidenx_cuda/src/lib.rs:39-152 --------------------
 * (cuda_malloc, cuda_free, cuda_memcpy_h2d/d2h/d2d, cuda_set_device, cuda_get_device,
 *  cuda_stream_create/destroy/synchronize).  Return 0 on success; hip_malloc returns 2 when the
 *  device is out of memory. */
int hip_set_device(int device_id);
int hip_get_device(int* device_id);
int hip_device_count(int* count);
int hip_malloc(void** ptr, size_t size);
int hip_free(void* ptr);
int hip_memcpy_h2d(void* dst, const void* src, size_t size);
int hip_memcpy_d2h(void* dst, const void* src, size_t size);
int hip_memcpy_d2d(void* dst, const void* src, size_t size);
int hip_stream_create(void** stream);
int hip_stream_destroy(void* stream);
int hip_stream_synchronize(void* stream);
int hip_set_stream(void* stream);       /* stream used by every later kernel/copy (NULL = default); waits for the work
                                           queued on the previous stream first (the scratch buffers are one per device),
                                           unless that stream is being captured */
void* hip_get_stream(void);
int hip_synchronize(void);              /* wait for everything queued on the backend's stream */
/* events recorded on the backend's stream (no counterpart in the reference; used for timing) */
int hip_event_create(void** event);
int hip_event_destroy(void* event);
int hip_event_record(void* event);
int hip_event_synchronize(void* event);
int hip_event_elapsed_ms(void* start, void* stop, float* ms);
/* Graph capture of a launch-bound call sequence (no counterpart in the reference).  begin_capture drains the
 * device and routes every later kernel of this library to a capture stream; end_capture returns an executable
 * graph and restores the previous stream; graph_launch replays it in stream order.  While capturing, the caller
 * must issue nothing that allocates, copies to the host or synchronises: warm the same sequence up eagerly first,
 * so that the library's scratch has its final size (a call that would have to grow it fails with
 * MX_HIP_ERR_INVALID instead).  Fill with hip_fill_*, not memset. */
int hip_graph_begin_capture(void);
int hip_graph_end_capture(void** graph_exec);
int hip_graph_launch(void* graph_exec);
int hip_graph_destroy(void* graph_exec);
/* A capture whose launches are all small kernels with an interpreter body (f32 elementwise, row reductions,
 * the per-thread and per-block small matmul kernels; tensors of at most 4096 elements) is kept as a "program": its
 * replay is ONE launch of a single work-group that runs the recorded kernels in order, which costs a fraction
 * of a microsecond per kernel instead of the 1.6 us and more of a graph node.  Any other capture is a plain HIP graph.
 * No counterpart in the reference.  hip_graph_is_program: 1 / 0 for a handle of hip_graph_end_capture;
 * hip_graph_set_programs: allow (1, default) or forbid (0) programs for later captures, returns the old value. */
int hip_graph_is_program(void* graph_exec);
int hip_graph_set_programs(int enabled);
/* Inside a capture that is not a program, consecutive f32 elementwise launches over one index space (at most two
 * collapsed dims, fewer than 2^20 elements) that meet each other's data only element for element are recorded as ONE
 * kernel node that applies them in order per element (each output is still written; same bytes as separate launches).
 * hip_graph_fused_launches: how many launches of the capture were fused, and into how many nodes;
 * hip_graph_set_fusion: allow (1, default) or forbid (0) this for later captures, returns the old value.
 * No counterpart in the reference. */
int hip_graph_fused_launches(void* graph_exec, int* nodes);
int hip_graph_set_fusion(int enabled);
/* A capture whose every launch is one of those the fused chains take (f32 elementwise over at most two collapsed dims,
 * the one-thread-per-output matmul, a row sum that one work-group does, the few-output long-reduction matmul, the fused MSE
 * loss), each over tensors of at most 8192 elements (hip_graph_set_resident), is kept as a "resident step program": nothing is launched while it is recorded, and a replay
 * is ONE launch of ONE 512-thread work-group that runs the recorded kernels in order with the tensors they write held
 * in LDS for as long as they are alive, a work-group barrier only in front of kernels that read across threads, and
 * memory written once, at the end, for what is still alive then.  Same functors, same device functions, same order of
 * additions as the eager kernels: the same bytes.  It takes the place of a "program" above (which it subsumes) unless
 * switched off.  No counterpart in the reference.
 * hip_graph_launch_n: `times` replays in a row; a resident step program makes them in one launch, with the tensors one
 *   replay hands to the next (parameters) staying in LDS - the final state of memory is that of `times` replays.
 * hip_graph_is_resident: number of recorded kernels of the resident step program behind a handle, 0 when it is not one;
 *   lds_operands / barriers (may be NULL): operand references served from LDS, barriers per replay.
 * hip_graph_set_resident: the largest tensor, in elements, that a launch of a later capture may touch for the capture
 *   to be kept this way: 0 never, at most 65536, default 8192 (one work-group's instruction stream is what a recorded
 *   kernel costs - about 0.7 us up to 2048 elements, 1.5 us for 10000, where the fused chains are ahead again: a
 *   Linear(3 -> 1) + MSE + SGD step on 1000 rows replays in 14.2 us this way and 19.0 us as chains, on 10000 rows in 34 and 23);
 *   returns the old value.
 * hip_buffer_discard: a hint that the contents of [ptr, ptr + bytes) are no longer needed (a caching allocator calls it
 *   when a buffer goes back to its pool, where the reference would call cuda_free, crates/maidenx_cuda/src/lib.rs:
 *   55-63).  Inside a capture it lets a resident step program leave such tensors in LDS only; otherwise it does nothing. */
int hip_graph_launch_n(void* graph_exec, size_t times);
int hip_graph_is_resident(void* graph_exec, int* lds_operands, int* barriers);
int hip_graph_set_resident(int max_elements);
void hip_buffer_discard(void* ptr, size_t bytes);

/* ---- binary: replaces crates/maidenx_cuda/src/ops/binary.rs:12-161 --------------------------------
 * metadata = dims[n] | lhs_strides[n] | rhs_strides[n] | lhs_offset | rhs_offset   (NULL: contiguous)
 * Semantics: crates/maidenx_cpu/src/ops/binary.rs:13-124 (out-of-place, contiguous output),
 * :126-248 (in place, written through the lhs strides), :250-368 (logical).
 * div: b == 0 gives (a == 0 ? 0 : +INF). */
#define MX_DECL_BINARY(T, S)                                                                              \
    void hip_add_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, T* out);     \
    void hip_sub_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, T* out);     \
    void hip_mul_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, T* out);     \
    void hip_div_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, T* out);     \
    void hip_maximum_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, T* out); \
    void hip_minimum_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, T* out); \
    void hip_logical_and_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, mx_bool* out); \
    void hip_logical_or_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, mx_bool* out);  \
    void hip_logical_xor_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, mx_bool* out); \
    void hip_eq_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, mx_bool* out); \
    void hip_ne_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, mx_bool* out); \
    void hip_lt_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, mx_bool* out); \
    void hip_le_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, mx_bool* out); \
    void hip_gt_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, mx_bool* out); \
    void hip_ge_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* lhs, const T* rhs, mx_bool* out); \
    void hip_add_inplace_##S(size_t num_els, size_t num_dims, const size_t* metadata, T* lhs, const T* rhs); \
    void hip_sub_inplace_##S(size_t num_els, size_t num_dims, const size_t* metadata, T* lhs, const T* rhs); \
    void hip_mul_inplace_##S(size_t num_els, size_t num_dims, const size_t* metadata, T* lhs, const T* rhs); \
    void hip_div_inplace_##S(size_t num_els, size_t num_dims, const size_t* metadata, T* lhs, const T* rhs);
MX_DECL_BINARY(float, f32)
MX_DECL_BINARY(mx_bf16, bf16)
MX_DECL_BINARY(mx_f16, f16)
/* The rest of the family's dtypes (crates/maidenx_cuda/src/ops/binary.rs:172-181).  Integers saturate on add / sub /
 * mul; a zero divisor gives 0 for 0/0 and otherwise the largest (negative dividend: the smallest) value, MIN / -1
 * gives MAX; bool: add = maximum = or, sub = div = minimum = and, mul = xor
 * (crates/maidenx_cpu/src/ops/binary.rs:374-410, 457-578, 584-606). */
MX_DECL_BINARY(double, f64)
MX_DECL_BINARY(mx_bool, bool)
MX_DECL_BINARY(uint8_t, u8)
MX_DECL_BINARY(uint16_t, u16)
MX_DECL_BINARY(uint32_t, u32)
MX_DECL_BINARY(uint64_t, u64)
MX_DECL_BINARY(int8_t, i8)
MX_DECL_BINARY(int16_t, i16)
MX_DECL_BINARY(int32_t, i32)
MX_DECL_BINARY(int64_t, i64)

/* ---- unary: replaces crates/maidenx_cuda/src/ops/unary.rs:21-77 ------------------------------------
 * metadata = dims[n] | strides[n] | offset   (NULL: contiguous).  input == NULL means "in place on
 * output" (crates/maidenx_cuda/kernels/ops/unary.cu:20).  Semantics:
 * crates/maidenx_cpu/src/ops/unary.rs:14-122; the constant has the input dtype. */
#define MX_DECL_UNARY1(NAME, T, S, O) \
    void hip_##NAME##_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* input, O* output);
#define MX_DECL_UNARYC(NAME, T, S, O) \
    void hip_##NAME##_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* input, T constant, O* output);
#define MX_DECL_UNARY(T, S)                                                                                 \
    MX_DECL_UNARY1(neg, T, S, T) MX_DECL_UNARY1(abs, T, S, T) MX_DECL_UNARY1(sign, T, S, T)                 \
    MX_DECL_UNARY1(square, T, S, T) MX_DECL_UNARY1(sqrt, T, S, T) MX_DECL_UNARY1(relu, T, S, T)             \
    MX_DECL_UNARY1(sigmoid, T, S, T) MX_DECL_UNARY1(tanh, T, S, T) MX_DECL_UNARY1(gelu, T, S, T)            \
    MX_DECL_UNARY1(sin, T, S, T) MX_DECL_UNARY1(cos, T, S, T) MX_DECL_UNARY1(tan, T, S, T)                  \
    MX_DECL_UNARY1(ln, T, S, T) MX_DECL_UNARY1(log10, T, S, T) MX_DECL_UNARY1(log2, T, S, T)                \
    MX_DECL_UNARY1(exp, T, S, T) MX_DECL_UNARY1(exp10, T, S, T) MX_DECL_UNARY1(exp2, T, S, T)               \
    MX_DECL_UNARY1(softplus, T, S, T) MX_DECL_UNARY1(recip, T, S, T) MX_DECL_UNARY1(logical_not, T, S, mx_bool) \
    MX_DECL_UNARYC(add_scalar, T, S, T) MX_DECL_UNARYC(sub_scalar, T, S, T) MX_DECL_UNARYC(mul_scalar, T, S, T) \
    MX_DECL_UNARYC(div_scalar, T, S, T) MX_DECL_UNARYC(maximum_scalar, T, S, T)                             \
    MX_DECL_UNARYC(minimum_scalar, T, S, T) MX_DECL_UNARYC(pow, T, S, T) MX_DECL_UNARYC(leaky_relu, T, S, T) \
    MX_DECL_UNARYC(elu, T, S, T) MX_DECL_UNARYC(eq_scalar, T, S, mx_bool) MX_DECL_UNARYC(ne_scalar, T, S, mx_bool) \
    MX_DECL_UNARYC(lt_scalar, T, S, mx_bool) MX_DECL_UNARYC(le_scalar, T, S, mx_bool)                       \
    MX_DECL_UNARYC(gt_scalar, T, S, mx_bool) MX_DECL_UNARYC(ge_scalar, T, S, mx_bool)
MX_DECL_UNARY(float, f32)
MX_DECL_UNARY(mx_bf16, bf16)
MX_DECL_UNARY(mx_f16, f16)

/* ---- unary for f64, bool and the integers: crates/maidenx_cuda/src/ops/unary.rs:97-136, 152-191 ---------------------
 * The forms that are exact everywhere (semantics: crates/maidenx_cpu/src/ops/unary.rs:124-230, 234-236, 354-369,
 * 374-560, 564, 585-589, 650-740): integer neg / abs / square wrap on overflow as the reference's release build does,
 * integer sqrt is `(x as f32).sqrt() as T` of |x| (i64 through f64), the scalar add / sub / mul saturate; bool: neg = not,
 * add_scalar = or, sub_scalar = xor, mul_scalar = div_scalar = and, the rest identity.  The f64 transcendental forms
 * use the device math library (within 2 ulp of the host libm).  Not built: the integer pow (a float powf and a cast
 * in the reference). */
void hip_logical_not_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, mx_bool* output);
void hip_sign_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_square_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_sqrt_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_neg_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_abs_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_relu_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_recip_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_add_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, double* output);
void hip_sub_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, double* output);
void hip_mul_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, double* output);
void hip_div_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, double* output);
void hip_maximum_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, double* output);
void hip_minimum_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, double* output);
void hip_eq_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, mx_bool* output);
void hip_ne_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, mx_bool* output);
void hip_lt_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, mx_bool* output);
void hip_le_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, mx_bool* output);
void hip_gt_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, mx_bool* output);
void hip_ge_scalar_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, mx_bool* output);
void hip_leaky_relu_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, double* output);
void hip_sigmoid_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_tanh_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_gelu_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_sin_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_cos_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_tan_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_ln_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_log10_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_log2_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_exp_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_exp10_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_exp2_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_softplus_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_pow_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, double* output);
void hip_elu_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double constant, double* output);
void hip_logical_not_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool* output);
void hip_neg_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool* output);
void hip_abs_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool* output);
void hip_sign_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool* output);
void hip_square_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool* output);
void hip_sqrt_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool* output);
void hip_relu_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool* output);
void hip_sigmoid_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool* output);
void hip_tanh_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool* output);
void hip_add_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_sub_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_mul_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_div_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_maximum_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_minimum_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_eq_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_ne_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_lt_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_le_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_gt_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_ge_scalar_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_pow_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool constant, mx_bool* output);
void hip_logical_not_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, mx_bool* output);
void hip_sign_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t* output);
void hip_square_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t* output);
void hip_sqrt_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t* output);
void hip_add_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, uint8_t* output);
void hip_sub_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, uint8_t* output);
void hip_mul_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, uint8_t* output);
void hip_div_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, uint8_t* output);
void hip_maximum_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, uint8_t* output);
void hip_minimum_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, uint8_t* output);
void hip_eq_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, mx_bool* output);
void hip_ne_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, mx_bool* output);
void hip_lt_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, mx_bool* output);
void hip_le_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, mx_bool* output);
void hip_gt_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, mx_bool* output);
void hip_ge_scalar_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, mx_bool* output);
void hip_logical_not_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, mx_bool* output);
void hip_sign_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t* output);
void hip_square_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t* output);
void hip_sqrt_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t* output);
void hip_add_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, uint16_t* output);
void hip_sub_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, uint16_t* output);
void hip_mul_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, uint16_t* output);
void hip_div_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, uint16_t* output);
void hip_maximum_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, uint16_t* output);
void hip_minimum_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, uint16_t* output);
void hip_eq_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, mx_bool* output);
void hip_ne_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, mx_bool* output);
void hip_lt_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, mx_bool* output);
void hip_le_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, mx_bool* output);
void hip_gt_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, mx_bool* output);
void hip_ge_scalar_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, mx_bool* output);
void hip_logical_not_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, mx_bool* output);
void hip_sign_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t* output);
void hip_square_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t* output);
void hip_sqrt_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t* output);
void hip_add_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, uint32_t* output);
void hip_sub_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, uint32_t* output);
void hip_mul_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, uint32_t* output);
void hip_div_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, uint32_t* output);
void hip_maximum_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, uint32_t* output);
void hip_minimum_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, uint32_t* output);
void hip_eq_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, mx_bool* output);
void hip_ne_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, mx_bool* output);
void hip_lt_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, mx_bool* output);
void hip_le_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, mx_bool* output);
void hip_gt_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, mx_bool* output);
void hip_ge_scalar_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, mx_bool* output);
void hip_logical_not_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, mx_bool* output);
void hip_sign_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t* output);
void hip_square_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t* output);
void hip_sqrt_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t* output);
void hip_add_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, uint64_t* output);
void hip_sub_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, uint64_t* output);
void hip_mul_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, uint64_t* output);
void hip_div_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, uint64_t* output);
void hip_maximum_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, uint64_t* output);
void hip_minimum_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, uint64_t* output);
void hip_eq_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, mx_bool* output);
void hip_ne_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, mx_bool* output);
void hip_lt_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, mx_bool* output);
void hip_le_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, mx_bool* output);
void hip_gt_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, mx_bool* output);
void hip_ge_scalar_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, mx_bool* output);
void hip_logical_not_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, mx_bool* output);
void hip_sign_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_square_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_sqrt_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_neg_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_abs_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_add_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, int8_t* output);
void hip_sub_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, int8_t* output);
void hip_mul_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, int8_t* output);
void hip_div_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, int8_t* output);
void hip_maximum_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, int8_t* output);
void hip_minimum_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, int8_t* output);
void hip_eq_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, mx_bool* output);
void hip_ne_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, mx_bool* output);
void hip_lt_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, mx_bool* output);
void hip_le_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, mx_bool* output);
void hip_gt_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, mx_bool* output);
void hip_ge_scalar_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, mx_bool* output);
void hip_logical_not_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, mx_bool* output);
void hip_sign_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_square_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_sqrt_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_neg_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_abs_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_add_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, int16_t* output);
void hip_sub_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, int16_t* output);
void hip_mul_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, int16_t* output);
void hip_div_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, int16_t* output);
void hip_maximum_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, int16_t* output);
void hip_minimum_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, int16_t* output);
void hip_eq_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, mx_bool* output);
void hip_ne_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, mx_bool* output);
void hip_lt_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, mx_bool* output);
void hip_le_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, mx_bool* output);
void hip_gt_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, mx_bool* output);
void hip_ge_scalar_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, mx_bool* output);
void hip_logical_not_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, mx_bool* output);
void hip_sign_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_square_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_sqrt_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_neg_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_abs_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_add_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, int32_t* output);
void hip_sub_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, int32_t* output);
void hip_mul_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, int32_t* output);
void hip_div_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, int32_t* output);
void hip_maximum_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, int32_t* output);
void hip_minimum_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, int32_t* output);
void hip_eq_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, mx_bool* output);
void hip_ne_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, mx_bool* output);
void hip_lt_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, mx_bool* output);
void hip_le_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, mx_bool* output);
void hip_gt_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, mx_bool* output);
void hip_ge_scalar_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, mx_bool* output);
void hip_logical_not_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, mx_bool* output);
void hip_sign_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t* output);
void hip_square_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t* output);
void hip_sqrt_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t* output);
void hip_neg_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t* output);
void hip_abs_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t* output);
void hip_add_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, int64_t* output);
void hip_sub_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, int64_t* output);
void hip_mul_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, int64_t* output);
void hip_div_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, int64_t* output);
void hip_maximum_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, int64_t* output);
void hip_minimum_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, int64_t* output);
void hip_eq_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, mx_bool* output);
void hip_ne_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, mx_bool* output);
void hip_lt_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, mx_bool* output);
void hip_le_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, mx_bool* output);
void hip_gt_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, mx_bool* output);
void hip_ge_scalar_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, mx_bool* output);

/* Integer pow: `(x as f64).powf(c as f64) as T`, u8 through f32 (crates/maidenx_cpu/src/ops/unary.rs:565-572; the CUDA
 * crate lists it at crates/maidenx_cuda/src/ops/unary.rs:105-136).  Evaluated in exact integer arithmetic: the result is
 * what a correctly rounded pow followed by Rust's saturating, truncating `as` gives. */
void hip_pow_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t constant, uint8_t* output);
void hip_pow_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t constant, uint16_t* output);
void hip_pow_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t constant, uint32_t* output);
void hip_pow_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t constant, uint64_t* output);
void hip_pow_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t constant, int8_t* output);
void hip_pow_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t constant, int16_t* output);
void hip_pow_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t constant, int32_t* output);
void hip_pow_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t constant, int64_t* output);

/* ---- reduction: replaces crates/maidenx_cuda/src/ops/reduction.rs:19-35 ---------------------------
 * sum/mean/max/min metadata = dims[n] | strides[n] | red_len[r] | red_stride[r] | offset, r = 1
 * (the only value the tensor layer produces, crates/maidenx_tensor/src/ops/reduction.rs:38).
 * sum_to_shape metadata = in_dims[n] | in_strides[n] | out_dims[n] | offset; every output dim is 1
 * or the input dim.  Semantics: crates/maidenx_cpu/src/ops/reduction.rs:6-183, 185-272, 383-553
 * (mean divides once at the end; max starts from f32::MIN, min from f32::MAX; NaNs never win).
 * Accumulation is f32 in a fixed order; bf16 results are rounded once.
 * fold metadata = dims[n] | strides[n] | fold_dim, window_dim, fold_size, step, window_size, offset: the
 * adjoint of unfold, crates/maidenx_cpu/src/ops/reduction.rs:274-380 (output = the input shape without
 * window_dim and with fold_dim resized to fold_size; num_els counts the input). */
#define MX_DECL_REDUCE(T, S)                                                                                \
    void hip_sum_##S(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const T* inp, T* out);  \
    void hip_mean_##S(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const T* inp, T* out); \
    void hip_max_##S(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const T* inp, T* out);  \
    void hip_min_##S(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const T* inp, T* out);  \
    void hip_sum_to_shape_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* inp, T* out);  \
    void hip_fold_##S(size_t num_els, size_t num_dims, const size_t* metadata, const T* inp, T* out);
MX_DECL_REDUCE(float, f32)
MX_DECL_REDUCE(mx_bf16, bf16)
MX_DECL_REDUCE(mx_f16, f16)

/* Fused loss and optimizer steps (no counterpart in the reference's backend: its MSELoss is four tensor ops and six more
 * backward, crates/maidenx_nn/src/losses/mse.rs:21-29, its SGD two per parameter, optimizers/sgd.rs:17-27).  The same
 * element functions in the same order on values held in registers, contiguous f32 buffers:
 *   hip_mse_loss_f32           loss[0] = (sum of square(pred[i] - target[i])) / n          (16-byte aligned operands)
 *   hip_mse_loss_backward_f32  grad_pred[i] = 0 + (((grad_loss[0] / n) * 2) * (pred[i] - target[i])),
 *                              grad_target[i] = 0 + (-(that product)); either output may be NULL; grad_loss == NULL
 *                              stands for a gradient of 1 (the seed of backward(), which then need not be written)
 *   hip_sgd_step_f32           param[i] = param[i] - grad[i] * lr
 * Gradients and parameters are bit for bit what sub / pow / sum_all / div_scalar and their backward, or mul_scalar and
 * sub_inplace, give; the loss is a sum of n terms added in a fixed tree of its own (within the f32 tolerance of a
 * reduction of the op sequence's, whose order the reference does not fix either).  Inside a graph capture, at sizes
 * where a launch is latency bound, the three join the fused chains like the ops they replace (the step as an elementwise
 * member, the loss of at most 65536 elements as a stage of the serial phase, the backward pass as a member of the
 * parallel phase): the replayed bytes are those of the calls made one by one. */
void hip_mse_loss_f32(size_t n, const float* pred, const float* target, float* loss);
void hip_mse_loss_backward_f32(size_t n, const float* pred, const float* target, const float* grad_loss, float* grad_pred, float* grad_target);
void hip_sgd_step_f32(size_t n, float* param, const float* grad, float lr);

/* hip_sum_f32 for callers that cannot allocate.  No counterpart in the reference: it is for code that runs under HIP
 * graph capture, tight serving loops and harnesses that forbid allocation, where hip_sum_f32's grown-on-demand scratch
 * (its chunk partials when the reduced axis is cut to fill the chip) is not acceptable.  Same arguments and kernels as
 * hip_sum_f32, and for a contiguous input the same result bits; the partials live in a fixed 4 MiB array inside the
 * library's code object (one copy per GPU, held until the process ends: 3 MiB for chunk partials, 1 MiB for the partial
 * rows of a narrow-row reduction), so the call performs no hipMalloc, hipFree or stream synchronisation.  A strided
 * (e.g. transposed) input is summed one thread per output in ascending order - the reference's sequential order -
 * because hip_sum_f32's logical-order copy of such an input lives in grown scratch: equal to hip_sum_f32 to rounding,
 * not bit for bit.  A shape whose partials would not fit is refused: hip_get_last_status() == 3 (too large) and nothing
 * is queued — [8192,8192] and [64,512,1024] along any axis fit.  All calls on a GPU share that GPU's array: calls that overlap in time on one GPU race.
 * hip_noalloc_prepare() resolves the array's device address on the current device ahead of time (optional; the first
 * hip_sum_f32_noalloc on a device does it otherwise).  Returns 0 on success. */
void hip_sum_f32_noalloc(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const float* inp, float* out);
int hip_noalloc_prepare(void);
/* How many times the library's scratch buffers were allocated or grown (hipMalloc) since the process began; a caller
 * that must not allocate can watch it.  No counterpart in the reference. */
size_t hip_scratch_allocations(void);

/* The same for f64 and the integers (crates/maidenx_cuda/src/ops/reduction.rs:59-113; mean for f64 only, as in
 * crates/maidenx_cpu/src/ops/reduction.rs:581-586).  The accumulator is the storage type: integer sums wrap (the
 * reference's release build), so they are bit-exact in any order; f64 sums differ from the sequential order by
 * rounding.  sum_to_shape takes contiguous inputs only for these dtypes.  fold (crates/maidenx_cpu/src/ops/reduction.rs:
 * 591-599): f64 adds its windows in ascending order in f64, the integers wrap. */
void hip_fold_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_fold_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t* output);
void hip_fold_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t* output);
void hip_fold_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t* output);
void hip_fold_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t* output);
void hip_fold_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_fold_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_fold_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_fold_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t* output);
void hip_sum_f64(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const double* input, double* output);
void hip_max_f64(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const double* input, double* output);
void hip_min_f64(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const double* input, double* output);
void hip_mean_f64(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const double* input, double* output);
void hip_sum_to_shape_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_sum_u8(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint8_t* input, uint8_t* output);
void hip_max_u8(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint8_t* input, uint8_t* output);
void hip_min_u8(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint8_t* input, uint8_t* output);
void hip_sum_to_shape_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t* output);
void hip_sum_u16(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint16_t* input, uint16_t* output);
void hip_max_u16(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint16_t* input, uint16_t* output);
void hip_min_u16(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint16_t* input, uint16_t* output);
void hip_sum_to_shape_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t* output);
void hip_sum_u32(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint32_t* input, uint32_t* output);
void hip_max_u32(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint32_t* input, uint32_t* output);
void hip_min_u32(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint32_t* input, uint32_t* output);
void hip_sum_to_shape_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t* output);
void hip_sum_u64(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint64_t* input, uint64_t* output);
void hip_max_u64(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint64_t* input, uint64_t* output);
void hip_min_u64(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const uint64_t* input, uint64_t* output);
void hip_sum_to_shape_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t* output);
void hip_sum_i8(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_max_i8(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_min_i8(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_sum_to_shape_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_sum_i16(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_max_i16(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_min_i16(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_sum_to_shape_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_sum_i32(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_max_i32(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_min_i32(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_sum_to_shape_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_sum_i64(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int64_t* input, int64_t* output);
void hip_max_i64(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int64_t* input, int64_t* output);
void hip_min_i64(size_t num_els, size_t num_dims, size_t num_red_dims, const size_t* metadata, const int64_t* input, int64_t* output);
void hip_sum_to_shape_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t* output);

/* ---- matmul: replaces crates/maidenx_cuda/src/ops/matmul.rs:12-29 ---------------------------------
 * metadata = out_ndim, a_ndim, b_ndim | out_shape | a_shape | b_shape | a_strides | b_strides | a_off | b_off
 * Semantics: crates/maidenx_cpu/src/ops/matmul.rs:5-122 (forward; strided operands use strides[0]
 * as the batch stride) and :124-268 (backward; contiguous indexing, either gradient may be NULL).
 * f32 accumulate; bf16 results are rounded once. */
#define MX_DECL_MATMUL(T, S)                                                                                \
    void hip_matmul_##S(size_t num_els, const size_t* metadata, const T* a, const T* b, T* c);              \
    void hip_matmul_backward_##S(size_t num_els_a, size_t num_els_b, const size_t* metadata, const T* grad_output, \
                                 const T* a, const T* b, T* grad_a, T* grad_b);
MX_DECL_MATMUL(float, f32)
MX_DECL_MATMUL(mx_bf16, bf16)
MX_DECL_MATMUL(mx_f16, f16)

/* The same for f64 and the integers (crates/maidenx_cuda/src/ops/matmul.rs:36-50): LDS-tiled products without a
 * matrix instruction, each output accumulated in the storage type with the reduction index ascending and multiply and
 * add unfused - the order of crates/maidenx_cpu/src/ops/matmul.rs:60-86 - so f64 results carry the reference's bits and
 * integer results wrap as its release build does. */
void hip_matmul_f64(size_t num_els, const size_t* metadata, const double* a, const double* b, double* c);
void hip_matmul_backward_f64(size_t num_els_a, size_t num_els_b, const size_t* metadata, const double* grad_output, const double* a, const double* b, double* grad_a, double* grad_b);
void hip_matmul_u8(size_t num_els, const size_t* metadata, const uint8_t* a, const uint8_t* b, uint8_t* c);
void hip_matmul_backward_u8(size_t num_els_a, size_t num_els_b, const size_t* metadata, const uint8_t* grad_output, const uint8_t* a, const uint8_t* b, uint8_t* grad_a, uint8_t* grad_b);
void hip_matmul_u16(size_t num_els, const size_t* metadata, const uint16_t* a, const uint16_t* b, uint16_t* c);
void hip_matmul_backward_u16(size_t num_els_a, size_t num_els_b, const size_t* metadata, const uint16_t* grad_output, const uint16_t* a, const uint16_t* b, uint16_t* grad_a, uint16_t* grad_b);
void hip_matmul_u32(size_t num_els, const size_t* metadata, const uint32_t* a, const uint32_t* b, uint32_t* c);
void hip_matmul_backward_u32(size_t num_els_a, size_t num_els_b, const size_t* metadata, const uint32_t* grad_output, const uint32_t* a, const uint32_t* b, uint32_t* grad_a, uint32_t* grad_b);
void hip_matmul_u64(size_t num_els, const size_t* metadata, const uint64_t* a, const uint64_t* b, uint64_t* c);
void hip_matmul_backward_u64(size_t num_els_a, size_t num_els_b, const size_t* metadata, const uint64_t* grad_output, const uint64_t* a, const uint64_t* b, uint64_t* grad_a, uint64_t* grad_b);
void hip_matmul_i8(size_t num_els, const size_t* metadata, const int8_t* a, const int8_t* b, int8_t* c);
void hip_matmul_backward_i8(size_t num_els_a, size_t num_els_b, const size_t* metadata, const int8_t* grad_output, const int8_t* a, const int8_t* b, int8_t* grad_a, int8_t* grad_b);
void hip_matmul_i16(size_t num_els, const size_t* metadata, const int16_t* a, const int16_t* b, int16_t* c);
void hip_matmul_backward_i16(size_t num_els_a, size_t num_els_b, const size_t* metadata, const int16_t* grad_output, const int16_t* a, const int16_t* b, int16_t* grad_a, int16_t* grad_b);
void hip_matmul_i32(size_t num_els, const size_t* metadata, const int32_t* a, const int32_t* b, int32_t* c);
void hip_matmul_backward_i32(size_t num_els_a, size_t num_els_b, const size_t* metadata, const int32_t* grad_output, const int32_t* a, const int32_t* b, int32_t* grad_a, int32_t* grad_b);
void hip_matmul_i64(size_t num_els, const size_t* metadata, const int64_t* a, const int64_t* b, int64_t* c);
void hip_matmul_backward_i64(size_t num_els_a, size_t num_els_b, const size_t* metadata, const int64_t* grad_output, const int64_t* a, const int64_t* b, int64_t* grad_a, int64_t* grad_b);

/* ---- padding: replaces crates/maidenx_cuda/src/ops/padding.rs:13-71 (constant mode) ---------------
 * metadata = in_dims[n] | in_strides[n] | in_offset | out_dims[n] | (pad_before, pad_after)[n]
 * Semantics: crates/maidenx_cpu/src/ops/padding.rs:7-113 and :327-436.  Bit-exact. */
#define MX_DECL_PAD(T, S)                                                                                   \
    void hip_pad_with_constant_##S(size_t num_els_in, size_t num_els_out, size_t num_dims, const size_t* metadata, \
                                   const T* inp, T* out, T pad_value);                                      \
    void hip_pad_with_constant_backward_##S(size_t num_els_in, size_t num_els_out, size_t num_dims,         \
                                            const size_t* metadata, const T* grad_out, T* grad_in);
MX_DECL_PAD(float, f32)
MX_DECL_PAD(mx_bf16, bf16)
MX_DECL_PAD(mx_f16, f16)

/* reflection / replication modes of the same file (same metadata, no pad value).
 * Semantics: crates/maidenx_cpu/src/ops/padding.rs:115-325 (forward, bit-exact) and :438-665 (backward:
 * each input position receives the sum of the output gradients read from it, f32 accumulation in
 * ascending output order).  Reflection of a padded dim of size 1 is refused (the reference never returns). */
#define MX_DECL_PAD_EDGE(T, S)                                                                              \
    void hip_pad_with_reflection_##S(size_t num_els_in, size_t num_els_out, size_t num_dims, const size_t* metadata, \
                                     const T* inp, T* out);                                                 \
    void hip_pad_with_replication_##S(size_t num_els_in, size_t num_els_out, size_t num_dims, const size_t* metadata, \
                                      const T* inp, T* out);                                                \
    void hip_pad_with_reflection_backward_##S(size_t num_els_in, size_t num_els_out, size_t num_dims,       \
                                              const size_t* metadata, const T* grad_out, T* grad_in);       \
    void hip_pad_with_replication_backward_##S(size_t num_els_in, size_t num_els_out, size_t num_dims,      \
                                               const size_t* metadata, const T* grad_out, T* grad_in);
MX_DECL_PAD_EDGE(float, f32)
MX_DECL_PAD_EDGE(mx_bf16, bf16)
MX_DECL_PAD_EDGE(mx_f16, f16)

/* The three pad modes for f64 as well (crates/maidenx_cuda/src/ops/padding.rs:82); backward sums are formed in f64. */
void hip_pad_with_constant_f64(size_t num_els_in, size_t num_els_out, size_t num_dims, const size_t* metadata, const double* input, double* output, double pad_value);
void hip_pad_with_constant_backward_f64(size_t num_els_in, size_t num_els_out, size_t num_dims, const size_t* metadata, const double* grad_out, double* grad_in);
void hip_pad_with_reflection_f64(size_t num_els_in, size_t num_els_out, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_pad_with_replication_f64(size_t num_els_in, size_t num_els_out, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_pad_with_reflection_backward_f64(size_t num_els_in, size_t num_els_out, size_t num_dims, const size_t* metadata, const double* grad_out, double* grad_in);
void hip_pad_with_replication_backward_f64(size_t num_els_in, size_t num_els_out, size_t num_dims, const size_t* metadata, const double* grad_out, double* grad_in);

/* ... and for the integers (crates/maidenx_cuda/src/ops/padding.rs:83-90; CPU instantiations at
 * crates/maidenx_cpu/src/ops/padding.rs:670-677, 683-690, 696-703, 710-717, 723-730, 736-743): the forward modes copy,
 * the backward sums are formed in the storage type and wrap, as the reference's release build does. */
MX_DECL_PAD(uint8_t, u8)   MX_DECL_PAD_EDGE(uint8_t, u8)
MX_DECL_PAD(uint16_t, u16) MX_DECL_PAD_EDGE(uint16_t, u16)
MX_DECL_PAD(uint32_t, u32) MX_DECL_PAD_EDGE(uint32_t, u32)
MX_DECL_PAD(uint64_t, u64) MX_DECL_PAD_EDGE(uint64_t, u64)
MX_DECL_PAD(int8_t, i8)    MX_DECL_PAD_EDGE(int8_t, i8)
MX_DECL_PAD(int16_t, i16)  MX_DECL_PAD_EDGE(int16_t, i16)
MX_DECL_PAD(int32_t, i32)  MX_DECL_PAD_EDGE(int32_t, i32)
MX_DECL_PAD(int64_t, i64)  MX_DECL_PAD_EDGE(int64_t, i64)

/* ---- conv: replaces crates/maidenx_cuda/src/nn/conv.rs:12-24 --------------------------------------
 * metadata = 12 slots B, C, H, W, kh, kw, oh, ow, pad_h, pad_w, stride_h, stride_w as the kernel
 * reads them (crates/maidenx_cpu/src/nn/conv.rs:20-34).  im2col writes [B][C*kh*kw][oh*ow];
 * col2im sums in the reference's order and skips column indices >= num_els (:135).  Bit-exact. */
#define MX_DECL_CONV(T, S)                                                                                  \
    void hip_conv2d_im2col_##S(size_t num_els, const size_t* metadata, const T* input, T* col);             \
    void hip_conv2d_col2im_##S(size_t num_els, const size_t* metadata, const T* col, T* output);
MX_DECL_CONV(float, f32)
MX_DECL_CONV(mx_bf16, bf16)
MX_DECL_CONV(mx_f16, f16)

/* col2im accumulated into a gradient that exists (no backend symbol in the reference: its backward() adds the input
 * gradient that conv2d_col2im wrote with a separate add_, crates/maidenx_tensor/src/lib.rs:221-241):
 *   grad[i] = grad[i] + (the value hip_conv2d_col2im_f32 writes to output[i])
 * - the sum formed as there, then one f32 add: the bits of the two calls, without writing the intermediate and reading it
 * back. */
void hip_conv2d_col2im_add_f32(size_t num_els, const size_t* metadata, const float* col, float* grad);

/* f64 as well (crates/maidenx_cuda/src/nn/conv.rs:35): the same kernels, two elements per 16-byte vector. */
void hip_conv2d_im2col_f64(size_t num_els, const size_t* metadata, const double* input, double* col);
void hip_conv2d_col2im_f64(size_t num_els, const size_t* metadata, const double* col, double* output);

/* ---- the Conv2d layer's products with the column matrix, the matrix never stored --------------------------------
 * No backend symbol exists for this in the reference: crates/maidenx_nn/src/layers/conv.rs:206-222 writes the column
 * matrix with conv2d_im2col and multiplies it, reading the buffer [B][C*kh*kw][oh*ow] as a row-major matrix
 * cols[M = B*oh*ow, K = C*kh*kw]; :279 multiplies its transpose with the output gradient.  One call here is that
 * product with the entries of the matrix gathered from `input` while the tiles are staged (a ninth of the memory
 * traffic for a 3x3 kernel, and no buffer of M*K elements):
 *   transposed == 0:  out[M, n] = cols x rhs,     rhs [K, n]
 *   transposed != 0:  out[K, n] = cols^T x rhs,   rhs [M, n]
 * metadata: the 12 slots of hip_conv2d_im2col_f32; rhs_strides: element strides of rhs's two dims (one of them must
 * be 1), rhs already points at its first element; out is contiguous.  Same tiles, same order of additions as
 * hip_conv2d_im2col_f32 followed by hip_matmul_f32 on products that the latter runs on the matrix cores, so the
 * same bits there.  M*K and B*C*H*W must be below 2^31. */
void hip_conv2d_cols_matmul_f32(const size_t* metadata, int transposed, const float* input, const float* rhs, size_t n,
                                const size_t* rhs_strides, float* out);

/* The forward product of the layer with what follows it in the store (no backend symbol in the reference:
 * crates/maidenx_nn/src/layers/conv.rs:217-232 multiplies, reshapes to [B, oh, ow, Cout], transposes twice and adds the
 * bias - a second pass over the output through a transposed view):
 *   out[b][j][p] = (x[b*P + p][:] . w[j][:]) + bias[j]      x [M = B*P, K] and w [J, K] row-major, out [B, J, P]
 * The product's tiles and order of additions are hip_matmul_f32's, the addition is hip_add_f32's: the same bits as the
 * three calls.  Returns 1 when it ran, 0 when the shapes are not for it and nothing was queued (whole 64-row tiles,
 * J = 64, K a multiple of 32, 16-byte aligned operands, more than 128 tiles): the caller then makes the separate calls. */
int hip_conv2d_forward_product_f32(size_t M, size_t K, size_t J, size_t P, const float* x, const float* w, const float* bias, float* out);

/* ---- softmax: replaces crates/maidenx_cuda/src/nn/activation/softmax.rs (cuda_softmax_<T>) ------------
 * metadata = dims[n] | strides[n] | offset; dim >= num_dims means the last dim.
 * Semantics: crates/maidenx_cpu/src/nn/activation/softmax.rs:62-207 (max from -inf, the sum seeded
 * with exp(-inf - max), output contiguous; a strided input is indexed with the reference's own rule,
 * which walks the leading dims from dim 0 upwards).  The sum is f32 in a fixed order. */
void hip_softmax_f32(size_t num_els, size_t num_dims, size_t dim, const size_t* metadata, const float* input, float* output);
void hip_softmax_bf16(size_t num_els, size_t num_dims, size_t dim, const size_t* metadata, const mx_bf16* input, mx_bf16* output);
void hip_softmax_f16(size_t num_els, size_t num_dims, size_t dim, const size_t* metadata, const mx_f16* input, mx_f16* output);
/* f64 (crates/maidenx_cuda/src/nn/activation/softmax.rs:26-31): formed in f64 throughout. */
void hip_softmax_f64(size_t num_els, size_t num_dims, size_t dim, const size_t* metadata, const double* input, double* output);

/* ---- index ops -----------------------------------------------------------------------------------
 * No backend symbol exists for these in the reference: crates/maidenx_tensor/src/ops/indexing.rs runs them
 * as host loops over get / set / add_at_index (index_select :93-124, index_add_ :15-91, gather :315-363,
 * scatter_add_ :403-461, bincount :463-522; add_at_index utils/indexing.rs:96-140).  A layout is
 * dims[n] | strides[n] | offset of one tensor; outputs of index_select / gather are contiguous; indices
 * are read as i32 like the reference does; gather and scatter_add_ wrap negative indices; the in-place
 * ops add in the storage dtype in the reference's order (bit-identical, deterministic).  An index
 * outside its range is skipped and reported by hip_get_last_status() as an invalid argument
 * (the reference returns IndexOutOfBounds); that call waits for the stream when index ops ran. */
#define MX_DECL_INDEX(T, S, I, IS)                                                                                     \
    void hip_index_select_##S##_##IS(size_t num_dims, size_t dim, const size_t* in_layout, size_t n_idx, size_t idx_stride, \
                                     size_t idx_offset, const I* indices, const T* input, T* output);                  \
    void hip_gather_##S##_##IS(size_t num_dims, size_t dim, const size_t* in_layout, const size_t* idx_layout,         \
                               const I* index, const T* input, T* output);                                             \
    void hip_index_add_##S##_##IS(size_t num_dims, size_t dim, const size_t* self_layout, const size_t* src_layout,    \
                                  size_t n_idx, size_t idx_stride, size_t idx_offset, const I* indices, const T* src,  \
                                  T* self);                                                                            \
    void hip_scatter_add_##S##_##IS(size_t num_dims, size_t dim, const size_t* self_layout, const size_t* idx_layout,  \
                                    const size_t* src_layout, const I* index, const T* src, T* self);                  \
    void hip_bincount_weighted_##S##_##IS(size_t n, size_t stride, size_t offset, const I* input, size_t w_stride,     \
                                          size_t w_offset, const T* weights, size_t out_size, T* output);
/* ---- fused Adam step --------------------------------------------------------------------------------
 * No backend symbol exists for this in the reference: crates/maidenx_nn/src/optimizers/adam.rs:46-86 updates a
 * parameter with fourteen tensor ops (mul_scalar, add, square, div_scalar, sqrt, add_scalar, div, sub_).  One call
 * here applies the same element functions in the same order to contiguous param / grad / m / v of n elements and
 * leaves exactly the bits that sequence leaves in param, m and v.  The scalars are the ones the reference passes to
 * its *_scalar ops, in the tensor's dtype: beta1, 1-beta1, beta2, 1-beta2, the two bias terms 1-beta^(t+1) that m
 * and v are divided by, epsilon, and lr_t = lr*sqrt(bias2)/bias1. */
#define MX_DECL_ADAM(T, S)                                                                                                 \
    void hip_adam_step_##S(size_t n, T* param, const T* grad, T* m, T* v, T beta1, T one_minus_beta1, T beta2,              \
                           T one_minus_beta2, T bias1, T bias2, T epsilon, T lr_t);
MX_DECL_ADAM(float, f32)
MX_DECL_ADAM(mx_bf16, bf16)
MX_DECL_ADAM(mx_f16, f16)

/* index_put_ (indexing.rs:182-311): `indices` (host array) fixes the leading dims of self, src is copied into the
 * sub-tensor that remains (its shape must equal those dims); with every dim fixed a 0-d src is one element and any
 * other src goes element by element behind indices[0] of a 1-d self.  A shape mismatch, an index out of bounds or a
 * source that does not fit is an error status and nothing is written. */
#define MX_DECL_INDEX_PUT(T, S)                                                                                            \
    void hip_index_put_##S(size_t self_num_dims, const size_t* self_layout, size_t num_indices, const size_t* indices,     \
                           size_t src_num_dims, const size_t* src_layout, const T* src, T* self);
MX_DECL_INDEX_PUT(float, f32)
MX_DECL_INDEX_PUT(mx_bf16, bf16)
MX_DECL_INDEX_PUT(mx_f16, f16)
MX_DECL_INDEX(float, f32, int32_t, i32)
MX_DECL_INDEX(float, f32, int64_t, i64)
MX_DECL_INDEX(mx_bf16, bf16, int32_t, i32)
MX_DECL_INDEX(mx_bf16, bf16, int64_t, i64)
MX_DECL_INDEX(mx_f16, f16, int32_t, i32)
MX_DECL_INDEX(mx_f16, f16, int64_t, i64)
/* f64, bool and the integers: the reference's index ops are dtype-generic (they move Scalars, indexing.rs:15, 93, 182,
 * 315, 403), so every storage dtype has them.  The in-place adds follow add_at_index (utils/indexing.rs:121-135): f64
 * adds in f64, bool is `||`, the integers wrap.  The weighted bincount takes float weights: f64 besides the three above. */
#define MX_DECL_INDEX_WIDE(T, S, I, IS)                                                                                \
    void hip_index_select_##S##_##IS(size_t num_dims, size_t dim, const size_t* in_layout, size_t n_idx, size_t idx_stride, \
                                     size_t idx_offset, const I* indices, const T* input, T* output);                  \
    void hip_gather_##S##_##IS(size_t num_dims, size_t dim, const size_t* in_layout, const size_t* idx_layout,         \
                               const I* index, const T* input, T* output);                                             \
    void hip_index_add_##S##_##IS(size_t num_dims, size_t dim, const size_t* self_layout, const size_t* src_layout,    \
                                  size_t n_idx, size_t idx_stride, size_t idx_offset, const I* indices, const T* src,  \
                                  T* self);                                                                            \
    void hip_scatter_add_##S##_##IS(size_t num_dims, size_t dim, const size_t* self_layout, const size_t* idx_layout,  \
                                    const size_t* src_layout, const I* index, const T* src, T* self);
#define MX_DECL_INDEX_WIDE_ALL(T, S) MX_DECL_INDEX_WIDE(T, S, int32_t, i32) MX_DECL_INDEX_WIDE(T, S, int64_t, i64) MX_DECL_INDEX_PUT(T, S)
MX_DECL_INDEX_WIDE_ALL(double, f64)
MX_DECL_INDEX_WIDE(mx_bool, bool, int32_t, i32)      /* (spelled out: `bool` is a macro in C and must reach ## unexpanded) */
MX_DECL_INDEX_WIDE(mx_bool, bool, int64_t, i64)
MX_DECL_INDEX_PUT(mx_bool, bool)
MX_DECL_INDEX_WIDE_ALL(uint8_t, u8)
MX_DECL_INDEX_WIDE_ALL(uint16_t, u16)
MX_DECL_INDEX_WIDE_ALL(uint32_t, u32)
MX_DECL_INDEX_WIDE_ALL(uint64_t, u64)
MX_DECL_INDEX_WIDE_ALL(int8_t, i8)
MX_DECL_INDEX_WIDE_ALL(int16_t, i16)
MX_DECL_INDEX_WIDE_ALL(int32_t, i32)
MX_DECL_INDEX_WIDE_ALL(int64_t, i64)
void hip_bincount_weighted_f64_i32(size_t n, size_t stride, size_t offset, const int32_t* input, size_t w_stride, size_t w_offset, const double* weights, size_t out_size, double* output);
void hip_bincount_weighted_f64_i64(size_t n, size_t stride, size_t offset, const int64_t* input, size_t w_stride, size_t w_offset, const double* weights, size_t out_size, double* output);
void hip_bincount_i32(size_t n, size_t stride, size_t offset, const int32_t* input, size_t out_size, int32_t* output);
void hip_bincount_i64(size_t n, size_t stride, size_t offset, const int64_t* input, size_t out_size, int64_t* output);

/* ---- device-side fill / convert / strided copy --------------------------------------------------
 * No backend symbol exists for these in the reference: it builds host vectors
 * (crates/maidenx_tensor/src/creation.rs:144-164), converts dtypes on the host
 * (crates/maidenx_core/src/buffer/mod.rs:155-196) and makes views contiguous element by element
 * (crates/maidenx_tensor/src/f.rs:19-30).  hip_copy_strided takes the unary metadata layout. */
void hip_fill_f32(size_t num_els, float* out, float value);
void hip_fill_bf16(size_t num_els, mx_bf16* out, mx_bf16 value);
void hip_fill_f16(size_t num_els, mx_f16* out, mx_f16 value);
void hip_fill_bool(size_t num_els, mx_bool* out, mx_bool value);
void hip_copy_strided_f32(size_t num_els, size_t num_dims, const size_t* metadata, const float* input, float* output);
void hip_copy_strided_bf16(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bf16* input, mx_bf16* output);
void hip_copy_strided_f16(size_t num_els, size_t num_dims, const size_t* metadata, const mx_f16* input, mx_f16* output);
void hip_cast_bool_f32(size_t num_els, const mx_bool* input, float* output);
void hip_cast_bool_bf16(size_t num_els, const mx_bool* input, mx_bf16* output);
void hip_cast_f32_bf16(size_t num_els, const float* input, mx_bf16* output);
void hip_cast_bf16_f32(size_t num_els, const mx_bf16* input, float* output);
void hip_cast_f32_bool(size_t num_els, const float* input, mx_bool* output);
void hip_cast_bf16_bool(size_t num_els, const mx_bf16* input, mx_bool* output);
void hip_cast_bool_f16(size_t num_els, const mx_bool* input, mx_f16* output);
void hip_cast_f32_f16(size_t num_els, const float* input, mx_f16* output);
void hip_cast_f16_f32(size_t num_els, const mx_f16* input, float* output);
void hip_cast_f16_bool(size_t num_els, const mx_f16* input, mx_bool* output);
/* The same three for f64, the integers and bool, and conversions between every pair of the plain-number dtypes
 * (f32, f64, bool, u8 … i64) with the results of the reference's host conversion
 * (crates/maidenx_core/src/buffer/mod.rs:155-196, pair table :414-560): Rust's `as` — float to integer drops the
 * fraction, saturates and sends NaN to 0; integer to float rounds to nearest even; integer to integer keeps the low
 * bits; to bool is `!= 0`. */
void hip_fill_f64(size_t num_els, double* out, double value);
void hip_fill_u8(size_t num_els, uint8_t* out, uint8_t value);
void hip_fill_u16(size_t num_els, uint16_t* out, uint16_t value);
void hip_fill_u32(size_t num_els, uint32_t* out, uint32_t value);
void hip_fill_u64(size_t num_els, uint64_t* out, uint64_t value);
void hip_fill_i8(size_t num_els, int8_t* out, int8_t value);
void hip_fill_i16(size_t num_els, int16_t* out, int16_t value);
void hip_fill_i32(size_t num_els, int32_t* out, int32_t value);
void hip_fill_i64(size_t num_els, int64_t* out, int64_t value);
void hip_copy_strided_f64(size_t num_els, size_t num_dims, const size_t* metadata, const double* input, double* output);
void hip_copy_strided_bool(size_t num_els, size_t num_dims, const size_t* metadata, const mx_bool* input, mx_bool* output);
void hip_copy_strided_u8(size_t num_els, size_t num_dims, const size_t* metadata, const uint8_t* input, uint8_t* output);
void hip_copy_strided_u16(size_t num_els, size_t num_dims, const size_t* metadata, const uint16_t* input, uint16_t* output);
void hip_copy_strided_u32(size_t num_els, size_t num_dims, const size_t* metadata, const uint32_t* input, uint32_t* output);
void hip_copy_strided_u64(size_t num_els, size_t num_dims, const size_t* metadata, const uint64_t* input, uint64_t* output);
void hip_copy_strided_i8(size_t num_els, size_t num_dims, const size_t* metadata, const int8_t* input, int8_t* output);
void hip_copy_strided_i16(size_t num_els, size_t num_dims, const size_t* metadata, const int16_t* input, int16_t* output);
void hip_copy_strided_i32(size_t num_els, size_t num_dims, const size_t* metadata, const int32_t* input, int32_t* output);
void hip_copy_strided_i64(size_t num_els, size_t num_dims, const size_t* metadata, const int64_t* input, int64_t* output);
void hip_cast_f32_f64(size_t num_els, const float* input, double* output);
void hip_cast_f32_u8(size_t num_els, const float* input, uint8_t* output);
void hip_cast_f32_u16(size_t num_els, const float* input, uint16_t* output);
void hip_cast_f32_u32(size_t num_els, const float* input, uint32_t* output);
void hip_cast_f32_u64(size_t num_els, const float* input, uint64_t* output);
void hip_cast_f32_i8(size_t num_els, const float* input, int8_t* output);
void hip_cast_f32_i16(size_t num_els, const float* input, int16_t* output);
void hip_cast_f32_i32(size_t num_els, const float* input, int32_t* output);
void hip_cast_f32_i64(size_t num_els, const float* input, int64_t* output);
void hip_cast_f64_f32(size_t num_els, const double* input, float* output);
void hip_cast_f64_bool(size_t num_els, const double* input, mx_bool* output);
void hip_cast_f64_u8(size_t num_els, const double* input, uint8_t* output);
void hip_cast_f64_u16(size_t num_els, const double* input, uint16_t* output);
void hip_cast_f64_u32(size_t num_els, const double* input, uint32_t* output);
void hip_cast_f64_u64(size_t num_els, const double* input, uint64_t* output);
void hip_cast_f64_i8(size_t num_els, const double* input, int8_t* output);
void hip_cast_f64_i16(size_t num_els, const double* input, int16_t* output);
void hip_cast_f64_i32(size_t num_els, const double* input, int32_t* output);
void hip_cast_f64_i64(size_t num_els, const double* input, int64_t* output);
void hip_cast_bool_f64(size_t num_els, const mx_bool* input, double* output);
void hip_cast_bool_u8(size_t num_els, const mx_bool* input, uint8_t* output);
void hip_cast_bool_u16(size_t num_els, const mx_bool* input, uint16_t* output);
void hip_cast_bool_u32(size_t num_els, const mx_bool* input, uint32_t* output);
void hip_cast_bool_u64(size_t num_els, const mx_bool* input, uint64_t* output);
void hip_cast_bool_i8(size_t num_els, const mx_bool* input, int8_t* output);
void hip_cast_bool_i16(size_t num_els, const mx_bool* input, int16_t* output);
void hip_cast_bool_i32(size_t num_els, const mx_bool* input, int32_t* output);
void hip_cast_bool_i64(size_t num_els, const mx_bool* input, int64_t* output);
void hip_cast_u8_f32(size_t num_els, const uint8_t* input, float* output);
void hip_cast_u8_f64(size_t num_els, const uint8_t* input, double* output);
void hip_cast_u8_bool(size_t num_els, const uint8_t* input, mx_bool* output);
void hip_cast_u8_u16(size_t num_els, const uint8_t* input, uint16_t* output);
void hip_cast_u8_u32(size_t num_els, const uint8_t* input, uint32_t* output);
void hip_cast_u8_u64(size_t num_els, const uint8_t* input, uint64_t* output);
void hip_cast_u8_i8(size_t num_els, const uint8_t* input, int8_t* output);
void hip_cast_u8_i16(size_t num_els, const uint8_t* input, int16_t* output);
void hip_cast_u8_i32(size_t num_els, const uint8_t* input, int32_t* output);
void hip_cast_u8_i64(size_t num_els, const uint8_t* input, int64_t* output);
void hip_cast_u16_f32(size_t num_els, const uint16_t* input, float* output);
void hip_cast_u16_f64(size_t num_els, const uint16_t* input, double* output);
void hip_cast_u16_bool(size_t num_els, const uint16_t* input, mx_bool* output);
void hip_cast_u16_u8(size_t num_els, const uint16_t* input, uint8_t* output);
void hip_cast_u16_u32(size_t num_els, const uint16_t* input, uint32_t* output);
void hip_cast_u16_u64(size_t num_els, const uint16_t* input, uint64_t* output);
void hip_cast_u16_i8(size_t num_els, const uint16_t* input, int8_t* output);
void hip_cast_u16_i16(size_t num_els, const uint16_t* input, int16_t* output);
void hip_cast_u16_i32(size_t num_els, const uint16_t* input, int32_t* output);
void hip_cast_u16_i64(size_t num_els, const uint16_t* input, int64_t* output);
void hip_cast_u32_f32(size_t num_els, const uint32_t* input, float* output);
void hip_cast_u32_f64(size_t num_els, const uint32_t* input, double* output);
void hip_cast_u32_bool(size_t num_els, const uint32_t* input, mx_bool* output);
void hip_cast_u32_u8(size_t num_els, const uint32_t* input, uint8_t* output);
void hip_cast_u32_u16(size_t num_els, const uint32_t* input, uint16_t* output);
void hip_cast_u32_u64(size_t num_els, const uint32_t* input, uint64_t* output);
void hip_cast_u32_i8(size_t num_els, const uint32_t* input, int8_t* output);
void hip_cast_u32_i16(size_t num_els, const uint32_t* input, int16_t* output);
void hip_cast_u32_i32(size_t num_els, const uint32_t* input, int32_t* output);
void hip_cast_u32_i64(size_t num_els, const uint32_t* input, int64_t* output);
void hip_cast_u64_f32(size_t num_els, const uint64_t* input, float* output);
void hip_cast_u64_f64(size_t num_els, const uint64_t* input, double* output);
void hip_cast_u64_bool(size_t num_els, const uint64_t* input, mx_bool* output);
void hip_cast_u64_u8(size_t num_els, const uint64_t* input, uint8_t* output);
void hip_cast_u64_u16(size_t num_els, const uint64_t* input, uint16_t* output);
void hip_cast_u64_u32(size_t num_els, const uint64_t* input, uint32_t* output);
void hip_cast_u64_i8(size_t num_els, const uint64_t* input, int8_t* output);
void hip_cast_u64_i16(size_t num_els, const uint64_t* input, int16_t* output);
void hip_cast_u64_i32(size_t num_els, const uint64_t* input, int32_t* output);
void hip_cast_u64_i64(size_t num_els, const uint64_t* input, int64_t* output);
void hip_cast_i8_f32(size_t num_els, const int8_t* input, float* output);
void hip_cast_i8_f64(size_t num_els, const int8_t* input, double* output);
void hip_cast_i8_bool(size_t num_els, const int8_t* input, mx_bool* output);
void hip_cast_i8_u8(size_t num_els, const int8_t* input, uint8_t* output);
void hip_cast_i8_u16(size_t num_els, const int8_t* input, uint16_t* output);
void hip_cast_i8_u32(size_t num_els, const int8_t* input, uint32_t* output);
void hip_cast_i8_u64(size_t num_els, const int8_t* input, uint64_t* output);
void hip_cast_i8_i16(size_t num_els, const int8_t* input, int16_t* output);
void hip_cast_i8_i32(size_t num_els, const int8_t* input, int32_t* output);
void hip_cast_i8_i64(size_t num_els, const int8_t* input, int64_t* output);
void hip_cast_i16_f32(size_t num_els, const int16_t* input, float* output);
void hip_cast_i16_f64(size_t num_els, const int16_t* input, double* output);
void hip_cast_i16_bool(size_t num_els, const int16_t* input, mx_bool* output);
void hip_cast_i16_u8(size_t num_els, const int16_t* input, uint8_t* output);
void hip_cast_i16_u16(size_t num_els, const int16_t* input, uint16_t* output);
void hip_cast_i16_u32(size_t num_els, const int16_t* input, uint32_t* output);
void hip_cast_i16_u64(size_t num_els, const int16_t* input, uint64_t* output);
void hip_cast_i16_i8(size_t num_els, const int16_t* input, int8_t* output);
void hip_cast_i16_i32(size_t num_els, const int16_t* input, int32_t* output);
void hip_cast_i16_i64(size_t num_els, const int16_t* input, int64_t* output);
void hip_cast_i32_f32(size_t num_els, const int32_t* input, float* output);
void hip_cast_i32_f64(size_t num_els, const int32_t* input, double* output);
void hip_cast_i32_bool(size_t num_els, const int32_t* input, mx_bool* output);
void hip_cast_i32_u8(size_t num_els, const int32_t* input, uint8_t* output);
void hip_cast_i32_u16(size_t num_els, const int32_t* input, uint16_t* output);
void hip_cast_i32_u32(size_t num_els, const int32_t* input, uint32_t* output);
void hip_cast_i32_u64(size_t num_els, const int32_t* input, uint64_t* output);
void hip_cast_i32_i8(size_t num_els, const int32_t* input, int8_t* output);
void hip_cast_i32_i16(size_t num_els, const int32_t* input, int16_t* output);
void hip_cast_i32_i64(size_t num_els, const int32_t* input, int64_t* output);
void hip_cast_i64_f32(size_t num_els, const int64_t* input, float* output);
void hip_cast_i64_f64(size_t num_els, const int64_t* input, double* output);
void hip_cast_i64_bool(size_t num_els, const int64_t* input, mx_bool* output);
void hip_cast_i64_u8(size_t num_els, const int64_t* input, uint8_t* output);
void hip_cast_i64_u16(size_t num_els, const int64_t* input, uint16_t* output);
void hip_cast_i64_u32(size_t num_els, const int64_t* input, uint32_t* output);
void hip_cast_i64_u64(size_t num_els, const int64_t* input, uint64_t* output);
void hip_cast_i64_i8(size_t num_els, const int64_t* input, int8_t* output);
void hip_cast_i64_i16(size_t num_els, const int64_t* input, int16_t* output);
void hip_cast_i64_i32(size_t num_els, const int64_t* input, int32_t* output);

#ifdef __cplusplus
}
#endif
#endif /* MAIDENX_HIP_H */
