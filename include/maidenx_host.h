/* maidenx_host.h — C ABI of the host layer (libmaidenx_host.so).
 *
 * The host layer replays MaidenX's tensor / autograd / nn calls above the backend kernels of
 * maidenx_hip.h: each function below names the reference function whose backend-call sequence it issues.
 * Tensors are opaque handles; a handle is released with mxt_release.  Float tensors are f32 or bf16 (comparisons
 * give bool); mixed operands and non-integer scalars promote as the reference does (utils/promotion.rs:16-33,
 * ops/unary.rs:872-876).  Conv2d is f32 only.
 *
 * Functions that return a handle return NULL on error, functions that return int return non-zero;
 * mxt_last_error() then gives the error kind (the variant of crates/maidenx_core/src/error.rs that the
 * reference would return) and its text.
 */
#ifndef MAIDENX_HOST_H
#define MAIDENX_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* mxt_tensor;
typedef void* mxt_module;

/* error kinds */
#define MXT_OK 0
#define MXT_ERR_INVALID_SHAPE 1
#define MXT_ERR_SHAPE_MISMATCH 2
#define MXT_ERR_DIM_OUT_OF_BOUNDS 3
#define MXT_ERR_INCOMPATIBLE_SHAPE 4
#define MXT_ERR_INVALID_OPERATION 5
#define MXT_ERR_INVALID_ARGUMENT 6
#define MXT_ERR_UNSUPPORTED_DTYPE 7
#define MXT_ERR_OUT_OF_MEMORY 8
#define MXT_ERR_BACKEND 9
int mxt_last_error(char* text, size_t cap);      /* kind of the last failure on this thread; copies its text */
const char* mxt_backend_name(void);

/* dtypes */
#define MXT_F32 0
#define MXT_BF16 1
#define MXT_BOOL 2

/* creation: crates/maidenx_tensor/src/creation.rs:25-84 (new), :253-305 (fill); randn is seeded here.  The _dtype
 * forms take f32 values and store them in the given float dtype; the plain forms are f32. */
mxt_tensor mxt_new(const float* data, const size_t* shape, size_t ndim);
mxt_tensor mxt_fill(const size_t* shape, size_t ndim, float value);
mxt_tensor mxt_new_dtype(const float* data, const size_t* shape, size_t ndim, int dtype);
mxt_tensor mxt_fill_dtype(const size_t* shape, size_t ndim, float value, int dtype);
mxt_tensor mxt_randn(const size_t* shape, size_t ndim, uint64_t seed);
void mxt_release(mxt_tensor t);

/* metadata */
size_t mxt_ndim(mxt_tensor t);
size_t mxt_size(mxt_tensor t);
size_t mxt_offset(mxt_tensor t);
void mxt_shape(mxt_tensor t, size_t* out);
void mxt_strides(mxt_tensor t, size_t* out);
int mxt_dtype(mxt_tensor t);
mxt_tensor mxt_to_dtype(mxt_tensor t, int dtype);   /* wt.rs:86-90: converts the whole buffer, keeps the layout */
int mxt_requires_grad(mxt_tensor t);
int mxt_is_contiguous(mxt_tensor t);
int mxt_to_host(mxt_tensor t, float* out);       /* logical (row-major) order; bool tensors as 0/1 */

/* autograd: crates/maidenx_tensor/src/wt.rs:92-104, src/lib.rs:213-323 */
int mxt_with_grad(mxt_tensor t);
mxt_tensor mxt_grad(mxt_tensor t);               /* NULL without error text if the tensor has no grad */
int mxt_backward(mxt_tensor t);
int mxt_zero_grad(mxt_tensor t);
mxt_tensor mxt_detach(mxt_tensor t);

/* ops: crates/maidenx_tensor/src/ops/{binary,unary,reduction,matmul,transform}.rs
 *   binary         : add sub mul div matmul
 *   binary_inplace : add_ sub_
 *   unary          : neg square relu tanh gelu exp sum_all mean_all contiguous squeeze_all
 *   unary_scalar   : add_scalar mul_scalar div_scalar pow gt_scalar
 *   reduce         : sum mean                      (dim may be negative)
 *   shape_op       : view reshape (-1 allowed) broadcast broadcast_left sum_to_shape transpose (2 args) squeeze unsqueeze (1 arg) */
mxt_tensor mxt_binary(const char* op, mxt_tensor a, mxt_tensor b);
int mxt_binary_inplace(const char* op, mxt_tensor a, mxt_tensor b);
mxt_tensor mxt_unary(const char* op, mxt_tensor a);
mxt_tensor mxt_unary_scalar(const char* op, mxt_tensor a, float c);
mxt_tensor mxt_reduce(const char* op, mxt_tensor a, int dim, int keep_dim);
mxt_tensor mxt_shape_op(const char* op, mxt_tensor a, const int64_t* args, size_t nargs);

/* nn: crates/maidenx_nn/src/layers/linear.rs:20-98, layers/conv.rs:100-322, losses/mse.rs:21-29,
 * optimizers/sgd.rs:17-33.  Modules take their parameters as tensors (bias may be NULL). */
mxt_module mxt_linear_new(mxt_tensor weight, mxt_tensor bias);
mxt_module mxt_linear_new_seeded(size_t in_features, size_t out_features, int with_bias, uint64_t seed);
mxt_module mxt_conv2d_new(mxt_tensor weight, mxt_tensor bias, size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                          size_t pad_h, size_t pad_w);
mxt_tensor mxt_module_forward(mxt_module m, mxt_tensor input);
mxt_tensor mxt_module_weight(mxt_module m);
mxt_tensor mxt_module_bias(mxt_module m);        /* NULL if the module has none */
void mxt_module_release(mxt_module m);
mxt_tensor mxt_mse_loss(mxt_tensor pred, mxt_tensor target);
int mxt_sgd_step(mxt_module m, float lr);
int mxt_sgd_zero_grad(mxt_module m);
/* optimizers/adam.rs:16-99 with f64 hyper-parameters; the moments live in the optimizer object, one pair per
 * parameter of the module it is first stepped with.  On the HIP build a contiguous f32 parameter is updated by one
 * hip_adam_step_f32 call instead of the reference's fourteen ops (same bits); mxt_adam_set_fused(opt, 0) keeps the ops. */
void* mxt_adam_new(double lr, double beta1, double beta2, double epsilon);
void mxt_adam_release(void* opt);
void mxt_adam_set_fused(void* opt, int enabled);
int mxt_adam_step(void* opt, mxt_module m);

/* The loop of examples/device/cpu.rs:32-38 (forward, MSE, backward, SGD step, zero_grad), `epochs` times,
 * without leaving native code.  losses (may be NULL) receives the loss of every epoch; reading it costs one
 * device-to-host copy per epoch, so pass NULL when timing. */
int mxt_train(mxt_module m, mxt_tensor input, mxt_tensor target, float lr, size_t epochs, float* losses);
/* With losses == NULL and at least 32 epochs the HIP build runs eagerly until the buffer addresses of a step repeat
 * (8 to 64 epochs), then records that many steps as a graph and replays it (the loop is launch-bound); results are
 * those of the eager loop.  mxt_set_graph_replay(0) keeps every
 * epoch eager; mxt_last_train_replayed() tells how many epochs of the last mxt_train call were replays. */
void mxt_set_graph_replay(int enabled);
size_t mxt_last_train_replayed(void);
/* The same for any step: calls fn(user, e) for e = 0 .. steps-1 (a non-zero return ends the loop with an error), or - on
 * the HIP build, from 32 steps on - runs it eagerly until the buffer addresses of a step repeat, records some more steps as
 * a graph and replays that for the rest; mxt_last_train_replayed() counts the replays.  The step must issue the same
 * tensor calls every time, must not read values back from the device, and hands results on only through tensors it
 * updates (parameters, gradients): tensors it creates are gone when it returns.  No counterpart in the reference, whose
 * loops are written in the caller's Rust. */
typedef int (*mxt_step_fn)(void* user, size_t step);
int mxt_run_steps(mxt_step_fn fn, void* user, size_t steps);
/* sum_all() (crates/maidenx_tensor/src/ops/reduction.rs:76-83) sums one dim after the other.  By default a contiguous f32
 * tensor is summed by one sum_to_shape call to [1, .., 1] instead: the gradients are the same bytes, the sum is added
 * up in another order (both within the f32 tolerance of a reduction).  enabled = 0: dim by dim. */
void mxt_set_sum_all_in_one_pass(int enabled);
/* backward() leaves out what cannot change a bit of any gradient (enabled = 0: does it all, as the reference does): the
 * gradient of a binary op's operand that requires none (computed and dropped in the reference,
 * crates/maidenx_tensor/src/lib.rs:93-111), x.pow(1) in the backward of pow(2), the zero fill in front of the first
 * accumulation when the gradient is a broadcast view, and the first accumulation itself (0 + g) when g is a fresh
 * sum_to_shape result, whose buffer then becomes the gradient. */
void mxt_set_autograd_shortcuts(int enabled);
/* MSELoss (crates/maidenx_nn/src/losses/mse.rs:21-29: sub, pow(2), sum_all, div_scalar) and SGD::step
 * (optimizers/sgd.rs:17-27: mul_scalar, in-place sub) are one backend call each on the HIP build (hip_mse_loss_f32 and
 * its backward, hip_sgd_step_f32) for contiguous f32 tensors: every gradient and every updated parameter is the same
 * bytes as the op sequence gives, the loss is summed in another order (within the f32 tolerance of a reduction).
 * enabled = 0: the op sequences. */
void mxt_set_fused_nn_kernels(int enabled);
/* Conv2d backward (nn/layers/conv.rs:253-268): col2im is handed num_els = B*C*H*W and reads no entry of grad_cols at
 * or beyond that flat index (crates/maidenx_cpu/src/nn/conv.rs:135), so by default only the leading
 * ceil(B*C*H*W / (C*kh*kw)) rows of grad_cols are computed; the input gradient is the same bytes either way.
 * enabled = 0 computes the whole product as the reference does. */
void mxt_set_conv_skip_unread_grad_cols(int enabled);
/* Conv2d forward (conv.rs:206-222) and its weight gradient (:279) multiply the column matrix.  The HIP build can
 * gather the entries of that matrix from the input inside the product (hip_conv2d_cols_matmul_f32) instead of storing
 * it with conv2d_im2col first.  mode 0: always store, as the reference does; 1 (default): gather when the input does
 * not require a gradient, i.e. when no backward is recorded (the forward alone is faster that way; a training step is
 * faster with the one stored matrix that serves both products); 2: gather in forward and backward (about 6 % slower
 * per step on a 64-channel 3x3 layer, and no buffer of B*oh*ow x C*kh*kw elements is held for the backward).  The
 * products are the same bits wherever the stored product runs on the matrix cores. */
void mxt_set_conv_gathered_products(int mode);

/* bookkeeping */
size_t mxt_backend_calls(void);                  /* kernels dispatched since the last reset */
void mxt_reset_backend_calls(void);
size_t mxt_cast_calls(void);                     /* whole-buffer dtype conversions since the last reset */
size_t mxt_device_allocations(void);             /* allocations that reached the backend (pool misses) */
int mxt_synchronize(void);

#ifdef __cplusplus
}
#endif
#endif
