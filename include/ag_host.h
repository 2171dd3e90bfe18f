/*
 * ag_host.h -- C ABI of the host-side operator layer (libag_host.so).
 *
 * libag_host.so is the C++ mirror of the part of rust-autograd that CALLS the GPU kernels: the
 * `op::Op` compute/grad interface (src/op.rs:90-101), the lazy graph and `TensorBuilder`
 * (src/tensor.rs:609-803), reverse-mode `grad()` (src/gradient.rs:20-84, src/tensor_ops/mod.rs:
 * 94-114), the evaluator (src/evaluation.rs:251-363), `VariableEnvironment` (src/variable.rs) and
 * the `Adam` optimizer (src/optimizers/adam.rs, src/optimizers/mod.rs:21-99).  The functions below
 * expose that layer through opaque handles so that a test harness in any language can build the
 * same graphs the reference's examples and tests build.  Tensors are identified by their node id
 * inside a context; every function returns -1 (or NULL) on misuse and leaves a message in
 * agh_last_error() -- the counterpart of a Rust panic.  Arrays cross this boundary as host f32.
 */
#ifndef AG_HOST_H
#define AG_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

typedef struct agh_env agh_env;   /* VariableEnvironment            src/variable.rs:152-155 */
typedef struct agh_ctx agh_ctx;   /* Context (graph + environment)  src/graph.rs            */
typedef struct agh_adam agh_adam; /* optimizers::Adam               src/optimizers/adam.rs  */

const char *agh_last_error(void);

/* ---- variables ------------------------------------------------------------------------------ */
agh_env *agh_env_new(void);
void agh_env_free(agh_env *env);
/* env.namespace_mut(ns).slot().name(name).set(array): returns the VariableID.  ns "" = default. */
int agh_env_set(agh_env *env, const char *ns, const char *name, const float *data, const int64_t *shape, int rank);
int agh_env_find(agh_env *env, const char *ns, const char *name);
int agh_env_shape(agh_env *env, int var_id, int64_t *shape_out, int max_rank); /* returns the rank */
int agh_env_read(agh_env *env, int var_id, float *out, size_t n);
/* Overwrites the variable's array in place (same element count), as writing through
 * env.get_array_by_id(id).borrow_mut() does (src/variable.rs:695-703). */
int agh_env_write(agh_env *env, int var_id, const float *data, size_t n);
int agh_env_len(agh_env *env); /* number of variable arrays (named or not) */
/* Persistence in the reference's own on-disk format: serde_json of {"array_list":[{"v":1,"dim":[..],
 * "data":[..]},..],"name_to_id":{"ns\u0001name":id,..}} (src/variable.rs:470-480).
 * agh_env_save = VariableEnvironment::save (:549-554); agh_env_load = ::load (:487-490), NULL on error;
 * agh_env_initialize = ::initialize (:493-503), replacing the arrays and names of `env`.
 * A file that cannot be opened or parsed gives -1 / NULL and a message in agh_last_error(). */
int agh_env_save(agh_env *env, const char *path);
agh_env *agh_env_load(const char *path);
int agh_env_initialize(agh_env *env, const char *path);
/* Reads a saved environment and writes it again, in host memory only (no device is touched):
 * checks a file and brings it to the exact text agh_env_save produces. */
int agh_env_file_rewrite(const char *src_path, const char *dst_path);

/* ---- graph construction (one context = one `env.run(|ctx| ...)` closure) --------------------- */
agh_ctx *agh_ctx_new(agh_env *env);
void agh_ctx_free(agh_ctx *ctx);
int agh_variable(agh_ctx *ctx, int var_id);
int agh_placeholder(agh_ctx *ctx, const char *name, const int64_t *shape, int rank); /* -1 = unknown extent */
int agh_scalar(agh_ctx *ctx, float value);
int agh_conv2d(agh_ctx *ctx, int x, int w, int pad, int stride, int dilation);           /* conv2d / dilated_conv2d */
/* the same operator made to materialise the im2col columns as its second output, like the reference,
 * whatever the geometry (the default takes the column-free path for large stride-1 / stride-2 cases) */
int agh_conv2d_with_columns(agh_ctx *ctx, int x, int w, int pad, int stride, int dilation);
int agh_conv2d_transpose(agh_ctx *ctx, int x, int w, int pad, int stride, int dilation); /* (dilated_)conv2d_transpose */
int agh_max_pool2d(agh_ctx *ctx, int x, int pool_size, int pad, int stride);
int agh_matmul(agh_ctx *ctx, int a, int b);
int agh_batch_matmul(agh_ctx *ctx, int a, int b, int trans_a, int trans_b);
int agh_reduce_sum(agh_ctx *ctx, int x, const int *axes, int n_axes, int keep_dims);
int agh_reduce_mean(agh_ctx *ctx, int x, const int *axes, int n_axes, int keep_dims);
int agh_sum_all(agh_ctx *ctx, int x);
int agh_relu(agh_ctx *ctx, int x);
int agh_add(agh_ctx *ctx, int a, int b);
int agh_mul(agh_ctx *ctx, int a, int b);
int agh_add_n(agh_ctx *ctx, const int *xs, int n);
int agh_nth_tensor(agh_ctx *ctx, int x, int n);
int agh_reshape(agh_ctx *ctx, int x, const int64_t *shape, int rank);
int agh_sparse_softmax_cross_entropy(agh_ctx *ctx, int logits, int labels);
int agh_stop_gradient(agh_ctx *ctx, int x);
/* tensor_ops::grad(ys, xs): writes nx tensor ids to out. */
int agh_grad(agh_ctx *ctx, const int *ys, int ny, const int *xs, int nx, int *out);
/* tensor_ops::grad_with_default(ys, xs, ys_grads): ys_grads[i] is the known gradient of ys[i]. */
int agh_grad_with_default(agh_ctx *ctx, const int *ys, const int *ys_grads, int ny, const int *xs, int nx, int *out);
/* optimizers::grad_helper(losses, namespace): returns the number of (variable, gradient) pairs. */
int agh_grad_helper(agh_ctx *ctx, const int *losses, int n, const char *ns, int *vars_out, int *grads_out, int max_out);

/* ---- introspection -------------------------------------------------------------------------- */
int agh_num_nodes(agh_ctx *ctx);
/* Pairs of nodes that the evaluations of this context so far ran as one launch (a ReLU, or the ReLU of a sum, with the
 * 2 x 2 max pooling behind it); the results are those of the nodes evaluated in turn. */
int agh_fused_pairs(agh_ctx *ctx);
/* How often an op of the calling thread found the rearranged copy it needed already made by an earlier op (the
 * zero-bordered upstream gradient that the two gradients of a column-free convolution share), since the thread began. */
long long agh_reused_copies(void);
/* Switches the evaluator's shortcuts (the fused pairs and the reused copies above) off or on for the whole process; on
 * by default.  The results are the same bits either way: the switch exists to show that, and to time the difference. */
void agh_set_shortcuts(int on);
const char *agh_op_name(agh_ctx *ctx, int tensor);
int agh_topo_rank(agh_ctx *ctx, int tensor);
int agh_num_inputs(agh_ctx *ctx, int tensor);

/* ---- optimizer ------------------------------------------------------------------------------ */
agh_adam *agh_adam_new(agh_env *env, const char *adam_ns, const int *var_ids, int n, float alpha, float eps, float b1,
                       float b2);
void agh_adam_free(agh_adam *adam);
/* Optimizer::get_update_op: one tensor whose evaluation applies every update. */
int agh_adam_update_op(agh_adam *adam, agh_ctx *ctx, const int *params, const int *grads, int n);

/* ---- evaluation ----------------------------------------------------------------------------- */
/* ctx.evaluator().extend(tensors).feed(name, array)...run().  Results stay in the context until
 * the next agh_eval; agh_result_* read them.  Returns 0, or -1 if evaluation panicked. */
int agh_eval(agh_ctx *ctx, const int *tensors, int n, const char *const *feed_names, const float *const *feed_data,
             const int64_t *const *feed_shapes, const int *feed_ranks, int n_feeds);
/* The same evaluation without waiting for the device: the work is enqueued and the call returns.  The
 * statuses of the results are known (operator errors are found on the host while the work is enqueued);
 * agh_result_read and every other read of device data wait as needed.  For steps whose results are not
 * read, Optimizer::update above all (optimizers/mod.rs:63-81 only unwraps them): the host builds the next
 * graph while the device runs this one.  Feed buffers may be reused when the call returns. */
int agh_eval_nowait(agh_ctx *ctx, const int *tensors, int n, const char *const *feed_names,
                    const float *const *feed_data, const int64_t *const *feed_shapes, const int *feed_ranks,
                    int n_feeds);
/* Waits until the device has finished everything enqueued so far. */
int agh_synchronize(void);
int agh_result_status(agh_ctx *ctx, int i); /* 0 = Ok, 1..5 = OpError variant, 100 = HIP error */
const char *agh_result_message(agh_ctx *ctx, int i);
int agh_result_shape(agh_ctx *ctx, int i, int64_t *shape_out, int max_rank); /* returns the rank */
int agh_result_read(agh_ctx *ctx, int i, float *out, size_t n);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* AG_HOST_H */
