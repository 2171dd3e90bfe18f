// extern "C" wrapper of the host operator layer (see include/ag_host.h).
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>

#include "ag_host.h"
#include "ag_host.hpp"

using namespace ag::host;

struct agh_env {
    VariableEnvironment env;
};
struct agh_ctx {
    Context ctx;
    std::vector<EvalResult> results;
    explicit agh_ctx(VariableEnvironment *e) : ctx(e) {}
};
struct agh_adam {
    optimizers::Adam adam;
};

static thread_local std::string g_err;

template <typename F>
static int guard(F f)
{
    try {
        return f();
    } catch (const std::exception &e) {
        g_err = e.what();
        return -1;
    }
}

static Tensor T(agh_ctx *c, int id)
{
    if (id < 0 || (size_t)id >= c->ctx.num_nodes()) throw Panic("tensor id out of range");
    return c->ctx.tensor(id);
}

static Shape to_shape(const int64_t *s, int rank) { return Shape(s, s + (rank > 0 ? rank : 0)); }

extern "C" {

const char *agh_last_error(void) { return g_err.c_str(); }

agh_env *agh_env_new(void) { return new agh_env(); }
void agh_env_free(agh_env *env) { delete env; }

int agh_env_set(agh_env *env, const char *ns, const char *name, const float *data, const int64_t *shape, int rank)
{
    return guard([&] { return env->env.set(ns ? ns : "", name, NdArray::from_host(to_shape(shape, rank), data)); });
}

int agh_env_find(agh_env *env, const char *ns, const char *name)
{
    return guard([&] {
        auto id = env->env.find(ns ? ns : "", name);
        return id ? *id : -1;
    });
}

int agh_env_shape(agh_env *env, int var_id, int64_t *shape_out, int max_rank)
{
    return guard([&] {
        const Shape &s = env->env.array(var_id).shape();
        for (int i = 0; i < (int)s.size() && i < max_rank; ++i) shape_out[i] = s[(size_t)i];
        return (int)s.size();
    });
}

int agh_env_read(agh_env *env, int var_id, float *out, size_t n)
{
    return guard([&] {
        const std::vector<float> h = env->env.array(var_id).to_host();
        if (h.size() != n) throw Panic("agh_env_read: element count differs");
        std::memcpy(out, h.data(), n * sizeof(float));
        return 0;
    });
}

int agh_env_write(agh_env *env, int var_id, const float *data, size_t n)
{
    return guard([&] {
        NdArray &a = env->env.array(var_id);
        if (a.len() != n) throw Panic("agh_env_write: element count differs");
        a.copy_from_host(data);
        return 0;
    });
}

int agh_env_len(agh_env *env) { return (int)env->env.size(); }

int agh_env_save(agh_env *env, const char *path)
{
    return guard([&] {
        env->env.save(path);
        return 0;
    });
}

agh_env *agh_env_load(const char *path)
{
    agh_env *env = new agh_env();
    if (guard([&] {
            env->env.initialize(path);
            return 0;
        }) != 0) {
        delete env;
        return nullptr;
    }
    return env;
}

int agh_env_initialize(agh_env *env, const char *path)
{
    return guard([&] {
        env->env.initialize(path);
        return 0;
    });
}

int agh_env_file_rewrite(const char *src_path, const char *dst_path)
{
    return guard([&] {
        write_saved_environment(read_saved_environment(src_path), dst_path);
        return 0;
    });
}

agh_ctx *agh_ctx_new(agh_env *env) { return new agh_ctx(&env->env); }
void agh_ctx_free(agh_ctx *ctx) { delete ctx; }

int agh_variable(agh_ctx *c, int var_id) { return guard([&] { return c->ctx.variable(var_id).id; }); }

int agh_placeholder(agh_ctx *c, const char *name, const int64_t *shape, int rank)
{
    return guard([&] { return c->ctx.placeholder(name, to_shape(shape, rank)).id; });
}

int agh_scalar(agh_ctx *c, float v) { return guard([&] { return tensor_ops::scalar(v, &c->ctx).id; }); }

int agh_conv2d(agh_ctx *c, int x, int w, int pad, int stride, int dilation)
{
    return guard([&] { return tensor_ops::dilated_conv2d(T(c, x), T(c, w), pad, stride, dilation).id; });
}

int agh_conv2d_with_columns(agh_ctx *c, int x, int w, int pad, int stride, int dilation)
{
    return guard([&] { return tensor_ops::conv2d_with_columns(T(c, x), T(c, w), pad, stride, dilation).id; });
}

int agh_conv2d_transpose(agh_ctx *c, int x, int w, int pad, int stride, int dilation)
{
    return guard([&] { return tensor_ops::dilated_conv2d_transpose(T(c, x), T(c, w), pad, stride, dilation).id; });
}

int agh_max_pool2d(agh_ctx *c, int x, int pool_size, int pad, int stride)
{
    return guard([&] { return tensor_ops::max_pool2d(T(c, x), pool_size, pad, stride).id; });
}

int agh_matmul(agh_ctx *c, int a, int b) { return guard([&] { return tensor_ops::matmul(T(c, a), T(c, b)).id; }); }

int agh_batch_matmul(agh_ctx *c, int a, int b, int ta, int tb)
{
    return guard([&] { return tensor_ops::batch_matmul_t(T(c, a), T(c, b), ta != 0, tb != 0).id; });
}

int agh_reduce_sum(agh_ctx *c, int x, const int *axes, int n, int keep)
{
    return guard([&] { return tensor_ops::reduce_sum(T(c, x), std::vector<int>(axes, axes + n), keep != 0).id; });
}

int agh_reduce_mean(agh_ctx *c, int x, const int *axes, int n, int keep)
{
    return guard([&] { return tensor_ops::reduce_mean(T(c, x), std::vector<int>(axes, axes + n), keep != 0).id; });
}

int agh_sum_all(agh_ctx *c, int x) { return guard([&] { return tensor_ops::sum_all(T(c, x)).id; }); }
int agh_relu(agh_ctx *c, int x) { return guard([&] { return tensor_ops::relu(T(c, x)).id; }); }
int agh_add(agh_ctx *c, int a, int b) { return guard([&] { return tensor_ops::add(T(c, a), T(c, b)).id; }); }
int agh_mul(agh_ctx *c, int a, int b) { return guard([&] { return tensor_ops::mul(T(c, a), T(c, b)).id; }); }

int agh_add_n(agh_ctx *c, const int *xs, int n)
{
    return guard([&] {
        std::vector<Tensor> ts;
        for (int i = 0; i < n; ++i) ts.push_back(T(c, xs[i]));
        return tensor_ops::add_n(ts).id;
    });
}

int agh_nth_tensor(agh_ctx *c, int x, int n) { return guard([&] { return tensor_ops::nth_tensor(T(c, x), n).id; }); }

int agh_reshape(agh_ctx *c, int x, const int64_t *shape, int rank)
{
    return guard([&] { return tensor_ops::reshape(T(c, x), to_shape(shape, rank)).id; });
}

int agh_sparse_softmax_cross_entropy(agh_ctx *c, int logits, int labels)
{
    return guard([&] { return tensor_ops::sparse_softmax_cross_entropy(T(c, logits), T(c, labels)).id; });
}

int agh_stop_gradient(agh_ctx *c, int x) { return guard([&] { return tensor_ops::stop_gradient(T(c, x)).id; }); }

int agh_grad(agh_ctx *c, const int *ys, int ny, const int *xs, int nx, int *out)
{
    return guard([&] {
        std::vector<Tensor> y, x;
        for (int i = 0; i < ny; ++i) y.push_back(T(c, ys[i]));
        for (int i = 0; i < nx; ++i) x.push_back(T(c, xs[i]));
        const std::vector<Tensor> g = tensor_ops::grad(y, x);
        for (int i = 0; i < nx; ++i) out[i] = g[(size_t)i].id;
        return 0;
    });
}

int agh_grad_with_default(agh_ctx *c, const int *ys, const int *ys_grads, int ny, const int *xs, int nx, int *out)
{
    return guard([&] {
        std::vector<Tensor> y, gy, x;
        for (int i = 0; i < ny; ++i) {
            y.push_back(T(c, ys[i]));
            gy.push_back(T(c, ys_grads[i]));
        }
        for (int i = 0; i < nx; ++i) x.push_back(T(c, xs[i]));
        const std::vector<Tensor> g = tensor_ops::grad_with_default(y, x, gy);
        for (int i = 0; i < nx; ++i) out[i] = g[(size_t)i].id;
        return 0;
    });
}

int agh_grad_helper(agh_ctx *c, const int *losses, int n, const char *ns, int *vars_out, int *grads_out, int max_out)
{
    return guard([&] {
        std::vector<Tensor> l;
        for (int i = 0; i < n; ++i) l.push_back(T(c, losses[i]));
        const auto vg = optimizers::grad_helper(l, c->ctx, ns ? ns : "");
        const int cnt = (int)vg.first.size();
        if (cnt > max_out) throw Panic("agh_grad_helper: output arrays too small");
        for (int i = 0; i < cnt; ++i) {
            vars_out[i] = vg.first[(size_t)i].id;
            grads_out[i] = vg.second[(size_t)i].id;
        }
        return cnt;
    });
}

int agh_num_nodes(agh_ctx *c) { return (int)c->ctx.num_nodes(); }
int agh_fused_pairs(agh_ctx *c) { return (int)c->ctx.fused_pairs(); }
long long agh_reused_copies(void) { return (long long)reused_copies(); }
void agh_set_shortcuts(int on) { set_shortcuts(on != 0); }

const char *agh_op_name(agh_ctx *c, int t)
{
    try {
        return T(c, t).graph->node(t).op->name();
    } catch (const std::exception &e) {
        g_err = e.what();
        return nullptr;
    }
}

int agh_topo_rank(agh_ctx *c, int t) { return guard([&] { return T(c, t).graph->node(t).topo_rank; }); }
int agh_num_inputs(agh_ctx *c, int t) { return guard([&] { return (int)T(c, t).graph->node(t).incoming_nodes.size(); }); }

agh_adam *agh_adam_new(agh_env *env, const char *adam_ns, const int *var_ids, int n, float alpha, float eps, float b1,
                       float b2)
{
    try {
        return new agh_adam{optimizers::Adam(alpha, eps, b1, b2, std::vector<VariableID>(var_ids, var_ids + n), env->env,
                                             adam_ns)};
    } catch (const std::exception &e) {
        g_err = e.what();
        return nullptr;
    }
}

void agh_adam_free(agh_adam *adam) { delete adam; }

int agh_adam_update_op(agh_adam *adam, agh_ctx *c, const int *params, const int *grads, int n)
{
    return guard([&] {
        std::vector<Tensor> p, g;
        for (int i = 0; i < n; ++i) {
            p.push_back(T(c, params[i]));
            g.push_back(T(c, grads[i]));
        }
        return adam->adam.get_update_op(p, g, c->ctx).id;
    });
}

static int eval_impl(agh_ctx *c, const int *tensors, int n, const char *const *feed_names, const float *const *feed_data,
                     const int64_t *const *feed_shapes, const int *feed_ranks, int n_feeds, bool wait)
{
    return guard([&] {
        std::vector<Tensor> ts;
        for (int i = 0; i < n; ++i) ts.push_back(T(c, tensors[i]));
        static const bool timing = [] {
            const char *e = std::getenv("AG_HOST_TRACE");
            return e && std::string(e) == "time";
        }();
        const auto t0 = std::chrono::steady_clock::now();
        std::vector<std::pair<std::string, NdArray>> feeds;
        for (int i = 0; i < n_feeds; ++i)
            feeds.emplace_back(feed_names[i], NdArray::from_host(to_shape(feed_shapes[i], feed_ranks[i]), feed_data[i]));
        const auto t1 = std::chrono::steady_clock::now();
        c->results = c->ctx.eval(ts, feeds);
        const auto t2 = std::chrono::steady_clock::now();
        if (wait) synchronize();
        if (timing) {
            const auto t3 = std::chrono::steady_clock::now();
            auto us = [](auto a, auto b) { return std::chrono::duration<double, std::micro>(b - a).count(); };
            std::fprintf(stderr, "[ag_host] eval: feeds %.1f us, enqueue %.1f us, wait %.1f us\n", us(t0, t1), us(t1, t2), us(t2, t3));
        }
        return 0;
    });
}

int agh_eval(agh_ctx *c, const int *tensors, int n, const char *const *feed_names, const float *const *feed_data,
             const int64_t *const *feed_shapes, const int *feed_ranks, int n_feeds)
{
    return eval_impl(c, tensors, n, feed_names, feed_data, feed_shapes, feed_ranks, n_feeds, true);
}

int agh_eval_nowait(agh_ctx *c, const int *tensors, int n, const char *const *feed_names, const float *const *feed_data,
                    const int64_t *const *feed_shapes, const int *feed_ranks, int n_feeds)
{
    return eval_impl(c, tensors, n, feed_names, feed_data, feed_shapes, feed_ranks, n_feeds, false);
}

int agh_synchronize(void)
{
    return guard([&] {
        synchronize();
        return 0;
    });
}

int agh_result_status(agh_ctx *c, int i)
{
    return guard([&] { return (int)c->results.at((size_t)i).error.kind; });
}

const char *agh_result_message(agh_ctx *c, int i)
{
    try {
        return c->results.at((size_t)i).error.message.c_str();
    } catch (const std::exception &e) {
        g_err = e.what();
        return nullptr;
    }
}

int agh_result_shape(agh_ctx *c, int i, int64_t *shape_out, int max_rank)
{
    return guard([&] {
        const Shape &s = c->results.at((size_t)i).array.shape();
        for (int k = 0; k < (int)s.size() && k < max_rank; ++k) shape_out[k] = s[(size_t)k];
        return (int)s.size();
    });
}

int agh_result_read(agh_ctx *c, int i, float *out, size_t n)
{
    return guard([&] {
        const std::vector<float> h = c->results.at((size_t)i).array.to_host();
        if (h.size() != n) throw Panic("agh_result_read: element count differs");
        std::memcpy(out, h.data(), n * sizeof(float));
        return 0;
    });
}

}  // extern "C"
