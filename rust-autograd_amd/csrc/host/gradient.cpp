// Reverse-mode gradient construction (src/gradient.rs:20-247, src/tensor_ops/mod.rs:94-114,
// src/optimizers/mod.rs:21-46).  Only graph nodes are built here; no numerics run.
#include <queue>
#include <unordered_map>

#include "ag_host.hpp"

namespace ag {
namespace host {

namespace {

struct GradientInfo {  // src/gradient.rs:150-174
    std::vector<Tensor> gradients;
    bool on_backprop_path = false;
    // the accumulated gradients are added together when first asked for
    Tensor gradient()
    {
        if (gradients.size() > 1) gradients[0] = tensor_ops::add_n(gradients);
        gradients.resize(1);
        return gradients[0];
    }
};

using GradientMap = std::unordered_map<TensorID, GradientInfo>;

bool is_given_xs(TensorID id, const std::vector<Tensor> &xs)
{
    for (const Tensor &x : xs)
        if (x.id == id) return true;
    return false;
}

// Go backward from ys and mark the nodes between ys and xs (src/gradient.rs:203-247).
GradientMap init_gradient_map(Graph &g, const std::vector<Tensor> &ys, const std::vector<Tensor> &xs)
{
    GradientMap map;
    std::vector<std::pair<TensorID, bool>> dfs;
    for (const Tensor &y : ys) dfs.emplace_back(y.id, false);
    while (!dfs.empty()) {
        const auto [id, should_visit] = dfs.back();
        dfs.pop_back();
        const TensorInternal &n = g.node(id);
        if (should_visit) {
            bool child_on_path = false;
            for (const IncomingTensor &c : n.get_backprop_inputs()) child_on_path |= map.at(c.id).on_backprop_path;
            GradientInfo info;
            info.on_backprop_path = n.is_differentiable && (is_given_xs(id, xs) || child_on_path);
            map[id] = std::move(info);
        } else {
            dfs.emplace_back(id, true);
            for (const IncomingTensor &c : n.get_backprop_inputs()) {
                if (map.count(id)) continue;
                const TensorInternal &child = g.node(c.id);
                if (child.is_source() || !child.is_differentiable) {
                    // no xs can lie beyond it: record it and stop the search in this direction
                    GradientInfo info;
                    info.on_backprop_path = child.is_differentiable && is_given_xs(child.id, xs);
                    map[child.id] = std::move(info);
                } else {
                    dfs.emplace_back(child.id, false);
                }
            }
        }
    }
    return map;
}

struct HeapNode {
    TensorID id;
    int topo_rank;
    bool operator<(const HeapNode &o) const { return topo_rank < o.topo_rank; }  // max-heap by rank
};

// `gys`: already known gradients of `ys` (gradient.rs:36-50); null = a scalar one for every y.
GradientMap compute_gradients(Graph &g, const std::vector<Tensor> &ys, const std::vector<Tensor> &xs,
                              const std::vector<Tensor> *gys = nullptr)
{
    GradientMap map = init_gradient_map(g, ys, xs);
    if (gys && gys->size() != ys.size()) throw Panic("grad_with_default: ys and ys_grads differ in length");
    std::priority_queue<HeapNode> heap;
    for (size_t i = 0; i < ys.size(); ++i) {
        const Tensor &y = ys[i];
        map.at(y.id).gradients.push_back(gys ? (*gys)[i] : tensor_ops::scalar(1.f, &g));
        heap.push(HeapNode{y.id, g.node(y.id).topo_rank});
    }
    while (!heap.empty()) {
        const HeapNode top = heap.top();
        heap.pop();
        const Tensor gy = map.at(top.id).gradient();
        GradientContext ctx(gy, g.tensor(top.id), &g);
        g.node(top.id).op->grad(ctx);  // builds new nodes only
        // snapshot: Op::grad may have grown the node table
        const std::vector<IncomingTensor> bp = g.node(top.id).get_backprop_inputs();
        std::vector<std::optional<Tensor>> &gxs = ctx.input_grads();
        if (gxs.size() != bp.size())
            throw Panic(std::string("Bad Op impl: ") + g.node(top.id).op->name() + "::grad appended " +
                        std::to_string(gxs.size()) + " gradients for " + std::to_string(bp.size()) + " back-prop inputs");
        for (size_t i = 0; i < bp.size(); ++i) {
            auto it = map.find(bp[i].id);
            if (it == map.end() || !it->second.on_backprop_path || !gxs[i]) continue;
            const bool x_not_visited = it->second.gradients.empty();
            it->second.gradients.push_back(*gxs[i]);
            const TensorInternal &x = g.node(bp[i].id);
            if (!x.is_source() && x_not_visited) heap.push(HeapNode{x.id, x.topo_rank});
        }
    }
    return map;
}

}  // namespace

namespace tensor_ops {

std::vector<Tensor> grad(const std::vector<Tensor> &ys, const std::vector<Tensor> &xs)
{
    if (ys.empty()) throw Panic("grad: no ys");
    Graph &g = *ys[0].graph;
    std::vector<Tensor> sums;
    for (const Tensor &y : ys) sums.push_back(sum_all(y));  // every y is wrapped in sum_all (mod.rs:102)
    GradientMap map = compute_gradients(g, sums, xs);
    std::vector<Tensor> ret;
    for (const Tensor &x : xs) {
        auto it = map.find(x.id);
        if (it != map.end() && it->second.on_backprop_path && !it->second.gradients.empty())
            ret.push_back(it->second.gradient());
        else
            ret.push_back(zeros_like(x));  // not differentiable (mod.rs:108-111)
    }
    return ret;
}

std::vector<Tensor> grad_with_default(const std::vector<Tensor> &ys, const std::vector<Tensor> &xs,
                                      const std::vector<Tensor> &ys_grads)
{
    // mod.rs:130-153: no sum_all wrapping, the given gradients start the back-propagation
    if (ys.empty()) throw Panic("grad_with_default: no ys");
    Graph &g = *ys[0].graph;
    GradientMap map = compute_gradients(g, ys, xs, &ys_grads);
    std::vector<Tensor> ret;
    for (const Tensor &x : xs) {
        auto it = map.find(x.id);
        if (it != map.end() && it->second.on_backprop_path && !it->second.gradients.empty())
            ret.push_back(it->second.gradient());
        else
            ret.push_back(zeros_like(x));
    }
    return ret;
}

}  // namespace tensor_ops

namespace optimizers {

std::pair<std::vector<Tensor>, std::vector<Tensor>> grad_helper(const std::vector<Tensor> &losses, Context &ctx,
                                                                const std::string &namespace_id)
{
    std::vector<Tensor> ys, xs;
    for (const Tensor &y : losses) ys.push_back(tensor_ops::sum_all(y));
    for (const auto &nv : ctx.env().names_in(namespace_id)) xs.push_back(ctx.variable(nv.second));
    GradientMap map = compute_gradients(ctx, ys, xs);
    std::pair<std::vector<Tensor>, std::vector<Tensor>> out;
    for (const Tensor &x : xs) {
        auto it = map.find(x.id);
        if (it != map.end() && it->second.on_backprop_path && !it->second.gradients.empty()) {
            out.first.push_back(x);
            out.second.push_back(it->second.gradient());
        }
    }
    return out;
}

}  // namespace optimizers

}  // namespace host
}  // namespace ag
