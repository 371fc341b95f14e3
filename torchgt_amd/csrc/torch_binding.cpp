// PyTorch-ROCm binding of the library's hot operators: TORCH_LIBRARY ops with C++ autograd functions over the C ABI
// of include/torchgt_hip.h.  Host code only (g++): it validates the tensors, allocates the outputs with torch's
// allocator, takes the current HIP stream and calls the C entry points; nothing else happens between Python and
// the kernels.  The reference has no such layer - its hot path is a chain of ATen / torch_scatter calls from Python
// (attn_module.py:133-189, models/graphormer_dist_node_level.py:246-314) - these ops stand where that chain stood.
//
//   torchgt::sparse_attention(q, k, v, bias?, plan holder, bias_mode, workspace) -> (out, Z)
//   torchgt::dense_attention(q, k, v, bias?, p_drop, seed, bf16_products) -> out
//   torchgt::linear(x, weights[], biases?[]) -> Tensor[]                      (1 to 3 layers of one shape)
//   torchgt::add_layer_norm(x, r?, gamma, beta, eps) -> (sum, y)
//   torchgt::encoder_layer(x, residual?, params[16], plan holder, workspace, heads, eps1, eps2) -> (x + attention, ffn output)
//   torchgt::dense_encoder_layer(x, residual?, params[16], extra[], attn_bias?, sp16?, et16?, heads, eps1, eps2, p_drop, seed,
//                                bf16_products) -> (x + attention, ffn output)      the graph-level layer around the dense attention
//   torchgt::add(x, r) -> sum
//   torchgt::gelu(u) / torchgt::relu(u) -> h
//   torchgt::nll_loss(log_probs, target, ignore_index) -> loss                (mean over the rows that count)
//   torchgt::ffn(x, W1, b1, W2, b2) -> layer2(gelu(layer1(x)))
//   torchgt::multi_head_attention(x, params[6 | 8], plan holder, workspace, heads) -> y     (sparse attention, no bias)
#include <torch/library.h>
#include <torch/custom_class.h>
#include <torch/autograd.h>
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <c10/hip/HIPCachingAllocator.h>
#include <c10/core/DeviceGuard.h>

#include "../../include/torchgt_hip.h"

namespace {

using at::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

void check(int rc, const char* what) {
    TORCH_CHECK(rc == TGT_OK, what, ": ", tgt_error_string(rc), " (", tgt_last_error(), ")");
}
int dtype_code(const Tensor& t) {
    if (t.scalar_type() == at::kFloat) return TGT_DTYPE_F32;
    if (t.scalar_type() == at::kBFloat16) return TGT_DTYPE_BF16;
    TORCH_CHECK(false, "torchgt: unsupported dtype ", t.scalar_type(), " (float32 or bfloat16)");
}
void* stream_of(const Tensor& t) { return c10::hip::getCurrentHIPStream(t.device().index()).stream(); }
const void* ptr(const c10::optional<Tensor>& t) { return (t.has_value() && t->defined()) ? t->data_ptr() : nullptr; }
void on_gpu(const Tensor& t, const char* op) {
    TORCH_CHECK(t.is_cuda(), op, " needs GPU tensors (there is no CPU implementation)");
}

// The library's own device memory (plans, tile sets, scratch of the edge preparation) comes from torch's caching
// allocator once this extension is loaded: a plan built per training iteration then costs no hipMalloc / hipFree.
void* torch_alloc(size_t bytes, void* stream, void*) {
    try {
        return c10::hip::HIPCachingAllocator::raw_alloc_with_stream(bytes, static_cast<hipStream_t>(stream));
    } catch (const std::exception&) {
        return nullptr;
    }
}
void torch_free(void* p, void*) { c10::hip::HIPCachingAllocator::raw_delete(p); }
struct AllocatorRegistration {
    AllocatorRegistration() { tgt_set_allocator(&torch_alloc, &torch_free, nullptr); }
};
const AllocatorRegistration allocator_registration;

// Owner of a tgt_plan_t: the Python plan object holds one, and so does every autograd node that will need the plan
// in its backward - the plan lives until the last of them lets go.
struct PlanHolder : torch::CustomClassHolder {
    int64_t h;
    explicit PlanHolder(int64_t handle) : h(handle) {}
    ~PlanHolder() override {
        if (h) tgt_plan_destroy(reinterpret_cast<tgt_plan_t*>(h));
    }
    int64_t handle() const { return h; }
};

// the attention entry points take the number of rows from the plan: tensors of another length must not reach them
void rows_match_plan(const c10::intrusive_ptr<PlanHolder>& holder, int64_t N, const char* op) {
    int64_t info[16];
    check(tgt_plan_info(reinterpret_cast<const tgt_plan_t*>(holder->h), info), "tgt_plan_info");
    TORCH_CHECK(info[0] == N, op, ": ", N, " rows, but the plan was built for ", info[0], " nodes");
}

// ---------------------------------------------------------------------------------------------------------------
// sparse attention
// ---------------------------------------------------------------------------------------------------------------
struct SparseAttention : public torch::autograd::Function<SparseAttention> {
    static variable_list forward(AutogradContext* ctx, Tensor q, Tensor k, Tensor v, c10::optional<Tensor> bias,
                                 c10::intrusive_ptr<PlanHolder> holder, int64_t mode, Tensor ws) {
        const int64_t plan = holder->h;
        on_gpu(q, "sparse attention");
        TORCH_CHECK(q.dim() == 3 && q.sizes() == k.sizes() && q.sizes() == v.sizes(), "q, k, v must be [N, H, d] with equal shapes");
        TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "q/k/v must share a dtype");
        const int code = dtype_code(q);
        q = q.contiguous(); k = k.contiguous(); v = v.contiguous();
        Tensor b;
        if (bias.has_value() && bias->defined()) {
            TORCH_CHECK(bias->scalar_type() == q.scalar_type(), "edge bias must have the dtype of q");
            b = bias->contiguous();
        }
        const int64_t N = q.size(0), H = q.size(1), d = q.size(2);
        rows_match_plan(holder, N, "sparse_attention");
        c10::DeviceGuard guard(q.device());
        Tensor out = at::empty_like(q);
        Tensor Z = at::empty({N, H}, q.options().dtype(at::kFloat));
        check(tgt_sparse_attn_fwd(reinterpret_cast<const tgt_plan_t*>(plan), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                  b.defined() ? b.data_ptr() : nullptr, (int)mode, (int)H, (int)d, code, out.data_ptr(),
                                  Z.data_ptr<float>(), ws.data_ptr(), ws.numel(), stream_of(q)),
              "tgt_sparse_attn_fwd");
        ctx->save_for_backward({q, k, v, b, out, Z, ws});
        ctx->saved_data["plan"] = holder;
        ctx->saved_data["mode"] = mode;
        ctx->saved_data["bias_grad"] = b.defined() && bias->requires_grad();
        ctx->mark_non_differentiable({Z});
        ctx->set_materialize_grads(false);       // no zero tensor is made for Z's absent gradient
        return {out, Z};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        auto saved = ctx->get_saved_variables();
        const Tensor &q = saved[0], &k = saved[1], &v = saved[2], &b = saved[3], &out = saved[4], &Z = saved[5], &ws = saved[6];
        const int64_t plan = ctx->saved_data["plan"].toCustomClass<PlanHolder>()->h, mode = ctx->saved_data["mode"].toInt();
        const int64_t H = q.size(1), d = q.size(2);
        if (!grads[0].defined()) return {Tensor(), Tensor(), Tensor(), Tensor(), Tensor(), Tensor(), Tensor()};
        Tensor dout = grads[0].contiguous();
        c10::DeviceGuard guard(q.device());
        Tensor dq = at::empty_like(q), dk = at::empty_like(k), dv = at::empty_like(v), dbias;
        if (b.defined() && ctx->saved_data["bias_grad"].toBool()) {
            dbias = at::empty_like(b);
            if (mode & TGT_BIAS_BOTH_ORDERS) dbias.narrow(0, b.size(0) / 2, b.size(0) / 2).zero_();   // the source-sorted copy gets none
        }
        check(tgt_sparse_attn_bwd(reinterpret_cast<const tgt_plan_t*>(plan), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                  b.defined() ? b.data_ptr() : nullptr, (int)mode, (int)H, (int)d, dtype_code(q), out.data_ptr(),
                                  Z.data_ptr<float>(), dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                  dbias.defined() ? dbias.data_ptr() : nullptr, ws.data_ptr(), ws.numel(), stream_of(q)),
              "tgt_sparse_attn_bwd");
        return {dq, dk, dv, dbias, Tensor(), Tensor(), Tensor()};
    }
};
std::tuple<Tensor, Tensor> sparse_attention(const Tensor& q, const Tensor& k, const Tensor& v, const c10::optional<Tensor>& bias,
                                            const c10::intrusive_ptr<PlanHolder>& plan, int64_t mode, const Tensor& ws) {
    auto r = SparseAttention::apply(q, k, v, bias, plan, mode, ws);
    return {r[0], r[1]};
}

// ---------------------------------------------------------------------------------------------------------------
// dense attention
// ---------------------------------------------------------------------------------------------------------------
struct DenseAttention : public torch::autograd::Function<DenseAttention> {
    static Tensor forward(AutogradContext* ctx, Tensor q, Tensor k, Tensor v, c10::optional<Tensor> bias, double p_drop,
                          int64_t seed, bool bf16_products) {
        on_gpu(q, "dense attention");
        TORCH_CHECK(q.dim() == 4 && q.sizes() == k.sizes() && q.sizes() == v.sizes(), "q, k, v must be [b, S, H, d] with equal shapes");
        TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "q/k/v must share a dtype");
        int code = dtype_code(q);
        if (code == TGT_DTYPE_F32 && bf16_products) code = TGT_DTYPE_F32_BF16_PRODUCTS;
        q = q.contiguous(); k = k.contiguous(); v = v.contiguous();
        const int64_t b = q.size(0), S = q.size(1), H = q.size(2), d = q.size(3);
        Tensor bb;
        if (bias.has_value() && bias->defined()) {
            TORCH_CHECK(bias->scalar_type() == q.scalar_type() && bias->dim() == 4 && bias->size(0) == b && bias->size(1) == H &&
                            bias->size(2) == S && bias->size(3) == S,
                        "attn_bias must be [b, H, S, S] of q's dtype");
            bb = bias->contiguous();
        }
        c10::DeviceGuard guard(q.device());
        Tensor out = at::empty({b, S, H * d}, q.options());
        Tensor lse = at::empty({b, H, S}, q.options().dtype(at::kFloat));
        check(tgt_dense_attn_dropout_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), bb.defined() ? bb.data_ptr() : nullptr, (int)b,
                                         (int)S, (int)H, (int)d, code, (float)p_drop, (uint64_t)seed, out.data_ptr(),
                                         lse.data_ptr<float>(), stream_of(q)),
              "tgt_dense_attn_dropout_fwd");
        ctx->save_for_backward({q, k, v, bb, out, lse});
        ctx->saved_data["code"] = (int64_t)code;
        ctx->saved_data["p"] = p_drop;
        ctx->saved_data["seed"] = seed;
        ctx->saved_data["bias_grad"] = bb.defined() && bias->requires_grad();
        return out;
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        auto saved = ctx->get_saved_variables();
        const Tensor &q = saved[0], &k = saved[1], &v = saved[2], &bb = saved[3], &out = saved[4], &lse = saved[5];
        const int64_t b = q.size(0), S = q.size(1), H = q.size(2), d = q.size(3);
        Tensor dout = grads[0].contiguous();
        c10::DeviceGuard guard(q.device());
        Tensor dq = at::empty_like(q), dk = at::empty_like(k), dv = at::empty_like(v), dbias;
        if (bb.defined() && ctx->saved_data["bias_grad"].toBool()) dbias = at::empty_like(bb);
        check(tgt_dense_attn_dropout_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), bb.defined() ? bb.data_ptr() : nullptr, (int)b,
                                         (int)S, (int)H, (int)d, (int)ctx->saved_data["code"].toInt(),
                                         (float)ctx->saved_data["p"].toDouble(), (uint64_t)ctx->saved_data["seed"].toInt(),
                                         out.data_ptr(), lse.data_ptr<float>(), dout.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                         dv.data_ptr(), dbias.defined() ? dbias.data_ptr() : nullptr, stream_of(q)),
              "tgt_dense_attn_dropout_bwd");
        return {dq, dk, dv, dbias, Tensor(), Tensor(), Tensor()};
    }
};
Tensor dense_attention(const Tensor& q, const Tensor& k, const Tensor& v, const c10::optional<Tensor>& bias, double p_drop,
                       int64_t seed, bool bf16_products) {
    return DenseAttention::apply(q, k, v, bias, p_drop, seed, bf16_products);
}

// ---------------------------------------------------------------------------------------------------------------
// dense attention with the bias formed in the kernels from packed ids and the three tables
// ---------------------------------------------------------------------------------------------------------------
struct DenseAttentionIds : public torch::autograd::Function<DenseAttentionIds> {
    static Tensor forward(AutogradContext* ctx, Tensor q, Tensor k, Tensor v, c10::optional<Tensor> attn_bias, Tensor sp16,
                          Tensor et16, Tensor sp_tab, Tensor e_tab, Tensor vd, double p_drop, int64_t seed, bool bf16_products) {
        on_gpu(q, "dense attention from ids");
        TORCH_CHECK(q.dim() == 4 && q.sizes() == k.sizes() && q.sizes() == v.sizes(), "q, k, v must be [b, S, H, d] with equal shapes");
        TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "q/k/v must share a dtype");
        int code = dtype_code(q);
        TORCH_CHECK(code != TGT_DTYPE_F32 || bf16_products,
                    "dense attention from ids computes with bf16 matrix products: pass bf16 tensors, or float32 with bf16_products");
        if (code == TGT_DTYPE_F32) code = TGT_DTYPE_F32_BF16_PRODUCTS;
        q = q.contiguous(); k = k.contiguous(); v = v.contiguous();
        const int64_t b = q.size(0), S = q.size(1), H = q.size(2), d = q.size(3);
        TORCH_CHECK(sp16.scalar_type() == at::kShort && sp16.dim() == 3 && sp16.size(0) == b && sp16.size(1) == S && sp16.size(2) == S &&
                        sp16.is_contiguous(), "sp16 must be a contiguous int16 [b, S, S] (tgt_dense_ids_pack)");
        TORCH_CHECK(et16.scalar_type() == at::kShort && et16.dim() == 4 && et16.size(0) == b && et16.size(1) == S && et16.size(2) == S &&
                        et16.is_contiguous(), "et16 must be a contiguous int16 [b, S, S, F] (tgt_dense_ids_pack)");
        const int64_t F = et16.size(3);
        TORCH_CHECK(sp_tab.dim() == 2 && e_tab.dim() == 2 && sp_tab.size(1) == H && e_tab.size(1) == H && vd.numel() == H &&
                        sp_tab.scalar_type() == q.scalar_type() && e_tab.scalar_type() == q.scalar_type() &&
                        vd.scalar_type() == q.scalar_type(), "tables must be [rows, H] / [H] of q's dtype");
        Tensor ab;
        if (attn_bias.has_value() && attn_bias->defined()) {
            TORCH_CHECK(attn_bias->scalar_type() == q.scalar_type() && attn_bias->dim() == 3 && attn_bias->size(0) == b &&
                            attn_bias->size(1) == S && attn_bias->size(2) == S, "attn_bias must be [b, S, S] of q's dtype");
            ab = attn_bias->contiguous();
        }
        Tensor st = sp_tab.contiguous(), et = e_tab.contiguous(), vdc = vd.reshape({-1}).contiguous();
        c10::DeviceGuard guard(q.device());
        Tensor out = at::empty({b, S, H * d}, q.options());
        Tensor lse = at::empty({b, H, S}, q.options().dtype(at::kFloat));
        check(tgt_dense_attn_ids_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), ab.defined() ? ab.data_ptr() : nullptr,
                                     reinterpret_cast<const uint16_t*>(sp16.data_ptr()), reinterpret_cast<const uint16_t*>(et16.data_ptr()),
                                     (int)F, st.data_ptr(), (int)st.size(0), et.data_ptr(), (int)et.size(0), vdc.data_ptr(), (int)b,
                                     (int)S, (int)H, (int)d, code, (float)p_drop, (uint64_t)seed, out.data_ptr(),
                                     lse.data_ptr<float>(), stream_of(q)),
              "tgt_dense_attn_ids_fwd");
        ctx->save_for_backward({q, k, v, ab, sp16, et16, st, et, vdc, out, lse});
        ctx->saved_data["code"] = (int64_t)code;
        ctx->saved_data["p"] = p_drop;
        ctx->saved_data["seed"] = seed;
        ctx->saved_data["vd_shape"] = vd.sizes().vec();
        return out;
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        auto saved = ctx->get_saved_variables();
        const Tensor &q = saved[0], &k = saved[1], &v = saved[2], &ab = saved[3], &sp16 = saved[4], &et16 = saved[5], &st = saved[6],
                     &et = saved[7], &vd = saved[8], &out = saved[9], &lse = saved[10];
        const int64_t b = q.size(0), S = q.size(1), H = q.size(2), d = q.size(3), F = et16.size(3);
        Tensor dout = grads[0].contiguous();
        c10::DeviceGuard guard(q.device());
        Tensor dq = at::empty_like(q), dk = at::empty_like(k), dv = at::empty_like(v), dst, det, dvd, ws;
        const bool tables = ctx->needs_input_grad(6) || ctx->needs_input_grad(7) || ctx->needs_input_grad(8);
        int64_t ws_bytes = 0;
        if (tables) {
            dst = at::empty_like(st); det = at::empty_like(et); dvd = at::empty_like(vd);
            ws_bytes = tgt_dense_attn_ids_bwd_workspace_bytes((int)b, (int)H, (int)st.size(0), (int)et.size(0));
            ws = at::empty({ws_bytes}, q.options().dtype(at::kByte));
        }
        check(tgt_dense_attn_ids_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), ab.defined() ? ab.data_ptr() : nullptr,
                                     reinterpret_cast<const uint16_t*>(sp16.data_ptr()), reinterpret_cast<const uint16_t*>(et16.data_ptr()),
                                     (int)F, st.data_ptr(), (int)st.size(0), et.data_ptr(), (int)et.size(0), vd.data_ptr(), (int)b, (int)S,
                                     (int)H, (int)d, (int)ctx->saved_data["code"].toInt(), (float)ctx->saved_data["p"].toDouble(),
                                     (uint64_t)ctx->saved_data["seed"].toInt(), out.data_ptr(), lse.data_ptr<float>(), dout.data_ptr(),
                                     dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), tables ? dst.data_ptr() : nullptr,
                                     tables ? det.data_ptr() : nullptr, tables ? dvd.data_ptr() : nullptr,
                                     tables ? ws.data_ptr() : nullptr, ws_bytes, stream_of(q)),
              "tgt_dense_attn_ids_bwd");
        if (tables) dvd = dvd.view(ctx->saved_data["vd_shape"].toIntVector());
        return {dq, dk, dv, Tensor(), Tensor(), Tensor(), dst, det, dvd, Tensor(), Tensor(), Tensor()};
    }
};
Tensor dense_attention_ids(const Tensor& q, const Tensor& k, const Tensor& v, const c10::optional<Tensor>& attn_bias, const Tensor& sp16,
                           const Tensor& et16, const Tensor& sp_tab, const Tensor& e_tab, const Tensor& vd, double p_drop, int64_t seed,
                           bool bf16_products) {
    return DenseAttentionIds::apply(q, k, v, attn_bias, sp16, et16, sp_tab, e_tab, vd, p_drop, seed, bf16_products);
}
// the reference's int64 ids to the packed form, once per batch
std::tuple<Tensor, Tensor> dense_ids_pack(const Tensor& spatial_pos, const Tensor& edge_type, int64_t num_spatial, int64_t num_edges) {
    on_gpu(spatial_pos, "dense_ids_pack");
    TORCH_CHECK(spatial_pos.dim() == 3 && edge_type.dim() == 4 && spatial_pos.size(1) == spatial_pos.size(2) &&
                    edge_type.size(0) == spatial_pos.size(0) && edge_type.size(1) == spatial_pos.size(1) &&
                    edge_type.size(2) == spatial_pos.size(1), "spatial_pos [b, s, s] and attn_edge_type [b, s, s, F] expected");
    Tensor sp = spatial_pos.to(at::kLong).contiguous(), et = edge_type.to(at::kLong).contiguous();
    const int64_t b = sp.size(0), s = sp.size(1), F = et.size(3);
    c10::DeviceGuard guard(sp.device());
    Tensor sp16 = at::empty({b, s + 1, s + 1}, sp.options().dtype(at::kShort));
    Tensor et16 = at::empty({b, s + 1, s + 1, F}, sp.options().dtype(at::kShort));
    check(tgt_dense_ids_pack(sp.data_ptr<int64_t>(), et.data_ptr<int64_t>(), (int)b, (int)s, (int)F, (int)num_spatial, (int)num_edges,
                             reinterpret_cast<uint16_t*>(sp16.data_ptr()), reinterpret_cast<uint16_t*>(et16.data_ptr()), stream_of(sp)),
          "tgt_dense_ids_pack");
    return {sp16, et16};
}

// ---------------------------------------------------------------------------------------------------------------
// 1 to 3 linear layers of one shape on the same input
// ---------------------------------------------------------------------------------------------------------------
struct Linear : public torch::autograd::Function<Linear> {
    // wb: the n weights, then the biases that exist (bit j of bias_mask: layer j has one), in layer order
    static variable_list forward(AutogradContext* ctx, Tensor x, at::TensorList wb, int64_t n64, int64_t bias_mask) {
        on_gpu(x, "linear");
        const int n = (int)n64;
        TORCH_CHECK(n >= 1 && n <= 3 && (int)wb.size() >= n, "linear takes 1 to 3 (weight, bias) pairs");
        const int code = dtype_code(x);
        const int64_t out_f = wb[0].size(0), in_f = wb[0].size(1);
        TORCH_CHECK(x.size(-1) == in_f, "x has ", x.size(-1), " features, the weights take ", in_f);
        Tensor x2 = x.reshape({-1, in_f}).contiguous();
        const int64_t N = x2.size(0);
        std::vector<Tensor> save{x2};
        const void *W[3] = {nullptr, nullptr, nullptr}, *B[3] = {nullptr, nullptr, nullptr};
        void* Y[3] = {nullptr, nullptr, nullptr};
        variable_list ys;
        c10::DeviceGuard guard(x.device());
        std::vector<Tensor> keep;
        int next_bias = n;
        for (int j = 0; j < n; ++j) {
            const Tensor& w = wb[j];
            TORCH_CHECK(w.dim() == 2 && w.size(0) == out_f && w.size(1) == in_f && w.scalar_type() == x.scalar_type(),
                        "all weights must be [out, in] of x's dtype");
            Tensor wc = w.contiguous();
            save.push_back(wc);
            W[j] = wc.data_ptr();
            if (bias_mask & (1 << j)) {
                TORCH_CHECK(next_bias < (int)wb.size(), "fewer biases than the mask says");
                const Tensor& bj = wb[next_bias++];
                TORCH_CHECK(bj.numel() == out_f && bj.scalar_type() == x.scalar_type(), "all biases must be [out] of x's dtype");
                keep.push_back(bj.contiguous());
                B[j] = keep.back().data_ptr();
            }
            ys.push_back(at::empty({N, out_f}, x.options()));
            Y[j] = ys.back().data_ptr();
        }
        check(tgt_linear_fwd(x2.data_ptr(), W, B, Y, n, N, (int)in_f, (int)out_f, code, stream_of(x)), "tgt_linear_fwd");
        ctx->save_for_backward(save);
        ctx->saved_data["bias_mask"] = bias_mask;
        ctx->saved_data["x_shape"] = x.sizes().vec();
        std::vector<int64_t> oshape(x.sizes().vec());
        oshape.back() = out_f;
        for (auto& y : ys) y = y.view(oshape);
        return ys;
    }
    static variable_list backward(AutogradContext* ctx, variable_list dys) {
        auto saved = ctx->get_saved_variables();
        const Tensor& x2 = saved[0];
        const int n = (int)saved.size() - 1;
        const int64_t out_f = saved[1].size(0), in_f = saved[1].size(1), N = x2.size(0);
        const int64_t bias_mask = ctx->saved_data["bias_mask"].toInt();
        int n_bias = 0;
        for (int j = 0; j < n; ++j) n_bias += (bias_mask >> j) & 1;
        const bool need_dx = ctx->needs_input_grad(0);
        bool need_dw = false;
        for (int j = 0; j < n + n_bias; ++j) need_dw = need_dw || ctx->needs_input_grad(1 + j);
        c10::DeviceGuard guard(x2.device());
        const void *W[3] = {nullptr, nullptr, nullptr}, *DY[3] = {nullptr, nullptr, nullptr};
        void *DW[3] = {nullptr, nullptr, nullptr}, *DB[3] = {nullptr, nullptr, nullptr};
        std::vector<Tensor> dyc, dWs(n), dbs(n);
        for (int j = 0; j < n; ++j) {
            W[j] = saved[1 + j].data_ptr();
            dyc.push_back(dys[j].defined() ? dys[j].reshape({N, out_f}).contiguous() : at::zeros({N, out_f}, x2.options()));
            DY[j] = dyc.back().data_ptr();
            if (need_dw) {
                dWs[j] = at::empty_like(saved[1 + j]);
                DW[j] = dWs[j].data_ptr();
                if (bias_mask & (1 << j)) {
                    dbs[j] = at::empty({out_f}, x2.options());
                    DB[j] = dbs[j].data_ptr();
                }
            }
        }
        Tensor dx, ws;
        if (need_dx) dx = at::empty_like(x2);
        int64_t ws_bytes = 0;
        if (need_dw) {
            ws_bytes = tgt_linear_bwd_workspace_bytes(n, (int)in_f, (int)out_f);
            ws = at::empty({ws_bytes}, x2.options().dtype(at::kByte));
        }
        check(tgt_linear_bwd(x2.data_ptr(), W, DY, n, N, (int)in_f, (int)out_f, dtype_code(x2), need_dx ? dx.data_ptr() : nullptr,
                             need_dw ? DW : nullptr, need_dw ? DB : nullptr, need_dw ? ws.data_ptr() : nullptr, ws_bytes,
                             stream_of(x2)),
              "tgt_linear_bwd");
        variable_list out;
        out.push_back(need_dx ? dx.view(ctx->saved_data["x_shape"].toIntVector()) : Tensor());
        for (int j = 0; j < n; ++j) out.push_back(dWs[j]);
        for (int j = 0; j < n; ++j)
            if (bias_mask & (1 << j)) out.push_back(dbs[j]);
        out.push_back(Tensor());     // n
        out.push_back(Tensor());     // bias_mask
        return out;
    }
};
std::vector<Tensor> linear(const Tensor& x, at::TensorList weights, const c10::List<c10::optional<Tensor>>& biases) {
    TORCH_CHECK(weights.size() == biases.size(), "one bias slot per weight");
    variable_list wb(weights.begin(), weights.end());
    int64_t mask = 0;
    for (size_t j = 0; j < biases.size(); ++j) {
        c10::optional<Tensor> b = biases.get(j);
        if (b.has_value() && b->defined()) {
            wb.push_back(*b);
            mask |= (int64_t)1 << j;
        }
    }
    return Linear::apply(x, at::TensorList(wb), (int64_t)weights.size(), mask);      // a TensorList: every entry is an autograd input
}

// ---------------------------------------------------------------------------------------------------------------
// residual add + LayerNorm, add, GELU / ReLU
// ---------------------------------------------------------------------------------------------------------------
struct AddLayerNorm : public torch::autograd::Function<AddLayerNorm> {
    static variable_list forward(AutogradContext* ctx, Tensor x, c10::optional<Tensor> r, Tensor gamma, Tensor beta, double eps) {
        on_gpu(x, "add_layer_norm");
        const int code = dtype_code(x);
        const int64_t C = x.size(-1);
        Tensor x2 = x.reshape({-1, C}).contiguous(), r2;
        const bool has_r = r.has_value() && r->defined();
        if (has_r) r2 = r->reshape({-1, C}).contiguous();
        const int64_t N = x2.size(0);
        c10::DeviceGuard guard(x.device());
        Tensor s = has_r ? at::empty_like(x2) : x2, y = at::empty_like(x2);
        Tensor mean = at::empty({N}, x.options().dtype(at::kFloat)), rstd = at::empty({N}, x.options().dtype(at::kFloat));
        Tensor g = gamma.contiguous(), b = beta.contiguous();
        check(tgt_add_layer_norm_fwd(x2.data_ptr(), has_r ? r2.data_ptr() : nullptr, g.data_ptr(), b.data_ptr(), N, (int)C, (float)eps,
                                     code, has_r ? s.data_ptr() : nullptr, y.data_ptr(), mean.data_ptr<float>(),
                                     rstd.data_ptr<float>(), stream_of(x)),
              "tgt_add_layer_norm_fwd");
        ctx->save_for_backward({s, g, mean, rstd});
        ctx->saved_data["has_r"] = has_r;
        ctx->saved_data["shape"] = x.sizes().vec();
        ctx->set_materialize_grads(false);       // an output nobody differentiates costs no zero tensor
        return {s.view(x.sizes()), y.view(x.sizes())};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        auto saved = ctx->get_saved_variables();
        const Tensor &s = saved[0], &g = saved[1], &mean = saved[2], &rstd = saved[3];
        const int64_t N = s.size(0), C = s.size(1);
        c10::DeviceGuard guard(s.device());
        Tensor dy = grads[1].defined() ? grads[1].reshape({N, C}).contiguous() : at::zeros_like(s);
        Tensor extra;
        if (grads[0].defined()) extra = grads[0].reshape({N, C}).contiguous();
        Tensor ds = at::empty_like(s), dg = at::empty_like(g), db = at::empty_like(g);
        const int64_t nbytes = tgt_layer_norm_bwd_workspace_bytes((int)C);
        Tensor ws = at::empty({nbytes}, s.options().dtype(at::kByte));
        check(tgt_layer_norm_bwd(s.data_ptr(), g.data_ptr(), mean.data_ptr<float>(), rstd.data_ptr<float>(), dy.data_ptr(),
                                 extra.defined() ? extra.data_ptr() : nullptr, N, (int)C, dtype_code(s), ds.data_ptr(), dg.data_ptr(),
                                 db.data_ptr(), ws.data_ptr(), nbytes, stream_of(s)),
              "tgt_layer_norm_bwd");
        Tensor dsv = ds.view(ctx->saved_data["shape"].toIntVector());
        return {dsv, ctx->saved_data["has_r"].toBool() ? dsv : Tensor(), dg, db, Tensor()};
    }
};
std::tuple<Tensor, Tensor> add_layer_norm(const Tensor& x, const c10::optional<Tensor>& r, const Tensor& gamma, const Tensor& beta,
                                          double eps) {
    auto o = AddLayerNorm::apply(x, r, gamma, beta, eps);
    return {o[0], o[1]};
}

struct Add : public torch::autograd::Function<Add> {
    static Tensor forward(AutogradContext* ctx, Tensor x, Tensor r) {
        on_gpu(x, "add");
        const int64_t C = x.size(-1);
        Tensor x2 = x.reshape({-1, C}).contiguous(), r2 = r.reshape({-1, C}).contiguous();
        c10::DeviceGuard guard(x.device());
        Tensor s = at::empty_like(x2);
        check(tgt_add_layer_norm_fwd(x2.data_ptr(), r2.data_ptr(), nullptr, nullptr, x2.size(0), (int)C, 0.f, dtype_code(x), s.data_ptr(),
                                     nullptr, nullptr, nullptr, stream_of(x)),
              "tgt_add_layer_norm_fwd");
        return s.view(x.sizes());
    }
    static variable_list backward(AutogradContext*, variable_list grads) { return {grads[0], grads[0]}; }
};
Tensor add(const Tensor& x, const Tensor& r) { return Add::apply(x, r); }

template <bool GELU>
struct Activation : public torch::autograd::Function<Activation<GELU>> {
    static Tensor forward(AutogradContext* ctx, Tensor u) {
        on_gpu(u, GELU ? "gelu" : "relu");
        Tensor u2 = u.contiguous();
        c10::DeviceGuard guard(u.device());
        Tensor h = at::empty_like(u2);
        check((GELU ? tgt_gelu_fwd : tgt_relu_fwd)(u2.data_ptr(), u2.numel(), dtype_code(u), h.data_ptr(), stream_of(u)),
              GELU ? "tgt_gelu_fwd" : "tgt_relu_fwd");
        ctx->save_for_backward({u2});
        return h;
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const Tensor u = ctx->get_saved_variables()[0];
        Tensor dh = grads[0].contiguous();
        c10::DeviceGuard guard(u.device());
        Tensor du = at::empty_like(u);
        check((GELU ? tgt_gelu_bwd : tgt_relu_bwd)(u.data_ptr(), dh.data_ptr(), u.numel(), dtype_code(u), du.data_ptr(), stream_of(u)),
              GELU ? "tgt_gelu_bwd" : "tgt_relu_bwd");
        return {du};
    }
};
Tensor gelu(const Tensor& u) { return Activation<true>::apply(u); }
Tensor relu(const Tensor& u) { return Activation<false>::apply(u); }

// F.nll_loss(log_probs [N, C], target [N] int64), reduction 'mean' (main_sp_sparse_node_level.py:200)
struct NllLoss : public torch::autograd::Function<NllLoss> {
    static Tensor forward(AutogradContext* ctx, Tensor logp, Tensor target, int64_t ignore_index) {
        on_gpu(logp, "nll_loss");
        TORCH_CHECK(logp.dim() == 2, "nll_loss: log_probs must be [N, C]");
        TORCH_CHECK(target.is_cuda() && target.scalar_type() == at::kLong && target.dim() == 1 && target.size(0) == logp.size(0),
                    "nll_loss: target must be an int64 GPU tensor [N]");
        Tensor lp = logp.contiguous(), t = target.contiguous();
        c10::DeviceGuard guard(logp.device());
        const int64_t N = lp.size(0), C = lp.size(1);
        Tensor loss = at::empty({}, lp.options()), count = at::empty({1}, lp.options().dtype(at::kFloat));
        const int64_t nbytes = tgt_nll_loss_workspace_bytes(N);
        Tensor ws = at::empty({nbytes}, lp.options().dtype(at::kByte));
        check(tgt_nll_loss_fwd(lp.data_ptr(), t.data_ptr<int64_t>(), N, (int)C, dtype_code(lp), ignore_index, loss.data_ptr(),
                               count.data_ptr<float>(), ws.data_ptr(), nbytes, stream_of(lp)),
              "tgt_nll_loss_fwd");
        ctx->save_for_backward({t, count});
        ctx->saved_data["C"] = C;
        ctx->saved_data["ignore"] = ignore_index;
        ctx->saved_data["bf16"] = lp.scalar_type() == at::kBFloat16;
        return loss;
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        auto sv = ctx->get_saved_variables();
        const Tensor &t = sv[0], &count = sv[1];
        c10::DeviceGuard guard(t.device());
        const int64_t N = t.size(0), C = ctx->saved_data["C"].toInt();
        const auto dt = ctx->saved_data["bf16"].toBool() ? at::kBFloat16 : at::kFloat;
        Tensor g = grads[0].to(dt).contiguous();
        Tensor d = at::empty({N, C}, t.options().dtype(dt));
        check(tgt_nll_loss_bwd(t.data_ptr<int64_t>(), g.data_ptr(), count.data_ptr<float>(), N, (int)C, dtype_code(d),
                               ctx->saved_data["ignore"].toInt(), d.data_ptr(), stream_of(d)),
              "tgt_nll_loss_bwd");
        return {d, Tensor(), Tensor()};
    }
};
Tensor nll_loss(const Tensor& logp, const Tensor& target, int64_t ignore_index) { return NllLoss::apply(logp, target, ignore_index); }

// ---------------------------------------------------------------------------------------------------------------
// one whole encoder layer of the node-level Graphormer (models/graphormer_dist_node_level.py:276-314) with sparse
// attention, no bias, no dropout: the seven kernels of the forward and the nine of the backward launched from one
// operator and one autograd node instead of eight of each.  The same numbers as the modules give op by op; what goes
// away is the per-operator cost of the dispatcher and of autograd between the launches, and what only a whole layer
// can do: GELU rides on the FFN linears (tgt_linear_act_fwd / _bwd) and the six sums over weight-gradient partials
// share one launch at the end of the backward (tgt_reduce_partials).
//   s1 = x (+ residual); y1 = LN1(s1); q, k, v = y1 W^T + b; o = attention(q, k, v); a = o Wo^T + bo
//   s2 = s1 + a; y2 = LN2(s2); u = y2 W1^T + b1; h = gelu(u); f = h W2^T + b2;  returns (s2, f)
// params: n1.weight, n1.bias, Wq, bq, Wk, bk, Wv, bv, Wo, bo, n2.weight, n2.bias, W1, b1, W2, b2
// ---------------------------------------------------------------------------------------------------------------
namespace layer {
// The sums over workgroup partials that the backward kernels of a layer leave behind, for one launch at the layer's end.
struct Deferred {
    std::vector<tgt_reduce_desc> sums;
    std::vector<Tensor> workspaces;       // hold the partials until the launch
    void run(int code, void* stream) {
        for (size_t i = 0; i < sums.size(); i += 8)
            check(tgt_reduce_partials(sums.data() + i, (int)std::min<size_t>(8, sums.size() - i), code, stream), "tgt_reduce_partials");
        sums.clear();
    }
};
void ln_fwd(const Tensor& x, const Tensor& r, const Tensor& g, const Tensor& b, double eps, Tensor& sum, Tensor& y, Tensor& mean,
            Tensor& rstd) {
    const int64_t N = x.size(0), C = x.size(1);
    sum = r.defined() ? at::empty_like(x) : x;
    y = at::empty_like(x);
    mean = at::empty({N}, x.options().dtype(at::kFloat));
    rstd = at::empty({N}, x.options().dtype(at::kFloat));
    check(tgt_add_layer_norm_fwd(x.data_ptr(), r.defined() ? r.data_ptr() : nullptr, g.data_ptr(), b.data_ptr(), N, (int)C, (float)eps,
                                 dtype_code(x), r.defined() ? sum.data_ptr() : nullptr, y.data_ptr(), mean.data_ptr<float>(),
                                 rstd.data_ptr<float>(), stream_of(x)),
          "tgt_add_layer_norm_fwd");
}
// ds = LN backward of dy (+ extra), dgamma, dbeta
void ln_bwd(const Tensor& s, const Tensor& g, const Tensor& mean, const Tensor& rstd, const Tensor& dy, const Tensor& extra, Tensor& ds,
            Tensor& dg, Tensor& db, Deferred& later) {
    const int64_t N = s.size(0), C = s.size(1);
    ds = at::empty_like(s); dg = at::empty_like(g); db = at::empty_like(g);
    const int64_t nbytes = tgt_layer_norm_bwd_workspace_bytes((int)C);
    Tensor ws = at::empty({nbytes}, s.options().dtype(at::kByte));
    tgt_reduce_desc sum;
    check(tgt_layer_norm_bwd_deferred(s.data_ptr(), g.data_ptr(), mean.data_ptr<float>(), rstd.data_ptr<float>(), dy.data_ptr(),
                                      extra.defined() ? extra.data_ptr() : nullptr, N, (int)C, dtype_code(s), ds.data_ptr(), dg.data_ptr(),
                                      db.data_ptr(), ws.data_ptr(), nbytes, stream_of(s), &sum),
          "tgt_layer_norm_bwd_deferred");
    later.sums.push_back(sum);
    later.workspaces.push_back(ws);
}
// ys[j] = x W[j]^T + b[j]
void lin_fwd(const Tensor& x, std::initializer_list<const Tensor*> W, std::initializer_list<const Tensor*> b, std::vector<Tensor>& ys) {
    const int n = (int)W.size();
    const int64_t N = x.size(0), in_f = x.size(1), out_f = (*W.begin())->size(0);
    const void *Wp[3] = {nullptr, nullptr, nullptr}, *Bp[3] = {nullptr, nullptr, nullptr};
    void* Yp[3] = {nullptr, nullptr, nullptr};
    ys.clear();
    int j = 0;
    for (const Tensor* w : W) Wp[j++] = w->data_ptr();
    j = 0;
    for (const Tensor* bb : b) Bp[j++] = bb->data_ptr();
    for (j = 0; j < n; ++j) { ys.push_back(at::empty({N, out_f}, x.options())); Yp[j] = ys.back().data_ptr(); }
    check(tgt_linear_fwd(x.data_ptr(), Wp, Bp, Yp, n, N, (int)in_f, (int)out_f, dtype_code(x), stream_of(x)), "tgt_linear_fwd");
}
// dx = sum_j dy[j] W[j]; dW[j] = dy[j]^T x; db[j] = column sums of dy[j]
void lin_bwd(const Tensor& x, std::initializer_list<const Tensor*> W, std::initializer_list<const Tensor*> dy, Tensor& dx,
             std::vector<Tensor>& dW, std::vector<Tensor>& db, Deferred& later) {
    const int n = (int)W.size();
    const int64_t N = x.size(0), in_f = x.size(1), out_f = (*W.begin())->size(0);
    const void *Wp[3] = {nullptr, nullptr, nullptr}, *DYp[3] = {nullptr, nullptr, nullptr};
    void *DWp[3] = {nullptr, nullptr, nullptr}, *DBp[3] = {nullptr, nullptr, nullptr};
    dW.clear(); db.clear();
    int j = 0;
    for (const Tensor* w : W) { Wp[j] = w->data_ptr(); dW.push_back(at::empty_like(*w)); DWp[j] = dW.back().data_ptr();
                                db.push_back(at::empty({out_f}, x.options())); DBp[j] = db.back().data_ptr(); ++j; }
    j = 0;
    for (const Tensor* d : dy) DYp[j++] = d->data_ptr();
    dx = at::empty_like(x);
    const int64_t ws_bytes = tgt_linear_bwd_workspace_bytes(n, (int)in_f, (int)out_f);
    Tensor ws = at::empty({ws_bytes}, x.options().dtype(at::kByte));
    tgt_reduce_desc sum;
    check(tgt_linear_bwd_deferred(x.data_ptr(), Wp, DYp, n, N, (int)in_f, (int)out_f, dtype_code(x), dx.data_ptr(), DWp, DBp, ws.data_ptr(),
                                  ws_bytes, stream_of(x), &sum),
          "tgt_linear_bwd_deferred");
    later.sums.push_back(sum);
    later.workspaces.push_back(ws);
}
// u = x W^T + b, h = gelu(u) from one kernel
void lin_gelu_fwd(const Tensor& x, const Tensor& W, const Tensor& b, Tensor& u, Tensor& h) {
    const int64_t N = x.size(0), in_f = x.size(1), out_f = W.size(0);
    u = at::empty({N, out_f}, x.options());
    h = at::empty({N, out_f}, x.options());
    check(tgt_linear_act_fwd(x.data_ptr(), W.data_ptr(), b.data_ptr(), N, (int)in_f, (int)out_f, dtype_code(x), TGT_ACT_GELU, u.data_ptr(),
                             h.data_ptr(), stream_of(x)),
          "tgt_linear_act_fwd");
}
// backward of y = h W^T + b with h = gelu(u): du = (dy W) gelu'(u), dW = dy^T h, db
void lin_gelu_bwd(const Tensor& h, const Tensor& W, const Tensor& dy, const Tensor& u, Tensor& du, std::vector<Tensor>& dW,
                  std::vector<Tensor>& db, Deferred& later) {
    const int64_t N = h.size(0), in_f = h.size(1), out_f = W.size(0);
    du = at::empty_like(u);
    dW.assign(1, at::empty_like(W));
    db.assign(1, at::empty({out_f}, h.options()));
    const int64_t ws_bytes = tgt_linear_bwd_workspace_bytes(1, (int)in_f, (int)out_f);
    Tensor ws = at::empty({ws_bytes}, h.options().dtype(at::kByte));
    tgt_reduce_desc sum;
    check(tgt_linear_act_bwd(h.data_ptr(), W.data_ptr(), dy.data_ptr(), u.data_ptr(), N, (int)in_f, (int)out_f, dtype_code(h), TGT_ACT_GELU,
                             du.data_ptr(), dW[0].data_ptr(), db[0].data_ptr(), ws.data_ptr(), ws_bytes, stream_of(h), &sum),
          "tgt_linear_act_bwd");
    later.sums.push_back(sum);
    later.workspaces.push_back(ws);
}
}  // namespace layer

// FeedForwardNetwork.forward (models/graphormer_dist_node_level.py:35-39): layer2(gelu(layer1(x))) as one operator and
// one autograd node: the activation rides on the linears and the two sums of weight-gradient partials share a launch.
struct FfnFn : public torch::autograd::Function<FfnFn> {
    static Tensor forward(AutogradContext* ctx, Tensor x, Tensor W1, Tensor b1, Tensor W2, Tensor b2) {
        on_gpu(x, "ffn");
        const int64_t C = x.size(-1);
        for (const Tensor* t : {&W1, &b1, &W2, &b2})
            TORCH_CHECK(t->defined() && t->is_cuda() && t->scalar_type() == x.scalar_type(), "ffn: parameters must be GPU tensors of x's dtype");
        TORCH_CHECK(W1.dim() == 2 && W1.size(1) == C && W2.dim() == 2 && W2.size(1) == W1.size(0) && b1.numel() == W1.size(0) &&
                    b2.numel() == W2.size(0), "ffn: weight shapes do not chain");
        c10::DeviceGuard guard(x.device());
        Tensor x2 = x.reshape({-1, C}).contiguous(), w1 = W1.contiguous(), w2 = W2.contiguous(), c1 = b1.contiguous(), c2 = b2.contiguous();
        Tensor u, h;
        std::vector<Tensor> f;
        layer::lin_gelu_fwd(x2, w1, c1, u, h);
        layer::lin_fwd(h, {&w2}, {&c2}, f);
        ctx->save_for_backward({x2, u, h, w1, w2});
        std::vector<int64_t> shape = x.sizes().vec();
        shape.back() = w2.size(0);
        return f[0].view(shape);
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        auto sv = ctx->get_saved_variables();
        const Tensor &x2 = sv[0], &u = sv[1], &h = sv[2], &w1 = sv[3], &w2 = sv[4];
        c10::DeviceGuard guard(x2.device());
        Tensor d_f = grads[0].reshape({x2.size(0), w2.size(0)}).contiguous();
        Tensor du, dx;
        std::vector<Tensor> dW2, db2, dW1, db1;
        layer::Deferred later;
        layer::lin_gelu_bwd(h, w2, d_f, u, du, dW2, db2, later);
        layer::lin_bwd(x2, {&w1}, {&du}, dx, dW1, db1, later);
        later.run(dtype_code(x2), stream_of(x2));
        std::vector<int64_t> shape = grads[0].sizes().vec();
        shape.back() = x2.size(1);
        return {dx.view(shape), dW1[0], db1[0], dW2[0], db2[0]};
    }
};
Tensor ffn(const Tensor& x, const Tensor& W1, const Tensor& b1, const Tensor& W2, const Tensor& b2) { return FfnFn::apply(x, W1, b1, W2, b2); }

// MultiHeadAttention.forward with sparse attention and no bias (models/graphormer_dist_node_level.py:246-273; the GT
// flavour of gt_dist_node_level.py:186-216 has no output layer) as one operator and one autograd node:
// q, k, v = x W^T + b from one kernel, the attention, the output layer; the backward ends with one launch for both
// sums of weight-gradient partials.  P: Wq, bq, Wk, bk, Wv, bv (, Wo, bo).
struct MhaFn : public torch::autograd::Function<MhaFn> {
    static Tensor forward(AutogradContext* ctx, Tensor x, at::TensorList P, c10::intrusive_ptr<PlanHolder> holder, Tensor ws, int64_t H) {
        on_gpu(x, "multi_head_attention");
        TORCH_CHECK(P.size() == 6 || P.size() == 8, "multi_head_attention takes 6 parameter tensors, or 8 with an output layer");
        for (const Tensor& t : P) TORCH_CHECK(t.defined() && t.is_cuda() && t.scalar_type() == x.scalar_type(), "parameters must be GPU tensors of x's dtype");
        const int64_t C = x.size(-1), HD = P[0].size(0);
        TORCH_CHECK(HD % H == 0, "projection width ", HD, " is not a multiple of ", H, " heads");
        std::vector<Tensor> p;
        for (const Tensor& t : P) p.push_back(t.contiguous());
        c10::DeviceGuard guard(x.device());
        Tensor x2 = x.reshape({-1, C}).contiguous();
        const int64_t N = x2.size(0), d = HD / H;
        rows_match_plan(holder, N, "multi_head_attention");
        std::vector<Tensor> qkv, y;
        layer::lin_fwd(x2, {&p[0], &p[2], &p[4]}, {&p[1], &p[3], &p[5]}, qkv);
        Tensor o = at::empty_like(qkv[0]), Z = at::empty({N, H}, x.options().dtype(at::kFloat));
        check(tgt_sparse_attn_fwd(reinterpret_cast<const tgt_plan_t*>(holder->h), qkv[0].data_ptr(), qkv[1].data_ptr(), qkv[2].data_ptr(), nullptr,
                                  TGT_BIAS_NONE, (int)H, (int)d, dtype_code(x), o.data_ptr(), Z.data_ptr<float>(), ws.data_ptr(), ws.numel(),
                                  stream_of(x)),
              "tgt_sparse_attn_fwd");
        const bool has_o = p.size() == 8;
        if (has_o) layer::lin_fwd(o, {&p[6]}, {&p[7]}, y);
        std::vector<Tensor> save{x2, qkv[0], qkv[1], qkv[2], o, Z, ws};
        save.insert(save.end(), p.begin(), p.end());
        ctx->save_for_backward(save);
        ctx->saved_data["plan"] = holder;
        ctx->saved_data["H"] = H;
        std::vector<int64_t> shape = x.sizes().vec();
        shape.back() = has_o ? p[6].size(0) : HD;
        return (has_o ? y[0] : o).view(shape);
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        auto sv = ctx->get_saved_variables();
        const Tensor &x2 = sv[0], &q = sv[1], &k = sv[2], &v = sv[3], &o = sv[4], &Z = sv[5], &ws = sv[6];
        const Tensor* p = &sv[7];
        const bool has_o = sv.size() == 7 + 8;
        const int64_t N = x2.size(0), H = ctx->saved_data["H"].toInt(), d = q.size(1) / H;
        c10::DeviceGuard guard(x2.device());
        const int code = dtype_code(x2);
        Tensor dy = grads[0].reshape({N, -1}).contiguous(), do_, dx;
        std::vector<Tensor> dWo, dbo, dWqkv, dbqkv;
        layer::Deferred later;
        if (has_o) layer::lin_bwd(o, {&p[6]}, {&dy}, do_, dWo, dbo, later);
        else do_ = dy;
        Tensor dq = at::empty_like(q), dk = at::empty_like(k), dv = at::empty_like(v);
        check(tgt_sparse_attn_bwd(reinterpret_cast<const tgt_plan_t*>(ctx->saved_data["plan"].toCustomClass<PlanHolder>()->h), q.data_ptr(),
                                  k.data_ptr(), v.data_ptr(), nullptr, TGT_BIAS_NONE, (int)H, (int)d, code, o.data_ptr(), Z.data_ptr<float>(),
                                  do_.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), nullptr, ws.data_ptr(), ws.numel(), stream_of(q)),
              "tgt_sparse_attn_bwd");
        layer::lin_bwd(x2, {&p[0], &p[2], &p[4]}, {&dq, &dk, &dv}, dx, dWqkv, dbqkv, later);
        later.run(code, stream_of(x2));
        std::vector<int64_t> shape = grads[0].sizes().vec();
        shape.back() = x2.size(1);
        variable_list out{dx.view(shape), dWqkv[0], dbqkv[0], dWqkv[1], dbqkv[1], dWqkv[2], dbqkv[2]};
        if (has_o) { out.push_back(dWo[0]); out.push_back(dbo[0]); }
        for (int i = 0; i < 3; ++i) out.push_back(Tensor());
        return out;
    }
};
Tensor multi_head_attention(const Tensor& x, at::TensorList params, const c10::intrusive_ptr<PlanHolder>& plan, const Tensor& ws, int64_t H) {
    return MhaFn::apply(x, params, plan, ws, H);
}

struct EncoderLayerFn : public torch::autograd::Function<EncoderLayerFn> {
    static variable_list forward(AutogradContext* ctx, Tensor x, c10::optional<Tensor> residual, at::TensorList P,
                                 c10::intrusive_ptr<PlanHolder> holder, Tensor ws, int64_t H, double eps1, double eps2) {
        on_gpu(x, "encoder_layer");
        TORCH_CHECK(P.size() == 16, "encoder_layer takes 16 parameter tensors");
        const int64_t C = x.size(-1);
        TORCH_CHECK(C % H == 0, "hidden size ", C, " is not a multiple of ", H, " heads");
        for (const Tensor& p : P) TORCH_CHECK(p.defined() && p.is_cuda() && p.scalar_type() == x.scalar_type(), "parameters must be GPU tensors of x's dtype");
        std::vector<Tensor> p;
        for (const Tensor& t : P) p.push_back(t.contiguous());
        c10::DeviceGuard guard(x.device());
        Tensor x2 = x.reshape({-1, C}).contiguous(), r2;
        if (residual.has_value() && residual->defined()) r2 = residual->reshape({-1, C}).contiguous();
        const int64_t N = x2.size(0), d = C / H;
        rows_match_plan(holder, N, "encoder_layer");
        Tensor s1, y1, mean1, rstd1, s2, y2, mean2, rstd2;
        std::vector<Tensor> qkv, a, u, f;
        layer::ln_fwd(x2, r2, p[0], p[1], eps1, s1, y1, mean1, rstd1);
        layer::lin_fwd(y1, {&p[2], &p[4], &p[6]}, {&p[3], &p[5], &p[7]}, qkv);
        Tensor o = at::empty_like(qkv[0]), Z = at::empty({N, H}, x.options().dtype(at::kFloat));
        check(tgt_sparse_attn_fwd(reinterpret_cast<const tgt_plan_t*>(holder->h), qkv[0].data_ptr(), qkv[1].data_ptr(), qkv[2].data_ptr(), nullptr,
                                  TGT_BIAS_NONE, (int)H, (int)d, dtype_code(x), o.data_ptr(), Z.data_ptr<float>(), ws.data_ptr(), ws.numel(),
                                  stream_of(x)),
              "tgt_sparse_attn_fwd");
        layer::lin_fwd(o, {&p[8]}, {&p[9]}, a);
        layer::ln_fwd(s1, a[0], p[10], p[11], eps2, s2, y2, mean2, rstd2);
        Tensor h;
        u.resize(1);
        layer::lin_gelu_fwd(y2, p[12], p[13], u[0], h);
        layer::lin_fwd(h, {&p[14]}, {&p[15]}, f);
        std::vector<Tensor> save{s1, mean1, rstd1, y1, qkv[0], qkv[1], qkv[2], o, Z, s2, mean2, rstd2, y2, u[0], h, ws};
        save.insert(save.end(), p.begin(), p.end());
        ctx->save_for_backward(save);
        ctx->saved_data["plan"] = holder;
        ctx->saved_data["H"] = H;
        ctx->saved_data["has_r"] = r2.defined();
        ctx->saved_data["shape"] = x.sizes().vec();
        ctx->set_materialize_grads(false);
        return {s2.view(x.sizes()), f[0].view(x.sizes())};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        auto sv = ctx->get_saved_variables();
        const Tensor &s1 = sv[0], &mean1 = sv[1], &rstd1 = sv[2], &y1 = sv[3], &q = sv[4], &k = sv[5], &v = sv[6], &o = sv[7], &Z = sv[8],
                     &s2 = sv[9], &mean2 = sv[10], &rstd2 = sv[11], &y2 = sv[12], &u = sv[13], &h = sv[14], &ws = sv[15];
        const Tensor* p = &sv[16];
        const int64_t N = s1.size(0), C = s1.size(1), H = ctx->saved_data["H"].toInt(), d = C / H;
        c10::DeviceGuard guard(s1.device());
        Tensor d_s2, d_f;
        if (grads[0].defined()) d_s2 = grads[0].reshape({N, C}).contiguous();
        d_f = grads[1].defined() ? grads[1].reshape({N, C}).contiguous() : at::zeros_like(s1);
        const int code = dtype_code(s1);
        Tensor du, dy2, ds2, do_, dy1, dx;
        std::vector<Tensor> dW2, db2, dW1, db1, dWo, dbo, dWqkv, dbqkv;
        layer::Deferred later;
        layer::lin_gelu_bwd(h, p[14], d_f, u, du, dW2, db2, later);
        layer::lin_bwd(y2, {&p[12]}, {&du}, dy2, dW1, db1, later);
        Tensor dg2, dbn2, dg1, dbn1;
        layer::ln_bwd(s2, p[10], mean2, rstd2, dy2, d_s2, ds2, dg2, dbn2, later);           // gradient of s2 = s1 + a: to both
        layer::lin_bwd(o, {&p[8]}, {&ds2}, do_, dWo, dbo, later);
        Tensor dq = at::empty_like(q), dk = at::empty_like(k), dv = at::empty_like(v);
        check(tgt_sparse_attn_bwd(reinterpret_cast<const tgt_plan_t*>(ctx->saved_data["plan"].toCustomClass<PlanHolder>()->h), q.data_ptr(),
                                  k.data_ptr(), v.data_ptr(), nullptr, TGT_BIAS_NONE, (int)H, (int)d, code, o.data_ptr(), Z.data_ptr<float>(),
                                  do_.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), nullptr, ws.data_ptr(), ws.numel(), stream_of(q)),
              "tgt_sparse_attn_bwd");
        layer::lin_bwd(y1, {&p[2], &p[4], &p[6]}, {&dq, &dk, &dv}, dy1, dWqkv, dbqkv, later);
        layer::ln_bwd(s1, p[0], mean1, rstd1, dy1, ds2, dx, dg1, dbn1, later);              // gradient of s1 = x (+ residual)
        later.run(dtype_code(s1), stream_of(s1));        // the six weight-gradient sums of the layer in one launch
        Tensor dxv = dx.view(ctx->saved_data["shape"].toIntVector());
        variable_list out{dxv, ctx->saved_data["has_r"].toBool() ? dxv : Tensor(),
                          dg1, dbn1, dWqkv[0], dbqkv[0], dWqkv[1], dbqkv[1], dWqkv[2], dbqkv[2], dWo[0], dbo[0], dg2, dbn2, dW1[0], db1[0],
                          dW2[0], db2[0]};
        for (int i = 0; i < 5; ++i) out.push_back(Tensor());
        return out;
    }
};
std::tuple<Tensor, Tensor> encoder_layer(const Tensor& x, const c10::optional<Tensor>& residual, at::TensorList params,
                                         const c10::intrusive_ptr<PlanHolder>& plan, const Tensor& ws, int64_t H, double eps1, double eps2) {
    auto r = EncoderLayerFn::apply(x, residual, params, plan, ws, H, eps1, eps2);
    return {r[0], r[1]};
}

// The same layer around the dense attention of the graph-level models (models/graphormer_graph_level.py:267-306).
// x: [b, S, C].  extra: nothing, [bias [b, H, S, S]] (kind 1: its gradient is returned when it needs one), or
// [spatial_table, edge_table, virtual_dist] (kind 2: the bias is formed in the kernels from ab / sp16 / et16, the
// table gradients are returned).  Attention dropout runs inside the kernels from (p_drop, seed).
struct DenseEncoderLayerFn : public torch::autograd::Function<DenseEncoderLayerFn> {
    static variable_list forward(AutogradContext* ctx, Tensor x, c10::optional<Tensor> residual, at::TensorList P, at::TensorList extra,
                                 c10::optional<Tensor> ab_o, c10::optional<Tensor> sp16_o, c10::optional<Tensor> et16_o, int64_t H,
                                 double eps1, double eps2, double p_drop, int64_t seed, bool bf16_products) {
        on_gpu(x, "dense_encoder_layer");
        TORCH_CHECK(x.dim() == 3, "x must be [b, S, C]");
        TORCH_CHECK(P.size() == 16, "dense_encoder_layer takes 16 parameter tensors");
        TORCH_CHECK(extra.size() == 0 || extra.size() == 1 || extra.size() == 3, "extra: nothing, a bias tensor, or the three tables");
        const int kind = extra.size() == 3 ? 2 : (int)extra.size();
        const int64_t b = x.size(0), S = x.size(1), C = x.size(2);
        TORCH_CHECK(C % H == 0, "hidden size ", C, " is not a multiple of ", H, " heads");
        const int64_t d = C / H;
        for (const Tensor& t : P) TORCH_CHECK(t.defined() && t.is_cuda() && t.scalar_type() == x.scalar_type(), "parameters must be GPU tensors of x's dtype");
        for (const Tensor& t : extra) TORCH_CHECK(t.defined() && t.is_cuda() && t.scalar_type() == x.scalar_type(), "bias / tables must be GPU tensors of x's dtype");
        int code = dtype_code(x);
        if (code == TGT_DTYPE_F32 && bf16_products) code = TGT_DTYPE_F32_BF16_PRODUCTS;
        TORCH_CHECK(kind != 2 || code != TGT_DTYPE_F32, "the bias from ids needs bf16 tensors or bf16_products");
        std::vector<Tensor> p, ex;
        for (const Tensor& t : P) p.push_back(t.contiguous());
        for (const Tensor& t : extra) ex.push_back(t.contiguous());
        Tensor ab, sp16, et16;
        if (kind == 1) {
            TORCH_CHECK(ex[0].dim() == 4 && ex[0].size(0) == b && ex[0].size(1) == H && ex[0].size(2) == S && ex[0].size(3) == S,
                        "attn_bias must be [b, H, S, S]");
        } else if (kind == 2) {
            TORCH_CHECK(sp16_o.has_value() && et16_o.has_value(), "the id form needs sp16 and et16");
            sp16 = *sp16_o; et16 = *et16_o;
            TORCH_CHECK(sp16.scalar_type() == at::kShort && sp16.is_contiguous() && sp16.dim() == 3 && sp16.size(0) == b && sp16.size(1) == S &&
                            sp16.size(2) == S, "sp16 must be a contiguous int16 [b, S, S]");
            TORCH_CHECK(et16.scalar_type() == at::kShort && et16.is_contiguous() && et16.dim() == 4 && et16.size(0) == b && et16.size(1) == S &&
                            et16.size(2) == S, "et16 must be a contiguous int16 [b, S, S, F]");
            TORCH_CHECK(ex[0].dim() == 2 && ex[1].dim() == 2 && ex[0].size(1) == H && ex[1].size(1) == H && ex[2].numel() == H,
                        "tables must be [rows, H] / [H]");
            if (ab_o.has_value() && ab_o->defined()) {
                TORCH_CHECK(ab_o->scalar_type() == x.scalar_type() && ab_o->dim() == 3 && ab_o->size(0) == b && ab_o->size(1) == S &&
                                ab_o->size(2) == S, "attn_bias must be [b, S, S] of x's dtype");
                ab = ab_o->contiguous();
            }
        }
        c10::DeviceGuard guard(x.device());
        Tensor x2 = x.reshape({-1, C}).contiguous(), r2;
        if (residual.has_value() && residual->defined()) r2 = residual->reshape({-1, C}).contiguous();
        Tensor s1, y1, mean1, rstd1, s2, y2, mean2, rstd2;
        std::vector<Tensor> qkv, a, u, f;
        layer::ln_fwd(x2, r2, p[0], p[1], eps1, s1, y1, mean1, rstd1);
        layer::lin_fwd(y1, {&p[2], &p[4], &p[6]}, {&p[3], &p[5], &p[7]}, qkv);
        Tensor o = at::empty_like(qkv[0]), lse = at::empty({b, H, S}, x.options().dtype(at::kFloat));
        if (kind == 2) {
            Tensor vd = ex[2].reshape({-1});
            check(tgt_dense_attn_ids_fwd(qkv[0].data_ptr(), qkv[1].data_ptr(), qkv[2].data_ptr(), ab.defined() ? ab.data_ptr() : nullptr,
                                         reinterpret_cast<const uint16_t*>(sp16.data_ptr()), reinterpret_cast<const uint16_t*>(et16.data_ptr()),
                                         (int)et16.size(3), ex[0].data_ptr(), (int)ex[0].size(0), ex[1].data_ptr(), (int)ex[1].size(0),
                                         vd.data_ptr(), (int)b, (int)S, (int)H, (int)d, code, (float)p_drop, (uint64_t)seed, o.data_ptr(),
                                         lse.data_ptr<float>(), stream_of(x)),
                  "tgt_dense_attn_ids_fwd");
        } else {
            check(tgt_dense_attn_dropout_fwd(qkv[0].data_ptr(), qkv[1].data_ptr(), qkv[2].data_ptr(), kind == 1 ? ex[0].data_ptr() : nullptr, (int)b,
                                             (int)S, (int)H, (int)d, code, (float)p_drop, (uint64_t)seed, o.data_ptr(), lse.data_ptr<float>(),
                                             stream_of(x)),
                  "tgt_dense_attn_dropout_fwd");
        }
        layer::lin_fwd(o, {&p[8]}, {&p[9]}, a);
        layer::ln_fwd(s1, a[0], p[10], p[11], eps2, s2, y2, mean2, rstd2);
        Tensor h;
        u.resize(1);
        layer::lin_gelu_fwd(y2, p[12], p[13], u[0], h);
        layer::lin_fwd(h, {&p[14]}, {&p[15]}, f);
        std::vector<Tensor> save{s1, mean1, rstd1, y1, qkv[0], qkv[1], qkv[2], o, lse, s2, mean2, rstd2, y2, u[0], h, ab, sp16, et16};
        save.insert(save.end(), p.begin(), p.end());
        save.insert(save.end(), ex.begin(), ex.end());
        ctx->save_for_backward(save);
        ctx->saved_data["kind"] = (int64_t)kind;
        ctx->saved_data["H"] = H;
        ctx->saved_data["code"] = (int64_t)code;
        ctx->saved_data["p"] = p_drop;
        ctx->saved_data["seed"] = seed;
        ctx->saved_data["has_r"] = r2.defined();
        ctx->saved_data["bias_grad"] = kind == 1 && extra[0].requires_grad();
        ctx->saved_data["vd_shape"] = kind == 2 ? extra[2].sizes().vec() : std::vector<int64_t>{};
        ctx->set_materialize_grads(false);
        return {s2.view(x.sizes()), f[0].view(x.sizes())};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        auto sv = ctx->get_saved_variables();
        const Tensor &s1 = sv[0], &mean1 = sv[1], &rstd1 = sv[2], &y1 = sv[3], &q = sv[4], &k = sv[5], &v = sv[6], &o = sv[7], &lse = sv[8],
                     &s2 = sv[9], &mean2 = sv[10], &rstd2 = sv[11], &y2 = sv[12], &u = sv[13], &h = sv[14], &ab = sv[15], &sp16 = sv[16],
                     &et16 = sv[17];
        const Tensor* p = sv.data() + 18;
        const Tensor* ex = sv.data() + 34;
        const int kind = (int)ctx->saved_data["kind"].toInt(), code = (int)ctx->saved_data["code"].toInt();
        const int64_t H = ctx->saved_data["H"].toInt(), b = lse.size(0), S = lse.size(2), N = s1.size(0), C = s1.size(1), d = C / H;
        const float p_drop = (float)ctx->saved_data["p"].toDouble();
        const uint64_t seed = (uint64_t)ctx->saved_data["seed"].toInt();
        c10::DeviceGuard guard(s1.device());
        Tensor d_s2, d_f;
        if (grads[0].defined()) d_s2 = grads[0].reshape({N, C}).contiguous();
        d_f = grads[1].defined() ? grads[1].reshape({N, C}).contiguous() : at::zeros_like(s1);
        Tensor du, dy2, ds2, do_, dy1, dx, dg2, dbn2, dg1, dbn1;
        std::vector<Tensor> dW2, db2, dW1, db1, dWo, dbo, dWqkv, dbqkv;
        layer::Deferred later;
        layer::lin_gelu_bwd(h, p[14], d_f, u, du, dW2, db2, later);
        layer::lin_bwd(y2, {&p[12]}, {&du}, dy2, dW1, db1, later);
        layer::ln_bwd(s2, p[10], mean2, rstd2, dy2, d_s2, ds2, dg2, dbn2, later);
        layer::lin_bwd(o, {&p[8]}, {&ds2}, do_, dWo, dbo, later);
        Tensor dq = at::empty_like(q), dk = at::empty_like(k), dv = at::empty_like(v);
        variable_list dextra;
        if (kind == 2) {
            Tensor dst = at::empty_like(ex[0]), det = at::empty_like(ex[1]), vd = ex[2].reshape({-1}), dvd = at::empty_like(vd);
            const int64_t ws_bytes = tgt_dense_attn_ids_bwd_workspace_bytes((int)b, (int)H, (int)ex[0].size(0), (int)ex[1].size(0));
            Tensor ws = at::empty({ws_bytes}, s1.options().dtype(at::kByte));
            check(tgt_dense_attn_ids_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), ab.defined() ? ab.data_ptr() : nullptr,
                                         reinterpret_cast<const uint16_t*>(sp16.data_ptr()), reinterpret_cast<const uint16_t*>(et16.data_ptr()),
                                         (int)et16.size(3), ex[0].data_ptr(), (int)ex[0].size(0), ex[1].data_ptr(), (int)ex[1].size(0),
                                         vd.data_ptr(), (int)b, (int)S, (int)H, (int)d, code, p_drop, seed, o.data_ptr(), lse.data_ptr<float>(),
                                         do_.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dst.data_ptr(), det.data_ptr(),
                                         dvd.data_ptr(), ws.data_ptr(), ws_bytes, stream_of(q)),
                  "tgt_dense_attn_ids_bwd");
            dextra = {dst, det, dvd.view(ctx->saved_data["vd_shape"].toIntVector())};
        } else {
            Tensor dbias;
            if (kind == 1 && ctx->saved_data["bias_grad"].toBool()) dbias = at::empty_like(ex[0]);
            check(tgt_dense_attn_dropout_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), kind == 1 ? ex[0].data_ptr() : nullptr, (int)b, (int)S,
                                             (int)H, (int)d, code, p_drop, seed, o.data_ptr(), lse.data_ptr<float>(), do_.data_ptr(),
                                             dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dbias.defined() ? dbias.data_ptr() : nullptr,
                                             stream_of(q)),
                  "tgt_dense_attn_dropout_bwd");
            if (kind == 1) dextra = {dbias};
        }
        layer::lin_bwd(y1, {&p[2], &p[4], &p[6]}, {&dq, &dk, &dv}, dy1, dWqkv, dbqkv, later);
        layer::ln_bwd(s1, p[0], mean1, rstd1, dy1, ds2, dx, dg1, dbn1, later);
        later.run(dtype_code(s1), stream_of(s1));        // the six weight-gradient sums of the layer in one launch
        Tensor dxv = dx.view({b, S, C});
        variable_list out{dxv, ctx->saved_data["has_r"].toBool() ? dxv : Tensor(),
                          dg1, dbn1, dWqkv[0], dbqkv[0], dWqkv[1], dbqkv[1], dWqkv[2], dbqkv[2], dWo[0], dbo[0], dg2, dbn2, dW1[0], db1[0],
                          dW2[0], db2[0]};
        out.insert(out.end(), dextra.begin(), dextra.end());
        for (int i = 0; i < 9; ++i) out.push_back(Tensor());      // ab, sp16, et16, H, eps1, eps2, p_drop, seed, bf16_products
        return out;
    }
};
std::tuple<Tensor, Tensor> dense_encoder_layer(const Tensor& x, const c10::optional<Tensor>& residual, at::TensorList params,
                                               at::TensorList extra, const c10::optional<Tensor>& ab, const c10::optional<Tensor>& sp16,
                                               const c10::optional<Tensor>& et16, int64_t H, double eps1, double eps2, double p_drop,
                                               int64_t seed, bool bf16_products) {
    auto r = DenseEncoderLayerFn::apply(x, residual, params, extra, ab, sp16, et16, H, eps1, eps2, p_drop, seed, bf16_products);
    return {r[0], r[1]};
}

}  // namespace

TORCH_LIBRARY(torchgt, m) {
    m.class_<PlanHolder>("PlanHolder").def(torch::init<int64_t>()).def("handle", &PlanHolder::handle);
    m.def("sparse_attention(Tensor q, Tensor k, Tensor v, Tensor? bias, __torch__.torch.classes.torchgt.PlanHolder plan, int bias_mode, "
          "Tensor workspace) -> (Tensor, Tensor)");
    m.def("dense_attention(Tensor q, Tensor k, Tensor v, Tensor? bias, float p_drop, int seed, bool bf16_products) -> Tensor");
    m.def("dense_attention_ids(Tensor q, Tensor k, Tensor v, Tensor? attn_bias, Tensor sp16, Tensor et16, Tensor spatial_table, "
          "Tensor edge_table, Tensor virtual_dist, float p_drop, int seed, bool bf16_products) -> Tensor");
    m.def("dense_ids_pack(Tensor spatial_pos, Tensor edge_type, int num_spatial, int num_edges) -> (Tensor, Tensor)");
    m.def("linear(Tensor x, Tensor[] weights, Tensor?[] biases) -> Tensor[]");
    m.def("add_layer_norm(Tensor x, Tensor? r, Tensor gamma, Tensor beta, float eps) -> (Tensor, Tensor)");
    m.def("encoder_layer(Tensor x, Tensor? residual, Tensor[] params, __torch__.torch.classes.torchgt.PlanHolder plan, Tensor workspace, "
          "int num_heads, float eps1, float eps2) -> (Tensor, Tensor)");
    m.def("dense_encoder_layer(Tensor x, Tensor? residual, Tensor[] params, Tensor[] extra, Tensor? attn_bias, Tensor? sp16, Tensor? et16, "
          "int num_heads, float eps1, float eps2, float p_drop, int seed, bool bf16_products) -> (Tensor, Tensor)");
    m.def("add(Tensor x, Tensor r) -> Tensor");
    m.def("gelu(Tensor u) -> Tensor");
    m.def("relu(Tensor u) -> Tensor");
    m.def("nll_loss(Tensor log_probs, Tensor target, int ignore_index=-100) -> Tensor");
    m.def("ffn(Tensor x, Tensor W1, Tensor b1, Tensor W2, Tensor b2) -> Tensor");
    m.def("multi_head_attention(Tensor x, Tensor[] params, __torch__.torch.classes.torchgt.PlanHolder plan, Tensor workspace, int heads) -> Tensor");
}

// One implementation per op, registered for every backend and for autograd alike: each is an autograd function
// whose forward calls the C ABI directly (no further dispatch).
TORCH_LIBRARY_IMPL(torchgt, CompositeImplicitAutograd, m) {
    m.impl("sparse_attention", sparse_attention);
    m.impl("dense_attention", dense_attention);
    m.impl("dense_attention_ids", dense_attention_ids);
    m.impl("dense_ids_pack", dense_ids_pack);
    m.impl("linear", linear);
    m.impl("add_layer_norm", add_layer_norm);
    m.impl("encoder_layer", encoder_layer);
    m.impl("dense_encoder_layer", dense_encoder_layer);
    m.impl("add", add);
    m.impl("gelu", gelu);
    m.impl("relu", relu);
    m.impl("nll_loss", nll_loss);
    m.impl("ffn", ffn);
    m.impl("multi_head_attention", multi_head_attention);
}
