// Autograd node of the sparse attention modules, compiled against libtorch (host code only).
//
// It does what _BlockAttnFunction in attention_blockcuda.py does -- the reference's function is
// models/attention_blockcuda.py:20-112 (key-mask variant: models/attention_blockcuda_mask.py) -- with the node, the
// saved tensors and the output allocations on the C++ side of PyTorch: for small problems (the reference's L = 1024
// tasks) a training step is bound by the host, and the Python function spends about three times the kernels' run
// time between autograd's engine, ctypes and tensor bookkeeping.  The arithmetic is the library's: the row-major
// and strided entry points declared in include/spion_hip.h.  The Python function stays the statement of the
// behaviour; tests run both and compare.
#include <torch/extension.h>

#include <stdexcept>
#include <string>

#include "../../include/spion_hip.h"

namespace {

using torch::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

void check_library(const char* where) {
    if (!spion_error_pending()) return;
    std::string text = spion_last_error();
    spion_clear_error();
    throw std::runtime_error(std::string(where) + ": " + text);
}

// Layout of a [B, H, L, d] fp32 view for the strided entry points; false when they cannot take it (last dimension
// not unit-stride, strides not multiples of 16 bytes, storage not 16-byte aligned).
bool head_layout(const Tensor& t, spion_head_layout& lay) {
    if (t.dim() != 4) return false;
    const int64_t sb = t.stride(0), sh = t.stride(1), sl = t.stride(2), sf = t.stride(3);
    if (sf != 1 || reinterpret_cast<uintptr_t>(t.data_ptr()) % 16) return false;
    if (sb % 4 || sh % 4 || sl % 4 || sl < t.size(3) || sb < 0 || sh < 0) return false;
    if (t.size(2) * sl >= (int64_t(1) << 29)) return false;
    lay.batch_stride = sb;
    lay.head_stride = (int)sh;
    lay.row_stride = (int)sl;
    return true;
}

Tensor empty_heads(c10::IntArrayRef shape, bool interleaved, const torch::TensorOptions& opt) {
    if (!interleaved) return torch::empty(shape, opt);
    return torch::empty({shape[0], shape[2], shape[1], shape[3]}, opt).transpose(1, 2);  // memory [B, L, H, d]
}

bool same_strides(const Tensor& a, const Tensor& b) { return a.strides() == b.strides(); }

// q, k, v are the three slices of one [B, L, 3, H, d] buffer, in this order
bool adjacent_head_views(const Tensor& q, const Tensor& k, const Tensor& v) {
    const int64_t H = q.size(1), L = q.size(2), d = q.size(3);
    const int64_t want[4] = {L * 3 * H * d, d, 3 * H * d, 1};
    for (const Tensor* t : {&q, &k, &v})
        for (int i = 0; i < 4; ++i)
            if (t->stride(i) != want[i]) return false;
    const char *pq = (const char*)q.data_ptr(), *pk = (const char*)k.data_ptr(), *pv = (const char*)v.data_ptr();
    const int64_t step = H * d * 4;
    return pk - pq == step && pv - pk == step;
}

const float* fp(const Tensor& t) { return t.defined() ? static_cast<const float*>(t.data_ptr()) : nullptr; }
float* fpm(Tensor& t) { return static_cast<float*>(t.data_ptr()); }
const int* ip(const Tensor& t) { return static_cast<const int*>(t.data_ptr()); }

struct SparseAttnNode : public torch::autograd::Function<SparseAttnNode> {
    // pen_opt: [B, H*L] key penalties of the key-mask modules, or nothing.  stream: torch's current raw
    // stream at the call; autograd runs the backward of a node on the stream its forward ran on.
    static variable_list forward(AutogradContext* ctx, Tensor query, Tensor key, Tensor value,
                                 c10::optional<Tensor> pen_opt, Tensor offsets, Tensor columns, Tensor sum_mat, int64_t handle, int64_t nnz,
                                 int64_t num_heads, bool reads_views, int64_t stream) {
        void* h = reinterpret_cast<void*>(handle);
        const Tensor pen = pen_opt.has_value() ? *pen_opt : Tensor();
        spion_set_stream(h, reinterpret_cast<void*>(stream));
        TORCH_CHECK(query.dim() == 4 && key.sizes() == query.sizes() && value.sizes() == query.sizes(),
                    "query, key and value must be [B, H, L, d] tensors of one shape");
        TORCH_CHECK(query.scalar_type() == torch::kFloat32 && query.is_cuda(), "fp32 tensors on the GPU expected");
        const int64_t B = query.size(0), H = query.size(1);
        const auto opt = query.options();
        Tensor p_flat = torch::empty({B * H * nnz}, opt);
        spion_head_layout lin{}, lout{}, lk{}, lv{};
        bool strided = reads_views && !(query.is_contiguous() && key.is_contiguous() && value.is_contiguous()) &&
                       head_layout(query, lin) && head_layout(key, lk) && head_layout(value, lv) &&
                       same_strides(key, query) && same_strides(value, query);
        Tensor q, k, v, out;
        if (strided) {
            q = query;
            k = key;
            v = value;
            out = empty_heads(query.sizes(), query.stride(1) < query.stride(2), opt);
            head_layout(out, lout);
            spion_attn_forward_strided(h, fp(q), fp(k), fp(v), fp(pen), fpm(p_flat), fpm(out), ip(offsets), ip(columns),
                                       ip(sum_mat), (int)nnz, (int)num_heads, &lin, &lout);
        } else {
            q = query.contiguous();
            k = key.contiguous();
            v = value.contiguous();
            out = torch::empty(query.sizes(), opt);
            spion_attn_forward_rowmajor(h, fp(q), fp(k), fp(v), fp(pen), fpm(p_flat), fpm(out), ip(offsets), ip(columns),
                                        ip(sum_mat), (int)nnz);
        }
        check_library("attn_forward");
        // which kernel family serves THIS pattern (the handle may run other patterns before the backward)
        ctx->saved_data["tiled"] = spion_last_path(h) == 1;
        ctx->saved_data["handle"] = handle;
        ctx->saved_data["nnz"] = nnz;
        ctx->saved_data["heads"] = num_heads;
        ctx->saved_data["strided"] = strided;
        ctx->saved_data["stream"] = stream;
        ctx->save_for_backward({q, k, v, p_flat, offsets, columns, sum_mat, out});
        ctx->set_materialize_grads(false);  // the gradient of the returned probabilities is ignored anyway
        if (pen.defined()) ctx->mark_non_differentiable({p_flat});
        return {out, p_flat};
    }

    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const Tensor &q = saved[0], &k = saved[1], &v = saved[2], &p_flat = saved[3], &offsets = saved[4],
                     &columns = saved[5], &sum_mat = saved[6], &out = saved[7];
        void* h = reinterpret_cast<void*>(ctx->saved_data["handle"].toInt());
        const int64_t nnz = ctx->saved_data["nnz"].toInt();
        const int heads = (int)ctx->saved_data["heads"].toInt();
        spion_set_stream(h, reinterpret_cast<void*>(ctx->saved_data["stream"].toInt()));
        const auto opt = q.options();
        Tensor go = grads[0];
        if (!go.defined()) go = torch::zeros(q.sizes(), opt);  // only the probabilities were used downstream
        Tensor dq, dk, dv;
        if (ctx->saved_data["strided"].toBool()) {
            spion_head_layout lin{}, lout{}, lgrad{}, lgo{};
            if (!same_strides(go, out) || !head_layout(go, lgo)) go = torch::empty_like(out).copy_(go);  // out's strides
            if (adjacent_head_views(q, k, v)) {  // slices of one fused projection: the gradients likewise
                Tensor buf = torch::empty({q.size(0), q.size(2), 3, q.size(1), q.size(3)}, opt);
                dq = buf.select(2, 0).transpose(1, 2);
                dk = buf.select(2, 1).transpose(1, 2);
                dv = buf.select(2, 2).transpose(1, 2);
            } else {
                const bool inter = q.stride(1) < q.stride(2);
                dq = empty_heads(q.sizes(), inter, opt);
                dk = empty_heads(q.sizes(), inter, opt);
                dv = empty_heads(q.sizes(), inter, opt);
            }
            head_layout(q, lin);
            head_layout(out, lout);
            head_layout(dq, lgrad);
            spion_attn_backward_strided(h, fp(q), fp(k), fp(v), fp(p_flat), fp(out), fp(go), fpm(dq), fpm(dk), fpm(dv),
                                        ip(offsets), ip(columns), ip(sum_mat), (int)nnz, heads, &lin, &lout, &lgrad);
        } else {
            go = go.contiguous();
            // of the ABI's two [NB*nnz] scratch arguments (models/attention_blockcuda.py:83-84) the tile kernels use
            // neither and the element kernels only dS
            Tensor scratch;
            if (!ctx->saved_data["tiled"].toBool())
                scratch = torch::empty({std::max<int64_t>(q.size(0) * q.size(1) * nnz, 1)}, opt);
            dq = torch::empty(q.sizes(), opt);
            dk = torch::empty(q.sizes(), opt);
            dv = torch::empty(q.sizes(), opt);
            spion_attn_backward_rowmajor(h, fp(q), fp(k), fp(v), fp(p_flat), fp(out), fp(go),
                                         scratch.defined() ? fpm(scratch) : nullptr, fpm(dq), fpm(dk), fpm(dv),
                                         ip(offsets), ip(columns), ip(sum_mat), (int)nnz);
        }
        check_library("attn_backward");
        return {dq, dk, dv, Tensor(), Tensor(), Tensor(), Tensor(), Tensor(), Tensor(), Tensor(), Tensor(), Tensor()};
    }
};

std::vector<Tensor> sparse_attention(const Tensor& query, const Tensor& key, const Tensor& value,
                                     const c10::optional<Tensor>& pen, const Tensor& offsets, const Tensor& columns,
                                     const Tensor& sum_mat, int64_t handle, int64_t nnz, int64_t num_heads,
                                     bool reads_views, int64_t stream) {
    return SparseAttnNode::apply(query, key, value, pen, offsets, columns, sum_mat, handle, nnz, num_heads, reads_views,
                                 stream);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "C++ autograd node of the sparse attention modules";
    m.def("sparse_attention", &sparse_attention, "forward of the sparse attention modules; returns [out, p_flat]",
          py::arg("query"), py::arg("key"), py::arg("value"), py::arg("pen"), py::arg("offsets"), py::arg("columns"),
          py::arg("sum_mat"), py::arg("handle"), py::arg("nnz"), py::arg("num_heads"), py::arg("reads_views"),
          py::arg("stream"));
}
