// C++ autograd node for the most frequent call of the attention library: ONE bf16 KV chunk, one launch - the SDPA call
// sites of the reference (model/model.py:193-198, parallel/parallel_cp.py:224-229).  It is the host side of
// lightron_amd.attention.SingleChunkAttentionFunction moved out of Python: the same two C-ABI calls (ltr_attn_fwd,
// ltr_attn_bwd with LTR_DQ_BF16 | LTR_DKDV_BF16 | LTR_DELTA_FROM_O), but the backward runs on the autograd thread as a C++
// node - no interpreter lock to take, no Python frames - which is where the time of a call at the reference's default shapes
// (micro-batch 4, 12 heads of 64, sequence 128) goes.  No device code here: torch is used for tensors and autograd only,
// the kernels are those of libltr_attn.so.
#include <torch/extension.h>

#include <cmath>

#include "ltr_attn.h"

namespace {

using torch::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

void strides3(const Tensor &t, int64_t *out) {
    out[0] = t.stride(0);
    out[1] = t.stride(1);
    out[2] = t.stride(2);
}

void require_bshd(const Tensor &t, const char *name) {
    TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor (the HIP library has no CPU path)");
    TORCH_CHECK(t.dim() == 4 && (t.numel() == 0 || t.stride(3) == 1), name, " must be [B,S,H,D] with a contiguous last dim");
    TORCH_CHECK(t.scalar_type() == at::kBFloat16, name, " must be bf16");
}

void check_rc(int rc, const char *what) { TORCH_CHECK(rc == 0, what, " failed: ", ltr_strerror(rc), " (", rc, ")"); }

class SingleChunkNode : public torch::autograd::Function<SingleChunkNode> {
   public:
    // rope_opt: fp32 [n_pos, D/2, 2] (cos, sin) table indexed by global position, or nothing (no fused RoPE)
    static variable_list forward(AutogradContext *ctx, const Tensor &q, const Tensor &k, const Tensor &v, int64_t k_pos0, int64_t q_pos0a,
                                 int64_t q_pos0b, int64_t q_split, bool causal, double scale, int64_t stream, const c10::optional<Tensor> &rope_opt) {
        const Tensor rope = rope_opt.has_value() ? *rope_opt : Tensor();
        require_bshd(q, "q");
        const c10::DeviceGuard on_q_device(q.device());   // the library launches on the CURRENT device
        require_bshd(k, "k");
        require_bshd(v, "v");
        const int64_t B = q.size(0), Sq = q.size(1), Hq = q.size(2), D = q.size(3);
        TORCH_CHECK(k.sizes() == v.sizes() && k.size(0) == B && k.size(3) == D && k.device() == q.device() && v.device() == q.device(),
                    "k/v chunk shape or device mismatch");
        Tensor o = torch::empty({B, Sq, Hq, D}, q.options());
        Tensor lse = torch::empty({B, Hq, Sq}, q.options().dtype(at::kFloat));
        Tensor q_rot;
        const bool with_rope = rope.defined();
        if (with_rope) {
            TORCH_CHECK(rope.scalar_type() == at::kFloat && rope.dim() == 3 && rope.size(1) == D / 2 && rope.size(2) == 2 &&
                            rope.is_contiguous() && rope.device() == q.device(),
                        "the RoPE table must be a contiguous fp32 [n_pos, D/2, 2] (cos, sin) tensor on q's device");
            q_rot = torch::empty({B, Sq, Hq, D}, q.options());
        }
        if (Sq > 0) {
            ltr_attn_fwd_args a{};
            a.q = q.data_ptr();
            a.o = o.data_ptr();
            a.lse = lse.data_ptr<float>();
            a.B = (int32_t)B;
            a.Hq = (int32_t)Hq;
            a.Hkv = (int32_t)k.size(2);
            a.D = (int32_t)D;
            a.Sq = Sq;
            strides3(q, a.q_stride);
            strides3(o, a.o_stride);
            strides3(k, a.k_stride);
            strides3(v, a.v_stride);
            a.q_pos0[0] = q_pos0a;
            a.q_pos0[1] = q_pos0b;
            a.q_split = q_split;
            a.scale = (float)scale;
            a.flags = (causal ? LTR_CAUSAL : 0u) | (with_rope ? LTR_ROPE_Q : 0u);
            a.io_dtype = a.o_dtype = LTR_BF16;
            a.n_chunks = 1;
            a.chunk[0].k = k.data_ptr();
            a.chunk[0].v = v.data_ptr();
            a.chunk[0].sk = k.size(1);
            a.chunk[0].pos0 = k_pos0;
            if (with_rope) {
                a.rope_freqs = rope.data_ptr<float>();
                a.rope_pos0 = 0;
                a.rope_len = rope.size(0);
                a.q_rot = q_rot.data_ptr();
                strides3(q_rot, a.q_rot_stride);
            }
            check_rc(ltr_attn_fwd(&a, (void *)stream), "ltr_attn_fwd");
        }
        ctx->save_for_backward({with_rope ? q_rot : q, k, v, o, lse, with_rope ? rope : Tensor()});
        ctx->saved_data["k_pos0"] = k_pos0;
        ctx->saved_data["q_pos0a"] = q_pos0a;
        ctx->saved_data["q_pos0b"] = q_pos0b;
        ctx->saved_data["q_split"] = q_split;
        ctx->saved_data["causal"] = causal;
        ctx->saved_data["scale"] = scale;
        ctx->saved_data["stream"] = stream;   // the engine runs this node's backward on the forward's stream
        ctx->mark_non_differentiable({lse});
        return {o, lse};
    }

    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const Tensor &q = saved[0], &k = saved[1], &v = saved[2], &o = saved[3], &lse = saved[4], &rope = saved[5];
        const c10::DeviceGuard on_q_device(q.device());
        Tensor d_o = grads[0];
        if (d_o.scalar_type() != at::kBFloat16) d_o = d_o.to(at::kBFloat16);
        if (d_o.stride(3) != 1) d_o = d_o.contiguous();
        const int64_t B = q.size(0), Sq = q.size(1), Hq = q.size(2), D = q.size(3);
        Tensor dq = torch::empty({B, Sq, Hq, D}, q.options());
        Tensor dk = torch::empty(k.sizes(), k.options()), dv = torch::empty(k.sizes(), k.options());
        variable_list out(11);
        if (Sq == 0) {
            out[0] = dq;
            out[1] = dk.zero_();
            out[2] = dv.zero_();
            return out;
        }
        Tensor delta = torch::empty({B, Hq, Sq}, lse.options());   // workspace: filled by the dQ kernel from o
        ltr_attn_bwd_args a{};
        a.q = q.data_ptr();
        a.d_o = d_o.data_ptr();
        a.lse = lse.data_ptr<float>();
        a.delta = delta.data_ptr<float>();
        a.dq = dq.data_ptr();
        a.o = o.data_ptr();
        a.B = (int32_t)B;
        a.Hq = (int32_t)Hq;
        a.Hkv = (int32_t)k.size(2);
        a.D = (int32_t)D;
        a.Sq = Sq;
        strides3(q, a.q_stride);
        strides3(d_o, a.do_stride);
        strides3(dq, a.dq_stride);
        strides3(o, a.o_stride);
        strides3(k, a.k_stride);
        strides3(v, a.v_stride);
        strides3(dk, a.dk_stride);
        strides3(dv, a.dv_stride);
        a.q_pos0[0] = ctx->saved_data["q_pos0a"].toInt();
        a.q_pos0[1] = ctx->saved_data["q_pos0b"].toInt();
        a.q_split = ctx->saved_data["q_split"].toInt();
        a.scale = (float)ctx->saved_data["scale"].toDouble();
        // one call holds every key these rows see and every row that sees these keys: the kernels write bf16 results
        a.flags = (ctx->saved_data["causal"].toBool() ? LTR_CAUSAL : 0u) | LTR_DQ_BF16 | LTR_DKDV_BF16 | LTR_DELTA_FROM_O |
                  (rope.defined() ? LTR_ROPE_DQ : 0u);
        a.io_dtype = LTR_BF16;
        a.n_chunks = 1;
        a.chunk[0].k = k.data_ptr();
        a.chunk[0].v = v.data_ptr();
        a.chunk[0].dk = dk.data_ptr();
        a.chunk[0].dv = dv.data_ptr();
        a.chunk[0].sk = k.size(1);
        a.chunk[0].pos0 = ctx->saved_data["k_pos0"].toInt();
        if (rope.defined()) {
            a.rope_freqs = rope.data_ptr<float>();
            a.rope_pos0 = 0;
            a.rope_len = rope.size(0);
        }
        check_rc(ltr_attn_bwd(&a, (void *)ctx->saved_data["stream"].toInt()), "ltr_attn_bwd");
        out[0] = dq;
        out[1] = dk;
        out[2] = dv;
        return out;
    }
};

// (O [B,Sq,Hq,D] bf16, LSE [B,Hq,Sq] fp32); stream = hipStream_t of torch's current stream on q's device, as an integer
std::vector<Tensor> single_chunk(const Tensor &q, const Tensor &k, const Tensor &v, int64_t k_pos0, int64_t q_pos0a, int64_t q_pos0b,
                                 int64_t q_split, bool causal, double scale, int64_t stream, const c10::optional<Tensor> &rope) {
    return SingleChunkNode::apply(q, k, v, k_pos0, q_pos0a, q_pos0b, q_split, causal, scale, stream, rope);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("single_chunk", &single_chunk, "one bf16 KV chunk, forward with a C++ autograd node behind it");
    m.def("abi_version", []() { return ltr_abi_version(); });
}
