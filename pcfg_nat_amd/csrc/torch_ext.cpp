// Host side of the training operators as a torch extension: argument checks, output allocation, the autograd nodes and the
// call into the C-ABI of libpcfg_nat_hip.so, in C++.
//
// Takes the place of the reference's pybind module (fs_plugins/custom_ops/pcfg_loss.cpp:75-82) together with the autograd
// Functions that sit on top of it in Python (fs_plugins/custom_ops/pcfg_loss.py:49-85, 144-181): the same checks, the same
// in-place contract, the same eager backward inside the forward of the loss - only the arithmetic is behind the C-ABI.
// Nothing here touches device memory itself; the kernels are enqueued on torch's current stream of the tensors' device.
//
// Why it exists: a training step through the Python Functions costs the host about 0.25 ms (Function.apply, half a dozen
// torch.empty, ctypes marshalling of twenty arguments, twice), more than the 0.17 ms its kernels run.
#include <torch/extension.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include "../../include/pcfg_nat_hip.h"

namespace {

using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

void check_rc(int rc) { TORCH_CHECK(rc == PCFGNAT_OK, pcfgnat_last_error()); }

int dtype_code(const at::Tensor &t, const char *who) {
    switch (t.scalar_type()) {
        case at::kHalf: return PCFGNAT_F16;
        case at::kFloat: return PCFGNAT_F32;
        case at::kDouble: return PCFGNAT_F64;
        default: TORCH_CHECK(false, who, ": unsupported dtype ", t.scalar_type(), " (float16, float32, float64 are dispatched)");
    }
}

void *stream_of(const at::Tensor &t) { return (void *)c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

void need_gpu(const char *who, std::initializer_list<const at::Tensor *> ts) {
    const at::Tensor *first = nullptr;
    for (const at::Tensor *t : ts) {
        if (t == nullptr || !t->defined()) continue;
        TORCH_CHECK(t->is_cuda(), who, ": expected tensors on the GPU, got a ", t->device().type(), " tensor");
        if (first == nullptr) first = t;
        TORCH_CHECK(t->device() == first->device(), who, ": tensors are on different devices (", first->device(), " vs ", t->device(), ")");
    }
}

at::Tensor lengths(const char *who, const at::Tensor &t, int64_t B) {
    TORCH_CHECK(t.dim() == 1 && t.size(0) == B, who, ": length tensor must have shape [", B, "], got ", t.sizes());
    TORCH_CHECK(t.scalar_type() == at::kLong, who, ": lengths should be long");
    return t.contiguous();
}

struct PcfgDims {
    int64_t B, L, T, ml, Mc;
};
PcfgDims check_pcfg_inputs(const char *who, const at::Tensor &match_all, const at::Tensor &links, const at::Tensor &ol,
                           const at::Tensor &tl) {
    need_gpu(who, {&match_all, &links, &ol, &tl});
    TORCH_CHECK(match_all.dim() == 3, who, ": match_all dim != 3");
    TORCH_CHECK(links.dim() == 4, who, ": links dim != 4");
    const int64_t B = match_all.size(0), L = match_all.size(1), T = match_all.size(2);
    TORCH_CHECK(links.size(0) == B && links.size(1) == L && links.size(3) == L, who,
                ": links must be [bsz, prelen, max_left+1, prelen] = [", B, ", ", L, ", *, ", L, "], got ", links.sizes());
    const int64_t ml = links.size(2) - 1;
    return PcfgDims{B, L, T, ml, (L - 2) / (ml + 1) + 1};
}

// ---------------------------------------------------------------------------------------------------------------
// cuda_pcfg_loss (pcfg_loss.py:49-85), float32 tables
// ---------------------------------------------------------------------------------------------------------------
struct PcfgLossFn : public torch::autograd::Function<PcfgLossFn> {
    static variable_list forward(AutogradContext *ctx, at::Tensor match_all, at::Tensor links, at::Tensor output_length,
                                 at::Tensor target_length) {
        const bool need = match_all.requires_grad() || links.requires_grad();
        const PcfgDims d = check_pcfg_inputs("cuda_pcfg_loss", match_all, links, output_length, target_length);
        TORCH_CHECK(match_all.scalar_type() == at::kFloat && links.scalar_type() == at::kFloat,
                    "cuda_pcfg_loss: this entry takes float32 tables");
        match_all = match_all.contiguous();
        links = links.contiguous();
        const at::Tensor ol = lengths("cuda_pcfg_loss", output_length, d.B), tl = lengths("cuda_pcfg_loss", target_length, d.B);
        const c10::DeviceGuard guard(match_all.device());
        const auto f32 = match_all.options();
        at::Tensor S = at::empty({d.B, d.Mc, d.T + 2}, f32);
        at::Tensor aux = at::empty({(int64_t)std::max<size_t>(1, pcfgnat_pcfg_aux_floats(d.B, d.L, d.T, d.ml))}, f32);
        if (need) {
            // like the reference (pcfg_loss.py:71-73) the backward sweep runs eagerly with a unit upstream gradient
            at::Tensor ones = at::ones({d.B}, f32);
            at::Tensor mg = at::empty_like(match_all), lg = at::empty_like(links);
            check_rc(pcfgnat_pcfg_loss_forward_backward(ones.data_ptr<float>(), match_all.data_ptr<float>(), links.data_ptr<float>(),
                                                        ol.data_ptr<int64_t>(), tl.data_ptr<int64_t>(), S.data_ptr<float>(),
                                                        aux.data_ptr<float>(), mg.data_ptr<float>(), lg.data_ptr<float>(), d.B, d.L, d.T,
                                                        d.ml, stream_of(match_all)));
            ctx->save_for_backward({mg, lg});
        } else {
            check_rc(pcfgnat_pcfg_loss(match_all.data_ptr<float>(), links.data_ptr<float>(), ol.data_ptr<int64_t>(),
                                       tl.data_ptr<int64_t>(), S.data_ptr<float>(), aux.data_ptr<float>(), d.B, d.L, d.T, d.ml,
                                       stream_of(match_all)));
        }
        ctx->saved_data["need"] = need;
        return {S.select(1, 0).select(1, 0).clone()};
    }

    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        if (!ctx->saved_data["need"].toBool() || !grads[0].defined()) return {at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor()};
        const auto saved = ctx->get_saved_variables();
        const int64_t B = saved[0].size(0);
        const at::Tensor g = grads[0];
        return {saved[0] * g.view({B, 1, 1}), saved[1] * g.view({B, 1, 1, 1}), at::Tensor(), at::Tensor()};
    }
};

at::Tensor cuda_pcfg_loss(const at::Tensor &match_all, const at::Tensor &links, const at::Tensor &output_length,
                          const at::Tensor &target_length) {
    return PcfgLossFn::apply(match_all, links, output_length, target_length)[0];
}

// ---------------------------------------------------------------------------------------------------------------
// dag_logsoftmax_gather_inplace (pcfg_loss.py:144-181) in the log-sum-exp split: the forward only reads the logits, the
// backward turns the untouched logits into the gradient in place
// ---------------------------------------------------------------------------------------------------------------
struct GatherDims {
    int64_t B, L, V, T;
    int code;
};
GatherDims check_gather(const at::Tensor &word_ins_out, const at::Tensor &select_idx) {
    need_gpu("logsoftmax_gather", {&word_ins_out, &select_idx});
    TORCH_CHECK(word_ins_out.dim() == 3, "word_ins_out dim != 3");
    TORCH_CHECK(select_idx.dim() == 3, "select_idx dim != 3");
    GatherDims d{word_ins_out.size(0), word_ins_out.size(1), word_ins_out.size(2), select_idx.size(2), 0};
    TORCH_CHECK(select_idx.size(0) == d.B, "batch size not match");
    TORCH_CHECK(select_idx.size(1) == d.L, "prelen size not match");
    TORCH_CHECK(select_idx.scalar_type() == at::kLong, "select_idx should be long");
    TORCH_CHECK(word_ins_out.is_contiguous(), "word_ins_out is not contiguous");
    d.code = dtype_code(word_ins_out, "logsoftmax_gather");
    return d;
}

struct GatherFn : public torch::autograd::Function<GatherFn> {
    static variable_list forward(AutogradContext *ctx, at::Tensor word_ins_out, at::Tensor select_idx) {
        const bool need = word_ins_out.requires_grad();
        const GatherDims d = check_gather(word_ins_out, select_idx);
        const c10::DeviceGuard guard(word_ins_out.device());
        const auto out_opts = word_ins_out.options().dtype(word_ins_out.scalar_type() == at::kDouble ? at::kDouble : at::kFloat);
        at::Tensor selected = at::empty({d.B, d.L, d.T}, out_opts);
        const auto st = select_idx.strides();
        if (need) {
            at::Tensor row_lse = at::empty({d.B, d.L}, out_opts);
            check_rc(pcfgnat_logsoftmax_gather_lse(word_ins_out.data_ptr(), d.code, select_idx.data_ptr<int64_t>(), st[0], st[1], st[2],
                                                   selected.data_ptr(), row_lse.data_ptr(), nullptr, nullptr, d.B, d.L, d.V, d.T,
                                                   stream_of(word_ins_out)));
            ctx->save_for_backward({word_ins_out, select_idx, row_lse});
        } else {
            check_rc(pcfgnat_logsoftmax_gather(word_ins_out.data_ptr(), d.code, select_idx.data_ptr<int64_t>(), st[0], st[1], st[2],
                                               selected.data_ptr(), 0, d.B, d.L, d.V, d.T, stream_of(word_ins_out)));
        }
        // Note: the backward reuses word_ins_out as the gradient buffer
        ctx->mark_dirty({word_ins_out});
        ctx->set_materialize_grads(false);
        ctx->saved_data["need"] = need;
        ctx->saved_data["has_backward"] = false;
        return {word_ins_out, selected};
    }

    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        if (!ctx->saved_data["need"].toBool()) return {at::Tensor(), at::Tensor()};
        TORCH_CHECK(!grads[0].defined(), "Cannot reuse word_ins_out after logsoftmax_gather");
        if (!grads[1].defined()) return {at::Tensor(), at::Tensor()};
        TORCH_CHECK(!ctx->saved_data["has_backward"].toBool(), "Cannot backward twice in logsoftmax_gather");
        ctx->saved_data["has_backward"] = true;
        const auto saved = ctx->get_saved_variables();
        at::Tensor buf = saved[0];
        const at::Tensor &idx = saved[1], &row_lse = saved[2];
        const c10::DeviceGuard guard(buf.device());
        const at::Tensor g = grads[1].to(row_lse.scalar_type()).contiguous();
        const auto st = idx.strides();
        check_rc(pcfgnat_logsoftmax_gather_backward_lse(buf.data_ptr(), dtype_code(buf, "logsoftmax_gather"), idx.data_ptr<int64_t>(),
                                                        st[0], st[1], st[2], g.data_ptr(), row_lse.data_ptr(), buf.size(0), buf.size(1),
                                                        buf.size(2), idx.size(2), stream_of(buf)));
        return {buf, at::Tensor()};
    }
};

std::tuple<at::Tensor, at::Tensor> dag_logsoftmax_gather_inplace(const at::Tensor &word_ins_out, const at::Tensor &select_idx) {
    auto out = GatherFn::apply(word_ins_out, select_idx);
    return std::make_tuple(out[0], out[1]);
}

// ---------------------------------------------------------------------------------------------------------------
// The criterion's loss (nat_pcfg_loss.py:98-145) as one differentiable op: one native call in the forward (gather, both
// sweeps, posteriors at an upstream gradient of 1, loss), one in the backward (the single pass that turns the logits into
// their gradient, with the upstream gradient read from device memory).
// ---------------------------------------------------------------------------------------------------------------
struct CriterionFn : public torch::autograd::Function<CriterionFn> {
    static variable_list forward(AutogradContext *ctx, at::Tensor outputs, at::Tensor links, at::Tensor targets,
                                 at::Tensor output_length, at::Tensor target_length, c10::optional<at::Tensor> matchmask,
                                 c10::optional<at::Tensor> keep_word_mask) {
        const char *who = "pcfg_criterion";
        const bool need = outputs.requires_grad() || links.requires_grad();
        need_gpu(who, {&outputs, &targets, &links, &output_length, &target_length});
        TORCH_CHECK(outputs.dim() == 3 && outputs.is_contiguous(), who, ": logits must be a contiguous [bsz, prelen, vocab] tensor");
        const int64_t B = outputs.size(0), L = outputs.size(1), V = outputs.size(2);
        TORCH_CHECK(targets.dim() == 2 && targets.size(0) == B && targets.scalar_type() == at::kLong, who,
                    ": targets must be an int64 [bsz, tarlen] tensor");
        const int64_t T = targets.size(1);
        const int code = dtype_code(outputs, who);
        TORCH_CHECK(code != PCFGNAT_F64, who, ": logits must be float16 or float32");
        TORCH_CHECK(links.dim() == 4 && links.size(0) == B && links.size(1) == L && links.size(3) == L && links.scalar_type() == at::kFloat,
                    who, ": links must be float32 [bsz, prelen, max_left+1, prelen]");
        const int64_t ml = links.size(2) - 1, Mc = (L - 2) / (ml + 1) + 1;
        targets = targets.contiguous();
        links = links.contiguous();
        const at::Tensor ol = lengths(who, output_length, B), tl = lengths(who, target_length, B);
        TORCH_CHECK(matchmask.has_value() == keep_word_mask.has_value(), who, ": matchmask and keep_word_mask go together");
        at::Tensor mm8, keep8;
        if (matchmask.has_value()) {
            need_gpu(who, {&outputs, &*matchmask, &*keep_word_mask});
            TORCH_CHECK(matchmask->sizes() == at::IntArrayRef({B, T, L}) && keep_word_mask->sizes() == at::IntArrayRef({B, L}), who,
                        ": matchmask must be [bsz, tarlen, prelen] and keep_word_mask [bsz, prelen]");
            mm8 = matchmask->to(at::kByte).contiguous();
            keep8 = keep_word_mask->to(at::kByte).contiguous();
        }
        const c10::DeviceGuard guard(outputs.device());
        const auto f32 = links.options();
        // one allocation for the workspaces the backward does not need, one for what it keeps
        const int64_t n_match = B * L * T, n_S = B * Mc * (T + 2);
        const int64_t n_aux = (int64_t)std::max<size_t>(1, pcfgnat_pcfg_aux_floats(B, L, T, ml));
        at::Tensor work = at::empty({n_match + n_S + n_aux + 4}, f32);
        float *match = work.data_ptr<float>(), *S = match + n_match, *aux = S + n_S;
        aux += ((uintptr_t)aux & 15) ? (16 - ((uintptr_t)aux & 15)) / 4 : 0;  // (the kernels want it 16-byte aligned)
        at::Tensor mg = at::empty({B, L, T}, f32), lg = at::empty_like(links), row_lse = at::empty({B, L}, f32);
        at::Tensor out = at::empty({2 + B}, f32);  // loss, invalid count, ll with the invalid sentences zeroed
        const unsigned char *mm_ptr = mm8.defined() ? mm8.data_ptr<unsigned char>() : nullptr;
        const unsigned char *keep_ptr = keep8.defined() ? keep8.data_ptr<unsigned char>() : nullptr;
        int pad_zeroed = 0;
        if (need) {
            check_rc(pcfgnat_criterion_forward(outputs.data_ptr(), code, targets.data_ptr<int64_t>(), links.data_ptr<float>(),
                                               ol.data_ptr<int64_t>(), tl.data_ptr<int64_t>(), mm_ptr, keep_ptr, match, S, aux,
                                               mg.data_ptr<float>(), lg.data_ptr<float>(), row_lse.data_ptr<float>(),
                                               out.data_ptr<float>(), out.data_ptr<float>() + 2, &pad_zeroed, B, L, V, T, ml,
                                               stream_of(outputs)));
            ctx->save_for_backward({outputs, targets, mg, lg, row_lse, ol, keep8.defined() ? keep8 : at::Tensor()});
            ctx->saved_data["pad_zeroed"] = (int64_t)pad_zeroed;
            ctx->saved_data["ml"] = ml;
        } else {  // nothing to differentiate: the plain step (its gradients are discarded)
            check_rc(pcfgnat_criterion_step(outputs.data_ptr(), code, targets.data_ptr<int64_t>(), links.data_ptr<float>(),
                                            ol.data_ptr<int64_t>(), tl.data_ptr<int64_t>(), mm_ptr, keep_ptr, match, S, aux,
                                            mg.data_ptr<float>(), lg.data_ptr<float>(), row_lse.data_ptr<float>(), out.data_ptr<float>(), B,
                                            L, V, T, ml, 1.0f, nullptr, stream_of(outputs), nullptr));
        }
        ctx->saved_data["need"] = need;
        ctx->saved_data["has_backward"] = false;
        ctx->mark_dirty({outputs});
        ctx->set_materialize_grads(false);
        // ll with the invalid sentences (non-finite log-likelihood) zeroed, as nat_pcfg_loss.py:123-133 leaves it
        at::Tensor ll = need ? out.narrow(0, 2, B)
                             : at::nan_to_num(work.narrow(0, n_match, n_S).view({B, Mc * (T + 2)}).select(1, 0), 0.0, 0.0, 0.0);
        at::Tensor invalid = out.select(0, 1);
        ctx->mark_non_differentiable({invalid});
        return {outputs, out.select(0, 0), ll, invalid};
    }

    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        variable_list none(7);
        if (!ctx->saved_data["need"].toBool()) return none;
        TORCH_CHECK(!grads[0].defined(), "Cannot reuse the logits after pcfg_criterion");
        TORCH_CHECK(!grads[2].defined(), "pcfg_criterion: only the loss is differentiable (use cuda_pcfg_loss for per-sentence gradients)");
        if (!grads[1].defined()) return none;
        TORCH_CHECK(!ctx->saved_data["has_backward"].toBool(), "Cannot backward twice in pcfg_criterion");
        ctx->saved_data["has_backward"] = true;
        const auto saved = ctx->get_saved_variables();
        at::Tensor buf = saved[0], lg = saved[3];
        const at::Tensor &targets = saved[1], &mg = saved[2], &row_lse = saved[4], &ol = saved[5], &keep8 = saved[6];
        const c10::DeviceGuard guard(buf.device());
        const at::Tensor up = grads[1].detach().reshape({1}).to(buf.device(), at::kFloat);
        check_rc(pcfgnat_criterion_backward(buf.data_ptr(), dtype_code(buf, "pcfg_criterion"), targets.data_ptr<int64_t>(),
                                            mg.data_ptr<float>(), row_lse.data_ptr<float>(),
                                            keep8.defined() ? keep8.data_ptr<unsigned char>() : nullptr, ol.data_ptr<int64_t>(),
                                            (int)ctx->saved_data["pad_zeroed"].toInt(), up.data_ptr<float>(), lg.data_ptr<float>(),
                                            buf.size(0), buf.size(1), buf.size(2), targets.size(1), ctx->saved_data["ml"].toInt(),
                                            stream_of(buf)));
        none[0] = buf;
        none[1] = lg;
        return none;
    }
};

std::tuple<at::Tensor, at::Tensor, at::Tensor> pcfg_criterion(const at::Tensor &outputs, const at::Tensor &targets, const at::Tensor &links,
                                                              const at::Tensor &output_length, const at::Tensor &target_length,
                                                              c10::optional<at::Tensor> matchmask,
                                                              c10::optional<at::Tensor> keep_word_mask) {
    auto out = CriterionFn::apply(outputs, links, targets, output_length, target_length, matchmask, keep_word_mask);
    return std::make_tuple(out[1], out[2], out[3]);
}

// ---------------------------------------------------------------------------------------------------------------
// pcfg_extract_links with the products inside the kernels (glat_decomposed_with_link_two_hands_tri_pcfg.py:153-199 after
// the projections): one native call forward, one backward.  The caller (custom_ops.pcfg_extract_links) has made sure
// that the shape is one the library covers and passes the three tree masks as one byte per flag.
// ---------------------------------------------------------------------------------------------------------------
struct LinksFn : public torch::autograd::Function<LinksFn> {
    static at::Tensor forward(AutogradContext *ctx, at::Tensor query_chunks, at::Tensor key_chunks_left, at::Tensor key_chunks_right,
                              at::Tensor gate_logits, at::Tensor prev_output_tokens, int64_t pad_index, at::Tensor left_tree_mask,
                              at::Tensor right_tree_mask, at::Tensor main_chain) {
        const char *who = "pcfg_extract_links";
        need_gpu(who, {&query_chunks, &key_chunks_left, &key_chunks_right, &gate_logits, &prev_output_tokens, &left_tree_mask,
                       &right_tree_mask, &main_chain});
        TORCH_CHECK(query_chunks.dim() == 4 && key_chunks_left.sizes() == query_chunks.sizes() &&
                        key_chunks_right.sizes() == query_chunks.sizes(),
                    who, ": query and key chunks must share the shape [bsz, prelen, heads, head_dim]");
        TORCH_CHECK(query_chunks.scalar_type() == key_chunks_left.scalar_type() && query_chunks.scalar_type() == key_chunks_right.scalar_type(),
                    who, ": query and key chunks must share one of float16, float32");
        const int64_t B = query_chunks.size(0), L = query_chunks.size(1), H = query_chunks.size(2), F = query_chunks.size(3);
        TORCH_CHECK(gate_logits.dim() == 3 && gate_logits.size(0) == B && gate_logits.size(1) == L && gate_logits.size(2) == H &&
                        prev_output_tokens.dim() == 2 && prev_output_tokens.size(0) == B && prev_output_tokens.size(1) == L,
                    who, ": gate_logits must be [bsz, prelen, heads] and prev_output_tokens [bsz, prelen]");
        for (const at::Tensor *t : {&left_tree_mask, &right_tree_mask})
            TORCH_CHECK(t->scalar_type() == at::kByte && t->dim() == 2 && t->size(0) == L && t->size(1) == L && t->is_contiguous(), who,
                        ": tree masks must be contiguous uint8 [prelen, prelen]");
        TORCH_CHECK(main_chain.scalar_type() == at::kByte && main_chain.dim() == 1 && main_chain.size(0) == L && main_chain.is_contiguous(),
                    who, ": main_chain must be contiguous uint8 [prelen]");
        const int code = dtype_code(query_chunks, who);
        // (gradient mode is switched off inside a forward: whether a backward may follow is read off the inputs alone)
        const bool need = query_chunks.requires_grad() || key_chunks_left.requires_grad() || key_chunks_right.requires_grad() ||
                          gate_logits.requires_grad();
        TORCH_CHECK(pcfgnat_extract_links_fused_supported(code, L, H, F) &&
                        (!need || pcfgnat_extract_links_fused_backward_supported(code, L, H, F)),
                    who, ": shape not covered by the kernels with the products inside");
        const c10::DeviceGuard guard(query_chunks.device());
        const at::Tensor q = query_chunks.contiguous(), kl = key_chunks_left.contiguous(), kr = key_chunks_right.contiguous();
        const at::Tensor gate = gate_logits.to(at::kFloat).contiguous(), prev = prev_output_tokens.to(at::kLong).contiguous();
        const auto f32 = q.options().dtype(at::kFloat);
        at::Tensor links = at::empty({B, L, 2, L}, f32);
        const int64_t nw = 1 + (L + 31) / 32;
        at::Tensor side = at::empty({B * L * (H + (need ? nw : 0))}, f32);  // per-head normalisers, then the masks per parent as bits
        float *lse = side.data_ptr<float>();
        unsigned *tile_masks = need ? reinterpret_cast<unsigned *>(lse + B * L * H) : nullptr;
        check_rc(pcfgnat_extract_links_fused_forward(q.data_ptr(), kl.data_ptr(), kr.data_ptr(), code, gate.data_ptr<float>(),
                                                     prev.data_ptr<int64_t>(), pad_index, left_tree_mask.data_ptr<unsigned char>(),
                                                     right_tree_mask.data_ptr<unsigned char>(), main_chain.data_ptr<unsigned char>(),
                                                     links.data_ptr<float>(), lse, tile_masks, B, L, H, F, stream_of(q)));
        if (need) {
            ctx->save_for_backward({links, side, q, kl, kr, gate});
            ctx->saved_data["gate_dtype"] = (int64_t)gate_logits.scalar_type();
        }
        return links;
    }

    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        TORCH_CHECK(saved.size() == 6, "pcfg_extract_links: nothing was kept for a backward pass");
        const at::Tensor &links = saved[0], &side = saved[1], &q = saved[2], &kl = saved[3], &kr = saved[4], &gate = saved[5];
        const int64_t B = q.size(0), L = q.size(1), H = q.size(2), F = q.size(3);
        const c10::DeviceGuard guard(q.device());
        at::Tensor G = grads[0].to(at::kFloat).contiguous();
        if (reinterpret_cast<uintptr_t>(G.data_ptr()) % 16) G = G.clone();  // (a view at an odd offset: read in 16-byte pieces)
        at::Tensor d = at::empty({3, B, L, H, F}, q.options().requires_grad(false));
        const int64_t nws = (int64_t)((pcfgnat_extract_links_fused_backward_workspace_bytes(B, L, H, F) + 3) / 4);
        at::Tensor block = at::empty({nws + B * L * H}, q.options().dtype(at::kFloat).requires_grad(false));  // the workspace first: it wants 16-byte alignment
        float *ws = block.data_ptr<float>();
        const float *lse = side.data_ptr<float>();
        check_rc(pcfgnat_extract_links_fused_backward(G.data_ptr<float>(), links.data_ptr<float>(), lse,
                                                      reinterpret_cast<const unsigned *>(lse + B * L * H), q.data_ptr(), kl.data_ptr(),
                                                      kr.data_ptr(), dtype_code(q, "pcfg_extract_links"), gate.data_ptr<float>(),
                                                      d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), ws + nws, ws, B, L, H, F,
                                                      stream_of(q)));
        const at::Tensor dgate = block.narrow(0, nws, B * L * H).view({B, L, H});
        const auto gate_dtype = (at::ScalarType)ctx->saved_data["gate_dtype"].toInt();
        variable_list out(9);
        out[0] = d[0];
        out[1] = d[1];
        out[2] = d[2];
        out[3] = dgate.to(gate_dtype);
        return out;
    }
};

at::Tensor pcfg_extract_links_fused(const at::Tensor &query_chunks, const at::Tensor &key_chunks_left, const at::Tensor &key_chunks_right,
                                    const at::Tensor &gate_logits, const at::Tensor &prev_output_tokens, int64_t pad_index,
                                    const at::Tensor &left_tree_mask, const at::Tensor &right_tree_mask, const at::Tensor &main_chain) {
    return LinksFn::apply(query_chunks, key_chunks_left, key_chunks_right, gate_logits, prev_output_tokens, pad_index, left_tree_mask,
                          right_tree_mask, main_chain);
}

// ---------------------------------------------------------------------------------------------------------------
// The Viterbi decode as one native call (glat_decomposed_with_link_two_hands_tri_pcfg.py:414-416, 483-502): checks, the one
// allocation and the enqueue.  A decode of one short sentence is a few tens of microseconds of kernels; the same steps in
// Python (a dozen tensor-attribute calls, the device context, ctypes marshalling of twenty arguments) cost the host about
// ten more in front of the first launch.
//
// From the vocabulary logits [B,L,V] (float16 / float32; `node_scores`, `node_tokens` undefined) or from the node scores
// [B,L] float32 and node tokens [B,L] (`logits` undefined).  One block holds workspace | tokens [B,L] int64 | predicted
// lengths [B] | tokens [B,L] float32 | (from logits) node tokens [B,L] int64, node scores [B,L] float32.  The kernels write
// the per-sentence token counts to `counts_address` (pinned host memory owned by the caller, B int64); if `may_watch` and
// the stream is idle the entries are marked "not yet" (-2) first and the caller may watch them turn instead of waiting
// for the stream.  Returns (tokens float32 [B,L], predicted lengths [B], the block, whether the entries were marked).
// ---------------------------------------------------------------------------------------------------------------
std::tuple<at::Tensor, at::Tensor, at::Tensor, bool> viterbi_decode_enqueue(const c10::optional<at::Tensor> &logits,
                                                                            const c10::optional<at::Tensor> &node_scores,
                                                                            const c10::optional<at::Tensor> &node_tokens,
                                                                            const at::Tensor &links_in, const at::Tensor &output_length,
                                                                            const at::Tensor &left_tree_mask, int64_t pad_index,
                                                                            const at::Tensor &length_penalty, int64_t counts_address,
                                                                            bool may_watch) {
    const bool from_logits = logits.has_value() && logits->defined();
    const char *who = from_logits ? "pcfg_viterbi_decode_logits" : "pcfg_viterbi_decode";
    at::Tensor ob, tok;
    int64_t B, L, V = 0;
    if (from_logits) {
        need_gpu(who, {&*logits, &links_in, &output_length, &left_tree_mask, &length_penalty});
        TORCH_CHECK(logits->dim() == 3 && logits->is_contiguous(), who, ": logits must be a contiguous [bsz, prelen, vocab] tensor");
        TORCH_CHECK(logits->scalar_type() == at::kHalf || logits->scalar_type() == at::kFloat, who,
                    ": logits must be float16 or float32 (got ", logits->scalar_type(), ")");
        B = logits->size(0), L = logits->size(1), V = logits->size(2);
    } else {
        TORCH_CHECK(node_scores.has_value() && node_tokens.has_value(), who, ": node scores and node tokens are needed");
        need_gpu(who, {&*node_scores, &links_in, &output_length, &*node_tokens, &left_tree_mask, &length_penalty});
        TORCH_CHECK(node_scores->dim() == 2 && links_in.dim() == 4, who,
                    ": unreduced_logits must be [bsz, prelen] and links [bsz, prelen, max_left+1, prelen]");
        TORCH_CHECK(node_scores->scalar_type() == at::kFloat && links_in.scalar_type() == at::kFloat, who,
                    ": unreduced_logits and links must be float32");
        B = node_scores->size(0), L = node_scores->size(1);
        ob = node_scores->contiguous();
        tok = node_tokens->scalar_type() == at::kLong ? node_tokens->contiguous() : node_tokens->to(at::kLong).contiguous();
        TORCH_CHECK(tok.dim() == 2 && tok.size(0) == B && tok.size(1) == L, who, ": unreduced_tokens must be [bsz, prelen]");
    }
    TORCH_CHECK(links_in.dim() == 4 && links_in.scalar_type() == at::kFloat, who, ": links must be float32 [bsz, prelen, max_left+1, prelen]");
    TORCH_CHECK(links_in.size(0) == B && links_in.size(1) == L && links_in.size(3) == L, who, ": links shape ", links_in.sizes(),
                " does not match [bsz, prelen] = (", B, ", ", L, ")");
    TORCH_CHECK(left_tree_mask.dim() == 2 && left_tree_mask.size(0) == left_tree_mask.size(1), who, ": left_tree_mask must be square");
    const int64_t ml = links_in.size(2) - 1;
    TORCH_CHECK(length_penalty.scalar_type() == at::kFloat && length_penalty.is_contiguous() && length_penalty.numel() >= L / 4, who,
                ": length penalty must be float32 [prelen / 4]");
    const at::Tensor links = links_in.contiguous();
    const at::Tensor ol = lengths(who, output_length, B);
    const at::Tensor mask = left_tree_mask.scalar_type() == at::kLong ? left_tree_mask.contiguous() : left_tree_mask.to(at::kLong).contiguous();
    const c10::DeviceGuard guard(links.device());
    const int64_t nodes = B * L, fwords = (nodes + 1) / 2;
    const int64_t nwork = (int64_t)((pcfgnat_viterbi_decode_workspace_bytes(B, L, ml) + 7) / 8);
    const int64_t extra = from_logits ? nodes + fwords : 0;
    at::Tensor block = at::empty({nwork + nodes + B + fwords + extra}, links.options().dtype(at::kLong).requires_grad(false));
    int64_t *base = block.data_ptr<int64_t>();
    int64_t *out_tokens = base + nwork, *pred = out_tokens + nodes;
    float *tokens_f32 = reinterpret_cast<float *>(pred + B);
    const auto stream = c10::hip::getCurrentHIPStream(links.device().index());
    int64_t *counts = reinterpret_cast<int64_t *>(static_cast<intptr_t>(counts_address));
    TORCH_CHECK(counts != nullptr || B == 0, who, ": no buffer for the token counts");
    const bool marked = may_watch && B > 0 && stream.query();
    if (marked)
        for (int64_t i = 0; i < B; i++) counts[i] = -2;
    if (from_logits) {
        int64_t *best_idx = pred + B + fwords;
        float *best_lprob = reinterpret_cast<float *>(best_idx + nodes);
        check_rc(pcfgnat_viterbi_decode_logits(logits->data_ptr(), dtype_code(*logits, who), V, best_lprob, best_idx, links.data_ptr<float>(),
                                               ol.data_ptr<int64_t>(), mask.data_ptr<int64_t>(), mask.size(0), pad_index,
                                               length_penalty.data_ptr<float>(), base, out_tokens, tokens_f32, counts, pred, B, L, ml,
                                               (void *)stream.stream()));
    } else {
        check_rc(pcfgnat_viterbi_decode(ob.data_ptr<float>(), links.data_ptr<float>(), ol.data_ptr<int64_t>(), tok.data_ptr<int64_t>(),
                                        mask.data_ptr<int64_t>(), mask.size(0), pad_index, length_penalty.data_ptr<float>(), base, out_tokens,
                                        tokens_f32, counts, pred, B, L, ml, (void *)stream.stream()));
    }
    at::Tensor tokf = block.slice(0, nwork + nodes + B, nwork + nodes + B + fwords).view(at::kFloat).slice(0, 0, nodes).view({B, L});
    return std::make_tuple(tokf, block.slice(0, nwork + nodes, nwork + nodes + B), block, marked);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "host side of PCFG-NAT's training operators over libpcfg_nat_hip.so";
    m.def("abi_version", []() { return pcfgnat_abi_version(); });
    m.def("cuda_pcfg_loss", &cuda_pcfg_loss, "inside-algorithm log-likelihood, float32 (pcfg_loss.py:49-85)");
    m.def("dag_logsoftmax_gather_inplace", &dag_logsoftmax_gather_inplace, "fused log-softmax + gather (pcfg_loss.py:144-181)");
    m.def("pcfg_criterion", &pcfg_criterion, "the criterion's loss as one differentiable op (nat_pcfg_loss.py:98-145)", py::arg("outputs"),
          py::arg("targets"), py::arg("links"), py::arg("output_length"), py::arg("target_length"), py::arg("matchmask") = py::none(),
          py::arg("keep_word_mask") = py::none());
    m.def("viterbi_decode_enqueue", &viterbi_decode_enqueue,
          "checks, allocation and enqueue of the single-call Viterbi decode (glat_decomposed_with_link_two_hands_tri_pcfg.py:414-416, 483-502)");
    m.def("pcfg_extract_links_fused", &pcfg_extract_links_fused,
          "the link scorer after its projections, products inside the kernels (glat_decomposed_with_link_two_hands_tri_pcfg.py:153-199)");
}
