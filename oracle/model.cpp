// Llama-style target forward of the CPU oracle (test infrastructure only).
//
// The reference has no verify pass for this family (real_forward_traits.rs:323-328); it is
// composed here from the per-token decode graph (families/llama/mod.rs:197-316,
// attn.rs:152-369, dense.rs:45-120) under the batched-verify contract of
// families/qwen/batched.rs:92-456: M rows at positions base..base+M, K/V of row m stored at
// cache position base+m before any row attends, row m sees [0, base+m] (chain) or the
// committed prefix plus its root path (tree, batched_layers.rs:216-228,373-408).
// All arithmetic is the fp32 of crates/compute; the only fp16 roundings are the K/V cache
// store (optional) and the logits store, the two dtype boundaries the engine fixes.
#include "tsoracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <string>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

void tso_set_error(const std::string& s);

struct tso_model {
    tso_model_desc d;
    std::vector<tso_layer> layers;
    std::vector<float> rope_freqs;  // non-empty when rope_factors given
    std::vector<std::vector<float>> k, v;  // per layer [max_context][nkv*hd]
    int64_t position = 0;
    float route_margin = 1.0f;
    // the routing of the last verify call: [layer][row][8] expert ids in rank order (-1 past top_k) and
    // [layer][row] the relative gap between the last chosen and the first rejected logit
    std::vector<int32_t> route_sel;
    std::vector<float> route_gap;
    // test hook: expert ids to take instead of the top-k, same shape (empty: route normally)
    std::vector<int32_t> forced_sel;
    // TurboQuant KV: sign vectors, codebooks and midpoints of the key and the value side
    std::vector<float> tq_k_signs, tq_v_signs, tq_k_cb, tq_v_cb, tq_k_mid, tq_v_mid;
    // the residual stream of the last pass's rows after the last layer, before the final norm: [rows][hidden]
    std::vector<float> last_x;
    int last_rows = 0;
    bool quantized(int layer) const {  // model-io/src/kv_quant.rs:102-107
        if (d.kv_k_bits <= 0 || layers[layer].window != 0) return false;
        return d.n_layers <= 2 || layer + 1 < d.n_layers;
    }
};

namespace {

// Y[m][r] = sum_k dequant(W[r])[k] * X[m][k]; each (m, r) is the sequential fp32 sum of
// dequant_*_gemv (q4_k.rs:207-220).  The row is dequantized once and reused for all m,
// which changes no bit of any result.
void gemm_rows(const tso_tensor& w, const float* x, int m_rows, float* y, int threads) {
    int64_t rows = w.rows, cols = w.cols;
    int64_t rb = tso_row_bytes(w.dtype, cols);
    const uint8_t* base = (const uint8_t*)w.data;
#pragma omp parallel num_threads(threads)
    {
        std::vector<float> deq((size_t)cols);
#pragma omp for schedule(static)
        for (int64_t r = 0; r < rows; r++) {
            tso_dequantize_row(w.dtype, base + r * rb, cols, deq.data());
            for (int m = 0; m < m_rows; m++) {
                const float* xv = x + (int64_t)m * cols;
                float acc = 0.0f;
                for (int64_t kk = 0; kk < cols; kk++) acc += deq[kk] * xv[kk];
                y[(int64_t)m * rows + r] = acc;
            }
        }
    }
}

// Rows [r0, r0 + n) of a stacked matrix as a tensor of their own.
tso_tensor row_slice(const tso_tensor& t, int64_t r0, int64_t n) {
    tso_tensor v = t;
    v.data = (const uint8_t*)t.data + r0 * tso_row_bytes(t.dtype, t.cols);
    v.rows = n;
    return v;
}

// real_forward_dispatch.rs:1135-1158 (`router_topk_gemma4`, per_expert_scale all ones): top-k by
// logit, ties to the lower index; softmax over the selected logits only.
// `forced` (test hook, nullable): k expert ids to take, in this order, instead of the top-k -- the
// weights are still the softmax of this row's own logits over them.  `gap_out` (nullable): the
// relative gap between the last chosen and the first rejected logit of the unforced ranking.
void route_topk(const float* logits, int n, int k, int* sel, float* w, float* margin, const int32_t* forced = nullptr,
                float* gap_out = nullptr) {
    std::vector<int> order(n);
    for (int i = 0; i < n; i++) order[i] = i;
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return logits[a] > logits[b]; });
    for (int i = 0; i < k; i++) sel[i] = forced ? forced[i] : order[i];
    float mx = logits[sel[0]];
    for (int i = 1; i < k; i++) mx = std::max(mx, logits[sel[i]]);
    float sum = 0.0f, ex[8];
    for (int i = 0; i < k; i++) {
        ex[i] = std::exp(logits[sel[i]] - mx);
        sum += ex[i];
    }
    for (int i = 0; i < k; i++) w[i] = ex[i] / sum * 1.0f;
    if (k < n) {
        const float range = logits[order[0]] - logits[order[n - 1]];
        const float gap = (logits[order[k - 1]] - logits[order[k]]) / (range > 0.0f ? range : 1.0f);
        if (gap < *margin) *margin = gap;
        if (gap_out) *gap_out = gap;
    } else if (gap_out) {
        *gap_out = 1.0f;
    }
}

std::vector<float> norm_weight(const tso_tensor& t) {
    std::vector<float> w((size_t)t.cols);
    tso_dequantize_row(t.dtype, (const uint8_t*)t.data, t.cols, w.data());
    return w;
}

inline float round_f16(float x) { return tso_f16_to_f32(tso_f32_to_f16(x)); }

// y[m][i] += bias[i] for a one-row tensor of any dtype (absent: nothing)
void add_bias(const tso_tensor& b, float* y, int m_rows, int n) {
    if (!b.data) return;
    std::vector<float> bias = norm_weight(b);
    for (int m = 0; m < m_rows; m++)
        for (int i = 0; i < n; i++) y[(size_t)m * n + i] += bias[i];
}

}  // namespace

extern "C" tso_model* tso_model_create(const tso_model_desc* desc) {
    tso_model* m = new tso_model();
    m->d = *desc;
    m->layers.assign(desc->layers, desc->layers + desc->n_layers);
    m->d.layers = m->layers.data();
    if (m->d.threads < 1) m->d.threads = 1;
    int64_t stride = (int64_t)desc->n_kv_heads * desc->head_dim;
    m->k.resize(desc->n_layers);
    m->v.resize(desc->n_layers);
    for (int l = 0; l < desc->n_layers; l++) {
        m->k[l].assign((size_t)(desc->max_context * stride), 0.0f);
        m->v[l].assign((size_t)(desc->max_context * stride), 0.0f);
    }
    if (desc->rope_freqs) {
        m->rope_freqs.assign(desc->rope_freqs, desc->rope_freqs + desc->head_dim / 2);
        m->d.rope_freqs = nullptr;
        m->d.rope_factors = nullptr;
    } else if (desc->rope_factors) {
        m->rope_freqs.resize(desc->head_dim / 2);
        tso_rope_frequencies_with_factors(desc->head_dim, desc->rope_theta, desc->rope_factors,
                                          m->rope_freqs.data());
        m->d.rope_factors = nullptr;
    }
    if (!(m->d.rope_mscale > 0.0f)) m->d.rope_mscale = 1.0f;
    if (m->d.kv_k_bits > 0) {  // kv_quant_attention.rs:24-44: one table set per side, KEY_SEED 0 and VALUE_SEED 1
        if (m->d.kv_v_bits <= 0) m->d.kv_v_bits = m->d.kv_k_bits;
        const int hd = desc->head_dim;
        auto side = [&](int bits, uint64_t seed, std::vector<float>& signs, std::vector<float>& cb, std::vector<float>& mid) {
            signs.resize(hd);
            tso_tq_sign_vector(hd, seed, signs.data());
            cb.resize((size_t)1 << bits);
            tso_tq_codebook(hd, bits, cb.data());
            mid.resize(cb.size());  // one spare
            tso_tq_midpoints(cb.data(), (int)cb.size(), mid.data());
        };
        side(m->d.kv_k_bits, 0, m->tq_k_signs, m->tq_k_cb, m->tq_k_mid);
        side(m->d.kv_v_bits, 1, m->tq_v_signs, m->tq_v_cb, m->tq_v_mid);
    }
    return m;
}
extern "C" int tso_model_layer_quantized(const tso_model* m, int layer) { return m->quantized(layer) ? 1 : 0; }

extern "C" void tso_model_destroy(tso_model* m) { delete m; }
extern "C" float tso_model_route_margin(const tso_model* m) { return m->route_margin; }
extern "C" int tso_model_route_record(const tso_model* m, int32_t* sel, float* gap) {
    if (m->route_sel.empty()) return -1;
    std::copy(m->route_sel.begin(), m->route_sel.end(), sel);
    std::copy(m->route_gap.begin(), m->route_gap.end(), gap);
    return 0;
}
extern "C" void tso_model_force_route(tso_model* m, const int32_t* sel, int64_t n) {
    m->forced_sel.assign(sel, sel + (sel ? n : 0));
}
extern "C" void tso_model_reset(tso_model* m) { m->position = 0; }
extern "C" int64_t tso_model_position(const tso_model* m) { return m->position; }
// kv_cache_rewind.rs:46-55: a cursor move; rows are addressed by absolute position and
// nothing is erased.
extern "C" void tso_model_rewind_to(tso_model* m, int64_t position) { m->position = position; }
extern "C" float* tso_model_k(tso_model* m, int layer) { return m->k[layer].data(); }
extern "C" float* tso_model_v(tso_model* m, int layer) { return m->v[layer].data(); }

// `x0` (nullable): the rows that enter the first layer, in place of the embedding lookup of `feed`.
static int verify_impl(tso_model* mdl, const int32_t* feed, const int32_t* parent, int M, int64_t base,
                       uint16_t* logits_f16, float* logits_f32, int n_layers_run, const float* x0) {
    const tso_model_desc& d = mdl->d;
    // batched.rs:106-185 refusals
    if (M <= 0) {
        tso_set_error("verify: empty feed");
        return -1;
    }
    if (base != mdl->position) {
        tso_set_error("verify: start position does not match the KV cursor");
        return -2;
    }
    if (base + M > d.max_context) {
        tso_set_error("verify: block would write past the KV capacity");
        return -3;
    }
    for (int m = 0; m < M; m++)
        if (feed[m] < 0 || feed[m] >= d.vocab) {
            tso_set_error("verify: token id outside the vocabulary");
            return -4;
        }
    std::vector<int> depth(M, 0);
    if (parent) {
        if (parent[0] != -1) {
            tso_set_error("verify_tree: slot 0 must be the anchor (parent -1)");
            return -5;
        }
        for (int s = 1; s < M; s++) {
            if (parent[s] < 0 || parent[s] >= s) {
                tso_set_error("verify_tree: parent[s] must be in [0, s)");
                return -5;
            }
            depth[s] = depth[parent[s]] + 1;
        }
    } else {
        for (int m = 0; m < M; m++) depth[m] = m;
    }

    const int H = d.hidden, nq = d.n_q_heads, nkv = d.n_kv_heads, hd = d.head_dim, F = d.ffn;
    const int qd = nq * hd, kvd = nkv * hd;
    const int T = d.threads;
    std::vector<float> x((size_t)M * H), xn((size_t)M * H);
    // embed lookup (real_forward_dispatch.rs:154): one dequantized row per token
    if (x0) {
        std::memcpy(x.data(), x0, sizeof(float) * (size_t)M * H);
    } else {
        int64_t rb = tso_row_bytes(d.embed.dtype, H);
        for (int m = 0; m < M; m++)
            tso_dequantize_row(d.embed.dtype, (const uint8_t*)d.embed.data + (int64_t)feed[m] * rb, H,
                               &x[(size_t)m * H]);
    }
    std::vector<float> q((size_t)M * qd), kk((size_t)M * kvd), vv((size_t)M * kvd),
        att((size_t)M * qd), proj((size_t)M * H), gate((size_t)M * F), up((size_t)M * F);

    int L = n_layers_run < 0 ? d.n_layers : std::min(n_layers_run, (int)d.n_layers);
    mdl->route_margin = 1.0f;
    for (int l = 0; l < L; l++) {
        const tso_layer& ly = d.layers[l];
        std::vector<float> wn = norm_weight(ly.attn_norm);
        for (int m = 0; m < M; m++)
            tso_rms_norm(&x[(size_t)m * H], wn.data(), H, d.rms_eps, &xn[(size_t)m * H]);
        gemm_rows(ly.wq, xn.data(), M, q.data(), T);
        gemm_rows(ly.wk, xn.data(), M, kk.data(), T);
        gemm_rows(ly.wv, xn.data(), M, vv.data(), T);
        // families/gptoss/attn.rs:88-101: the projection biases, before the rotation
        add_bias(ly.bq, q.data(), M, qd);
        add_bias(ly.bk, kk.data(), M, kvd);
        add_bias(ly.bv, vv.data(), M, kvd);
        if (ly.q_norm.data) {  // per-head q/k RMSNorm (families/llama/state.rs:344-347)
            std::vector<float> qw = norm_weight(ly.q_norm), kw = norm_weight(ly.k_norm);
            std::vector<float> tmp(hd);
            for (int m = 0; m < M; m++) {
                for (int h = 0; h < nq; h++) {
                    float* p = &q[(size_t)m * qd + (size_t)h * hd];
                    tso_rms_norm(p, qw.data(), hd, d.rms_eps, tmp.data());
                    std::memcpy(p, tmp.data(), sizeof(float) * hd);
                }
                for (int h = 0; h < nkv; h++) {
                    float* p = &kk[(size_t)m * kvd + (size_t)h * hd];
                    tso_rms_norm(p, kw.data(), hd, d.rms_eps, tmp.data());
                    std::memcpy(p, tmp.data(), sizeof(float) * hd);
                }
            }
        }
        float* kc = mdl->k[l].data();
        float* vc = mdl->v[l].data();
        for (int m = 0; m < M; m++) {
            int64_t pos = base + depth[m];
            if (!mdl->rope_freqs.empty()) {
                tso_rope_neox_freqs_scaled(&q[(size_t)m * qd], 1, nq, hd, hd / 2, pos, mdl->rope_freqs.data(),
                                           d.rope_mscale);
                tso_rope_neox_freqs_scaled(&kk[(size_t)m * kvd], 1, nkv, hd, hd / 2, pos,
                                           mdl->rope_freqs.data(), d.rope_mscale);
            } else {
                tso_rope_neox(&q[(size_t)m * qd], 1, nq, hd, hd / 2, pos, d.rope_theta);
                tso_rope_neox(&kk[(size_t)m * kvd], 1, nkv, hd, hd / 2, pos, d.rope_theta);
            }
            // K,V land in the cache slot of row m (batched_layers.rs:84-113)
            float* kd = kc + (base + m) * kvd;
            float* vd = vc + (base + m) * kvd;
            for (int i = 0; i < kvd; i++) {
                kd[i] = d.round_kv_f16 ? round_f16(kk[(size_t)m * kvd + i]) : kk[(size_t)m * kvd + i];
                vd[i] = d.round_kv_f16 ? round_f16(vv[(size_t)m * kvd + i]) : vv[(size_t)m * kvd + i];
            }
            if (mdl->quantized(l)) {
                // kv_write.rs:66-118: the fp16 staging row is quantized into the slot, head by head;
                // attention then sees what the codes decode to (kv_quant_attention.rs:58-136 computes
                // the same sums in the rotated space)
                std::vector<uint32_t> words((size_t)hd + 1);
                std::vector<float> back((size_t)hd);
                for (int h = 0; h < nkv; h++) {
                    float norm;
                    tso_tq_quantize_row(kd + (size_t)h * hd, hd, mdl->tq_k_signs.data(), mdl->tq_k_mid.data(), d.kv_k_bits, &norm,
                                        words.data());
                    tso_tq_dequantize_row(norm, words.data(), mdl->tq_k_signs.data(), mdl->tq_k_cb.data(), d.kv_k_bits, hd,
                                          back.data());
                    std::memcpy(kd + (size_t)h * hd, back.data(), sizeof(float) * hd);
                    tso_tq_quantize_row(vd + (size_t)h * hd, hd, mdl->tq_v_signs.data(), mdl->tq_v_mid.data(), d.kv_v_bits, &norm,
                                        words.data());
                    tso_tq_dequantize_row(norm, words.data(), mdl->tq_v_signs.data(), mdl->tq_v_cb.data(), d.kv_v_bits, hd,
                                          back.data());
                    std::memcpy(vd + (size_t)h * hd, back.data(), sizeof(float) * hd);
                }
            }
        }
        std::vector<float> sinks;
        if (ly.sinks.data) sinks = norm_weight(ly.sinks);
        const float* sk = sinks.empty() ? nullptr : sinks.data();
#pragma omp parallel for num_threads(T) schedule(static)
        for (int m = 0; m < M; m++) {
            if (!parent) {
                // window: families/gptoss/attn.rs:120-137 (kv_start = seq_len - window, saturating)
                tso_causal_attention(&q[(size_t)m * qd], kc, vc, hd, nq, nkv, base + m + 1, ly.window,
                                     d.attn_scale, sk, &att[(size_t)m * qd]);
            } else {
                int64_t path[64];
                int n = 0;
                for (int s = m; s >= 0; s = parent[s]) path[n++] = base + s;
                for (int i = 0; i < n / 2; i++) std::swap(path[i], path[n - 1 - i]);
                // the row's sequence is the committed prefix followed by its root path; a window
                // keeps the last `window` members of that sequence
                int64_t seq_len = base + n, kv_start = 0;
                if (ly.window > 0 && seq_len > ly.window) kv_start = seq_len - ly.window;
                int skip = kv_start > base ? (int)(kv_start - base) : 0;
                tso_attention_core(&q[(size_t)m * qd], kc, vc, hd, nq, nkv, std::min(kv_start, base), base,
                                   path + skip, n - skip, d.attn_scale, sk, &att[(size_t)m * qd]);
            }
        }
        gemm_rows(ly.wo, att.data(), M, proj.data(), T);
        add_bias(ly.bo, proj.data(), M, H);
        for (size_t i = 0; i < (size_t)M * H; i++) x[i] = x[i] + proj[i];

        std::vector<float> wf = norm_weight(ly.ffn_norm);
        for (int m = 0; m < M; m++)
            tso_rms_norm(&x[(size_t)m * H], wf.data(), H, d.rms_eps, &xn[(size_t)m * H]);
        if (ly.n_experts > 0) {
            // families/llama/moe.rs + compute/src/moe.rs:47-73: y = x + sum over slots, in the
            // router's rank order, of w_slot * down_e(silu(gate_e xn) * up_e xn)
            const int E = ly.n_experts, K = ly.top_k;
            std::vector<float> rl((size_t)M * E);
            gemm_rows(ly.router, xn.data(), M, rl.data(), T);
            add_bias(ly.router_bias, rl.data(), M, E);  // families/gptoss/moe.rs:82-87: before the top-k
            std::vector<float> routed(H);
            for (int m = 0; m < M; m++) {
                int sel[8] = {0};
                float w[8];
                // the record (and the forced routing of the test hook) covers the first 16 rows of a call
                const bool rec = m < 16;
                const size_t slot = (size_t)l * 16 + (size_t)(rec ? m : 0);
                const int32_t* forced = rec && mdl->forced_sel.size() >= (slot + 1) * 8 ? &mdl->forced_sel[slot * 8] : nullptr;
                if (mdl->route_sel.size() < (size_t)d.n_layers * 16 * 8) {
                    mdl->route_sel.assign((size_t)d.n_layers * 16 * 8, -1);
                    mdl->route_gap.assign((size_t)d.n_layers * 16, 1.0f);
                }
                float gap_row = 1.0f;
                route_topk(&rl[(size_t)m * E], E, K, sel, w, &mdl->route_margin, forced, &gap_row);
                if (rec) {
                    mdl->route_gap[slot] = gap_row;
                    for (int s2 = 0; s2 < 8; s2++) mdl->route_sel[slot * 8 + s2] = s2 < K ? sel[s2] : -1;
                }
                // families/llama/moe.rs:193-198: the routed sum starts from zero, is accumulated in
                // rank order, and is then added to the stream
                std::fill(routed.begin(), routed.end(), 0.0f);
                for (int s = 0; s < K; s++) {
                    const int e = sel[s];
                    gemm_rows(row_slice(ly.we_gate, (int64_t)e * F, F), &xn[(size_t)m * H], 1, gate.data(), T);
                    gemm_rows(row_slice(ly.we_up, (int64_t)e * F, F), &xn[(size_t)m * H], 1, up.data(), T);
                    add_bias(row_slice(ly.be_gate, e, 1), gate.data(), 1, F);  // moe_gguf.metal:592-600
                    add_bias(row_slice(ly.be_up, e, 1), up.data(), 1, F);
                    for (int i = 0; i < F; i++)
                        gate[i] = d.act_alpha > 0.0f ? tso_swiglu_oai(gate[i], up[i], d.act_alpha, d.act_limit)
                                                     : tso_silu(gate[i]) * up[i];
                    gemm_rows(row_slice(ly.we_down, (int64_t)e * H, H), gate.data(), 1, proj.data(), T);
                    add_bias(row_slice(ly.be_down, e, 1), proj.data(), 1, H);
                    for (int i = 0; i < H; i++) routed[i] += w[s] * proj[i];
                }
                for (int i = 0; i < H; i++) x[(size_t)m * H + i] += routed[i];
            }
        } else {
            gemm_rows(ly.w_gate, xn.data(), M, gate.data(), T);
            gemm_rows(ly.w_up, xn.data(), M, up.data(), T);
            for (size_t i = 0; i < (size_t)M * F; i++) gate[i] = tso_silu(gate[i]) * up[i];
            gemm_rows(ly.w_down, gate.data(), M, proj.data(), T);
            for (size_t i = 0; i < (size_t)M * H; i++) x[i] = x[i] + proj[i];
        }
    }

    mdl->last_x = x;
    mdl->last_rows = M;
    // head (verify_layers.rs:270-333): final norm, lm_head, raw logits (mod.rs:421-423)
    if (!logits_f16 && !logits_f32) {  // a pass taken for its cache rows alone (produce_prefill, mtp_prime_step)
        mdl->position = base + M;
        return 0;
    }
    std::vector<float> wfin = norm_weight(d.final_norm);
    for (int m = 0; m < M; m++)
        tso_rms_norm(&x[(size_t)m * H], wfin.data(), H, d.rms_eps, &xn[(size_t)m * H]);
    const tso_tensor& head = d.lm_head.data ? d.lm_head : d.embed;
    std::vector<float> logits((size_t)M * d.vocab);
    gemm_rows(head, xn.data(), M, logits.data(), T);
    if (logits_f32) std::memcpy(logits_f32, logits.data(), logits.size() * sizeof(float));
    if (logits_f16)
        for (size_t i = 0; i < logits.size(); i++) logits_f16[i] = tso_f32_to_f16(logits[i]);
    mdl->position = base + M;
    return 0;
}

extern "C" int tso_model_verify(tso_model* mdl, const int32_t* feed, const int32_t* parent, int M, int64_t base,
                                uint16_t* logits_f16, float* logits_f32, int n_layers_run) {
    return verify_impl(mdl, feed, parent, M, base, logits_f16, logits_f32, n_layers_run, nullptr);
}

extern "C" int tso_model_last_hidden(const tso_model* m, int row, float* out) {
    if (row < 0 || row >= m->last_rows) {
        tso_set_error("last_hidden: no such row in the last pass");
        return -1;
    }
    std::memcpy(out, &m->last_x[(size_t)row * m->d.hidden], sizeof(float) * m->d.hidden);
    return 0;
}

// The drafter head's recurrence (docs/MTP.md:53-60; families/qwen/mtp.rs:441-700, batched rows :146-400):
//   x0 = fc([ norm_e(embed(t_{i+1})) ; norm_h(trunk_final_norm(h_i)) ])   embedding half first
// then the head model's one decoder layer over its OWN cache at position i, its own final norm
// (mtp.norm) and the trunk's output head.  h_i is a row of the trunk's residual stream (what its final
// norm consumes), or -- a chained step -- the head's own residual of the step before, through the same
// two norms.  The norms are the plain RMSNorm of this family's layers (the reference's qwen3.5 head keeps
// its weights as offsets from one; a plain-norm file holds the effective scale).
extern "C" int tso_mtp_step(tso_model* head, const tso_mtp_desc* mtp, const int32_t* next_tokens, const float* h_rows,
                            int M, int64_t position, uint16_t* logits_f16, float* logits_f32, float* x0_out) {
    const tso_model_desc& d = head->d;
    const int H = d.hidden;
    if (M <= 0) {
        tso_set_error("mtp_step: no rows");
        return -1;
    }
    if (mtp->fc.rows != H || mtp->fc.cols != 2 * H) {
        tso_set_error("mtp_step: fc must be hidden x (2 * hidden)");
        return -6;
    }
    for (int m = 0; m < M; m++)
        if (next_tokens[m] < 0 || next_tokens[m] >= d.vocab) {  // mtp.rs:461-465
            tso_set_error("mtp_step: draft token id outside the vocabulary");
            return -4;
        }
    if (position != head->position) {  // mtp.rs:484-491
        tso_set_error("mtp_step: the step's position is not where the head's cache ends");
        return -2;
    }
    std::vector<float> we = norm_weight(mtp->norm_embedding), wh = norm_weight(mtp->norm_hidden),
                       wt = norm_weight(mtp->trunk_norm);
    std::vector<float> cat((size_t)M * 2 * H), e(H), t(H), x0((size_t)M * H);
    const int64_t rb = tso_row_bytes(d.embed.dtype, H);
    for (int m = 0; m < M; m++) {
        tso_dequantize_row(d.embed.dtype, (const uint8_t*)d.embed.data + (int64_t)next_tokens[m] * rb, H, e.data());
        tso_rms_norm(e.data(), we.data(), H, d.rms_eps, &cat[(size_t)m * 2 * H]);
        tso_rms_norm(h_rows + (size_t)m * H, wt.data(), H, d.rms_eps, t.data());
        tso_rms_norm(t.data(), wh.data(), H, d.rms_eps, &cat[(size_t)m * 2 * H + H]);
    }
    gemm_rows(mtp->fc, cat.data(), M, x0.data(), d.threads);
    if (x0_out) std::memcpy(x0_out, x0.data(), sizeof(float) * x0.size());
    std::vector<int32_t> feed(next_tokens, next_tokens + M);
    return verify_impl(head, feed.data(), nullptr, M, position, logits_f16, logits_f32, -1, x0.data());
}

// families/qwen/dflash_tree.rs:106-207: gather the accepted path's rows into consecutive
// slots; safe in place because path[i] >= i.
extern "C" void tso_model_compact_tree(tso_model* m, int64_t base, const uint32_t* path, int n) {
    int64_t stride = (int64_t)m->d.n_kv_heads * m->d.head_dim;
    for (int l = 0; l < m->d.n_layers; l++)
        for (int i = 0; i < n; i++) {
            if ((int64_t)path[i] == i) continue;
            std::memmove(&m->k[l][(base + i) * stride], &m->k[l][(base + path[i]) * stride],
                         sizeof(float) * stride);
            std::memmove(&m->v[l][(base + i) * stride], &m->v[l][(base + path[i]) * stride],
                         sizeof(float) * stride);
        }
}
