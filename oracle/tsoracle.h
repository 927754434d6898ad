/*
 * tsoracle.h -- CPU restatement of the reference's speculative-verify path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT THE PRODUCT.  Nothing under turbospark_amd/
 * may include, link or call it.  It exists so the HIP path has something to be
 * compared against: plain scalar C++ that follows the reference's own CPU
 * sources function by function (each function cites the file:line it restates),
 * compiled with -ffp-contract=off so no multiply-add is fused that the Rust
 * original keeps separate.
 *
 * Pinned parts (what proves each restatement, besides reading it):
 *   - Q4_K decode / scale unpack ....... the reference's hand-packed superblock literal
 *   - Q8_0, Q4_K encode ................ round-trip bounds, idempotence, zero blocks
 *   - MXFP4 decode ..................... ggml-produced bytes -> floats fixture, all 256 scale bytes
 *   - rope / llama-3 factors ........... the reference's literal factor profile + closed forms
 *   - attention, rms_norm .............. closed-form small cases and brute-force restatements
 *   - whole fp32 Llama-style forward ... MLX known-answer logits (three fixtures), 2e-4
 *   - residual, shaped distribution .... the reference's exact unit cases; brute-force enumeration
 *   - penalties ........................ the reference's unit vectors (attenuated once per distinct id,
 *                                        divide / multiply by sign, presence once, frequency per
 *                                        occurrence, both additive, prompt-only ids untouched, ids
 *                                        outside the domain skipped, position beyond the history)
 *   - greedy tree walk ................. the reference's unit case
 *   - mix / derive_step_value .......... the published splitmix64 output vectors (the reference
 *                                        only tests invariants; its mixer is that textbook routine)
 *   - rejection round .................. distributional law (first emitted token ~ target p,
 *                                        acceptance rate = sum min(p,q)) over thousands of seeds
 *   - Q6_K decode / encode ............. the reference's hand-packed superblock literal; round-trip
 *                                        bound, both scale signs, zero block
 *   - Q5_K decode ...................... ggml-produced bytes -> floats fixture (two superblocks), ==; dropping
 *                                        the fifth-bit run changes the values
 *   - YaRN table ....................... the reference's gpt-oss scalars -> mscale 1.3465736, untouched
 *                                        fast end, fully interpolated slow end, ramp between ggml's
 *                                        correction dimensions, swapped betas differ
 *   - swiglu_oai ....................... closed forms on both sides of every clamp, the (up + 1) term
 *   - gpt-oss layer graph .............. an independent float64 numpy forward (biases, sinks, window,
 *                                        YaRN, router bias, expert biases, clamped SwiGLU), 2e-4; each
 *                                        term's removal moves the logits
 *   - adaptive depth ................... the reference's unit scenarios, one by one
 *   - generation loop .................. greedy output == plain greedy decoding for any drafter, exact
 *                                        budget, stop tokens, context cap, a self-drafting target is
 *                                        always accepted, draw counter = 2 offered + 2 rounds - 1
 * PARITY UNPINNED (no golden value exists anywhere in the reference):
 *   - tso_tree_round_sampled: multi-branch rejection sampling on a tree is not
 *     defined by the reference at all; the definition here is this project's own
 *     (checked only against the chain round on chain-shaped trees and in law).  With penalties
 *     a node is shaped with the history of its own root path, the chain round's rule.
 *   - tso_quantize_mxfp4: the reference has no MXFP4 encoder; checked by brute force
 *     against "nearest codebook value under the tightest covering exponent".
 *   - tso_quantize_q5_k: the reference only decodes Q5_K; the encoder is Q4_K's min/max fitter with 31
 *     levels, checked by decode(encode(x)) within half a step.
 */
#ifndef TSORACLE_H
#define TSORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Weight storage types; values are the ggml type ids the reference's GGUF
 * intake uses, so a tensor description reads the same on both sides. */
enum {
    TSO_F32 = 0,
    TSO_F16 = 1,
    TSO_Q8_0 = 8,
    TSO_Q4_K = 12,
    TSO_Q5_K = 13, /* 176 B / 256 elems: Q4_K's header, 32 bytes of fifth bits, 128 nibble bytes */
    TSO_Q6_K = 14, /* 210 B / 256 elems: 4 low bits + 2 high bits per element, 16 signed int8 scales, f16 d */
    TSO_BF16 = 30,
    TSO_MXFP4 = 39,
};

/* ---- scalar conversions ------------------------------------------------ */
uint16_t tso_f32_to_f16(float x);   /* IEEE round-to-nearest-even, as the `half` crate */
float tso_f16_to_f32(uint16_t h);
uint16_t tso_f32_to_bf16(float x);  /* crates/compute/src/quant.rs:28-39 */
float tso_bf16_to_f32(uint16_t b);  /* crates/compute/src/quant.rs:14-17 */

/* ---- block formats ----------------------------------------------------- */
int64_t tso_row_bytes(int dtype, int64_t n);
void tso_quantize_q8_0(const float* row, int64_t n, uint8_t* out);
void tso_dequantize_q8_0(const uint8_t* blocks, int64_t n, float* out);
void tso_quantize_q4_k(const float* row, int64_t n, uint8_t* out);
void tso_dequantize_q4_k(const uint8_t* blocks, int64_t n, float* out);
void tso_q4_k_scale_min(int j, const uint8_t* packed12, uint8_t* sc, uint8_t* mn);
/* crates/compute/src/quant_gguf/q6_k.rs:44-88 (decode), :101-194 (largest-magnitude encoder) */
void tso_dequantize_q5_k(const uint8_t* blocks, int64_t n, float* out); /* crates/compute/src/quant_gguf/q5_k.rs:47-96 */
void tso_quantize_q5_k(const float* row, int64_t n, uint8_t* out);      /* not in the reference: Q4_K's fitter, 31 levels */
void tso_dequantize_q6_k(const uint8_t* blocks, int64_t n, float* out);
void tso_quantize_q6_k(const float* row, int64_t n, uint8_t* out);
float tso_mxfp4_scale(uint8_t e);
void tso_dequantize_mxfp4(const uint8_t* blocks, int64_t n, float* out);
void tso_quantize_mxfp4(const float* row, int64_t n, uint8_t* out); /* ours: reference has no encoder */
void tso_dequantize_row(int dtype, const uint8_t* row, int64_t n, float* out);
/* y[r] = sum_k dequant(W[r,:])[k] * x[k], sequential fp32 sum (q4_k.rs:207-220). */
void tso_gemv(int dtype, const uint8_t* w, int64_t rows, int64_t cols, const float* x, float* y);

/* ---- ops --------------------------------------------------------------- */
void tso_rms_norm(const float* x, const float* w, int64_t n, float eps, float* y);
void tso_rope_neox(float* x, int num_tokens, int num_heads, int head_dim, int rotated_pairs,
                   int64_t position, float theta);
void tso_rope_neox_freqs(float* x, int num_tokens, int num_heads, int head_dim, int rotated_pairs,
                         int64_t position, const float* freqs);
int tso_llama3_rope_factors(int rotary_dim, double base, double factor, double low_freq_factor,
                            double high_freq_factor, double original_context, float* out);
void tso_rope_frequencies_with_factors(int rotary_dim, float base, const float* factors, float* out);
/* crates/compute/src/rope.rs:324-372 (YaRN): per-pair frequencies and the magnitude scale. */
void tso_yarn_frequencies(int rotary_dim, float base, float factor, int64_t original_context,
                          float beta_fast, float beta_slow, float* freqs, float* mscale);
/* The table rotation with a magnitude scale on cos and sin (crates/runtime/src/families/gptoss/
 * attn.rs:104-118 binds crates/gpu's rope_neox_freqs with state.rope_mscale). */
void tso_rope_neox_freqs_scaled(float* x, int num_tokens, int num_heads, int head_dim,
                                int rotated_pairs, int64_t position, const float* freqs, float mscale);
/* crates/gpu/src/shaders/moe_gguf.metal:528-556 (ggml's swiglu_oai). */
float tso_swiglu_oai(float gate, float up, float alpha, float limit);
/* window <= 0: full; sinks NULL: none; scale <= 0: 1/sqrt(head_dim). */
void tso_causal_attention(const float* q, const float* k, const float* v, int head_dim, int nq,
                          int nkv, int64_t seq_len, int64_t window, float scale, const float* sinks,
                          float* out);
void tso_attention_core(const float* q, const float* k, const float* v, int head_dim, int nq,
                        int nkv, int64_t kv_start, int64_t prefix_end, const int64_t* extra,
                        int n_extra, float scale, const float* sinks, float* out);
float tso_silu(float x);

/* ---- TurboQuant KV-cache codec (tq.cpp; crates/compute/src/kv_quant.rs, kv_quant_attention.rs, wht.rs) ---- */
void tso_tq_sign_vector(int dim, uint64_t seed, float* out);                        /* kv_quant.rs:68-81 */
void tso_tq_wht(const float* x, int n, float* y);                                   /* wht.rs:5-29, normalized */
void tso_tq_rht_forward(const float* x, const float* signs, int n, float* y);       /* kv_quant.rs:90-94 */
void tso_tq_rht_inverse(const float* x, const float* signs, int n, float* y);       /* kv_quant.rs:102-107 */
int tso_tq_codebook(int dim, int bits, float* out);                                 /* kv_quant.rs:166-256 */
void tso_tq_midpoints(const float* codebook, int levels, float* out);               /* kv_quant.rs:262-264 */
int tso_tq_packed_words(int length, int bits);                                      /* kv_quant.rs:276-282 */
int tso_tq_pack(const uint32_t* indices, int length, int bits, uint32_t* packed);   /* kv_quant.rs:289-312; -1: refused */
int tso_tq_unpack(const uint32_t* packed, int bits, int length, uint32_t* indices); /* kv_quant.rs:315-334 */
void tso_tq_quantize_row(const float* x, int dim, const float* signs, const float* midpoints, int bits, float* norm_out,
                         uint32_t* words);                                           /* kv_quant.rs:349-362 */
void tso_tq_dequantize_row(float norm, const uint32_t* words, const float* signs, const float* codebook, int bits, int dim,
                           float* out);                                              /* kv_quant.rs:367-379 */
void tso_tq_roundtrip_rows(const float* x, int64_t n, int dim, const float* signs, const float* codebook, const float* midpoints,
                           int bits, float* out);                                    /* dequantize(quantize(row)), n rows */
void tso_tq_attention(const float* q, const uint32_t* k_words, const float* k_norms, const uint32_t* v_words,
                      const float* v_norms, int hd, int nq, int nkv, int seq_len, float scale, const float* sinks,
                      const float* k_signs, const float* k_codebook, const float* v_signs, const float* v_codebook, int k_bits,
                      int v_bits, float* out);                                                   /* kv_quant_attention.rs:58-136 */

/* ---- selection --------------------------------------------------------- */
typedef struct {
    double temperature;
    uint32_t top_k;
    int32_t has_top_p;
    double top_p;
    double repetition_penalty;
    int32_t has_seed; /* benchmarks always pass a seed; 0 here is refused */
    uint64_t seed;
    double presence_penalty;
    double frequency_penalty;
    int32_t has_min_p;
    double min_p;
} tso_shaping;

uint64_t tso_mix(uint64_t x);
uint64_t tso_derive_step_value(uint64_t seed, uint64_t position);
double tso_to_unit_interval(uint64_t v);
/* Returns 0 on success, <0 on the reference's refusals (empty domain, non-finite). */
int tso_select(const uint16_t* logits, int64_t vocab, const tso_shaping* cfg, const int32_t* history,
               int64_t n_history, uint64_t position, int32_t* out_token);
/* support/probs must hold `vocab` entries. */
int tso_shaped_distribution(const uint16_t* logits, int64_t vocab, const tso_shaping* cfg,
                            const int32_t* history, int64_t n_history, uint64_t position,
                            uint32_t* support, double* probs, int64_t* n_out);
double tso_dist_probability(const uint32_t* support, const double* probs, int64_t n, uint32_t token);
uint32_t tso_dist_draw(const uint32_t* support, const double* probs, int64_t n, uint64_t seed,
                       uint64_t position);
/* Returns 1 and fills out (capacity np) when mass survives, 0 for the None case. */
int tso_residual(const uint32_t* ps, const double* pp, int64_t np, const uint32_t* qs,
                 const double* qp, int64_t nq, uint32_t* out_support, double* out_probs,
                 int64_t* n_out);

/* ---- one speculative round's host half -------------------------------- */
typedef struct {
    int32_t accepted;       /* proposals accepted this round */
    int32_t committed;      /* tokens pushed to history this round (excludes a stopping token) */
    int32_t next;           /* corrected / bonus token; -1 when the round stopped */
    int32_t stopped;        /* 0 none, 1 stop token, 2 budget */
    uint64_t draw_step;     /* counter after the round */
    int32_t path[17];       /* tree rounds: accepted slots, path[0] = 0 */
    int32_t path_len;
} tso_round_result;

/* Draft half of a sampled chain round (speculative.rs:606-660): draws k proposals,
 * one from each row of draft_logits, then advances draw_step once more for the
 * row-only step.  Greedy: argmax per row, draw_step untouched. */
int tso_draft_chain(const uint16_t* draft_logits, int k, int64_t vocab, const tso_shaping* cfg,
                    const int32_t* history, int64_t n_history, uint64_t generated,
                    uint64_t* draw_step, int32_t* proposals);
/* Acceptance + bonus (speculative.rs:694-754, 861-879).  target_logits is (k+1) x vocab.
 * stop_tokens may be NULL.  max_new_tokens bounds `generated` as the sink does. */
int tso_chain_round(const uint16_t* target_logits, const uint16_t* draft_logits,
                    const int32_t* proposals, int k, int64_t vocab, const tso_shaping* cfg,
                    const int32_t* history, int64_t n_history, uint64_t generated,
                    uint64_t max_new_tokens, const int32_t* stop_tokens, int n_stop,
                    uint64_t draw_step, tso_round_result* out);
/* Greedy tree walk (speculative.rs:494-550); parent[] are SLOT parents, parent[0] = -1. */
int tso_tree_round_greedy(const uint16_t* target_logits, const int32_t* feed, const int32_t* parent,
                          int m, int64_t vocab, const tso_shaping* cfg, const int32_t* history,
                          int64_t n_history, uint64_t generated, uint64_t max_new_tokens,
                          const int32_t* stop_tokens, int n_stop, tso_round_result* out);
/* Multi-branch rejection on a tree.  NOT IN THE REFERENCE -- this project's definition:
 * at each accepted node, children are tried in slot order; child c (token x, drawn from
 * the drafter row q of its parent) is accepted iff r*q(x) <= p(x) with a fresh uniform;
 * on rejection p <- normalise(max(p - q, 0)) and the next sibling is tried; when all
 * siblings are rejected (or there are none) the next token is drawn from the current p.
 * draft_logits is m x vocab: row s is the drafter distribution the children of slot s
 * were drawn from. */
int tso_tree_round_sampled(const uint16_t* target_logits, const uint16_t* draft_logits,
                           const int32_t* feed, const int32_t* parent, int m, int64_t vocab,
                           const tso_shaping* cfg, const int32_t* history, int64_t n_history,
                           uint64_t generated, uint64_t draw_step, tso_round_result* out);

/* ---- adaptive depth and the generation loop ---------------------------------------- */
/* crates/runtime/src/speculative_adaptive.rs:105-227; params = {climb_low, climb_mid, climb_high, drop} */
typedef struct {
    int floor, cap, cur, climb, pressure;
    int params[4];
} tso_adaptive;
void tso_adaptive_new(tso_adaptive* a, int floor, int cap);
void tso_adaptive_observe(tso_adaptive* a, int offered, int accepted);
int tso_adaptive_tile_cap(int cap, int tile_rows); /* tile_rows <= 0: None */

/* The producer traits of crates/runtime/src/producer.rs:17-387 as callbacks (non-zero = error). */
typedef struct {
    void* user;
    int (*reset)(void* user);
    int (*produce)(void* user, int32_t token, int64_t position, uint16_t* logits);
    int (*prefill)(void* user, int32_t token, int64_t position); /* produce_prefill: no logits */
    int (*verify)(void* user, const int32_t* feed, int m, int64_t base, uint16_t* logits);
    int (*rollback_retaining)(void* user, int64_t point, int keep_rows);
    int (*prime)(void* user, int32_t next_token, int64_t position);
    int (*step)(void* user, int32_t token, int64_t position, uint16_t* logits);
    int (*rewind)(void* user, int64_t position);
    /* Tree rounds (producer.rs:253-294), all NULL / 0 for a producer that verifies chains only.
     * tree_nodes: nodes per tree round; draft_tree fills node_parent[i] (the node index under which
     * node i hangs, -1 for a child of the anchor; parents before children) and tokens[i];
     * verify_tree takes slot parents (slot 0 = the anchor, node i at slot i + 1); compact_tree moves
     * the accepted path's slots to rows 0 .. n. */
    int tree_nodes;
    int (*draft_tree)(void* user, int32_t anchor, int64_t base, int nodes, int32_t* node_parent, int32_t* tokens);
    int (*verify_tree)(void* user, const int32_t* feed, const int32_t* parent, int m, int64_t base, uint16_t* logits);
    int (*compact_tree)(void* user, int64_t base, const uint32_t* path, int n);
} tso_producer;
typedef struct {
    tso_shaping shaping;
    uint64_t max_new_tokens;
    const int32_t* stop_tokens;
    int32_t n_stop;
    int32_t block, adaptive_floor; /* adaptive_floor 0: fixed block */
} tso_generation;
typedef struct {
    int32_t* tokens; /* caller's buffer, >= max_new_tokens */
    int64_t n_tokens;
    int32_t stop_reason, final_depth; /* 1 stop token, 2 budget */
    int64_t rounds, offered, accepted, rollbacks;
    uint64_t draw_step;
} tso_generation_result;
/* crates/runtime/src/speculative.rs:194-900 for the step-wise drafter: chain rounds, and greedy tree
 * rounds (:467-575) when the producer drafts trees of `block` nodes and the depth is fixed. */
int tso_run_speculative(const tso_producer* p, const int32_t* prompt, int64_t n_prompt,
                        const tso_generation* g, int64_t max_context, int64_t vocab,
                        tso_generation_result* out);

/* ---- Llama-style target model ------------------------------------------ */
typedef struct {
    const void* data; /* row-major, one byte run per output row */
    int32_t dtype;
    int64_t rows, cols;
} tso_tensor;

typedef struct {
    tso_tensor attn_norm, wq, wk, wv, wo, q_norm, k_norm; /* q_norm/k_norm data NULL when absent */
    tso_tensor ffn_norm, w_gate, w_up, w_down;
    /* routed experts instead of the dense FFN when n_experts > 0: router n_experts x hidden;
     * we_gate / we_up (n_experts * ffn) x hidden, we_down (n_experts * hidden) x ffn, stacked */
    int32_t n_experts, top_k;
    tso_tensor router, we_gate, we_up, we_down;
    /* gpt-oss additions (families/gptoss/mod.rs:11-23); every data pointer may be NULL:
     * projection biases added before the rotation (attn.rs:88-101) / after the output projection,
     * one attention sink per q head, router bias added before the top-k (moe.rs:82-87), per-expert
     * biases n_experts x ffn (gate, up; added before the activation) and n_experts x hidden (down).
     * window > 0: the row sees only the last `window` positions of its sequence. */
    tso_tensor bq, bk, bv, bo, sinks, router_bias, be_gate, be_up, be_down;
    int32_t window;
} tso_layer;

typedef struct {
    int32_t n_layers, hidden, n_q_heads, n_kv_heads, head_dim, ffn, vocab, max_context;
    float rms_eps, rope_theta, attn_scale; /* attn_scale <= 0: 1/sqrt(head_dim) */
    const float* rope_factors;             /* NULL or head_dim/2 per-pair divisors */
    int32_t round_kv_f16;                  /* store K,V through fp16 (the engine's cache dtype) */
    int32_t threads;                       /* OpenMP threads for the row loops; 1 = scalar reference */
    tso_tensor embed, final_norm, lm_head; /* lm_head.data NULL => tied to embed */
    const tso_layer* layers;
    const float* rope_freqs; /* NULL, or head_dim/2 explicit per-pair frequencies (YaRN table) */
    float rope_mscale;       /* multiplies cos and sin; <= 0 means 1 */
    float act_alpha, act_limit; /* act_alpha > 0: gpt-oss clamped SwiGLU instead of silu(g) * u */
    /* TurboQuant KV (crates/model-io/src/kv_quant.rs:25-40,102-107): bits per key / value coordinate,
     * 0 = fp16 rows.  Quantized are the full-attention layers (window == 0), all of them in a stack of
     * at most two layers, else all but the last.  A quantized layer's row goes through fp16 (the staging
     * row of crates/runtime/src/kv_write.rs:66-118), is quantized per head, and every later read sees
     * the decoded row. */
    int32_t kv_k_bits, kv_v_bits;
} tso_model_desc;

typedef struct tso_model tso_model;
/* Smallest distance, over every routing decision of the last verify call, between the last
 * selected and the first rejected router logit, relative to the row's logit range: a caller
 * comparing against an implementation with different rounding can see that no choice was close. */
float tso_model_route_margin(const tso_model* m);
/* The routing of the last verify call: sel [n_layers][16][8] expert ids in rank order (-1 past
 * top_k), gap [n_layers][16] the relative gap between the last chosen and the first rejected router
 * logit (real_forward_dispatch.rs:1135-1158 ranks by logit, ties to the lower index).  -1: no routed
 * layer has run. */
int tso_model_route_record(const tso_model* m, int32_t* sel, float* gap);
/* Test hook: expert ids to take in place of the top-k ([n_layers][16][8], n values; n = 0 restores
 * the ranking).  The weights remain the softmax of the row's own logits over the forced experts: how
 * the logits come out had the router decided a near tie the other way. */
void tso_model_force_route(tso_model* m, const int32_t* sel, int64_t n);
tso_model* tso_model_create(const tso_model_desc* desc);
void tso_model_destroy(tso_model* m);
void tso_model_reset(tso_model* m);
int64_t tso_model_position(const tso_model* m);
void tso_model_rewind_to(tso_model* m, int64_t position); /* kv_cache_rewind.rs:46-55 */
/* Raw access to the fp32 KV store of one layer: [position][kv_head][head_dim]. */
float* tso_model_k(tso_model* m, int layer);
float* tso_model_v(tso_model* m, int layer);
/* 1 when the layer's rows are kept quantized (the rule above). */
int tso_model_layer_quantized(const tso_model* m, int layer);
/* One batched pass over `m_rows` fed tokens at base (batched.rs:92-456 semantics for a
 * pure-attention target).  parent NULL => chain (row i at position base+i, sees [0, base+i]).
 * parent given => tree (row s rotated at base+depth[s], sees [0,base) + its root path; K/V of
 * slot s stored at cache position base+s).  logits_f16 (m_rows x vocab) and logits_f32 are
 * both optional; with neither, the pass stops after the last layer (produce_prefill, producer.rs:92-103).  n_layers_run < 0 => all layers (a positive value runs a prefix of the
 * stack and then the head; used only to bound the timed CPU baseline sample).
 * Advances the cursor by m_rows. */
int tso_model_verify(tso_model* m, const int32_t* feed, const int32_t* parent, int m_rows,
                     int64_t base, uint16_t* logits_f16, float* logits_f32, int n_layers_run);
/* Row `row` of the last pass's residual stream after the last layer -- what the final norm consumes
 * (hidden floats).  -1: the last pass had no such row. */
int tso_model_last_hidden(const tso_model* m, int row, float* out);

/* The drafter head that predicts one token further from the trunk's own state (docs/MTP.md:53-60,
 * crates/runtime/src/families/qwen/mtp.rs): `head` is a model of ONE decoder layer whose final_norm is
 * the head's own norm, whose embed / lm_head are the trunk's, and whose cache is the head's own. */
typedef struct {
    tso_tensor fc;                          /* hidden x (2 * hidden) */
    tso_tensor norm_embedding, norm_hidden; /* the norms of fc's two input halves */
    tso_tensor trunk_norm;                  /* the TRUNK's final norm: h goes through it first */
} tso_mtp_desc;
/* m_rows steps at positions position .. position + m_rows - 1 (mtp.rs:146-400 batches them over a
 * prompt; one row is mtp_step, :441-700): row r pairs next_tokens[r] -- the token at position + r + 1 --
 * with h_rows[r], the residual-stream row of position + r (the trunk's, or for a chained step the
 * head's own from the step before).  Both logits outputs NULL = a priming step: the cache rows alone
 * (mtp_prime_step, :110-116).  x0_out (nullable): fc's output rows.  The head's residual after the
 * block is then tso_model_last_hidden(head, r).  Advances the head's cursor by m_rows. */
int tso_mtp_step(tso_model* head, const tso_mtp_desc* mtp, const int32_t* next_tokens, const float* h_rows,
                 int m_rows, int64_t position, uint16_t* logits_f16, float* logits_f32, float* x0_out);
/* Tree compaction (families/qwen/dflash_tree.rs:106-207): move the K/V rows of slots
 * path[0..n) to cache positions base..base+n. */
void tso_model_compact_tree(tso_model* m, int64_t base, const uint32_t* path, int n);

const char* tso_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
