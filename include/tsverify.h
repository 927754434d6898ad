/*
 * tsverify.h -- C ABI of the MI355X speculative-decoding verify engine.
 *
 * One handle (tsv_ctx) is one target model resident in HBM plus its fp16 KV cache:
 * the drop-in for the reference's `SpeculativeProducer` on a pure-attention target
 * (crates/runtime/src/producer.rs:164-387).  Each entry point names the trait method
 * (or reference function) it replaces.  Conventions are the reference's own outbound
 * C ABI conventions (crates/ffi/include/turbospark.h:10-34): int32 status (0 = OK),
 * a thread-local last-error string, borrowed const inputs, opaque handles, no
 * unwinding across the boundary, one generation at a time per handle.
 *
 * All pointers are plain host pointers unless a parameter says "device".
 */
#ifndef TSVERIFY_H
#define TSVERIFY_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TSV_MAX_ROWS 16 /* rows one verify pass takes (reference: MAX_BATCH_ROWS, crates/gpu/src/dequant_int4_batch.rs:50) */

/* Status codes. */
enum {
    TSV_OK = 0,
    TSV_ERR_INVALID = -1,     /* a refusal by name: bad argument, cursor mismatch, unsupported shaping */
    TSV_ERR_DEVICE = -2,      /* a HIP call failed */
    TSV_ERR_UNSUPPORTED = -3, /* a shape or dtype this build has no kernel for */
};

/* Weight storage types; the values are ggml type ids, as in the reference's GGUF intake. */
enum {
    TSV_F32 = 0,
    TSV_F16 = 1,
    TSV_Q8_0 = 8,  /* 34 B / 32 elems  (crates/compute/src/quant_gguf/q8_0.rs) */
    TSV_Q4_K = 12, /* 144 B / 256 elems (crates/compute/src/quant_gguf/q4_k.rs) */
    TSV_Q5_K = 13, /* 176 B / 256 elems: Q4_K's header, 32 bytes of fifth bits, 128 nibble bytes (q5_k.rs) */
    TSV_Q6_K = 14, /* 210 B / 256 elems (crates/compute/src/quant_gguf/q6_k.rs): the other half of a Q4_K_M file */
    TSV_BF16 = 30,
    TSV_MXFP4 = 39, /* 17 B / 32 elems: e8m0 scale + 32 e2m1 nibbles (crates/compute/src/quant_gguf_mxfp4.rs) */
};

/* A host tensor in GGUF layout: one byte run per output row, rows x cols elements. */
typedef struct {
    const void* data;
    int32_t dtype;
    int64_t rows, cols;
} tsv_tensor;

/* One decoder layer (crates/runtime/src/families/llama/{attn,dense}.rs).  q_norm/k_norm
 * (per-head RMSNorm, qwen3 style) have data == NULL when absent. */
typedef struct {
    tsv_tensor attn_norm, wq, wk, wv, wo, q_norm, k_norm;
    tsv_tensor ffn_norm, w_gate, w_up, w_down;
    /* Routed experts in place of the dense FFN (crates/runtime/src/families/llama/moe.rs; router
     * real_forward_dispatch.rs:1135-1158): n_experts == 0 means the dense matrices above are used.
     * router: n_experts x hidden.  we_gate / we_up: all experts' matrices stacked,
     * (n_experts * ffn) x hidden, expert e owning rows [e * ffn, (e + 1) * ffn); we_down:
     * (n_experts * hidden) x ffn.  `ffn` of the model description is the expert width. */
    int32_t n_experts, top_k;
    tsv_tensor router, we_gate, we_up, we_down;
    /* gpt-oss layer additions (crates/runtime/src/families/gptoss/mod.rs:11-23); data == NULL when
     * absent.  bq/bk/bv: projection biases, added BEFORE the rotation (gptoss/attn.rs:88-101); bo:
     * output-projection bias; sinks: one attention sink logit per q head, joining the softmax
     * maximum and denominator only (crates/compute/src/attention.rs:29-137); router_bias:
     * n_experts values added to the router logits before the top-k (gptoss/moe.rs:82-87);
     * be_gate / be_up (n_experts x ffn, added before the activation) and be_down (n_experts x
     * hidden): per-expert biases (crates/gpu/src/shaders/moe_gguf.metal:592-600).  All f32 / f16 /
     * bf16 vectors.  window > 0: a row sees only the last `window` positions of its sequence
     * (gptoss/attn.rs:120-137); it must exceed TSV_MAX_ROWS. */
    tsv_tensor bq, bk, bv, bo, sinks, router_bias, be_gate, be_up, be_down;
    /* ring != 0 (window > 0 only): the layer keeps a ring of window + 2 * TSV_MAX_ROWS positions
     * (rounded to 16) instead of the whole context, position p in slot p % capacity -- the
     * reference's fp16 ring for sliding-window layers (crates/gpu/src/kv_cache.rs:122-131,360-378).
     * Rollbacks are then bounded by tsv_max_safe_rewind. */
    int32_t window, ring;
} tsv_layer;

typedef struct {
    int32_t n_layers, hidden, n_q_heads, n_kv_heads, head_dim, ffn, vocab, max_context;
    float rms_eps, rope_theta, attn_scale; /* attn_scale <= 0 means 1/sqrt(head_dim) */
    const float* rope_factors;             /* NULL, or head_dim/2 llama-3 per-pair divisors */
    tsv_tensor embed, final_norm, lm_head; /* lm_head.data NULL: tied to embed */
    const tsv_layer* layers;
    /* NULL, or head_dim/2 explicit per-pair rotation frequencies (a YaRN table from
     * tsv_yarn_frequencies; overrides rope_theta / rope_factors), and the magnitude scale that
     * multiplies cos and sin (<= 0 means 1): crates/compute/src/rope.rs:286-372. */
    const float* rope_freqs;
    float rope_mscale;
    /* act_alpha > 0 selects gpt-oss's clamped SwiGLU for the routed experts,
     * (min(g, limit) / (1 + exp(-alpha * min(g, limit)))) * (clamp(u, -limit, limit) + 1)
     * (crates/gpu/src/shaders/moe_gguf.metal:528-556), instead of silu(g) * u. */
    float act_alpha, act_limit;
    /* TurboQuant KV rows (crates/model-io/src/kv_quant.rs:25-72): bits per key and per value coordinate,
     * both 0 for fp16 rows everywhere; the pairs --kv-bits can name are 2/2, 3/3, 3/4 ("3.5") and 4/4.
     * Quantized are the full-attention layers (window == 0), all of them in a stack of at most two, else
     * all but the last (kv_quant.rs:102-107); such a layer keeps one f32 norm and the packed codebook
     * indices per position and kv head, 4 + 4 * ceil(head_dim * bits / 32) bytes (kv_quant.rs:141-144; the
     * value side at 3 bits takes 4 + head_dim / 2 bytes here, its indices being kept 16 positions to 64 bits). */
    int32_t kv_k_bits, kv_v_bits;
    /* --session-slots (crates/runtime/src/session_pool.rs; RealForwardRunner::open_with_session_slots,
     * real_forward_api.rs:526-556): how many conversations' KV state the handle keeps, the live one included.
     * 0 or 1: none parked.  With n > 1, n - 1 further sets of KV buffers are allocated at open; tsv_reset then
     * parks the live conversation (promoting the least recently used slot) instead of overwriting it, and
     * tsv_try_reuse_prefix first swaps in the parked conversation that continues the prompt furthest, if it
     * beats the live one.  A swap exchanges buffer pointers, never rows. */
    int32_t session_slots;
} tsv_model_desc;

typedef struct tsv_ctx tsv_ctx;

/* Shaping configuration: crates/selection/src/shaping.rs:44-123 (`ShapingConfig`). */
typedef struct {
    double temperature;
    uint32_t top_k;
    int32_t has_top_p;
    double top_p;
    double repetition_penalty;
    int32_t has_seed;
    uint64_t seed;
    double presence_penalty;
    double frequency_penalty;
    int32_t has_min_p;
    double min_p;
} tsv_shaping;

/* A rollback point: `SpeculativeProducer::Checkpoint` (real_forward_rollback.rs:19-28)
 * for a target with no recurrent state. */
typedef struct {
    int64_t position;
} tsv_point;

/* One round handed to the fused entry point. */
typedef struct {
    const int32_t* feed;   /* feed[0] = the confirmed token, feed[1..m) = proposals / tree nodes */
    const int32_t* parent; /* NULL: chain.  Else slot parents, parent[0] = -1, parent[s] < s */
    int32_t m;             /* rows, 1..TSV_MAX_ROWS */
    int64_t base;          /* position of feed[0]; must equal the KV cursor */
    tsv_shaping shaping;
    /* Drafter logits, fp16, host or device memory.  Chain: (m-1) x vocab, row i is the
     * distribution proposal i was drawn from.  Tree: m x vocab, row s is the distribution
     * the children of slot s were drawn from.  NULL at temperature 0. */
    const uint16_t* draft_logits;
    uint64_t draw_step; /* the loop's monotone uniform counter (speculative.rs:396-402) */
    const int32_t* stop_tokens;
    int32_t n_stop;
    uint64_t generated;      /* tokens reported so far (TokenSink::generated) */
    uint64_t max_new_tokens; /* budget; 0 = unbounded */
    uint16_t* logits_out;    /* optional: m x vocab fp16 copy of the verify logits */
    /* TokenSink::history when the round starts (prompt + every reported token, feed[0] last), host
     * memory; read only when a repetition / presence / frequency penalty is set at temperature > 0
     * (crates/selection/src/penalty.rs:15-82).  Its last min(generated, n_history) tokens are the
     * generated suffix the presence / frequency penalties count over (choose.rs:138-154). */
    const int32_t* history;
    int64_t n_history;
} tsv_round;

typedef struct {
    int32_t accepted;  /* proposals (tree: nodes) accepted */
    int32_t committed; /* tokens pushed to history (a stopping token is counted, not pushed) */
    int32_t next;      /* corrected / bonus token, -1 if the round stopped */
    int32_t stopped;   /* 0 no, 1 stop token, 2 budget */
    uint64_t draw_step;
    int32_t path[TSV_MAX_ROWS + 1]; /* accepted slots, path[0] = 0 (chain: 0,1,..,accepted) */
    int32_t path_len;
    int64_t kv_position; /* KV cursor after truncation: base + committed + 1 */
    /* Smallest relative distance of any f64 comparison this round (acceptance tests and
     * the cumulative draw) from flipping; decisions are bit-stable against host libm /
     * summation-order differences while this is >> 1e-12. */
    double min_margin;
} tsv_round_result;

/* ---- lifetime ------------------------------------------------------------- */
/* Uploads and re-tiles the weights, allocates the KV cache.  Replaces
 * `RealForwardRunner::open` for the scope of this path. */
int32_t tsv_open(const tsv_model_desc* desc, tsv_ctx** out);
void tsv_close(tsv_ctx* ctx);
/* Copies the calling thread's last error text (NUL-terminated) into buf; returns its length. */
int32_t tsv_last_error(char* buf, int32_t cap);
/* The HIP stream every kernel of this handle is launched on (a hipStream_t). */
void* tsv_stream(tsv_ctx* ctx);

/* ---- LogitProducer (producer.rs:17-104) ------------------------------------ */
int32_t tsv_reset(tsv_ctx* ctx);               /* LogitProducer::reset (with a session pool: real_forward_traits.rs:12-31) */
/* What KV rows cost, on the host and without a handle (crates/model-io/src/kv_quant.rs:146-205 kv_layer_strides;
 * context_policy.rs:294-333 kv_bytes_for_context_with): bytes one position costs in one layer, K side and V side
 * -- fp16 rows, or a norm and packed indices per kv head on the layers kv_k_bits / kv_v_bits quantize -- and the
 * bytes one conversation's KV state takes at `context` positions (a ring layer stops growing at its capacity;
 * a session pool multiplies it by session_slots).  -1 / an error code on a bad description. */
int32_t tsv_kv_row_bytes(const tsv_model_desc* desc, int32_t layer, int64_t* k_bytes, int64_t* v_bytes);
int64_t tsv_kv_bytes_for_context(const tsv_model_desc* desc, int64_t context);
int32_t tsv_session_pool_size(const tsv_ctx* ctx);    /* RealForwardRunner::session_pool_size: parked slots + 1 */
int32_t tsv_session_slot_evicted(const tsv_ctx* ctx); /* 1: the last tsv_reset overwrote a parked conversation */
/* 1: the last tsv_try_reuse_prefix swapped a parked conversation in.  A caller that keeps state of its own beside
 * the handle's (a drafter's context) must not treat such a reuse as a continuation of what it holds
 * (real_forward_traits.rs:199-239: "nothing rewound, nothing swapped"); tsv_run_speculative starts over then. */
int32_t tsv_session_swapped(const tsv_ctx* ctx);
/* The pool's two selection rules on their own (host only; session_pool.rs:116-129): the index of the highest of n
 * common-prefix scores and that score (-1 and 0 when n == 0 or every score is zero), and the index of the smallest
 * of n parking ticks (-1 when n == 0). */
int64_t tsv_session_best_match(const int64_t* scores, int64_t n, int64_t* score_out);
int64_t tsv_session_lru(const uint64_t* ticks, int64_t n);
int64_t tsv_kv_position(const tsv_ctx* ctx);   /* kv.position() */
/* KvCacheManager::max_safe_rewind (crates/gpu/src/kv_cache_rewind.rs:26-35): how many rows a rollback
 * may drop and still leave every ring layer's window intact: the smallest capacity - window over the
 * layers opened with `ring`; INT64_MAX when nothing rings (every layer stores position p at slot p).
 * tsv_rollback, tsv_rollback_retaining and tsv_try_reuse_prefix refuse by name (:46-55) a cursor that
 * would land more than this many rows behind the last row ever written. */
int64_t tsv_max_safe_rewind(const tsv_ctx* ctx);
/* LogitProducer::produce: one token at `position`; logits: vocab fp16. */
int32_t tsv_produce(tsv_ctx* ctx, int32_t token, int64_t position, uint16_t* logits);
/* produce_prefill / ChunkedPrefillRunner::prefill_chunk: feeds n tokens from pos0 in
 * passes of TSV_MAX_ROWS rows; logits (nullable) receives the LAST token's row.  Passes whose
 * logits nobody reads skip the final norm and the output head (producer.rs:92-103): every pass but
 * the last, and the last too when logits is NULL -- then no rows are left for tsv_accept. */
int32_t tsv_prefill(tsv_ctx* ctx, const int32_t* ids, int64_t n, int64_t pos0, uint16_t* logits);

/* ---- SpeculativeProducer (producer.rs:164-387) ------------------------------ */
int32_t tsv_checkpoint(tsv_ctx* ctx, tsv_point* out);              /* checkpoint() */
int32_t tsv_rollback(tsv_ctx* ctx, const tsv_point* point);        /* rollback() */
/* rollback_retaining(point, keep_rows): new KV length = point + keep_rows. */
int32_t tsv_rollback_retaining(tsv_ctx* ctx, const tsv_point* point, int32_t keep_rows);
int32_t tsv_commit_pending(tsv_ctx* ctx, int32_t keep_rows); /* no-op without recurrent state */
int32_t tsv_discard_pending(tsv_ctx* ctx);

/* ---- what the KV rows were built from (crates/runtime/src/kv_prefix.rs:49-137) ---------
 * The record on its own: pure host state, no GPU.  fed[0..len) are the token ids behind positions
 * [0, len); a state that took in anything the ids do not describe is tainted until cleared. */
typedef struct tsv_prefix tsv_prefix;
tsv_prefix* tsv_prefix_new(void);
void tsv_prefix_free(tsv_prefix* p);
void tsv_prefix_clear(tsv_prefix* p);                                     /* clear() :60-63 */
void tsv_prefix_taint(tsv_prefix* p);                                     /* taint() :68-70 */
/* record(tokens, pos0) :79-92: starting inside the record replaces its tail, past its end taints. */
void tsv_prefix_record(tsv_prefix* p, const int32_t* tokens, int64_t n, int64_t pos0);
void tsv_prefix_rewind_to(tsv_prefix* p, int64_t position);               /* rewind_to() :96-100 */
int64_t tsv_prefix_untainted_len(const tsv_prefix* p);                    /* untainted_len() :104-106; -1 = None */
/* common_prefix(prompt) :129-137: longest common prefix, at most n - 1 (one token is always left to feed). */
int64_t tsv_prefix_common(const tsv_prefix* p, const int32_t* prompt, int64_t n);

/* The same record behind a handle.  It is written where tokens are fed: tsv_produce and
 * tsv_prefill on success (real_forward_traits.rs:135-152, :395-402; a failed pass taints),
 * tsv_record_committed after a verify round; tsv_reset clears it, the rollbacks and the fused
 * round's truncation shorten it, tsv_write_kv taints it (rows no ids describe).
 * RealForwardRunner::set_prefix_reuse: reuse answers 0 until the host opts in. */
int32_t tsv_set_prefix_reuse(tsv_ctx* ctx, int32_t on);
/* LogitProducer::try_reuse_prefix (producer.rs:24-47, real_forward_traits.rs:173-289): commits to
 * continuing from the current state for the leading N tokens of the prompt and returns N (0: no
 * reuse, the caller resets; < 0: error).  A cursor that runs past the agreed prefix is moved back
 * to it, within tsv_max_safe_rewind.  With a session pool the best-matching parked conversation is swapped in
 * first (select_session, :655-673), and a rewind deeper than the kept prefix on a live session nobody compared
 * favorably is refused (:283) so that the caller's reset parks that conversation instead of overwriting it. */
int64_t tsv_try_reuse_prefix(tsv_ctx* ctx, const int32_t* prompt, int64_t n);
/* SpeculativeProducer::record_committed(tokens, pos0) (producer.rs:322-330): the rows of a verify
 * pass that the round committed, `feed[..committed + 1]` at `base` (speculative.rs:828-836). */
int32_t tsv_record_committed(tsv_ctx* ctx, const int32_t* tokens, int64_t n, int64_t pos0);
/* Positions the handle's record describes; -1 when tainted. */
int64_t tsv_prefix_len(const tsv_ctx* ctx);
/* verify(feed, base, logits): m rows at base..base+m, row i sees [0, base+i].
 * logits nullable (m x vocab fp16): NULL keeps them on the device for tsv_accept. */
int32_t tsv_verify(tsv_ctx* ctx, const int32_t* feed, int32_t m, int64_t base, uint16_t* logits);
/* verify_tree(feed, parent, base, logits): row s rotated at base+depth[s], sees the
 * prefix plus its root path; K/V of slot s stored at cache position base+s. */
int32_t tsv_verify_tree(tsv_ctx* ctx, const int32_t* feed, const int32_t* parent, int32_t m,
                        int64_t base, uint16_t* logits);
/* compact_tree(base, path): gather the accepted path's K/V rows to base..base+n. */
int32_t tsv_compact_tree(tsv_ctx* ctx, int64_t base, const uint32_t* path, int32_t n);

/* ---- acceptance on the device ----------------------------------------------- */
/* The host half of a round (speculative.rs:694-754, 861-879; tree: 494-550) run as
 * kernels over the logits the last verify left on the device, followed by the KV
 * truncation (and, for a tree, compaction).  Uses round->{parent,m,base,shaping,
 * draft_logits,draw_step,stop_tokens,generated,max_new_tokens}; feed must be the feed
 * of that verify.  A tree at temperature > 0 runs multi-branch rejection (children in
 * slot order, r * q(x) <= p(x), residual max(p - q, 0) renormalised after a rejection);
 * the reference keeps tree rounds greedy (speculative.rs:390-392), so that mode has no
 * counterpart there, and it takes no stop tokens or budget.  m, base and the tree
 * (parent, or NULL for a chain) must be those of that verify: anything else is refused
 * as TSV_ERR_INVALID before a kernel runs. */
int32_t tsv_accept(tsv_ctx* ctx, const tsv_round* round, tsv_round_result* out);
/* verify + accept + truncate in one call: the whole verify step. */
int32_t tsv_verify_accept(tsv_ctx* ctx, const tsv_round* round, tsv_round_result* out);
/* The greedy round of tsv_accept for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Nothing
 * is allocated, copied from the host or waited for: the logits (m x vocab fp16) and the result are
 * DEVICE memory of the caller's, `stream` is the caller's hipStream_t (NULL: the default stream),
 * and the arg-max partial results live in a 4 KiB static device array that every GPU the library
 * runs on holds until the process ends.  Limits: 1..TSV_MAX_ROWS rows (more is refused by name),
 * at most 16 stop tokens.  There is no handle, so no KV truncation: result->kv_position = base +
 * committed + 1 is where the caller moves its cursor.  A non-finite logit is reported in band
 * (stopped = -1, next = -1, path_len = 0).  Calls on one GPU share that GPU's array: two calls that
 * overlap in time on one GPU race.  Under stream capture: the stream must be one of the caller's own (the
 * NULL stream cannot be captured), and the array's address must already be known on that GPU -- it is once
 * tsv_open has run there, or after one call of this entry point outside capture (the first call on a GPU asks
 * the runtime for the address, which is not a capturable operation). */
int32_t tsv_accept_greedy_noalloc(void* stream, const uint16_t* logits_dev, int32_t vocab, const int32_t* feed,
                                  const int32_t* parent, int32_t m, int64_t base, const int32_t* stop_tokens,
                                  int32_t n_stop, uint64_t generated, uint64_t max_new_tokens,
                                  tsv_round_result* result_dev);
/* Draft half of a sampled chain round (speculative.rs:606-660): draws k proposals, one
 * from each row of draft_logits (k x vocab fp16, host or device), advancing *draw_step by
 * k + 1; greedy: argmax per row. */
int32_t tsv_draft_chain(tsv_ctx* ctx, const uint16_t* draft_logits, int32_t k,
                        const tsv_shaping* shaping, uint64_t* draw_step, int32_t* proposals,
                        const int32_t* history, int64_t n_history, uint64_t generated);

/* ---- the generation loop (speculative.rs:194-900) and the adaptive depth ---------------- */
/* Per-round draft depth controller, speculative_adaptive.rs:105-227: pure state.  A streak of
 * fully accepted rounds (climb_low from depth 2-3, climb_mid from 4, climb_high from 5 up) climbs
 * one step, `drop` accumulated missed proposals fall one step; never below floor or above cap. */
typedef struct {
    int32_t floor, cap, cur, climb, pressure;
    int32_t climb_low, climb_mid, climb_high, drop;
} tsv_adaptive;
void tsv_adaptive_init(tsv_adaptive* a, int32_t floor, int32_t cap);       /* AdaptiveDepth::new, shipped tuning */
int32_t tsv_adaptive_depth(const tsv_adaptive* a);                          /* depth() */
void tsv_adaptive_observe(tsv_adaptive* a, int32_t offered, int32_t accepted); /* observe() */
int32_t tsv_adaptive_tile_cap(int32_t cap, int32_t tile_rows);              /* tile_cap(); tile_rows <= 0: none */

/* The draft side of SpeculativeProducer (producer.rs:164-260) as callbacks; non-zero = failure.
 * prime(next, position): write the drafter's row for a token whose proposal is not needed;
 * step(token, position, logits): the same and fill vocab fp16 logits (host memory);
 * rewind(position): the drafter continues after the accepted prefix that ended at `position`. */
typedef struct {
    void* user;
    int32_t (*prime)(void* user, int32_t next_token, int64_t position);
    int32_t (*step)(void* user, int32_t token, int64_t position, uint16_t* logits);
    int32_t (*rewind)(void* user, int64_t position);
    /* non-zero: `step` is handed DEVICE memory (a buffer of the loop's) and fills it on the GPU, finished
     * by the time it returns; the draws and the round then read the drafter's rows where they are.  No
     * counterpart in the reference, whose draft_step hands back host logits (producer.rs:196-204). */
    int32_t device_logits;
    /* optional (may be NULL): how many positions the drafter's own context covers.  The loop reuses
     * a prefix only when this is within one row of it (the drafter continuity guard of
     * real_forward_traits.rs:199-239); without it a run always starts from an empty state. */
    int64_t (*position)(void* user);
    /* optional (0 / NULL: chain rounds only): a drafter that offers TREES (producer.rs:253-274).
     * tree_nodes: nodes per tree round.  draft_tree(anchor, base, nodes, node_parent, tokens): a tree
     * anchored at `anchor` (the token at `base`), parents before children; node_parent[i] is the index
     * of the node under which node i hangs, -1 for a child of the anchor (DflashTreeNode::parent,
     * dflash_tree.rs:12-17), tokens[i] its token.  A round is a tree round when it is greedy, the
     * depth is fixed, nothing shortened it and tree_nodes == block (speculative.rs:386-392). */
    int32_t tree_nodes;
    int32_t (*draft_tree)(void* user, int32_t anchor, int64_t base, int32_t nodes, int32_t* node_parent, int32_t* tokens);
    /* optional (may be NULL): drafts_block_passes / draft_block (producer.rs:222-250, call site
     * speculative.rs:596-603).  draft_block(anchor, base, block, proposals): `block` proposals for positions
     * base + 1 .. base + block in ONE call, `anchor` being the token at `base`; the drafter keeps its own state
     * (no prime follows) and picks its own tokens.  A drafter that has it is asked for blocks in every greedy
     * round (the arg-max ignores penalties and truncation, crates/selection/src/choose.rs:84-88); sampled rounds
     * need the proposal distributions and go step by step, which a drafter without `step` refuses. */
    int32_t (*draft_block)(void* user, int32_t anchor, int64_t base, int32_t block, int32_t* proposals);
    /* optional (may be NULL): supports_chunked_drafter_prefill / prefill_chunk_priming_drafter
     * (producer.rs:193-211, call site speculative.rs:287-316).  prefill_chunk(tokens, n, start_position, logits,
     * next_token): the target's prefill of one prompt chunk, priming the drafter over every position whose next
     * token is known; next_token is the prompt token after the chunk, -1 when the chunk ends the prompt (that
     * last position is left for the first draft step).  logits (host, vocab fp16): the row after the chunk's
     * last token.  With it the loop hands the prompt to this callback instead of tsv_prefill + prime per token
     * (the loop prefills the whole prompt before it primes: a drafter whose prime reads the target's state of
     * the same position, as the head of tsv_mtp_open does, must offer this callback). */
    int32_t (*prefill_chunk)(void* user, const int32_t* tokens, int64_t n, int64_t start_position, uint16_t* logits,
                             int32_t next_token);
} tsv_drafter;

/* ---- a drafter inside the library: the head that predicts one token further from the target's own state ----
 * docs/MTP.md:53-60, crates/runtime/src/families/qwen/mtp.rs:
 *     x   = fc([ norm_embedding(embed(t_{i+1})) ; norm_hidden(target_final_norm(h_i)) ])     (embedding half first)
 *     x   = x + attn(attn_norm(x))      -- over the head's OWN cache, at position i
 *     x   = x + ffn(ffn_norm(x))
 *     out = target_lm_head(head_norm(x))
 * h_i is the target's residual stream at position i after its last layer (what its final norm consumes); a
 * chained step (depth > 1) feeds the head's own x of the step before in its place (mtp.rs:85-91).  The norms
 * are this family's plain RMSNorm (the reference's qwen3.5 head stores its norm weights as offsets from one,
 * docs/MTP.md:82-90: a caller with such a file adds the one before handing the vectors over).
 * `model`: n_layers == 1, that layer being the head's decoder block; final_norm the head's own norm; embed and
 * lm_head left empty (data NULL): the head uses the target's, where they already are on the device; widths,
 * head counts, vocabulary and rotation as the target's; max_context the positions the head's cache holds. */
typedef struct {
    tsv_model_desc model;
    tsv_tensor fc;                          /* hidden x (2 * hidden), any matmul storage type */
    tsv_tensor norm_embedding, norm_hidden; /* hidden-wide vectors */
} tsv_mtp_desc;
/* Opens the head on the target's device and stream and attaches it: from then on the target's prompt passes
 * keep their final residual rows for the head.  Close the head before the target. */
int32_t tsv_mtp_open(tsv_ctx* target, const tsv_mtp_desc* desc, tsv_ctx** head);
/* mtp_draft_step / mtp_prime_step (mtp.rs:92-116): the head's row at `position` (which must be where its cache
 * ends, mtp.rs:484-491) from next_token -- the token at position + 1 -- and the state at `position`: the
 * target's, when the target's last pass holds a row for that position and the head has not stepped since its
 * last rewind; else the head's own from the step before.  logits NULL: a priming step, cache row only.
 * Otherwise vocab fp16, host memory, or device memory when logits_on_device is non-zero. */
int32_t tsv_mtp_step(tsv_ctx* head, int32_t next_token, int64_t position, uint16_t* logits, int32_t logits_on_device);
/* mtp_rewind_to (mtp.rs:422-436): the head continues after the accepted prefix that ended at `position`. */
int32_t tsv_mtp_rewind(tsv_ctx* head, int64_t position);
/* prefill_chunk_priming_drafter for this head (real_forward_traits.rs:361-402, mtp_prime_rows_batched
 * mtp.rs:146-400): tsv_prefill of the target over the chunk, and after each pass the head's rows for every
 * position of it whose next token is known, sixteen at a time.  The head must stand at start_position. */
int32_t tsv_mtp_prefill_chunk(tsv_ctx* head, const int32_t* tokens, int64_t n, int64_t start_position, uint16_t* logits,
                              int32_t next_token);
/* `block` greedy proposals (1..15) chained on the device: the step at base - 1 from `anchor` and the target's
 * state, then each arg-max fed to the next step as a device-side token, no host round trip in between; ends
 * with the row-only step of the last proposal (speculative.rs:612-625), so the head stands at base + block. */
int32_t tsv_mtp_draft_block(tsv_ctx* head, int32_t anchor, int64_t base, int32_t block, int32_t* proposals);
/* Fills `out` with this head's callbacks (prime, step with device logits, rewind, position, draft_block,
 * prefill_chunk) for tsv_run_speculative on the target the head is attached to.  With these callbacks in place the
 * loop chains SAMPLED rounds on the device too: every step's row stays in the loop's device buffer (the proposal
 * distributions of the rejection test) and its proposal is drawn there, at the draw positions the step-by-step
 * walk would use -- same tokens, same counters, one host wait per block. */
int32_t tsv_mtp_drafter(tsv_ctx* head, tsv_drafter* out);

typedef struct {
    tsv_shaping shaping;
    uint64_t max_new_tokens;     /* GenerationConfig::max_new_tokens, > 0 */
    const int32_t* stop_tokens;  /* tokenizer stop ids + extra_stop_tokens */
    int32_t n_stop;
    int32_t block;               /* proposals per round (the cap when adaptive), 1..15 */
    int32_t adaptive_floor;      /* 0: fixed block; else AdaptiveDepth(adaptive_floor, block) */
} tsv_generation;

typedef struct {
    int32_t* tokens;   /* caller's buffer for the reported tokens */
    int64_t capacity;  /* >= max_new_tokens */
    int64_t n_tokens;
    int32_t stop_reason; /* 1 stop token (not reported), 2 budget (its last token is reported) */
    int32_t final_depth;
    int64_t rounds, offered, accepted, rollbacks;
    uint64_t draw_step;
    int64_t kv_position;
    double min_margin;
    int64_t reused;      /* leading prompt tokens taken over from the previous run's state */
} tsv_generation_result;

/* run_speculative for the step-wise drafter: chain rounds, and greedy tree rounds (speculative.rs:
 * 467-575: draft_tree -> verify_tree -> the walk -> compact_tree -> rollback_retaining, all of it but
 * the draft inside one tsv_verify_accept) for a drafter that offers trees: admission, prefix reuse or reset
 * (speculative.rs:240-251), headless prefill that primes the drafter, then rounds of draft ->
 * verify + accept + truncate on the device -> record_committed -> rewind_drafter, never proposing
 * past the budget or the context window (speculative.rs:448-459). */
int32_t tsv_run_speculative(tsv_ctx* ctx, const tsv_drafter* drafter, const int32_t* prompt, int64_t n_prompt,
                            const tsv_generation* config, tsv_generation_result* out);
/* Device address of the logits the last pass left on the GPU (rows x vocab fp16, valid until the next
 * pass of this handle, written on tsv_stream): lets a second handle be the drafter of a loop without a
 * host round trip. */
const uint16_t* tsv_device_logits(tsv_ctx* ctx);
int64_t tsv_max_context(const tsv_ctx* ctx);
int64_t tsv_vocab(const tsv_ctx* ctx);

/* ---- GGUF intake (host) -------------------------------------------------------- */
/* The header parser of crates/repack/src/gguf_header/parser.rs:124-239 over a read-only mapping of
 * the file: version 3 only, metadata keys and tensor names unique, at most four non-zero
 * dimensions, every offset a multiple of general.alignment (default 32, a power of two); the data
 * region starts at the aligned end of the tensor table.  Refusals are by name (tsv_last_error). */
typedef struct tsv_gguf tsv_gguf;
int32_t tsv_gguf_open(const char* path, tsv_gguf** out);
void tsv_gguf_close(tsv_gguf* g);
int64_t tsv_gguf_tensor_count(const tsv_gguf* g);
int64_t tsv_gguf_data_start(const tsv_gguf* g);
/* A tensor where it lies in the mapping (valid until tsv_gguf_close): dtype is the ggml type id,
 * cols the first dimension, rows the product of the others (stacked experts are expert-major row
 * runs); bounds-checked against the file. */
int32_t tsv_gguf_tensor(const tsv_gguf* g, const char* name, tsv_tensor* out);
int32_t tsv_gguf_meta_number(const tsv_gguf* g, const char* key, double* out);
int32_t tsv_gguf_meta_string(const tsv_gguf* g, const char* key, char* buf, int32_t cap);
/* Opens a llama-family GGUF as a verify target: tensor names of crates/repack/src/gguf_names/
 * llama.rs:14-60 (`llama`; `qwen2` adds the q / k / v biases; `qwen3` / `qwen3moe` the per-head
 * q / k norms; routed experts as the stacked *_exps tensors; `gpt-oss` by gguf_names/gpt_oss.rs:30-72
 * with its biases, sinks, YaRN keys and the window on even layers), sizes from the `<arch>.*` metadata,
 * the q / k rows of a `llama` file un-permuted from llama.cpp's adjacent-pair order
 * (crates/repack/src/gguf_checkpoint/conventions.rs:133-243).  rope_freqs.weight, which the
 * reference refuses for this family, is taken as the llama-3 per-pair divisors; any other context
 * extension (rope.scaling.type, but gpt-oss's yarn) and partial rotation are refused.  max_context <= 0: the file's
 * context_length.  The mapping is dropped before the call returns. */
int32_t tsv_open_gguf(const char* path, int32_t max_context, tsv_ctx** out);

/* ---- install-time helpers (host) --------------------------------------------- */
/* The reference's quantize-on-install encoders (q8_0.rs:56-77, q4_k.rs:126-204). */
int64_t tsv_row_bytes(int32_t dtype, int64_t cols);
/* yarn_frequencies (crates/compute/src/rope.rs:324-372): rotary_dim/2 per-pair frequencies and
 * the magnitude scale 1 + 0.1 ln(factor); factor <= 0 gives the unscaled table and scale 1. */
int32_t tsv_yarn_frequencies(int32_t rotary_dim, float base, float factor, int64_t original_context,
                             float beta_fast, float beta_slow, float* freqs, float* mscale);
int32_t tsv_quantize_rows(int32_t dtype, const float* src, int64_t rows, int64_t cols, void* dst);
/* Seeded synthetic tensor: rows x cols of N(0, sigma) from a counter-based generator
 * keyed by (seed, stream), quantized to dtype row by row (the random-init installs of
 * crates/repack/src/synthetic_*.rs).  dst holds rows * tsv_row_bytes(dtype, cols) bytes. */
int32_t tsv_synth_tensor(int32_t dtype, uint64_t seed, uint64_t stream, float sigma, int64_t rows,
                         int64_t cols, void* dst);

#ifdef __cplusplus
}
#endif
#endif
