/*
 * tsverify_testing.h -- test and measurement hooks of libtsverify.so.
 *
 * Nothing here belongs to the drop-in surface (include/tsverify.h maps the reference's producer
 * traits); these entry points exist for the parity tests and for bench.py: reading and writing the
 * KV cache and the logits directly, single kernels in isolation, per-kernel timing, and the routing
 * decisions of the last pass.  A host that embeds the library needs none of them.
 */
#ifndef TSVERIFY_TESTING_H
#define TSVERIFY_TESTING_H

#include "tsverify.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Copies layer `layer`'s K and V rows [pos0, pos0+n) to host as fp16 in the reference
 * layout [position][kv_head][head_dim] (crates/gpu/src/kv_cache.rs:1-10). */
int32_t tsv_read_kv(tsv_ctx* ctx, int32_t layer, int64_t pos0, int64_t n, uint16_t* k, uint16_t* v);
/* The inverse: stores n rows of K and V (same host layout) at cache positions [pos0, pos0+n) of
 * one layer and moves the cursor to at least pos0 + n -- a long context without the prefill that
 * would build it (the full-size parity cases; also how a saved prefix would be restored).  On a layer that
 * keeps quantized rows the rows are quantized on the way in, as the forward's own rows are. */
int32_t tsv_write_kv(tsv_ctx* ctx, int32_t layer, int64_t pos0, int64_t n, const uint16_t* k, const uint16_t* v);
/* Stores m x vocab fp16 logits (host memory) as if a verify pass of m rows at `base` had just left them on
 * the device: tsv_accept then judges exactly these scores (acceptance cases no model would produce: ties,
 * flat rows, the fp16 extremes).  The KV cache and the cursor are not touched. */
int32_t tsv_write_logits(tsv_ctx* ctx, const uint16_t* logits, int32_t m, int64_t base);
/* One quantized small-M matmul through the same kernels the forward uses:
 * y[m][r] = sum_k W[r][k] x[m][k]; x is m x cols fp32 (rounded to fp16 on entry), y is
 * m x rows fp32.  W host tensor in GGUF layout (re-tiled per call).  `splits` <= 0 picks
 * the engine's own split-K factor. */
int32_t tsv_matmul(const tsv_tensor* w, const float* x, int32_t m, float* y, int32_t splits);

/* Host arithmetic only: how many launches of the walk kernel a sampled tree round of this shape is given -- the most
 * child tests any walk through the tree can take (children are tested in slot order; a walk rejects all n children of
 * a node, or rejects j - 1, accepts the j-th and goes on below it).  -1 for a malformed tree. */
int32_t tsv_tree_walk_bound(const int32_t* parent, int32_t m);

/* The four measurement hooks below (tsv_set_profile, tsv_set_repeat, tsv_matmul_time, tsv_copy_time) answer only in
 * a process whose environment carries TSV_MEASUREMENT_HOOKS=1; anywhere else turning one on is refused by name
 * (TSV_ERR_UNSUPPORTED) and the library runs exactly its serving path. */
/* Per-kernel-class timing with HIP events on the handle's stream (one event pair per launch
 * while enabled).  Classes, in order: embed, norm, qkv matmul, rope+kv store, attention,
 * output projection, gate/up matmul, down matmul, output head, acceptance, and "event pair":
 * one pair per pass with nothing between the two events, i.e. what an event pair itself adds
 * to every other reading.  tsv_get_profile sums the elapsed milliseconds and launch counts
 * since the last call and clears them. */
#define TSV_PROFILE_CLASSES 11
int32_t tsv_set_profile(tsv_ctx* ctx, int32_t on);
int32_t tsv_get_profile(tsv_ctx* ctx, float* ms, int32_t* counts, int32_t n_classes);

/* Measurement hook (no reference counterpart): launch the kernels of one class `times` times
 * in a row in every following pass (1 restores normal operation).  The extra launches redo the
 * same work on the same buffers, so results do not change; timing a pass with and without the
 * repeat gives the class's in-pipeline duration without an event pair around every launch.
 * Classes that accumulate (norm, embed, acceptance) are refused. */
int32_t tsv_set_repeat(tsv_ctx* ctx, int32_t profile_class, int32_t times);

/* Measurement hook (no reference counterpart): average microseconds of `iters` back-to-back
 * launches of the verify matmul kernel on a rows x cols weight of `dtype` with m activation
 * rows; epi 0 = split-K partials, 1 = silu(gate)*up over interleaved tiles, 2 = fp16 logits;
 * `rotate` weight copies are cycled so the bytes come from HBM. */
int32_t tsv_matmul_time(int32_t dtype, int64_t rows, int64_t cols, int32_t m, int32_t epi, int32_t splits,
                        int32_t iters, int32_t rotate, float* avg_us);

/* Measurement hook: average duration of `iters` launches of a plain device-to-device copy kernel
 * over `bytes` bytes (read once, written once).  It is the copy kernel of known size that HBM
 * traffic counters are scaled against, and the streaming rate the part actually reaches. */
int32_t tsv_copy_time(int64_t bytes, int32_t iters, float* avg_us);

/* One verify-pass attention through the same kernels the forward uses.  q: m x nq x hd,
 * k, v: (base + m) x nkv x hd in the reference cache layout, all fp16; row i sits at cache
 * slot base+i and sees [0, base) plus the slots of its root path (parent NULL: chain).
 * window > 0 keeps the last `window` positions of each row's sequence; sinks (nullable): one f32
 * logit per q head (crates/compute/src/attention.rs:29-137).
 * out: m x nq x hd fp16.  (The per-kernel parity hook of crates/gpu/tests/attention_tree_parity.rs.) */
int32_t tsv_attention(const uint16_t* q, const uint16_t* k, const uint16_t* v, int32_t m, int32_t nq,
                      int32_t nkv, int32_t hd, int64_t base, const int32_t* parent, float scale,
                      int32_t window, const float* sinks, uint16_t* out);

/* The tables the quantized KV rows are coded with, computed on the host (no GPU needed): head_dim signs
 * (crates/compute/src/kv_quant.rs:68-81, seed 0 for keys and 1 for values), the 1 << bits Lloyd-Max levels
 * (kv_quant.rs:166-256) and their (1 << bits) - 1 midpoints (kv_quant.rs:262-264). */
int32_t tsv_kv_quant_tables(int32_t head_dim, int32_t bits, int32_t value_side, float* signs, float* codebook,
                            float* midpoints);

/* The stored rows of a quantized layer in the reference's row form: n x n_kv_heads x (1 + words) u32 per side,
 * the f32 norm first, then ceil(head_dim * bits / 32) words of LSB-first codebook indices -- the row
 * crates/gpu/tests/kv_quantize_parity.rs:22-38 reads back.  (In device memory the norms and the indices lie in
 * separate arrays and the value indices are grouped by dimension, sixteen positions to a group; this call
 * re-packs them.) */
int32_t tsv_read_kv_quantized(tsv_ctx* ctx, int32_t layer, int64_t pos0, int64_t n, uint32_t* k_rows, uint32_t* v_rows);

/* One verify-pass attention over quantized rows through the kernels the forward uses (the parity hook
 * of crates/gpu/tests/kv_quantize_parity.rs and attention_tq_parity.rs).  k, v: (base + m) x nkv x hd
 * fp16 staging rows; every one goes through staging slots and the quantizer, sixteen rows
 * at a time as passes do, the last m of them as the pass itself: row i of the pass sits at position
 * base + i and sees positions 0 .. base + i, all of them as stored.  out: m x nq x hd fp16;
 * k_rows / v_rows: the stored rows of all base + m positions in tsv_read_kv_quantized's form.
 * k_bits / v_bits: 2, 3 or 4. */
int32_t tsv_attention_quantized(const uint16_t* q, const uint16_t* k, const uint16_t* v, int32_t m, int32_t nq, int32_t nkv,
                                int32_t hd, int64_t base, int32_t k_bits, int32_t v_bits, float scale, const float* sinks,
                                uint16_t* out, uint32_t* k_rows, uint32_t* v_rows);

/* The experts every row of the last pass chose in every routed layer: out is [n_layers][16][8] expert
 * ids in rank order (row r of the pass at [layer][r], the first top_k entries of a row are valid).
 * What the bench counts the expert bytes actually read from, and what the routing tests compare with
 * the oracle's ranking (real_forward_dispatch.rs:1135-1158).  Passes of at most sixteen rows are meant: the
 * 64-row prompt passes keep their selections in buffers of their own. */
int32_t tsv_route_selected(tsv_ctx* ctx, int32_t* out, int32_t n_layers);

/* Makes the routed layers take the experts given instead of each row's own top-k: sel is
 * [n_layers][16][8] expert ids (row r of a pass at [layer][r], slot order as given; a row whose first
 * entry is negative routes freely); the weights stay the softmax of the row's own router logits over
 * the experts taken.  NULL restores free routing.  With the oracle's ranking forced onto the device
 * (or the device's onto the oracle, tso_model_force_route) the two sides run the same experts on any
 * input, also one whose ranking sits inside the fp16 rounding of a tie; the bench uses it to time the
 * expert matmuls under routing that is independent from row to row.  While selections are held, prompts go in
 * 16-row passes (the 64-row passes route freely). */
int32_t tsv_force_route(tsv_ctx* ctx, const int32_t* sel, int32_t n_layers);

#ifdef __cplusplus
}
#endif
#endif
