// The drafter head inside the library: a one-layer handle on the target's stream that predicts one token further from
// the target's own state (docs/MTP.md:53-60, crates/runtime/src/families/qwen/mtp.rs).  Its pass is the ordinary pass
// of runtime.hip with the embedding stage replaced (launch_pass); here are its entry points and the callbacks that
// make it a tsv_drafter.
#include "ctx.h"

using namespace tsv;

// ---- the drafter head (docs/MTP.md:53-60, crates/runtime/src/families/qwen/mtp.rs) ------------------------
// One pass of the head over m rows at position .. position + m - 1: row r pairs next_tokens[r] with h_rows' row r.
int tsv::mtp_pass(tsv_ctx* c, const int32_t* next_tokens, int m, int64_t position, const float* h_rows, bool want_logits) {
    if (position != c->position) {  // mtp.rs:484-491
        set_error("mtp: step at position " + std::to_string((long long)position) + " but the head's cache covers [0, " +
                  std::to_string((long long)c->position) + "): prime the head over the prompt and rewind it after a rejected draft");
        return TSV_ERR_INVALID;
    }
    c->mtp.h_src = h_rows;
    c->headless = !want_logits;
    const int rc = enqueue_verify(c, next_tokens, nullptr, m, position);
    c->headless = false;
    c->mtp.h_src = nullptr;
    // after a full step row 0 of x is the head's own finished residual: what a chained step reads (mtp.rs:85-91)
    c->mtp.own_valid = rc == TSV_OK && want_logits && m == 1;
    return rc;
}

// Where the state of `position` is: the head's own row after a step of its own, else the target's last pass.
static int mtp_source(tsv_ctx* c, int64_t position, const float** src) {
    const tsv_ctx* t = c->mtp.target;
    if (c->mtp.own_valid) {
        *src = c->x;
        return TSV_OK;
    }
    if (position >= t->x_base && position < t->x_base + t->x_rows) {
        *src = t->x + (size_t)(position - t->x_base) * t->hidden;
        return TSV_OK;
    }
    set_error("mtp: the target's last pass holds no row for position " + std::to_string((long long)position) +
              " and the head has no step of its own to chain from");
    return TSV_ERR_INVALID;
}

extern "C" int32_t tsv_mtp_open(tsv_ctx* target, const tsv_mtp_desc* d, tsv_ctx** out) {
    TSV_NEED(target && d && out, "mtp_open: null argument");
    if (target->mtp.on || target->mtp_head) {
        set_error("mtp_open: the target is itself a head, or already has one");
        return TSV_ERR_INVALID;
    }
    const tsv_model_desc& m = d->model;
    if (m.n_layers != 1 || m.hidden != target->hidden || m.vocab != target->vocab) {
        set_error("mtp_open: the head is ONE decoder layer of the target's width over the target's vocabulary");
        return TSV_ERR_INVALID;
    }
    if (m.kv_k_bits || m.kv_v_bits || m.session_slots > 1 || (m.layers && m.layers[0].ring)) {
        set_error("mtp_open: the head keeps one plain fp16 cache (no quantized rows, ring or session slots)");
        return TSV_ERR_UNSUPPORTED;
    }
    TSV_HIP(hipStreamSynchronize(target->stream));
    const int rc = open_impl(&m, target, d, out);
    if (rc) return rc;
    target->mtp_head = *out;
    return TSV_OK;
}

extern "C" int32_t tsv_mtp_step(tsv_ctx* c, int32_t next_token, int64_t position, uint16_t* logits, int32_t on_device) {
    TSV_NEED(c && c->mtp.on, "mtp_step: not a drafter head");
    const float* src = nullptr;
    int rc = mtp_source(c, position, &src);
    if (rc) return rc;
    if ((rc = mtp_pass(c, &next_token, 1, position, src, logits != nullptr))) return rc;
    if (!logits) return TSV_OK;
    if (on_device) {  // stays in stream order: whoever reads the row does so on the target's stream
        TSV_HIP(hipMemcpyAsync(logits, c->logits, (size_t)c->vocab * 2, hipMemcpyDeviceToDevice, c->stream));
        return TSV_OK;
    }
    return finish_verify(c, 1, logits);
}

extern "C" int32_t tsv_mtp_rewind(tsv_ctx* c, int64_t position) {
    TSV_NEED(c && c->mtp.on, "mtp_rewind: not a drafter head");
    if (position < 0 || position > c->position) {  // mtp.rs:422-436
        set_error("mtp_rewind: the head cannot be moved forward, or before position 0");
        return TSV_ERR_INVALID;
    }
    c->position = position;
    c->mtp.own_valid = false;
    return TSV_OK;
}

extern "C" int32_t tsv_mtp_prefill_chunk(tsv_ctx* c, const int32_t* tokens, int64_t n, int64_t start_position,
                                         uint16_t* logits, int32_t next_token) {
    TSV_NEED(c && c->mtp.on && tokens, "mtp_prefill_chunk: not a drafter head, or no tokens");
    if (n < 1) {
        set_error("mtp_prefill_chunk: empty token list");
        return TSV_ERR_INVALID;
    }
    if (c->position != start_position) {
        set_error("mtp_prefill_chunk: the head's cache must end where the chunk starts");
        return TSV_ERR_INVALID;
    }
    tsv_ctx* t = c->mtp.target;
    // recorded once the chunk has run to completion, tainted when it has not (real_forward_traits.rs:395-402)
    const int rc = prefill_passes(t, tokens, n, start_position, logits, c, next_token >= 0 && next_token < t->vocab ? next_token : -1);
    if (rc == TSV_OK) t->prefix.record(tokens, n, start_position);
    else t->prefix.taint();
    return rc;
}

// The parameter blocks of a block draft's steps (one row each at base - 1 + d, d = 0 .. block) to the device in ONE copy;
// step d then runs with vp_dev naming its block and stages nothing.
static int stage_block_params(tsv_ctx* c, int64_t base, int block) {
    tsv_ctx::Mtp& h = c->mtp;
    const int32_t none = 0;
    for (int d = 0; d <= block; d++)
        if (int rc = fill_params(h.vp_block_host[d], &none, nullptr, 1, base - 1 + d, c->vocab)) return rc;
    TSV_HIP(hipMemcpyAsync(h.vp_block, h.vp_block_host, (size_t)(block + 1) * sizeof(VerifyParams), hipMemcpyHostToDevice, c->stream));
    return TSV_OK;
}

extern "C" int32_t tsv_mtp_draft_block(tsv_ctx* c, int32_t anchor, int64_t base, int32_t block, int32_t* proposals) {
    TSV_NEED(c && c->mtp.on && proposals, "mtp_draft_block: not a drafter head, or no output");
    if (block < 1 || block > TSV_MAX_ROWS - 1 || base < 1) {
        set_error("mtp_draft_block: 1..15 proposals after a position the target has produced");
        return TSV_ERR_INVALID;
    }
    tsv_ctx::Mtp& h = c->mtp;
    int rc;
    const int32_t none = 0;
    if (anchor < 0 || anchor >= c->vocab) {
        set_error("mtp_draft_block: token id outside the vocabulary");
        return TSV_ERR_INVALID;
    }
    // every step takes its token from chain[d] on the device: the anchor is put there with the parameter blocks
    h.chain_host[30] = anchor;
    TSV_HIP(hipMemcpyAsync(h.chain, h.chain_host + 30, 4, hipMemcpyHostToDevice, c->stream));
    if ((rc = stage_block_params(c, base, block))) return rc;
    VerifyParams* const vp_own = c->vp_dev;
    for (int d = 0; d <= block; d++) {
        // step d pairs the state of base - 1 + d with the token at base + d: the anchor, then each pick of the
        // step before, read where the arg-max left it; the last step is the row-only one (speculative.rs:612-625)
        const float* src = nullptr;
        if ((rc = mtp_source(c, base - 1 + d, &src))) break;
        h.feed_dev = h.chain + d;
        h.params_staged = true;
        c->vp_dev = h.vp_block + d;
        rc = mtp_pass(c, &none, 1, base - 1 + d, src, d < block);
        c->vp_dev = vp_own;
        h.params_staged = false;
        h.feed_dev = nullptr;
        if (rc) return rc;
        if (d < block && (rc = launch_argmax_rows(c->stream, c->logits, 1, c->vocab, c->sc, h.chain + d + 1, d == 0))) return rc;
    }
    if (rc) return rc;
    h.own_valid = false;
    TSV_HIP(hipMemcpyAsync(h.chain_host, h.chain + 1, (size_t)block * 4, hipMemcpyDeviceToHost, c->stream));
    TSV_HIP(hipMemcpyAsync(h.chain_host + 31, c->sc.counters, 4, hipMemcpyDeviceToHost, c->stream));
    TSV_HIP(hipStreamSynchronize(c->stream));
    if (h.chain_host[31]) {
        set_error("mtp_draft_block: score vector must not contain a non-finite entry");
        return TSV_ERR_INVALID;
    }
    for (int i = 0; i < block; i++) proposals[i] = h.chain_host[i];
    return TSV_OK;
}

// The sampled counterpart, for the library's own loop (no reference counterpart: its draft_block hands back tokens
// only, so its sampled rounds go step by step, speculative.rs:612-660): every step's logits row stays in `rows`
// (device, block x vocab fp16: the proposal distributions the rejection test needs), the proposal is DRAWN on
// the device from the row's shaped distribution at draw position draw_step + d (the same kernels and parameters as
// tsv_draft_chain for that row) and fed to the next step where it lies.  One host wait per block.
int tsv_mtp_draft_block_sampled(tsv_ctx* c, int32_t anchor, int64_t base, int32_t block, const tsv_shaping* sh, uint64_t draw_step,
                                const int32_t* history, int64_t n_history, uint64_t generated, uint16_t* rows, int32_t* proposals) {
    TSV_NEED(c && c->mtp.on && sh && rows && proposals, "mtp_draft_block: not a drafter head, or a null argument");
    if (block < 1 || block > TSV_MAX_ROWS - 1 || base < 1) {
        set_error("mtp_draft_block: 1..15 proposals after a position the target has produced");
        return TSV_ERR_INVALID;
    }
    int rc = check_shaping(*sh, true);
    if (rc) return rc;
    tsv_ctx::Mtp& h = c->mtp;
    AcceptParams ap;
    std::memset(&ap, 0, sizeof ap);
    ap.m = 0;
    ap.k = 1;
    ap.vocab = c->vocab;
    ap.sampled = sh->temperature != 0.0;
    ap.temperature = sh->temperature;
    ap.seed = sh->seed;
    fill_truncation(&ap, *sh);
    if ((rc = setup_penalties(c, *sh, history, n_history, generated, &ap))) return rc;  // the same history for every step of a round
    const int32_t none = 0;
    if (anchor < 0 || anchor >= c->vocab) {
        set_error("mtp_draft_block: token id outside the vocabulary");
        return TSV_ERR_INVALID;
    }
    h.chain_host[30] = anchor;
    TSV_HIP(hipMemcpyAsync(h.chain, h.chain_host + 30, 4, hipMemcpyHostToDevice, c->stream));
    if ((rc = stage_block_params(c, base, block))) return rc;
    VerifyParams* const vp_own = c->vp_dev;
    for (int d = 0; d <= block; d++) {
        const float* src = nullptr;
        if ((rc = mtp_source(c, base - 1 + d, &src))) return rc;
        h.feed_dev = h.chain + d;
        h.params_staged = true;
        c->vp_dev = h.vp_block + d;
        rc = mtp_pass(c, &none, 1, base - 1 + d, src, d < block);
        c->vp_dev = vp_own;
        h.params_staged = false;
        h.feed_dev = nullptr;
        if (rc) return rc;
        if (d == block) break;
        uint16_t* row = rows + (size_t)d * c->vocab;
        TSV_HIP(hipMemcpyAsync(row, c->logits, (size_t)c->vocab * 2, hipMemcpyDeviceToDevice, c->stream));
        h.draw_host[d] = ap;
        h.draw_host[d].draw_step = draw_step + (uint64_t)d;
        TSV_HIP(hipMemcpyAsync(h.draw_dev + d, h.draw_host + d, sizeof(AcceptParams), hipMemcpyHostToDevice, c->stream));
        if ((rc = launch_draft_chain(c->stream, row, h.draw_dev + d, h.draw_host[d], c->sc, h.chain + d + 1))) return rc;
    }
    h.own_valid = false;
    TSV_HIP(hipMemcpyAsync(h.chain_host, h.chain + 1, (size_t)block * 4, hipMemcpyDeviceToHost, c->stream));
    TSV_HIP(hipMemcpyAsync(c->res_host, c->sc.result, sizeof(AcceptResult), hipMemcpyDeviceToHost, c->stream));
    TSV_HIP(hipStreamSynchronize(c->stream));
    if (c->res_host->error) {  // (each step's draw clears the flag first: this is the last step's)
        set_error(std::string("mtp_draft_block: ") + accept_error_text(c->res_host->error));
        return (c->res_host->error & 1) ? TSV_ERR_INVALID : TSV_ERR_UNSUPPORTED;
    }
    for (int i = 0; i < block; i++) proposals[i] = h.chain_host[i];
    return TSV_OK;
}

namespace {
int32_t mtp_cb_prime(void* u, int32_t next, int64_t position) { return tsv_mtp_step((tsv_ctx*)u, next, position, nullptr, 0); }
int32_t mtp_cb_step(void* u, int32_t tok, int64_t position, uint16_t* logits) { return tsv_mtp_step((tsv_ctx*)u, tok, position, logits, 1); }
int32_t mtp_cb_rewind(void* u, int64_t position) { return tsv_mtp_rewind((tsv_ctx*)u, position); }
int64_t mtp_cb_position(void* u) { return ((tsv_ctx*)u)->position; }
int32_t mtp_cb_block(void* u, int32_t anchor, int64_t base, int32_t block, int32_t* proposals) {
    return tsv_mtp_draft_block((tsv_ctx*)u, anchor, base, block, proposals);
}
int32_t mtp_cb_chunk(void* u, const int32_t* tokens, int64_t n, int64_t start, uint16_t* logits, int32_t next_token) {
    return tsv_mtp_prefill_chunk((tsv_ctx*)u, tokens, n, start, logits, next_token);
}
}  // namespace

// Whether a drafter is this library's own head with its block callback in place (the loop then chains sampled rounds too).
tsv_ctx* tsv_mtp_own_head(const tsv_drafter* d) {
    return d && d->draft_block == mtp_cb_block && d->step == mtp_cb_step && d->user && ((tsv_ctx*)d->user)->mtp.on ? (tsv_ctx*)d->user
                                                                                                                     : nullptr;
}

extern "C" int32_t tsv_mtp_drafter(tsv_ctx* c, tsv_drafter* out) {
    TSV_NEED(c && c->mtp.on && out, "mtp_drafter: not a drafter head, or no output");
    std::memset(out, 0, sizeof *out);
    out->user = c;
    out->prime = mtp_cb_prime;
    out->step = mtp_cb_step;
    out->rewind = mtp_cb_rewind;
    out->device_logits = 1;
    out->position = mtp_cb_position;
    out->draft_block = mtp_cb_block;
    out->prefill_chunk = mtp_cb_chunk;
    return TSV_OK;
}
