// Host loop of speculative generation over the device verify step, and the adaptive draft depth.
//
// Restates crates/runtime/src/speculative.rs:194-900 (`run_speculative`, step-wise drafter, chain
// rounds) for a target that lives behind this library: admission (raw_completion.rs:126-146),
// headless prefill priming the drafter, then rounds of  commit(next) -> cap the block by budget
// and context (:448-459) -> draft_step x block + the row-only prime (:606-660) -> ONE call that
// verifies, accepts on the device and truncates the KV -> observe (:760-765) -> rewind_drafter.
// The token sink is the token-id part of crates/runtime/src/token_sink.rs:64-124: a stop token is
// not reported, the token that exhausts the budget is; neither enters the history.
// The controller is crates/runtime/src/speculative_adaptive.rs:105-227.
#include <algorithm>
#include <vector>

#include "tsv_internal.h"

using namespace tsv;

// ---- adaptive depth ----------------------------------------------------------------------
extern "C" void tsv_adaptive_init(tsv_adaptive* a, int32_t floor, int32_t cap) {
    // shipped tuning (speculative_adaptive.rs:170-190): streaks of 8 / 6 / 4 clean rounds climb
    // from depth 2-3 / 4 / 5+, two missed proposals drop a step
    a->cap = std::max(cap, 1);
    a->floor = std::min(std::max(floor, 1), a->cap);
    a->cur = a->floor;
    a->climb = a->pressure = 0;
    a->climb_low = 8;
    a->climb_mid = 6;
    a->climb_high = 4;
    a->drop = 2;
}

extern "C" int32_t tsv_adaptive_depth(const tsv_adaptive* a) { return a->cur; }

extern "C" int32_t tsv_adaptive_tile_cap(int32_t cap, int32_t tile_rows) {
    return tile_rows > 0 ? std::min(cap, std::max(tile_rows - 1, 1)) : cap;
}

static int climb_needed(const tsv_adaptive* a, int depth) {
    return depth <= 1 ? 2 : depth <= 3 ? a->climb_low : depth == 4 ? a->climb_mid : a->climb_high;
}

extern "C" void tsv_adaptive_observe(tsv_adaptive* a, int32_t offered, int32_t accepted) {
    if (offered <= 0) return;  // an empty round is not a signal
    accepted = std::min(accepted, offered);
    if (accepted == offered) {
        a->pressure = 0;
        if (a->cur < a->cap && ++a->climb >= climb_needed(a, a->cur)) {
            a->cur += 1;
            a->climb = 0;
        }
        return;
    }
    a->climb = 0;
    if (a->cur > a->floor) {  // at the floor there is nowhere to fall and no pressure builds
        a->pressure += offered - accepted;
        if (a->pressure >= a->drop) {
            a->cur -= 1;
            a->pressure = 0;
        }
    }
}

// ---- the loop ------------------------------------------------------------------------------
namespace {

struct Emit {
    tsv_generation_result* out;
    int push(int32_t t) {
        if (out->n_tokens >= out->capacity) {
            set_error("run_speculative: the token buffer is smaller than the budget");
            return TSV_ERR_INVALID;
        }
        out->tokens[out->n_tokens++] = t;
        return TSV_OK;
    }
};

bool is_stop(const tsv_generation* g, int32_t t) {
    for (int i = 0; i < g->n_stop; i++)
        if (g->stop_tokens[i] == t) return true;
    return false;
}

// select() of one logits row at draw position `position` (choose.rs:61-98): arg-max, or a draw
// from the shaped distribution
int select_row(tsv_ctx* c, const uint16_t* row, const tsv_shaping* sh, uint64_t position, int32_t* token,
               const std::vector<int32_t>& hist, uint64_t generated) {
    uint64_t at = position;
    return tsv_draft_chain(c, row, 1, sh, &at, token, hist.data(), (int64_t)hist.size(), generated);
}

}  // namespace

extern "C" int32_t tsv_run_speculative(tsv_ctx* c, const tsv_drafter* dr, const int32_t* prompt, int64_t n,
                                       const tsv_generation* g, tsv_generation_result* out) {
    if (!c || !dr || !dr->rewind || !prompt || !g || !out || !out->tokens) {
        set_error("run_speculative: null argument");
        return TSV_ERR_INVALID;
    }
    // a step-wise drafter steps and primes; a block drafter (producer.rs:222-250) may leave both out, and is
    // then primed over the prompt by its own prefill_chunk
    if (!(dr->step && dr->prime) && !(dr->draft_block && dr->prefill_chunk)) {
        set_error("run_speculative: the drafter needs step and prime, or draft_block and prefill_chunk");
        return TSV_ERR_INVALID;
    }
    const int64_t max_context = tsv_max_context(c);
    const int64_t vocab = tsv_vocab(c);
    // check_admission
    if (n < 1) {
        set_error("run_speculative: empty prompt");
        return TSV_ERR_INVALID;
    }
    if (g->max_new_tokens == 0) {
        set_error("run_speculative: zero generation budget");
        return TSV_ERR_INVALID;
    }
    if ((uint64_t)n + g->max_new_tokens > (uint64_t)max_context) {
        set_error("run_speculative: prompt plus budget overflow the context window");
        return TSV_ERR_INVALID;
    }
    if (g->block < 1 || g->block > TSV_MAX_ROWS - 1) {
        set_error("run_speculative: block must be 1..15 (block size 0 proposes nothing)");
        return TSV_ERR_INVALID;
    }
    if (g->n_stop < 0 || g->n_stop > 16 || (g->n_stop && !g->stop_tokens)) {
        set_error("run_speculative: at most 16 stop tokens");
        return TSV_ERR_INVALID;
    }
    const bool sampled = g->shaping.temperature != 0.0;
    if (sampled && !dr->step) {
        set_error("run_speculative: this drafter is block-wise only; a sampled round needs draft_step's distributions");
        return TSV_ERR_UNSUPPORTED;
    }
    tsv_adaptive ad;
    const bool adaptive = g->adaptive_floor > 0;
    if (adaptive) tsv_adaptive_init(&ad, g->adaptive_floor, g->block);
    out->n_tokens = 0;
    out->stop_reason = 0;
    out->rounds = out->offered = out->accepted = out->rollbacks = 0;
    out->draw_step = 0;
    out->min_margin = 1.0;
    out->final_depth = adaptive ? ad.cur : g->block;
    Emit emit{out};

    int rc;
    // The reuse contract (speculative.rs:240-251): ask how much of this prompt the state already
    // covers and reset only when the answer is none.  The drafter's context is not part of the
    // target's state, so a prefix is taken over only as a pure continuation -- nothing rewound, and
    // the drafter within one row of the reuse point (real_forward_traits.rs:199-239); a drafter
    // that cannot say where it stands never reuses.
    int64_t reused = 0, drafter_at = 0;
    if (dr->position) {
        const int64_t cursor = tsv_kv_position(c);
        int64_t keep = tsv_try_reuse_prefix(c, prompt, n);
        if (keep < 0) return TSV_ERR_INVALID;
        keep = std::min<int64_t>(keep, n - 1);
        if (keep > 0) {
            drafter_at = dr->position(dr->user);
            if (tsv_kv_position(c) != cursor || tsv_session_swapped(c) || drafter_at < 0 || keep - drafter_at > 1) keep = 0;
            // a drafter primed by the prefill itself needs the target's pass over the row it lags by: the
            // target steps back that one row and both continue from the drafter's position
            if (keep > drafter_at && dr->prefill_chunk) {
                tsv_point back{drafter_at};
                keep = drafter_at > 0 && tsv_rollback(c, &back) == TSV_OK ? drafter_at : 0;
            }
        }
        reused = keep;
    }
    if (reused == 0) {
        if ((rc = tsv_reset(c))) return rc;
        if (dr->position && dr->position(dr->user) > 0 && dr->rewind(dr->user, 0)) {
            set_error("run_speculative: rewind_drafter failed");
            return TSV_ERR_INVALID;
        }
    } else if (drafter_at > reused && dr->rewind(dr->user, reused)) {
        set_error("run_speculative: rewind_drafter failed");
        return TSV_ERR_INVALID;
    }
    out->reused = reused;
    std::vector<uint16_t> logits((size_t)vocab), rows_host;
    // the drafter's rows of a round: host memory, or a device buffer a GPU drafter fills in place
    struct DeviceRows {
        uint16_t* p = nullptr;
        ~DeviceRows() {
            if (p) (void)hipFree(p);
        }
    } rows_dev;
    uint16_t* rows;
    if (dr->device_logits) {
        if (hipMalloc((void**)&rows_dev.p, (size_t)g->block * vocab * 2) != hipSuccess) {
            (void)hipGetLastError();
            set_error("run_speculative: cannot allocate the drafter's device rows");
            return TSV_ERR_DEVICE;
        }
        rows = rows_dev.p;
    } else {
        rows_host.resize((size_t)g->block * vocab);
        rows = rows_host.data();
    }
    // prefill: every prompt token but the last skips the output head; the drafter is primed with
    // each known next token
    // the reused positions are already in the cache (and, by the guard above, in the drafter's
    // context up to at most the one row it lags by, which is primed here with its known next token)
    if (dr->prefill_chunk) {
        // speculative.rs:287-316: the whole prompt through the drafter-priming prefill; the last position is left
        // for the first draft step
        set_error("");
        if (dr->prefill_chunk(dr->user, prompt + reused, n - reused, reused, logits.data(), -1)) {
            if (error_is_empty()) set_error("run_speculative: prefill_chunk_priming_drafter failed");
            return TSV_ERR_INVALID;
        }
    } else {
        if (n - 1 > reused && (rc = tsv_prefill(c, prompt + reused, n - 1 - reused, reused, nullptr))) return rc;
        for (int64_t i = reused ? std::min(drafter_at, reused) : 0; i + 1 < n; i++)
            if (dr->prime(dr->user, prompt[i + 1], i)) {
                set_error("run_speculative: prime_drafter failed");
                return TSV_ERR_INVALID;
            }
        if ((rc = tsv_produce(c, prompt[n - 1], n - 1, logits.data()))) return rc;
    }
    int64_t history = n;  // tokens backed by KV rows or about to be
    std::vector<int32_t> hist(prompt, prompt + n);  // TokenSink::history: what the penalties look at
    uint64_t generated = 0, draw_step = 0;
    int32_t next;
    if ((rc = select_row(c, logits.data(), &g->shaping, generated, &next, hist, generated))) return rc;

    int32_t feed[TSV_MAX_ROWS];
    for (;;) {
        // sink.commit(next)
        generated += 1;
        if (is_stop(g, next)) {
            out->stop_reason = 1;
            break;
        }
        if ((rc = emit.push(next))) return rc;
        if (generated >= g->max_new_tokens) {
            out->stop_reason = 2;
            break;
        }
        history += 1;
        hist.push_back(next);
        const int64_t base = history - 1, position = history;
        const uint64_t budget_room = g->max_new_tokens - generated;
        const int64_t context_room = max_context - position;
        const int wanted = adaptive ? std::min(tsv_adaptive_depth(&ad), g->block) : g->block;
        const int round_block = (int)std::min<uint64_t>(std::min<uint64_t>((uint64_t)wanted, budget_room),
                                                        (uint64_t)std::max<int64_t>(context_room, 0));
        const bool truncated = round_block < wanted;
        if (round_block == 0) {
            set_error("run_speculative: round_block is 0: no room after admission; invariant violation");
            return TSV_ERR_INVALID;
        }
        // speculative.rs:386-392, 467-575: a TREE round -- greedy, fixed depth, the full block, a drafter
        // whose trees have exactly `block` nodes.  Verify, the walk (at the current node's row the
        // target's pick is accepted when a child of that node carries it), the compaction of the
        // accepted path and the truncation are one tsv_verify_accept.
        if (dr->draft_tree && dr->tree_nodes == g->block && !sampled && round_block == g->block && !adaptive) {
            const int nodes = dr->tree_nodes;
            int32_t node_parent[TSV_MAX_ROWS], parents[TSV_MAX_ROWS];
            feed[0] = next;
            if (dr->draft_tree(dr->user, next, base, nodes, node_parent, feed + 1)) {
                set_error("run_speculative: draft_tree failed");
                return TSV_ERR_INVALID;
            }
            parents[0] = -1;  // dflash_tree.rs:119-123: slot 0 is the anchor, node i sits at slot i + 1
            for (int i = 0; i < nodes; i++) {
                if (node_parent[i] < -1 || node_parent[i] >= i) {
                    set_error("run_speculative: draft_tree must list parents before children");
                    return TSV_ERR_INVALID;
                }
                parents[i + 1] = node_parent[i] < 0 ? 0 : node_parent[i] + 1;
            }
            tsv_round r{};
            r.feed = feed;
            r.parent = parents;
            r.m = nodes + 1;
            r.base = base;
            r.shaping = g->shaping;
            r.draw_step = draw_step;
            r.stop_tokens = g->stop_tokens;
            r.n_stop = g->n_stop;
            r.generated = generated;
            r.max_new_tokens = g->max_new_tokens;
            tsv_round_result res{};
            if ((rc = tsv_verify_accept(c, &r, &res))) return rc;
            out->rounds += 1;
            out->offered += nodes;
            out->accepted += res.accepted;
            if (res.committed < nodes) out->rollbacks += 1;
            int32_t path_feed[TSV_MAX_ROWS + 1];
            for (int i = 0; i <= res.committed; i++) path_feed[i] = feed[res.path[i]];
            for (int i = 1; i <= res.committed; i++)
                if ((rc = emit.push(path_feed[i]))) return rc;
            // the budget's last token is reported: the node the walk accepted last
            if (res.stopped == 2 && (rc = emit.push(feed[res.path[res.committed + 1]]))) return rc;
            generated += (uint64_t)res.accepted;
            history += res.committed;
            hist.insert(hist.end(), path_feed + 1, path_feed + 1 + res.committed);
            if ((rc = tsv_record_committed(c, path_feed, res.committed + 1, base))) return rc;
            if (dr->rewind(dr->user, base + res.committed)) {
                set_error("run_speculative: rewind_drafter failed");
                return TSV_ERR_INVALID;
            }
            if (res.stopped) {
                out->stop_reason = res.stopped;
                break;
            }
            next = res.next;
            continue;
        }
        // draft: block steps, each proposal drawn from the drafter's own distribution (or its
        // arg-max), then the row-only step that primes the drafter with the last proposal
        feed[0] = next;
        int32_t chained = next;
        if (dr->draft_block && !sampled) {
            // speculative.rs:596-603: the whole block from one call; the drafter keeps its own state
            set_error("");
            if (dr->draft_block(dr->user, next, base, round_block, feed + 1)) {
                if (error_is_empty()) set_error("run_speculative: draft_block failed");
                return TSV_ERR_INVALID;
            }
        } else if (tsv_ctx* own = sampled ? tsv_mtp_own_head(dr) : nullptr) {
            // the library's own head chains a sampled round on the device as well: the rows stay in `rows`, the draws
            // are the ones the steps below would make (positions draw_step .. draw_step + block - 1, then the row-only step)
            if ((rc = tsv_mtp_draft_block_sampled(own, next, base, round_block, &g->shaping, draw_step, hist.data(), (int64_t)hist.size(),
                                                  generated, rows, feed + 1)))
                return rc;
            draw_step += (uint64_t)round_block + 1;
        } else
        for (int d = 0; d <= round_block; d++) {
            if (d == round_block) {
                if (dr->prime(dr->user, chained, base - 1 + d)) {
                    set_error("run_speculative: prime_drafter failed");
                    return TSV_ERR_INVALID;
                }
                if (sampled) draw_step += 1;
                break;
            }
            uint16_t* row = rows + (size_t)d * vocab;
            if (dr->step(dr->user, chained, base - 1 + d, row)) {
                set_error("run_speculative: draft_step failed");
                return TSV_ERR_INVALID;
            }
            if ((rc = select_row(c, row, &g->shaping, sampled ? draw_step : generated, &chained, hist, generated)))
                return rc;
            if (sampled) draw_step += 1;
            feed[1 + d] = chained;
        }
        // verify + accept + truncate
        tsv_round r{};
        r.feed = feed;
        r.m = round_block + 1;
        r.base = base;
        r.shaping = g->shaping;
        r.draft_logits = sampled ? rows : nullptr;
        r.draw_step = draw_step;
        r.stop_tokens = g->stop_tokens;
        r.n_stop = g->n_stop;
        r.generated = generated;
        r.max_new_tokens = g->max_new_tokens;
        r.history = hist.data();
        r.n_history = (int64_t)hist.size();
        tsv_round_result res{};
        if ((rc = tsv_verify_accept(c, &r, &res))) return rc;
        out->rounds += 1;
        out->offered += round_block;
        out->accepted += res.accepted;
        out->min_margin = std::min(out->min_margin, res.min_margin);
        if (adaptive && !truncated && !res.stopped) tsv_adaptive_observe(&ad, round_block, res.accepted);
        if (res.committed < round_block) out->rollbacks += 1;
        for (int i = 0; i < res.committed; i++)
            if ((rc = emit.push(feed[1 + i]))) return rc;
        if (res.stopped == 2 && (rc = emit.push(feed[1 + res.committed]))) return rc;  // the budget's last token is reported
        generated += (uint64_t)res.accepted;
        history += res.committed;
        hist.insert(hist.end(), feed + 1, feed + 1 + res.committed);
        draw_step = res.draw_step;
        // the record that lets the next turn reuse: the confirmed token plus every committed
        // proposal, rows base .. base + committed + 1 (speculative.rs:828-836)
        if ((rc = tsv_record_committed(c, feed, res.committed + 1, base))) return rc;
        if (dr->rewind(dr->user, base + res.committed)) {
            set_error("run_speculative: rewind_drafter failed");
            return TSV_ERR_INVALID;
        }
        if (res.stopped) {
            out->stop_reason = res.stopped;
            break;
        }
        next = res.next;
    }
    out->draw_step = draw_step;
    out->final_depth = adaptive ? ad.cur : g->block;
    out->kv_position = tsv_kv_position(c);
    return TSV_OK;
}
