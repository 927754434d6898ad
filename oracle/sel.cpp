// Selection pipeline and the host half of a speculative round (test infrastructure only).
// Follows crates/selection/src/{derive,choose,distribution,truncation,penalty}.rs and
// crates/runtime/src/{speculative,token_sink,dflash_tree}.rs.
#include "tsoracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

static thread_local std::string g_err;
extern "C" const char* tso_last_error(void) { return g_err.c_str(); }
void tso_set_error(const std::string& s) { g_err = s; }

// crates/selection/src/derive.rs:32-38
extern "C" uint64_t tso_mix(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
// crates/selection/src/derive.rs:19-22 (seeded arm only)
extern "C" uint64_t tso_derive_step_value(uint64_t seed, uint64_t position) {
    return tso_mix(seed ^ (position * 0x9E3779B97F4A7C15ull));
}
// crates/selection/src/derive.rs:42-45
extern "C" double tso_to_unit_interval(uint64_t v) {
    return (double)(v >> 11) * (1.0 / (double)(1ull << 53));
}

namespace {

struct Dist {
    std::vector<uint32_t> support;
    std::vector<double> probs;
};

bool deterministic(const tso_shaping* c) { return c->temperature == 0.0; }

// crates/selection/src/choose.rs:277-285
int32_t argmax_f32(const std::vector<float>& s) {
    size_t best = 0;
    for (size_t i = 1; i < s.size(); i++)
        if (s[i] > s[best]) best = i;
    return (int32_t)best;
}

// crates/selection/src/penalty.rs:15-39
void apply_repetition_penalty(std::vector<float>& scores, const int32_t* history, int64_t nh,
                              double penalty) {
    if (penalty == 1.0 || nh == 0) return;
    std::unordered_set<int32_t> seen(history, history + nh);
    float p = (float)penalty;
    p = std::min(std::max(p, 1.17549435e-38f), 3.40282347e+38f);
    for (int32_t id : seen) {
        if (id < 0 || (size_t)id >= scores.size()) continue;
        float s = scores[id];
        float a = s > 0.0f ? s / p : s * p;
        scores[id] = std::min(std::max(a, -3.40282347e+38f), 3.40282347e+38f);
    }
}

// crates/selection/src/penalty.rs:59-82
void apply_presence_frequency(std::vector<float>& scores, const int32_t* suffix, int64_t n,
                              double presence, double frequency) {
    if ((presence == 0.0 && frequency == 0.0) || n == 0) return;
    std::unordered_map<int32_t, uint32_t> counts;
    for (int64_t i = 0; i < n; i++) counts[suffix[i]]++;
    for (auto& kv : counts) {
        if (kv.first < 0 || (size_t)kv.first >= scores.size()) continue;
        double penalty = presence + frequency * (double)kv.second;
        scores[kv.first] -= (float)penalty;
    }
}

// crates/selection/src/choose.rs:111-228.  Returns <0 on refusal; otherwise fills
// surviving (rank order) and sum; exps is the unnormalised softmax.
int shape_candidates(const uint16_t* raw, int64_t vocab, const tso_shaping* cfg,
                     const int32_t* history, int64_t nh, uint64_t position,
                     std::vector<uint32_t>& surviving, std::vector<double>& exps, double* sum_out) {
    if (vocab <= 0) {
        tso_set_error("candidate domain must not be empty");
        return -1;
    }
    std::vector<float> working((size_t)vocab);
    bool all_finite = true;
    for (int64_t i = 0; i < vocab; i++) {
        float f = tso_f16_to_f32(raw[i]);
        all_finite &= std::isfinite(f);
        working[i] = f;
    }
    if (!all_finite) {
        tso_set_error("score vector must not contain a non-finite entry");
        return -2;
    }
    surviving.clear();
    exps.clear();
    if (deterministic(cfg)) {
        surviving.push_back((uint32_t)argmax_f32(working));
        *sum_out = 1.0;
        return 0;
    }
    apply_repetition_penalty(working, history, nh, cfg->repetition_penalty);
    int64_t generated = std::min<int64_t>((int64_t)position, nh);
    apply_presence_frequency(working, history + (nh - generated), generated, cfg->presence_penalty,
                             cfg->frequency_penalty);

    float maxf = -INFINITY;
    for (float w : working) maxf = std::fmax(maxf, w);
    double mx = (double)maxf;
    exps.resize((size_t)vocab);
    for (int64_t i = 0; i < vocab; i++) exps[i] = std::exp((double)working[i] - mx);
    double sum = 0.0;
    for (int64_t i = 0; i < vocab; i++) sum += exps[i];

    // truncation.rs:79-109,165-236: descending key, ties by ascending index.  The
    // comparator is a total order on NaN-free keys, so any correct sort yields the
    // one order the reference's sort_unstable_by yields; top-k is its prefix.
    std::vector<uint32_t> ranked((size_t)vocab);
    for (int64_t i = 0; i < vocab; i++) ranked[i] = (uint32_t)i;
    auto cmp = [&](uint32_t a, uint32_t b) {
        if (exps[a] != exps[b]) return exps[a] > exps[b];
        return a < b;
    };
    if (cfg->top_k == 0) {
        std::sort(ranked.begin(), ranked.end(), cmp);
    } else {
        size_t k = std::min<size_t>(cfg->top_k, ranked.size());
        std::partial_sort(ranked.begin(), ranked.begin() + k, ranked.end(), cmp);
        ranked.resize(k);
    }

    if (!cfg->has_top_p) {
        surviving = ranked;
    } else {
        double cumulative = 0.0;
        for (uint32_t i : ranked) {
            surviving.push_back(i);
            cumulative += exps[i] / sum;
            if (cumulative >= cfg->top_p) break;
        }
        if (surviving.empty() && !ranked.empty()) surviving.push_back(ranked[0]);
    }
    if (cfg->top_k != 0 && surviving.size() > cfg->top_k) surviving.resize(cfg->top_k);
    if (cfg->has_min_p && !ranked.empty()) {
        uint32_t top = ranked[0];
        double threshold = cfg->min_p * exps[top];
        std::vector<uint32_t> kept;
        for (uint32_t i : surviving)
            if (exps[i] >= threshold) kept.push_back(i);
        if (kept.empty()) kept.push_back(top);
        surviving.swap(kept);
    }
    if (surviving.empty()) {
        surviving.push_back((uint32_t)argmax_f32(working));
        *sum_out = 1.0;
        return 0;
    }
    *sum_out = sum;
    return 0;
}

// crates/selection/src/choose.rs:296-319
std::vector<double> reweight(const std::vector<uint32_t>& surviving, const std::vector<double>& exps,
                             double sum, double temperature) {
    double inv_t = 1.0 / temperature;
    double top = 0.0;
    for (uint32_t i : surviving) top = std::fmax(top, exps[i] / sum);
    std::vector<double> weighted(surviving.size());
    for (size_t j = 0; j < surviving.size(); j++) {
        double p = exps[surviving[j]] / sum;
        weighted[j] = top > 0.0 ? std::pow(p / top, inv_t) : std::pow(p, inv_t);
    }
    double total = 0.0;
    for (double w : weighted) total += w;
    if (total <= 0.0) {
        double n = (double)weighted.size();
        for (double& w : weighted) w = 1.0 / n;
        return weighted;
    }
    for (double& w : weighted) w = w / total;
    return weighted;
}

// crates/selection/src/choose.rs:239-273
int shaped(const uint16_t* logits, int64_t vocab, const tso_shaping* cfg, const int32_t* history,
           int64_t nh, uint64_t position, Dist& out) {
    std::vector<double> exps;
    double sum = 0.0;
    int rc = shape_candidates(logits, vocab, cfg, history, nh, position, out.support, exps, &sum);
    if (rc < 0) return rc;
    if (deterministic(cfg)) {
        out.probs.assign(1, 1.0);
        return 0;
    }
    out.probs = reweight(out.support, exps, sum, cfg->temperature);
    return 0;
}

// crates/selection/src/distribution.rs:61-66
double probability(const Dist& d, uint32_t token) {
    for (size_t i = 0; i < d.support.size(); i++)
        if (d.support[i] == token) return d.probs[i];
    return 0.0;
}

// crates/selection/src/distribution.rs:71-83 (== choose.rs:323-338)
uint32_t draw(const Dist& d, uint64_t seed, uint64_t position) {
    double target = tso_to_unit_interval(tso_derive_step_value(seed, position));
    double cumulative = 0.0;
    for (size_t i = 0; i < d.probs.size(); i++) {
        cumulative += d.probs[i];
        if (target < cumulative) return d.support[i];
    }
    return d.support.back();
}

// crates/selection/src/distribution.rs:96-126
bool residual(const Dist& p, const Dist& q, Dist& out) {
    const double RESIDUAL_EPSILON = 1e-12;
    std::unordered_map<uint32_t, double> q_mass;
    q_mass.reserve(q.support.size());
    for (size_t i = 0; i < q.support.size(); i++) q_mass.emplace(q.support[i], q.probs[i]);  // first wins
    out.support.clear();
    out.probs.clear();
    for (size_t i = 0; i < p.support.size(); i++) {
        auto it = q_mass.find(p.support[i]);
        double qm = it == q_mass.end() ? 0.0 : it->second;
        double mass = std::fmax(p.probs[i] - qm, 0.0);
        if (mass > 0.0) {
            out.support.push_back(p.support[i]);
            out.probs.push_back(mass);
        }
    }
    double total = 0.0;
    for (double m : out.probs) total += m;
    if (total < RESIDUAL_EPSILON || out.support.empty()) return false;
    for (double& m : out.probs) m /= total;
    return true;
}

// crates/selection/src/choose.rs:61-98
int select_token(const uint16_t* logits, int64_t vocab, const tso_shaping* cfg,
                 const int32_t* history, int64_t nh, uint64_t position, int32_t* out) {
    Dist d;
    int rc = shaped(logits, vocab, cfg, history, nh, position, d);
    if (rc < 0) return rc;
    if (deterministic(cfg)) {
        *out = (int32_t)d.support[0];
        return 0;
    }
    *out = (int32_t)draw(d, cfg->seed, position);
    return 0;
}

// The slice of crates/runtime/src/token_sink.rs:64-124 a token-id-only harness can see:
// stop-token ladder, exact budget; stop strings, cancellation and detokenisation have no
// counterpart without a tokenizer.
struct Sink {
    std::vector<int32_t> history;
    uint64_t generated;
    uint64_t max_new_tokens;
    const int32_t* stop_tokens;
    int n_stop;
    // 0: continue, 1: stop token, 2: budget
    int commit(int32_t token) {
        generated += 1;
        for (int i = 0; i < n_stop; i++)
            if (stop_tokens[i] == token) return 1;
        if (generated >= max_new_tokens) return 2;
        history.push_back(token);
        return 0;
    }
};

bool need_seed(const tso_shaping* cfg) {
    if (!deterministic(cfg) && !cfg->has_seed) {
        tso_set_error("a sampled round needs an explicit seed (the clock-derived arm is not reproducible)");
        return true;
    }
    return false;
}

}  // namespace

extern "C" int tso_select(const uint16_t* logits, int64_t vocab, const tso_shaping* cfg,
                          const int32_t* history, int64_t nh, uint64_t position, int32_t* out) {
    if (need_seed(cfg)) return -3;
    return select_token(logits, vocab, cfg, history, nh, position, out);
}

extern "C" int tso_shaped_distribution(const uint16_t* logits, int64_t vocab, const tso_shaping* cfg,
                                       const int32_t* history, int64_t nh, uint64_t position,
                                       uint32_t* support, double* probs, int64_t* n_out) {
    Dist d;
    int rc = shaped(logits, vocab, cfg, history, nh, position, d);
    if (rc < 0) return rc;
    std::memcpy(support, d.support.data(), d.support.size() * sizeof(uint32_t));
    std::memcpy(probs, d.probs.data(), d.probs.size() * sizeof(double));
    *n_out = (int64_t)d.support.size();
    return 0;
}

extern "C" double tso_dist_probability(const uint32_t* support, const double* probs, int64_t n,
                                       uint32_t token) {
    for (int64_t i = 0; i < n; i++)
        if (support[i] == token) return probs[i];
    return 0.0;
}

extern "C" uint32_t tso_dist_draw(const uint32_t* support, const double* probs, int64_t n,
                                  uint64_t seed, uint64_t position) {
    Dist d;
    d.support.assign(support, support + n);
    d.probs.assign(probs, probs + n);
    return draw(d, seed, position);
}

extern "C" int tso_residual(const uint32_t* ps, const double* pp, int64_t np, const uint32_t* qs,
                            const double* qp, int64_t nq, uint32_t* out_support, double* out_probs,
                            int64_t* n_out) {
    Dist p, q, r;
    p.support.assign(ps, ps + np);
    p.probs.assign(pp, pp + np);
    q.support.assign(qs, qs + nq);
    q.probs.assign(qp, qp + nq);
    if (!residual(p, q, r)) {
        *n_out = 0;
        return 0;
    }
    std::memcpy(out_support, r.support.data(), r.support.size() * sizeof(uint32_t));
    std::memcpy(out_probs, r.probs.data(), r.probs.size() * sizeof(double));
    *n_out = (int64_t)r.support.size();
    return 1;
}

// crates/runtime/src/speculative.rs:606-660 (step-wise drafter arm).  history and
// generated are NOT advanced between draft steps.
extern "C" int tso_draft_chain(const uint16_t* draft_logits, int k, int64_t vocab,
                               const tso_shaping* cfg, const int32_t* history, int64_t nh,
                               uint64_t generated, uint64_t* draw_step, int32_t* proposals) {
    if (need_seed(cfg)) return -3;
    bool sampled = !deterministic(cfg);
    for (int d = 0; d < k; d++) {
        const uint16_t* row = draft_logits + (int64_t)d * vocab;
        if (sampled) {
            Dist q;
            int rc = shaped(row, vocab, cfg, history, nh, generated, q);
            if (rc < 0) return rc;
            proposals[d] = (int32_t)draw(q, cfg->seed, *draw_step);
            *draw_step += 1;
        } else {
            int rc = select_token(row, vocab, cfg, history, nh, generated, &proposals[d]);
            if (rc < 0) return rc;
        }
    }
    if (sampled) *draw_step += 1;  // the row-only step (speculative.rs:618-624)
    return 0;
}

// crates/runtime/src/speculative.rs:694-754 (acceptance) and 861-879 (bonus).
extern "C" int tso_chain_round(const uint16_t* target_logits, const uint16_t* draft_logits,
                               const int32_t* proposals, int k, int64_t vocab, const tso_shaping* cfg,
                               const int32_t* history, int64_t nh, uint64_t generated,
                               uint64_t max_new_tokens, const int32_t* stop_tokens, int n_stop,
                               uint64_t draw_step, tso_round_result* out) {
    if (need_seed(cfg)) return -3;
    bool sampled = !deterministic(cfg);
    if (sampled && !draft_logits) {
        tso_set_error("a sampled round needs the drafter's logits");
        return -4;
    }
    Sink sink{std::vector<int32_t>(history, history + nh), generated, max_new_tokens, stop_tokens,
              n_stop};
    size_t base_len = sink.history.size();
    int accepted = 0, stopped = 0;
    bool have_corrected = false;
    int32_t corrected = -1;
    for (int i = 0; i < k; i++) {
        const uint16_t* row = target_logits + (int64_t)i * vocab;
        int32_t proposal = proposals[i];
        if (sampled) {
            Dist p, q;
            int rc = shaped(row, vocab, cfg, sink.history.data(), (int64_t)sink.history.size(),
                            sink.generated, p);
            if (rc < 0) return rc;
            // q was built in the draft phase with the pre-round history (speculative.rs:636-641).
            rc = shaped(draft_logits + (int64_t)i * vocab, vocab, cfg, history, nh, generated, q);
            if (rc < 0) return rc;
            double r = tso_to_unit_interval(tso_derive_step_value(cfg->seed, draw_step));
            draw_step += 1;
            if (r * probability(q, (uint32_t)proposal) <= probability(p, (uint32_t)proposal)) {
                accepted += 1;
                if ((stopped = sink.commit(proposal))) break;
            } else {
                Dist res;
                corrected = (int32_t)(residual(p, q, res) ? draw(res, cfg->seed, draw_step)
                                                          : draw(p, cfg->seed, draw_step));
                have_corrected = true;
                draw_step += 1;
                break;
            }
        } else {
            int32_t target;
            int rc = select_token(row, vocab, cfg, sink.history.data(),
                                  (int64_t)sink.history.size(), sink.generated, &target);
            if (rc < 0) return rc;
            if (target != proposal) break;
            accepted += 1;
            if ((stopped = sink.commit(proposal))) break;
        }
    }
    std::memset(out, 0, sizeof(*out));
    out->accepted = accepted;
    out->committed = (int32_t)(sink.history.size() - base_len);
    out->stopped = stopped;
    out->next = -1;
    if (!stopped) {
        const uint16_t* row = target_logits + (int64_t)accepted * vocab;
        if (have_corrected) {
            out->next = corrected;
        } else if (sampled) {
            Dist p;
            int rc = shaped(row, vocab, cfg, sink.history.data(), (int64_t)sink.history.size(),
                            sink.generated, p);
            if (rc < 0) return rc;
            out->next = (int32_t)draw(p, cfg->seed, draw_step);
            draw_step += 1;
        } else {
            int rc = select_token(row, vocab, cfg, sink.history.data(),
                                  (int64_t)sink.history.size(), sink.generated, &out->next);
            if (rc < 0) return rc;
        }
    }
    out->draw_step = draw_step;
    return 0;
}

// crates/runtime/src/speculative.rs:494-550 with slot parents from dflash_tree.rs:119-123.
extern "C" int tso_tree_round_greedy(const uint16_t* target_logits, const int32_t* feed,
                                     const int32_t* parent, int m, int64_t vocab,
                                     const tso_shaping* cfg, const int32_t* history, int64_t nh,
                                     uint64_t generated, uint64_t max_new_tokens,
                                     const int32_t* stop_tokens, int n_stop, tso_round_result* out) {
    if (!deterministic(cfg)) {
        tso_set_error("the reference's tree round is greedy only (speculative.rs:390-392)");
        return -5;
    }
    Sink sink{std::vector<int32_t>(history, history + nh), generated, max_new_tokens, stop_tokens,
              n_stop};
    size_t base_len = sink.history.size();
    std::memset(out, 0, sizeof(*out));
    out->path[0] = 0;
    out->path_len = 1;
    int at = 0;  // slot of the current node (0 = anchor)
    int stopped = 0;
    int32_t bonus = -1;
    for (;;) {
        int32_t target;
        int rc = select_token(target_logits + (int64_t)at * vocab, vocab, cfg, sink.history.data(),
                              (int64_t)sink.history.size(), sink.generated, &target);
        if (rc < 0) return rc;
        int hit = -1;
        for (int s = 1; s < m; s++)
            if (parent[s] == at && feed[s] == target) {
                hit = s;
                break;
            }
        if (hit < 0) {
            bonus = target;
            break;
        }
        out->path[out->path_len++] = hit;
        at = hit;
        if ((stopped = sink.commit(target))) break;
    }
    out->accepted = out->path_len - 1;
    out->committed = (int32_t)(sink.history.size() - base_len);
    out->stopped = stopped;
    out->next = stopped ? -1 : bonus;
    out->draw_step = 0;
    return 0;
}

// NOT IN THE REFERENCE (see the header): recursive multi-draft rejection per node.
extern "C" int tso_tree_round_sampled(const uint16_t* target_logits, const uint16_t* draft_logits,
                                      const int32_t* feed, const int32_t* parent, int m,
                                      int64_t vocab, const tso_shaping* cfg, const int32_t* history,
                                      int64_t nh, uint64_t generated, uint64_t draw_step,
                                      tso_round_result* out) {
    if (need_seed(cfg) || deterministic(cfg)) {
        if (deterministic(cfg)) tso_set_error("use tso_tree_round_greedy at temperature 0");
        return -3;
    }
    std::vector<int32_t> hist(history, history + nh);
    uint64_t gen = generated;
    std::memset(out, 0, sizeof(*out));
    out->path[0] = 0;
    out->path_len = 1;
    int at = 0;
    int32_t next = -1;
    for (;;) {
        Dist p, q;
        int rc = shaped(target_logits + (int64_t)at * vocab, vocab, cfg, hist.data(),
                        (int64_t)hist.size(), gen, p);
        if (rc < 0) return rc;
        rc = shaped(draft_logits + (int64_t)at * vocab, vocab, cfg, history, nh, generated, q);
        if (rc < 0) return rc;
        int hit = -1;
        for (int s = 1; s < m; s++) {
            if (parent[s] != at) continue;
            uint32_t x = (uint32_t)feed[s];
            double r = tso_to_unit_interval(tso_derive_step_value(cfg->seed, draw_step));
            draw_step += 1;
            if (r * probability(q, x) <= probability(p, x)) {
                hit = s;
                break;
            }
            Dist res;
            if (residual(p, q, res)) p = res;  // else keep p (the epsilon fallback)
        }
        if (hit < 0) {
            next = (int32_t)draw(p, cfg->seed, draw_step);
            draw_step += 1;
            break;
        }
        out->path[out->path_len++] = hit;
        at = hit;
        hist.push_back(feed[hit]);
        gen += 1;
    }
    out->accepted = out->path_len - 1;
    out->committed = out->accepted;
    out->next = next;
    out->draw_step = draw_step;
    return 0;
}

// ---- adaptive depth: crates/runtime/src/speculative_adaptive.rs:105-227 ---------------------
extern "C" void tso_adaptive_new(tso_adaptive* a, int floor, int cap) {
    cap = std::max(cap, 1);
    floor = std::min(std::max(floor, 1), cap);
    *a = tso_adaptive{floor, cap, floor, 0, 0, {8, 6, 4, 2}};  // AdaptiveParams::default (:46-55)
}
extern "C" int tso_adaptive_tile_cap(int cap, int tile_rows) {
    if (tile_rows <= 0) return cap;  // None
    return std::min(cap, std::max(tile_rows - 1, 1));
}
static int adaptive_climb(const tso_adaptive* a, int depth) {  // AdaptiveParams::climb (:60-67)
    if (depth <= 1) return 2;
    if (depth == 2 || depth == 3) return a->params[0];
    if (depth == 4) return a->params[1];
    return a->params[2];
}
extern "C" void tso_adaptive_observe(tso_adaptive* a, int offered, int accepted) {
    if (offered == 0) return;
    accepted = std::min(accepted, offered);
    if (accepted == offered) {
        a->pressure = 0;
        if (a->cur < a->cap) {
            a->climb += 1;
            if (a->climb >= adaptive_climb(a, a->cur)) {
                a->cur += 1;
                a->climb = 0;
            }
        }
    } else {
        a->climb = 0;
        if (a->cur > a->floor) {
            a->pressure += offered - accepted;
            if (a->pressure >= a->params[3]) {
                a->cur -= 1;
                a->pressure = 0;
            }
        }
    }
}

// ---- the loop: crates/runtime/src/speculative.rs:194-900, step-wise drafter, chain rounds ----
// Generic over the producer, like the reference (`run_speculative<P: SpeculativeProducer>`): the
// callbacks are the trait's methods.  Acceptance is the host code above.
extern "C" int tso_run_speculative(const tso_producer* p, const int32_t* prompt, int64_t n,
                                   const tso_generation* g, int64_t max_context, int64_t vocab,
                                   tso_generation_result* out) {
    // raw_completion.rs:126-146
    if (n < 1) {
        tso_set_error("empty prompt");
        return -1;
    }
    if (g->max_new_tokens == 0) {
        tso_set_error("zero budget");
        return -1;
    }
    if ((uint64_t)n + g->max_new_tokens > (uint64_t)max_context) {
        tso_set_error("context overflow");
        return -1;
    }
    if (g->block == 0) {
        tso_set_error("block size 0 proposes nothing");
        return -1;
    }
    if (need_seed(&g->shaping)) return -3;
    const tso_shaping* cfg = &g->shaping;
    const bool sampled = !deterministic(cfg);
    tso_adaptive ad;
    const bool adaptive = g->adaptive_floor > 0;
    if (adaptive) tso_adaptive_new(&ad, g->adaptive_floor, g->block);
    std::memset(&out->n_tokens, 0, sizeof(*out) - offsetof(tso_generation_result, n_tokens));

    p->reset(p->user);
    std::vector<uint16_t> logits((size_t)vocab), draft_rows((size_t)g->block * vocab),
        batch((size_t)(g->block + 1) * vocab);
    int64_t position = 0;
    std::vector<int32_t> history;
    for (int64_t i = 0; i < n; i++) {  // :337-372
        const bool last = i + 1 == n;
        int rc = last ? p->produce(p->user, prompt[i], position, logits.data())
                      : p->prefill(p->user, prompt[i], position);
        if (rc) return -10;
        if (i + 1 < n && p->prime(p->user, prompt[i + 1], i)) return -10;
        position += 1;
        history.push_back(prompt[i]);
    }
    Sink sink{history, 0, g->max_new_tokens, g->stop_tokens, g->n_stop};
    uint64_t draw_step = 0;
    int32_t next;
    int rc = select_token(logits.data(), vocab, cfg, sink.history.data(), (int64_t)sink.history.size(),
                          sink.generated, &next);
    if (rc < 0) return rc;
    auto report = [&](int32_t t) { out->tokens[out->n_tokens++] = t; };
    std::vector<int32_t> proposals, feed;
    for (;;) {
        // TokenSink::commit reports every token but a stop token (token_sink.rs:64-124)
        const bool stop_tok = std::find(g->stop_tokens, g->stop_tokens + g->n_stop, next) != g->stop_tokens + g->n_stop;
        if (!stop_tok) report(next);
        if (int why = sink.commit(next)) {
            out->stop_reason = why;
            break;
        }
        const int64_t base = (int64_t)sink.history.size() - 1;
        position = (int64_t)sink.history.size();
        // :448-459
        const uint64_t budget_room = g->max_new_tokens - sink.generated;
        const uint64_t context_room = (uint64_t)std::max<int64_t>(max_context - position, 0);
        const uint64_t wanted = adaptive ? (uint64_t)std::min(ad.cur, g->block) : (uint64_t)g->block;
        const int round_block = (int)std::min(std::min(wanted, budget_room), context_room);
        const bool truncated = (uint64_t)round_block < wanted;
        if (round_block == 0) {
            tso_set_error("round_block is 0: no room after admission; invariant violation");
            return -11;
        }
        // :386-392, :467-575: a TREE round -- greedy, fixed depth, the full block, a producer that drafts
        // trees of exactly `block` nodes.  The walk is the chain's acceptance generalised: at the current
        // node's row the target's pick is accepted when a child of that node carries it.
        if (p->draft_tree && p->tree_nodes == g->block && !sampled && round_block == g->block && !adaptive) {
            const int nodes = p->tree_nodes;
            std::vector<int32_t> node_parent((size_t)nodes), tokens((size_t)nodes), parents((size_t)nodes + 1);
            if (p->draft_tree(p->user, next, base, nodes, node_parent.data(), tokens.data())) return -10;
            parents[0] = -1;  // dflash_tree.rs:119-123: slot 0 is the anchor, node i sits at slot i + 1
            for (int i = 0; i < nodes; i++) parents[(size_t)i + 1] = node_parent[(size_t)i] < 0 ? 0 : node_parent[(size_t)i] + 1;
            feed.assign(1, next);
            feed.insert(feed.end(), tokens.begin(), tokens.end());
            const int64_t point = base;
            if (p->verify_tree(p->user, feed.data(), parents.data(), (int)feed.size(), base, batch.data())) return -10;
            out->rounds += 1;
            out->offered += nodes;
            std::vector<uint32_t> path(1, 0u);
            int at = -1, stopped = 0;
            int32_t bonus = -1;
            for (;;) {
                const int slot = at + 1;
                int32_t target;
                rc = select_token(batch.data() + (size_t)slot * vocab, vocab, cfg, sink.history.data(),
                                  (int64_t)sink.history.size(), sink.generated, &target);
                if (rc < 0) return rc;
                int hit = -1;
                for (int id = 0; id < nodes; id++)
                    if (node_parent[(size_t)id] == at && tokens[(size_t)id] == target) {
                        hit = id;
                        break;
                    }
                if (hit < 0) {
                    bonus = target;
                    break;
                }
                path.push_back((uint32_t)hit + 1u);
                at = hit;
                const bool st = std::find(g->stop_tokens, g->stop_tokens + g->n_stop, target) != g->stop_tokens + g->n_stop;
                if (!st) report(target);
                if ((stopped = sink.commit(target))) break;
            }
            out->accepted += (int64_t)path.size() - 1;
            const int committed = (int)((int64_t)sink.history.size() - (base + 1));
            if (p->compact_tree(p->user, base, path.data(), committed + 1)) return -10;
            if (committed + 1 < (int)feed.size()) {
                out->rollbacks += 1;
                if (p->rollback_retaining(p->user, point, committed + 1)) return -10;
            }
            if (p->rewind(p->user, base + committed)) return -10;
            if (stopped) {
                out->stop_reason = stopped;
                break;
            }
            next = bonus;
            continue;
        }
        // :606-660
        proposals.clear();
        int32_t chained = next;
        for (int d = 0; d <= round_block; d++) {
            if (d == round_block) {
                if (p->prime(p->user, chained, base - 1 + d)) return -10;
                if (sampled) draw_step += 1;
                break;
            }
            uint16_t* row = draft_rows.data() + (size_t)d * vocab;
            if (p->step(p->user, chained, base - 1 + d, row)) return -10;
            if (sampled) {
                Dist q;
                rc = shaped(row, vocab, cfg, sink.history.data(), (int64_t)sink.history.size(), sink.generated, q);
                if (rc < 0) return rc;
                chained = (int32_t)draw(q, cfg->seed, draw_step);
                draw_step += 1;
            } else {
                rc = select_token(row, vocab, cfg, sink.history.data(), (int64_t)sink.history.size(),
                                  sink.generated, &chained);
                if (rc < 0) return rc;
            }
            proposals.push_back(chained);
        }
        // :663-676
        feed.assign(1, next);
        feed.insert(feed.end(), proposals.begin(), proposals.end());
        const int64_t point = base;
        if (p->verify(p->user, feed.data(), (int)feed.size(), base, batch.data())) return -10;
        // :694-754, 861-879
        tso_round_result res;
        rc = tso_chain_round(batch.data(), sampled ? draft_rows.data() : nullptr, proposals.data(), round_block,
                             vocab, cfg, sink.history.data(), (int64_t)sink.history.size(), sink.generated,
                             g->max_new_tokens, g->stop_tokens, g->n_stop, draw_step, &res);
        if (rc < 0) return rc;
        out->rounds += 1;
        out->offered += round_block;
        out->accepted += res.accepted;
        if (adaptive && !truncated && !res.stopped) tso_adaptive_observe(&ad, round_block, res.accepted);
        for (int i = 0; i < res.accepted; i++) {
            const int32_t t = proposals[i];
            const bool st = std::find(g->stop_tokens, g->stop_tokens + g->n_stop, t) != g->stop_tokens + g->n_stop;
            if (!st) report(t);
            sink.commit(t);  // the same calls the round made on its copy of the sink
        }
        const int committed = res.committed;
        if (committed < round_block) {  // :800-814
            out->rollbacks += 1;
            if (p->rollback_retaining(p->user, point, committed + 1)) return -10;
        }
        if (p->rewind(p->user, base + committed)) return -10;  // :852-854
        draw_step = res.draw_step;
        if (res.stopped) {
            out->stop_reason = res.stopped;
            break;
        }
        next = res.next;
    }
    out->draw_step = draw_step;
    out->final_depth = adaptive ? ad.cur : g->block;
    return 0;
}
