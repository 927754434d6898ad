// Device-side acceptance for a speculative round: softmax statistics, greedy / rejection
// sampling acceptance, the residual or bonus draw, and the round's bookkeeping.
//
// Restates on the GPU what the reference runs on the host in f64
// (crates/runtime/src/speculative.rs:694-754,861-879; crates/selection/src/choose.rs:111-338,
// distribution.rs:61-126, derive.rs:19-45) so a round returns a few dozen bytes instead of
// m x vocab fp16 logits.
//
// Arithmetic: every probability is computed in f64 with the reference's operation sequence
//   e = exp(f64(w) - max);  p = e / sum;  weight = pow(p / top, 1/T);  prob = weight / total
// but `sum` and `total` are parallel (fixed-order, deterministic) reductions rather than one
// sequential loop, and the cumulative draw walks rank order (logit descending, index ascending)
// through a 65536-bin histogram keyed by the fp16 logit -- exp is monotone, so rank-by-exp is
// rank-by-logit -- instead of sorting the vocabulary.  Integer outputs can therefore differ
// from the host sequence only when a comparison is within ~1e-13 of flipping; every comparison's
// distance from flipping is folded into `min_margin` so a caller can see that it never was.
// Bin masses are accumulated as 2^-62 fixed point with integer atomics: order independent,
// hence bit-reproducible run to run.
//
// Repetition / presence / frequency penalties (sampled chain and tree rounds, the draft draws) are
// applied per candidate as it is read, from a per-token table of the history (see score_of);
// the kernels are compiled twice, and the variant without penalties is the code it always was.
#include <algorithm>
#include <cstring>

#include "tsv_internal.h"

namespace tsv {

namespace {

constexpr int NSEG = 64;          // index segments per vocabulary row
constexpr int MAX_DIST_ROWS = 32;  // target rows + drafter rows
constexpr int MAX_JOBS = 16;
constexpr int NSUB = 4;  // workgroups per segment in the mass / histogram pass
constexpr double FIX = 4611686018427387904.0;  // 2^62

struct RowStat {
    double mx, sum, total, top;
    double minp;               // penalised rounds: candidates with e < minp are out (0: off)
    int32_t cut_key, cut_idx;  // last surviving candidate in rank order (truncation off: 65536, INT_MAX)
    float cut_w;               // its score (penalised rounds: a rank bin can hold several values)
};
struct Cut {
    int32_t key, idx;
    float w, pad;
};

// Scratch layout inside AcceptScratch::stats (doubles):
//   [0, 4*32)                         truncation cut per distribution row (16 bytes each)
//   pmax / psum / ptot partials follow, then the residual pieces and the decisions
struct Layout {
    double* pmax;  // [rows][NSEG]
    double* psum;
    double* ptot;
    double* segtot;  // [jobs][NSEG * NSUB] residual mass per piece of a segment
    Cut* cut;        // [rows] truncation cut
};
__host__ __device__ inline Layout layout(double* base) {
    Layout l;
    l.pmax = base + 4 * MAX_DIST_ROWS;
    l.psum = l.pmax + MAX_DIST_ROWS * NSEG;
    l.ptot = l.psum + MAX_DIST_ROWS * NSEG;
    l.segtot = l.ptot + MAX_DIST_ROWS * NSEG;
    l.cut = (Cut*)base;
    return l;
}

struct Job {
    int32_t mode;  // 0 none, 1 draw from p, 2 draw from residual(p, q)
    int32_t row_p, row_q;
    double u;
};

struct Decision {
    Job job;
    int32_t accepted, committed, stopped, pad;
    uint64_t draw_step;
    double margin;
};

__device__ __forceinline__ float h2f(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }

// crates/selection/src/derive.rs:19-45
__device__ __forceinline__ uint64_t mix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
__device__ __forceinline__ double unit_draw(uint64_t seed, uint64_t position) {
    const uint64_t v = mix64(seed ^ (position * 0x9E3779B97F4A7C15ull));
    return (double)(v >> 11) * (1.0 / 9007199254740992.0);
}

// Rank key of an fp16 logit: 0 for the largest value, ascending as the logit falls; +0 and
// -0 share a key (they have the same exp, so the reference breaks their tie by index).
__device__ __forceinline__ uint32_t rank_key(uint16_t b) {
    if (b == 0x8000u) b = 0;
    const uint32_t asc = (b & 0x8000u) ? (uint32_t)(~b & 0xFFFFu) : (uint32_t)(b | 0x8000u);
    return 0xFFFFu - asc;
}

// Where the histogram keeps rank bin `key`: the two low 6-bit fields are swapped, so the 64
// consecutive keys one thread of the cumulative walk owns are 64 words apart and neighbouring
// threads read neighbouring words.
__device__ __forceinline__ uint32_t bin_addr(uint32_t key) {
    return (key & 0xF000u) | ((key & 63u) << 6) | ((key >> 6) & 63u);
}

// Whether candidate v (logit `bits`) is inside the row's truncated candidate set: the set is a
// prefix of the rank order (logit descending, index ascending), so it is described by its last
// member.
__device__ __forceinline__ bool survives(uint16_t bits, int v, const RowStat& s) {
    const int key = (int)rank_key(bits);
    return key < s.cut_key || (key == s.cut_key && v <= s.cut_idx);
}

// (p / top)^(1/T), choose.rs:296-311.  At T = 1 the power is the identity -- the host library's pow returns its
// argument exactly there -- and the device's software pow, the most expensive operation of these kernels, is skipped
// (a branch every lane takes the same way).
__device__ __forceinline__ double temper(double x, double inv_t) { return inv_t == 1.0 ? x : pow(x, inv_t); }

// choose.rs:296-319 for one candidate of a row whose statistics are known
__device__ __forceinline__ double prob_of(uint16_t bits, int v, const RowStat& s, double inv_t) {
    if (!survives(bits, v, s)) return 0.0;
    const double e = exp((double)h2f(bits) - s.mx);
    const double p = e / s.sum;
    return temper(p / s.top, inv_t) / s.total;
}

// ---- penalised scores -------------------------------------------------------------------------
// crates/selection/src/penalty.rs:15-82 through choose.rs:138-154: the repetition penalty divides
// (positive) or multiplies (other) the f32 score of every distinct token of the history once; the
// presence / frequency penalties subtract presence + frequency * count for every token of the
// generated suffix.  `pen_cnt[v]` holds, for the history the round started with, bit 31 = seen and
// the low bits = occurrences in the generated suffix; target row i of a chain round adds the i
// proposals committed before it was judged (speculative.rs:694-716: each accepted proposal goes
// through the sink before the next row is shaped) -- in general the tokens on the row's root path,
// which is the same rule for a tree node -- and drafter rows add nothing (speculative.rs:636-641).
//
// A penalised score is an f32 that need not be an fp16 value.  Its rank bin is the bin of the
// largest fp16 value not above it, so bins stay ordered; inside a bin the candidates with a score
// above the bin's own value come first (score descending, index ascending: the few "side"
// candidates), then the candidates exactly on the value in index order.
template <bool PEN>
__device__ __forceinline__ float score_of(const AcceptParams& ap, int row, int v, uint16_t bits) {
    float w = h2f(bits);
    if constexpr (PEN) {
        const uint32_t c = ap.pen_cnt[v];
        bool seen = (c >> 31) != 0;
        uint32_t gen = c & 0x7FFFFFFFu;
        // the tokens committed on the way to this row: its root path without the root (chain: rows 1..row)
        for (int s = row < ap.m ? row : 0; s > 0; s = ap.parent[s])
            if (ap.feed[s] == v) {
                seen = true;
                gen += 1;
            }
        if (ap.pen_has_rep && seen) {
            const float a = w > 0.0f ? __fdiv_rn(w, ap.pen_rep) : __fmul_rn(w, ap.pen_rep);
            w = fminf(fmaxf(a, -3.40282347e+38f), 3.40282347e+38f);
        }
        if (ap.pen_has_pf && gen != 0)
            w = __fsub_rn(w, (float)__dadd_rn(ap.pen_presence, __dmul_rn(ap.pen_frequency, (double)gen)));
    }
    return w;
}

// The largest fp16 value not above w (w clamped into the fp16 range first).
__device__ __forceinline__ uint16_t floor16(float w) {
    const float c = fminf(fmaxf(w, -65504.0f), 65504.0f);
    const _Float16 h = (_Float16)c;
    uint16_t b = __builtin_bit_cast(uint16_t, h);
    if ((float)h > c) {
        if ((b & 0x7FFFu) == 0)
            b = 0x8001u;  // below zero: the smallest negative value
        else if (b & 0x8000u)
            b += 1;
        else
            b -= 1;
    }
    return b;
}

template <bool PEN>
__device__ __forceinline__ uint32_t key_of(float w, uint16_t bits) {
    if constexpr (PEN) return rank_key(floor16(w));
    return rank_key(bits);
}

template <bool PEN>
__device__ __forceinline__ bool survives_w(float w, int key, int v, const RowStat& s) {
    if constexpr (PEN)
        return key < s.cut_key || (key == s.cut_key && (w > s.cut_w || (w == s.cut_w && v <= s.cut_idx)));
    return key < s.cut_key || (key == s.cut_key && v <= s.cut_idx);
}

// choose.rs:296-319 for a candidate given by its score
template <bool PEN>
__device__ __forceinline__ double prob_of_w(float w, int key, int v, const RowStat& s, double inv_t) {
    if (!survives_w<PEN>(w, key, v, s)) return 0.0;
    const double e = exp((double)w - s.mx);
    if constexpr (PEN) {
        if (e < s.minp) return 0.0;
    }
    const double p = e / s.sum;
    return temper(p / s.top, inv_t) / s.total;
}

template <typename T>
__device__ __forceinline__ T shfl_xor_t(T v, int o) {
    static_assert(sizeof(T) == 8, "64-bit only");
    uint64_t u = __builtin_bit_cast(uint64_t, v);
    uint32_t lo = __shfl_xor((uint32_t)u, o), hi = __shfl_xor((uint32_t)(u >> 32), o);
    return __builtin_bit_cast(T, ((uint64_t)hi << 32) | lo);
}

// Deterministic block sum: xor-butterfly inside a wave, then the waves in index order.
__device__ double block_sum_f64(double v, double* red) {
    for (int o = 32; o > 0; o >>= 1) v += shfl_xor_t(v, o);
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    double t = 0.0;
    for (int i = 0; i < nw; i++) t += red[i];
    return t;
}

__device__ __forceinline__ const uint16_t* row_ptr(const uint16_t* target, const uint16_t* draft, int m,
                                                   int vocab, int row) {
    return row < m ? target + (long)row * vocab : draft + (long)(row - m) * vocab;
}

// Wave-wide fold of a row's NSEG (= wave size) partials: lane s loads segment s, an xor
// butterfly combines them.  Both lanes of a pair add the same two operands, so every lane ends
// with the same bits, and every kernel that needs a row's statistics gets them this way.
__device__ __forceinline__ double wave_max_f64(double v) {
    for (int o = 32; o > 0; o >>= 1) v = fmax(v, shfl_xor_t(v, o));
    return v;
}
__device__ __forceinline__ double wave_sum_f64(double v) {
    for (int o = 32; o > 0; o >>= 1) v += shfl_xor_t(v, o);
    return v;
}
static_assert(NSEG == 64, "one lane per segment");

// ---- statistics, three short passes over every distribution row -------------------------
template <bool PEN>
__global__ __launch_bounds__(256) void k_row_max(const uint16_t* target, const uint16_t* draft, int m,
                                                 int vocab, double* scratch, int32_t* err,
                                                 unsigned long long* hist, int hist_words,
                                                 const AcceptParams* app) {
    __shared__ double red[4];
    const int row = blockIdx.y, seg = blockIdx.x;
    {
        // the rank histograms of this round's draws start from zero: every workgroup clears a slice
        const int nwg = gridDim.x * gridDim.y, wg = blockIdx.y * gridDim.x + blockIdx.x;
        const int per = (hist_words + nwg - 1) / nwg, h0 = wg * per, h1 = min(h0 + per, hist_words);
        for (int i = h0 + threadIdx.x; i < h1; i += 256) hist[i] = 0;
    }
    const uint16_t* p = row_ptr(target, draft, m, vocab, row);
    const int per = (vocab + NSEG - 1) / NSEG, v0 = seg * per, v1 = min(v0 + per, vocab);
    float mx = -INFINITY;
    bool bad = false;
    bool low = false;
    for (int v = v0 + threadIdx.x; v < v1; v += 256) {
        const uint16_t b = p[v];
        bad |= (b & 0x7C00u) == 0x7C00u;
        if constexpr (PEN) {
            const float w = score_of<true>(*app, row, v, b);
            low |= !(w >= -65504.0f);
            mx = fmaxf(mx, w);
        } else {
            mx = fmaxf(mx, h2f(b));
        }
    }
    if (bad) atomicOr(err, 1);
    if (low) atomicOr(err, 4);  // a penalised score below every fp16 value: no rank bin to put it in
    double d = (double)mx;
    for (int o = 32; o > 0; o >>= 1) d = fmax(d, shfl_xor_t(d, o));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = d;
    __syncthreads();
    if (threadIdx.x == 0) {
        Layout L = layout(scratch);
        L.pmax[row * NSEG + seg] = fmax(fmax(red[0], red[1]), fmax(red[2], red[3]));
        if (seg == 0) L.cut[row] = Cut{65536, 0x7FFFFFFF, 0.f, 0.f};  // no truncation until a cut is computed
    }
}

template <bool PEN>
__global__ __launch_bounds__(256) void k_row_sum(const uint16_t* target, const uint16_t* draft, int m,
                                                 int vocab, double* scratch, const AcceptParams* app) {
    __shared__ double red[4];
    const int row = blockIdx.y, seg = blockIdx.x;
    Layout L = layout(scratch);
    const double mx = wave_max_f64(L.pmax[row * NSEG + (threadIdx.x & 63)]);
    const uint16_t* p = row_ptr(target, draft, m, vocab, row);
    const int per = (vocab + NSEG - 1) / NSEG, v0 = seg * per, v1 = min(v0 + per, vocab);
    double acc = 0.0;
    for (int v = v0 + threadIdx.x; v < v1; v += 256) {
        float w;
        if constexpr (PEN)
            w = score_of<true>(*app, row, v, p[v]);
        else
            w = h2f(p[v]);
        acc += exp((double)w - mx);
    }
    acc = block_sum_f64(acc, red);
    if (threadIdx.x == 0) L.psum[row * NSEG + seg] = acc;
}

template <bool PEN>
__global__ __launch_bounds__(256) void k_row_total(const uint16_t* target, const uint16_t* draft, int m,
                                                   int vocab, double* scratch, double inv_t,
                                                   const AcceptParams* app) {
    __shared__ double red[4];
    const int row = blockIdx.y, seg = blockIdx.x;
    Layout L = layout(scratch);
    const double mx = wave_max_f64(L.pmax[row * NSEG + (threadIdx.x & 63)]);
    const double sum = wave_sum_f64(L.psum[row * NSEG + (threadIdx.x & 63)]);
    const double top = 1.0 / sum;  // the arg-max candidate has e == exp(0) == 1
    const uint16_t* p = row_ptr(target, draft, m, vocab, row);
    const int per = (vocab + NSEG - 1) / NSEG, v0 = seg * per, v1 = min(v0 + per, vocab);
    RowStat cs;
    cs.cut_key = L.cut[row].key;
    cs.cut_idx = L.cut[row].idx;
    cs.cut_w = L.cut[row].w;
    double acc = 0.0;
    for (int v = v0 + threadIdx.x; v < v1; v += 256) {
        const uint16_t b = p[v];
        if constexpr (PEN) {
            const float w = score_of<true>(*app, row, v, b);
            if (!survives_w<true>(w, (int)key_of<true>(w, b), v, cs)) continue;
            const double e = exp((double)w - mx);
            if (app->has_min_p && e < app->min_p) continue;
            acc += temper((e / sum) / top, inv_t);
        } else {
            if (!survives(b, v, cs)) continue;
            const double e = exp((double)h2f(b) - mx);
            acc += temper((e / sum) / top, inv_t);
        }
    }
    acc = block_sum_f64(acc, red);
    if (threadIdx.x == 0) L.ptot[row * NSEG + seg] = acc;
}

// Called by one whole wave: the finished statistics of `row`, identical in every lane.
__device__ RowStat load_stat(const Layout& L, int row) {
    const int lane = threadIdx.x & 63;
    RowStat s;
    s.mx = wave_max_f64(L.pmax[row * NSEG + lane]);
    s.sum = wave_sum_f64(L.psum[row * NSEG + lane]);
    s.top = 1.0 / s.sum;
    s.total = wave_sum_f64(L.ptot[row * NSEG + lane]);
    s.cut_key = L.cut[row].key;
    s.cut_idx = L.cut[row].idx;
    s.cut_w = L.cut[row].w;
    s.minp = 0.0;
    return s;
}

__device__ __forceinline__ void fold_margin(double& margin, double a, double b) {
    const double scale = fmax(fabs(a), fabs(b));
    if (scale == 0.0) return;  // two exact zeros (a candidate outside both truncated sets): nothing can flip
    margin = fmin(margin, fabs(a - b) / scale);
}

// TokenSink::commit restricted to what a token-id interface can see
// (crates/runtime/src/token_sink.rs:64-124): 0 continue, 1 stop token, 2 budget.
__device__ int sink_commit(const AcceptParams& ap, int32_t token, uint64_t& generated, int32_t& committed) {
    generated += 1;
    for (int i = 0; i < ap.n_stop; i++)
        if (ap.stop_tokens[i] == token) return 1;
    if (ap.max_new_tokens != 0 && generated >= ap.max_new_tokens) return 2;
    committed += 1;
    return 0;
}

// speculative.rs:694-754: the sequential walk over the proposals of a sampled chain round.
// pxs / qxs: p_i(x_i) and q_i(x_i) of every proposal, computed by the caller in parallel (one lane
// per proposal: an f64 exp + pow chain per value is long for a single thread to walk k times).
__device__ Decision decide_chain_sampled(const AcceptParams& ap, const double* pxs, const double* qxs) {
    Decision d;
    d.job.mode = 0;
    d.job.row_p = d.job.row_q = 0;
    d.job.u = 0.0;
    d.accepted = d.committed = d.stopped = d.pad = 0;
    d.margin = 1.0;
    uint64_t ds = ap.draw_step, gen = ap.generated;
    int reject = -1;
    for (int i = 0; i < ap.k; i++) {
        const int32_t x = ap.feed[i + 1];
        const double px = pxs[i], qx = qxs[i];
        const double r = unit_draw(ap.seed, ds);
        ds += 1;
        fold_margin(d.margin, r * qx, px);
        if (r * qx <= px) {
            d.accepted += 1;
            if ((d.stopped = sink_commit(ap, x, gen, d.committed))) break;
        } else {
            reject = i;
            break;
        }
    }
    if (!d.stopped) {
        d.job.u = unit_draw(ap.seed, ds);
        ds += 1;
        if (reject >= 0) {
            d.job.mode = 2;
            d.job.row_p = reject;
            d.job.row_q = ap.m + reject;
        } else {
            d.job.mode = 1;
            d.job.row_p = d.accepted;
        }
    }
    d.draw_step = ds;
    return d;
}

// ---- masses + rank histogram --------------------------------------------------------------
// kind 0: the job comes out of the chain decision (every workgroup re-derives it: a few
// dozen f64 ops).  kind 1: jobs are "draw from drafter row j at position draw_step + j".
template <bool PEN>
__global__ __launch_bounds__(256) void k_mass_hist(const uint16_t* target, const uint16_t* draft,
                                                   const AcceptParams* app, double* scratch, double* work,
                                                   unsigned long long* hist, Decision* dec_out, int kind) {
    __shared__ Decision dec;
    __shared__ double red[4];
    __shared__ RowStat stats[MAX_DIST_ROWS];
    __shared__ uint16_t s_tb[TSV_MAX_ROWS], s_db[TSV_MAX_ROWS];
    __shared__ double s_px[TSV_MAX_ROWS], s_qx[TSV_MAX_ROWS];
    const AcceptParams& ap = *app;
    const int seg = blockIdx.x, jobi = blockIdx.y, sub = blockIdx.z;
    Layout L = layout(scratch);
    if (kind == 0 && (int)threadIdx.x < ap.k) {
        const int i = threadIdx.x;
        const int32_t x = ap.feed[i + 1];
        s_tb[i] = target[(long)i * ap.vocab + x];
        s_db[i] = draft[(long)i * ap.vocab + x];
    }
    {
        // every row's statistics, one wave per row at a time
        const int rows = kind == 0 ? ap.m + ap.k : ap.k;
        for (int r = threadIdx.x >> 6; r < rows; r += 4) {
            RowStat st = load_stat(L, r);
            if (PEN && ap.has_min_p) st.minp = ap.min_p;
            if ((threadIdx.x & 63) == 0) stats[r] = st;
        }
    }
    __syncthreads();
    if (kind == 0 && (int)threadIdx.x < ap.k) {
        const int i = threadIdx.x;
        const double it = 1.0 / ap.temperature;
        const int32_t x = ap.feed[i + 1];
        const float wt = score_of<PEN>(ap, i, x, s_tb[i]), wd = score_of<PEN>(ap, ap.m + i, x, s_db[i]);
        s_px[i] = prob_of_w<PEN>(wt, (int)key_of<PEN>(wt, s_tb[i]), x, stats[i], it);
        s_qx[i] = prob_of_w<PEN>(wd, (int)key_of<PEN>(wd, s_db[i]), x, stats[ap.m + i], it);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        if (kind == 0) {
            dec = decide_chain_sampled(ap, s_px, s_qx);
        } else {
            dec.job.mode = 1;
            dec.job.row_p = ap.m + jobi;
            dec.job.row_q = 0;
            dec.job.u = unit_draw(ap.seed, ap.draw_step + jobi);
            dec.accepted = dec.committed = dec.stopped = 0;
            dec.draw_step = ap.draw_step;
            dec.margin = 1.0;
        }
        if (seg == 0 && sub == 0) dec_out[jobi] = dec;
    }
    __syncthreads();
    const Job job = dec.job;
    if (job.mode == 0) return;
    const int vocab = ap.vocab;
    const double inv_t = 1.0 / ap.temperature;
    const RowStat sp = stats[job.row_p];
    const RowStat sq = stats[job.mode == 2 ? job.row_q : job.row_p];
    const uint16_t* lp = row_ptr(target, draft, ap.m, vocab, job.row_p);
    const uint16_t* lq = row_ptr(target, draft, ap.m, vocab, job.row_q);
    double* wp = work + (long)jobi * 2 * vocab;
    double* wr = wp + vocab;
    unsigned long long* hp = hist + (long)jobi * 2 * 65536;
    unsigned long long* hr = hp + 65536;
    const int per = (vocab + NSEG - 1) / NSEG, v0 = seg * per, v1 = min(v0 + per, vocab);
    double racc = 0.0;
    for (int v = v0 + sub * 256 + threadIdx.x; v < v1; v += 256 * NSUB) {
        const uint16_t b = lp[v];
        const float w = score_of<PEN>(ap, job.row_p, v, b);
        const uint32_t rk = key_of<PEN>(w, b);
        const double pv = prob_of_w<PEN>(w, (int)rk, v, sp, inv_t);
        const uint32_t key = bin_addr(rk);
        wp[v] = pv;
        if (pv > 0.0) atomicAdd(hp + key, (unsigned long long)(pv * FIX));
        if (job.mode == 2) {
            const uint16_t bq = lq[v];
            const float wq = score_of<PEN>(ap, job.row_q, v, bq);
            const double mv = fmax(pv - prob_of_w<PEN>(wq, (int)key_of<PEN>(wq, bq), v, sq, inv_t), 0.0);
            wr[v] = mv;
            racc += mv;
            if (mv > 0.0) atomicAdd(hr + key, (unsigned long long)(mv * FIX));
        }
    }
    if (job.mode == 2) {
        racc = block_sum_f64(racc, red);
        if (threadIdx.x == 0) L.segtot[(jobi * NSEG + seg) * NSUB + sub] = racc;
    }
}

// Calls on_match(v) for every index v in [v0, v1) whose logit bits are `want` (or -0 when the
// bin is the zero bin), eight keys per 16-byte load when the row allows it.
template <class Fn>
__device__ __forceinline__ void scan_chunk(const uint16_t* lp, int v0, int v1, uint32_t want, bool zero_bin, bool vec,
                                           Fn&& on_match) {
    // sixty-four keys at a time while the range lasts: the eight loads are in flight together (the loop below, one
    // load per turn with the matches' own loads behind it, waits out a memory round trip per eight keys)
    if (vec) {
        for (; v0 + 64 <= v1; v0 += 64) {
            uint4 q[8];
#pragma unroll
            for (int i = 0; i < 8; i++) q[i] = *(const uint4*)(lp + v0 + 8 * i);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint32_t w[4] = {q[i].x, q[i].y, q[i].z, q[i].w};
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const uint32_t bits = (w[j >> 1] >> (16 * (j & 1))) & 0xFFFFu;
                    if (bits == want || (zero_bin && bits == 0x8000u)) on_match(v0 + 8 * i + j);
                }
            }
        }
    }
    for (int g = v0; g < v1; g += 8) {
        uint32_t w[4];
        if (vec && g + 8 <= v1) {
            const uint4 q = *(const uint4*)(lp + g);
            w[0] = q.x;
            w[1] = q.y;
            w[2] = q.z;
            w[3] = q.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t lo = g + 2 * j < v1 ? lp[g + 2 * j] : (want ^ 0x4000u);
                const uint32_t hi = g + 2 * j + 1 < v1 ? lp[g + 2 * j + 1] : (want ^ 0x4000u);
                w[j] = lo | (hi << 16);
            }
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t bits = (w[j >> 1] >> (16 * (j & 1))) & 0xFFFFu;
            if (bits == want || (zero_bin && bits == 0x8000u)) on_match(g + j);
        }
    }
}

// ---- truncation of the candidate set (top-k, top-p, min-p) ---------------------------------
// choose.rs:111-228 / truncation.rs:79-236: candidates are ranked by softmax mass descending, ties
// by ascending index; top-k keeps the first k, top-p the shortest prefix whose cumulative
// `e / sum` reaches top_p, min-p those with e >= min_p * e_top.  All three keep a PREFIX of the
// rank order, so the surviving set is described by its last member (rank bin, index); it is found
// from per-row histograms over the 65536 rank bins (candidates per bin, fixed-point mass per
// bin) instead of a sort, and the one bin the cut falls into is resolved in index order.
__global__ __launch_bounds__(256) void k_trunc_clear(unsigned long long* tmass, uint32_t* tcount, int rows) {
    const size_t n = (size_t)rows * 65536;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        tmass[i] = 0;
        tcount[i] = 0;
    }
}

template <bool PEN>
__global__ __launch_bounds__(256) void k_trunc_hist(const uint16_t* target, const uint16_t* draft, int m, int vocab,
                                                    double* scratch, unsigned long long* tmass, uint32_t* tcount,
                                                    int want_mass, const AcceptParams* app) {
    const int row = blockIdx.y, seg = blockIdx.x, lane = threadIdx.x & 63;
    Layout L = layout(scratch);
    const double mx = wave_max_f64(L.pmax[row * NSEG + lane]);
    const double sum = wave_sum_f64(L.psum[row * NSEG + lane]);
    const uint16_t* p = row_ptr(target, draft, m, vocab, row);
    const int per = (vocab + NSEG - 1) / NSEG, v0 = seg * per, v1 = min(v0 + per, vocab);
    unsigned long long* hm = tmass + (size_t)row * 65536;
    uint32_t* hc = tcount + (size_t)row * 65536;
    for (int v = v0 + threadIdx.x; v < v1; v += 256) {
        const uint16_t b = p[v];
        float w;
        if constexpr (PEN)
            w = score_of<true>(*app, row, v, b);
        else
            w = h2f(b);
        const uint32_t key = bin_addr(key_of<PEN>(w, b));
        unsigned long long mass = 0;
        if (want_mass) mass = (unsigned long long)((exp((double)w - mx) / sum) * FIX);
        // a run of equal logits (a flat row) would serialise on one address: one lane adds for all
        const uint32_t first = __builtin_amdgcn_readfirstlane(key);
        const unsigned long long active = __ballot(1);
        if (!PEN && __ballot(key == first) == active) {  // (equal keys are equal masses only without penalties)
            if (lane == (int)__builtin_ctzll(active)) {
                const int n = __builtin_popcountll(active);
                atomicAdd(hc + key, (uint32_t)n);
                if (want_mass) atomicAdd(hm + key, mass * (unsigned long long)n);
            }
        } else {
            atomicAdd(hc + key, 1u);
            if (want_mass && mass) atomicAdd(hm + key, mass);
        }
    }
}

// fp16 bits whose rank key is `key` (inverse of rank_key; the zero bin maps to +0)
__device__ __forceinline__ uint32_t key_bits(int key) {
    const uint32_t asc = 0xFFFFu - (uint32_t)key;
    return (asc & 0x8000u) ? (asc & 0x7FFFu) : (~asc & 0xFFFFu);
}

// The candidates of rank bin `bin` that sit exactly on the bin's value, in index order over
// [v0, v1).  Without penalties they are found by their fp16 bits.
template <bool PEN, class Fn>
__device__ __forceinline__ void scan_on(const AcceptParams& ap, int row, const uint16_t* lp, int v0, int v1, int bin,
                                        bool vec, Fn&& on_match) {
    const uint32_t want = key_bits(bin);
    if constexpr (PEN) {
        const float g = h2f((uint16_t)want);
        for (int v = v0; v < v1; v++)
            if (score_of<true>(ap, row, v, lp[v]) == g) on_match(v);
    } else {
        scan_chunk(lp, v0, v1, want, want == 0, vec, on_match);
    }
}

// Penalised rounds, whole workgroup of 1024 threads: the candidates of `row` whose score falls
// into rank bin `bin` without being the bin's own value, ordered by score descending, index
// ascending, in sorted[0 .. n).  They precede the bin's on-value candidates in rank order.
constexpr int SIDE_CAP = 1024;
struct SideEnt {
    float w;
    int32_t v;
};
__device__ int collect_side(const AcceptParams& ap, int row, const uint16_t* lp, int bin, SideEnt* raw,
                            SideEnt* sorted, int* counter, int32_t* err) {
    const int tid = threadIdx.x;
    const float g = h2f((uint16_t)key_bits(bin));
    __syncthreads();
    if (tid == 0) *counter = 0;
    __syncthreads();
    for (int v = tid; v < ap.vocab; v += 1024) {
        bool flagged = ap.pen_cnt[v] != 0;
        for (int s = row < ap.m ? row : 0; s > 0; s = ap.parent[s]) flagged |= ap.feed[s] == v;
        if (!flagged) continue;  // an untouched score is an fp16 value: on its bin's value
        const float w = score_of<true>(ap, row, v, lp[v]);
        if (w != g && (int)rank_key(floor16(w)) == bin) {
            const int i = atomicAdd(counter, 1);
            if (i < SIDE_CAP) raw[i] = SideEnt{w, v};
        }
    }
    __syncthreads();
    int n = *counter;
    if (n > SIDE_CAP) {  // refused: more penalised candidates between two neighbouring fp16 values than the list holds
        if (tid == 0) atomicOr(err, 8);
        n = SIDE_CAP;
    }
    for (int i = tid; i < n; i += 1024) {
        const SideEnt me = raw[i];
        int rank = 0;
        for (int j = 0; j < n; j++) rank += raw[j].w > me.w || (raw[j].w == me.w && raw[j].v < me.v);
        sorted[rank] = me;
    }
    __syncthreads();
    return n;
}

// Exclusive prefix of a 64-bit value over the 1024 threads of a workgroup; *total gets the sum.
__device__ unsigned long long block_scan_u64(unsigned long long loc, unsigned long long* wsum,
                                             unsigned long long* total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned long long inc = loc;
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t lo = __shfl_up((uint32_t)inc, o), hi = __shfl_up((uint32_t)(inc >> 32), o);
        const unsigned long long up = ((unsigned long long)hi << 32) | lo;
        if (lane >= o) inc += up;
    }
    __syncthreads();
    if (lane == 63) wsum[wave] = inc;
    __syncthreads();
    unsigned long long wbase = 0, t = 0;
    for (int i = 0; i < 16; i++) {
        if (i < wave) wbase += wsum[i];
        t += wsum[i];
    }
    *total = t;
    return wbase + inc - loc;
}

// One workgroup per distribution row.
template <bool PEN>
__global__ __launch_bounds__(1024) void k_trunc_cut(const uint16_t* target, const uint16_t* draft,
                                                    const AcceptParams* app, int m, double* scratch,
                                                    const unsigned long long* tmass, const uint32_t* tcount,
                                                    AcceptResult* res, int32_t* err) {
    __shared__ SideEnt s_raw[PEN ? SIDE_CAP : 1], s_sorted[PEN ? SIDE_CAP : 1];
    __shared__ int s_nside;
    __shared__ unsigned long long wsum[16];
    __shared__ unsigned long long s_before_p;
    __shared__ int s_bin_k, s_j_k, s_bin_p, s_cnt_p, s_minp_key, s_bin, s_j, s_idx;
    __shared__ double s_margin;
    const AcceptParams& ap = *app;
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int vocab = ap.vocab;
    Layout L = layout(scratch);
    const double mx = wave_max_f64(L.pmax[row * NSEG + lane]);
    const double sum = wave_sum_f64(L.psum[row * NSEG + lane]);
    const uint32_t* cmine = tcount + (size_t)row * 65536 + (tid >> 6) * 4096 + (tid & 63);
    const unsigned long long* mmine = tmass + (size_t)row * 65536 + (tid >> 6) * 4096 + (tid & 63);
    if (tid == 0) {
        s_bin_k = s_bin_p = s_minp_key = s_bin = -1;
        s_idx = 0x7FFFFFFF;
        s_margin = 1.0;
    }
    __syncthreads();
    unsigned long long total, total_p = 0;
    if (ap.top_k > 0) {
        unsigned long long loc = 0;
#pragma unroll 16
        for (int i = 0; i < 64; i++) loc += cmine[i * 64];
        const unsigned long long excl = block_scan_u64(loc, wsum, &total);
        const unsigned long long K = (unsigned long long)ap.top_k;
        if (excl < K && K <= excl + loc) {
            unsigned long long c = excl;
            for (int i = 0; i < 64; i++) {
                const unsigned long long cv = cmine[i * 64];
                if (K <= c + cv) {
                    s_bin_k = tid * 64 + i;
                    s_j_k = (int)(K - c);
                    break;
                }
                c += cv;
            }
        }
    }
    if (ap.has_top_p) {
        unsigned long long loc = 0;
#pragma unroll 16
        for (int i = 0; i < 64; i++) loc += mmine[i * 64];
        const unsigned long long excl = block_scan_u64(loc, wsum, &total);
        total_p = total;
        const unsigned long long tgt = (unsigned long long)(ap.top_p * FIX);
        if (excl < tgt && tgt <= excl + loc) {
            unsigned long long c = excl;
            for (int i = 0; i < 64; i++) {
                const unsigned long long mv = mmine[i * 64];
                if (mv > 0 && tgt <= c + mv) {
                    s_bin_p = tid * 64 + i;
                    s_before_p = c;
                    s_cnt_p = (int)cmine[i * 64];
                    break;
                }
                c += mv;
            }
        }
    }
    if (!PEN && ap.has_min_p) {  // (penalised rounds test e >= min_p per candidate instead)
        int best = -1;
        for (int i = 0; i < 64; i++) {
            const int key = tid * 64 + i;
            const uint32_t bits = key_bits(key);
            if ((bits & 0x7C00u) == 0x7C00u) continue;  // no finite logit has this key
            if (exp((double)h2f((uint16_t)bits) - mx) >= ap.min_p) best = key;  // e_top == exp(0) == 1
        }
        if (best >= 0) atomicMax(&s_minp_key, best);
    }
    __syncthreads();
    const uint16_t* lp = row_ptr(target, draft, m, vocab, row);
    int ns_p = 0;  // penalised rounds: the top-p bin's candidates above the bin's own value
    if constexpr (PEN) {
        if (s_bin_p >= 0) ns_p = collect_side(ap, row, lp, s_bin_p, s_raw, s_sorted, &s_nside, err);
    }
    if (tid == 0) {
        int bin = s_bin_k, j = s_bin_k >= 0 ? s_j_k : 0;
        if (s_bin_p >= 0) {
            // how many candidates of the bin it takes to reach top_p: each carries the same mass
            const double pm = exp((double)h2f((uint16_t)key_bits(s_bin_p)) - mx) / sum;
            double before = (double)s_before_p / FIX;
            long taken = 0;  // candidates above the bin's value, each with a mass of its own
            bool reached = false;
            double mg_side = 1.0;
            if constexpr (PEN) {
                for (int i = 0; i < ns_p && !reached; i++) {
                    before += exp((double)s_sorted[i].w - mx) / sum;
                    taken += 1;
                    fold_margin(mg_side, before, ap.top_p);
                    reached = before >= ap.top_p;
                }
                s_cnt_p -= ns_p;
            }
            long jp = reached || s_cnt_p <= 0 ? 0 : (long)ceil((ap.top_p - before) / pm);
            if (reached || s_cnt_p <= 0) {
                s_margin = mg_side;
                jp = taken;
                if (bin < 0 || s_bin_p < bin || (s_bin_p == bin && jp < j)) {
                    bin = s_bin_p;
                    j = (int)jp;
                }
            } else {
                jp = jp < 1 ? 1 : jp;
                while (jp > 1 && before + (double)(jp - 1) * pm >= ap.top_p) jp--;
                while (jp < s_cnt_p && before + (double)jp * pm < ap.top_p) jp++;
                jp = jp > s_cnt_p ? s_cnt_p : jp;
                double mg = 1.0;
                fold_margin(mg, before + (double)jp * pm, ap.top_p);
                if (jp > 1 || s_before_p > 0) fold_margin(mg, before + (double)(jp - 1) * pm, ap.top_p);
                s_margin = fmin(mg, mg_side);
                jp += taken;
                if (bin < 0 || s_bin_p < bin || (s_bin_p == bin && jp < j)) {
                    bin = s_bin_p;
                    j = (int)jp;
                }
            }
        }
        if (ap.has_top_p && s_bin_p < 0) {  // the cumulative mass never reached top_p: everything ranked survives
            double mg = 1.0;
            fold_margin(mg, (double)total_p / FIX, ap.top_p);
            s_margin = mg;
        }
        s_bin = bin;
        s_j = j;
    }
    __syncthreads();
    const int bin = s_bin;
    int j = s_j;
    float cut_w = bin >= 0 ? h2f((uint16_t)key_bits(bin)) : 0.f;
    if (bin >= 0 && j < (int)tcount[(size_t)row * 65536 + bin_addr(bin)]) {
        bool on_value = true;
        if constexpr (PEN) {
            // the bin's candidates above its own value come first in rank order
            const int ns = bin == s_bin_p ? ns_p : collect_side(ap, row, lp, bin, s_raw, s_sorted, &s_nside, err);
            if (j <= ns) {
                if (tid == 0) s_idx = s_sorted[j - 1].v;
                cut_w = s_sorted[j - 1].w;
                on_value = false;
            } else {
                j -= ns;
            }
        }
        if (on_value) {
            // the j-th candidate on the bin's value in index order
            const int per = ((vocab + 1023) / 1024 + 7) & ~7, v0 = min(tid * per, vocab), v1 = min(v0 + per, vocab);
            const bool vec = ((uintptr_t)lp & 15) == 0;
            int n = 0;
            scan_on<PEN>(ap, row, lp, v0, v1, bin, vec, [&](int) { n++; });
            const unsigned long long excl = block_scan_u64((unsigned long long)n, wsum, &total);
            if ((int)excl < j && j <= (int)excl + n) {
                int c = (int)excl;
                scan_on<PEN>(ap, row, lp, v0, v1, bin, vec, [&](int v) {
                    c++;
                    if (c == j) s_idx = v;
                });
            }
        }
        __syncthreads();
    }
    if (tid == 0) {
        Cut cut{65536, 0x7FFFFFFF, 0.f, 0.f};
        if (bin >= 0) cut = Cut{bin, s_idx, cut_w, 0.f};
        if (!PEN && ap.has_min_p && s_minp_key >= 0 && s_minp_key < cut.key) cut = Cut{s_minp_key, 0x7FFFFFFF, 0.f, 0.f};
        L.cut[row] = cut;
        atomicMin((unsigned long long*)&res->min_margin, __builtin_bit_cast(unsigned long long, s_margin));
    }
}

// ---- the cumulative walk --------------------------------------------------------------------
// One workgroup per job.  Finds the rank bin in which the cumulative mass first exceeds the
// uniform (exact integer prefix over the fixed-point bins, which the round's first kernel zeroed), then
// walks that bin's candidates in index order in f64.
constexpr int PICK_MASK_GROUPS = 32;  // groups of eight entries per thread the match mask holds: vocabularies to 262 144
template <bool PEN>
__global__ __launch_bounds__(1024) void k_pick(const uint16_t* target, const uint16_t* draft,
                                               const AcceptParams* app, double* scratch, const double* work,
                                               unsigned long long* hist, const Decision* dec_in,
                                               AcceptResult* res, int32_t* tokens_out, int32_t* err,
                                               int kind) {
    __shared__ SideEnt s_raw[PEN ? SIDE_CAP : 1], s_sorted[PEN ? SIDE_CAP : 1];
    __shared__ uint32_t s_mask[PEN ? 1 : 1024 * PICK_MASK_GROUPS / 4];  // one bit per vocabulary entry: on the bin's value
    __shared__ int s_nside, s_side_last;
    __shared__ double s_side_sum;
    __shared__ unsigned long long wsum[16];
    __shared__ double dsum[16];
    __shared__ unsigned long long s_total, s_before;
    __shared__ int s_bin, s_last_bin, s_token, s_fallback;
    __shared__ double s_cum_before, s_cum_at;
    const AcceptParams& ap = *app;
    const int jobi = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const Decision dec = dec_in[jobi];
    Layout L = layout(scratch);
    const int vocab = ap.vocab;
    int token = -1;
    double margin = dec.margin;

    if (dec.job.mode != 0) {
        int mode = dec.job.mode;
        double R = 1.0;
        if (mode == 2) {
            // residual mass: the pieces' partial sums folded in a fixed order
            static_assert(NSEG * NSUB == 256, "four waves fold the pieces");
            if (tid < 256) {
                const double part = wave_sum_f64(L.segtot[jobi * NSEG * NSUB + tid]);
                if (lane == 0) dsum[wave] = part;
            }
            __syncthreads();
            R = (dsum[0] + dsum[1]) + (dsum[2] + dsum[3]);
            __syncthreads();
            if (R < 1e-12) mode = 1;  // distribution.rs:96-126: residual underflow -> plain p draw
        }
        unsigned long long* hp = hist + (long)jobi * 2 * 65536;
        unsigned long long* hsel = mode == 2 ? hp + 65536 : hp;
        const double* w = kind == 2 ? work + (long)dec.pad * vocab : work + (long)jobi * 2 * vocab + (mode == 2 ? vocab : 0);
        const uint16_t* lp = row_ptr(target, draft, ap.m, vocab, dec.job.row_p);

        // 64 consecutive rank bins per thread (see bin_addr); integer sums are exact and order
        // independent
        const unsigned long long* hmine = hsel + (tid >> 6) * 4096 + (tid & 63);
        // (one workgroup reads the whole histogram: what bounds it is how many loads a wave keeps in flight, so the 64
        // bins come as two rounds of 32 loads)
        unsigned long long quarter[4], loc = 0;  // the bins' sum in four runs of sixteen: the rescan below needs one run
#pragma unroll
        for (int half = 0; half < 2; half++) {
            unsigned long long hv[32];
#pragma unroll
            for (int i = 0; i < 32; i++) hv[i] = hmine[(half * 32 + i) * 64];
#pragma unroll
            for (int b = 0; b < 2; b++) {
                unsigned long long q = 0;
#pragma unroll
                for (int i = 0; i < 16; i++) q += hv[b * 16 + i];
                quarter[half * 2 + b] = q;
                loc += q;
            }
        }
        unsigned long long inc = loc;
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t lo = __shfl_up((uint32_t)inc, o), hi = __shfl_up((uint32_t)(inc >> 32), o);
            const unsigned long long up = ((unsigned long long)hi << 32) | lo;
            if (lane >= o) inc += up;
        }
        if (lane == 63) wsum[wave] = inc;
        if (tid == 0) {
            s_bin = -1;
            s_last_bin = -1;
            s_token = -1;
            s_fallback = 0;
        }
        __syncthreads();
        unsigned long long wbase = 0, total = 0;
        for (int i = 0; i < 16; i++) {
            if (i < wave) wbase += wsum[i];
            total += wsum[i];
        }
        const unsigned long long excl = wbase + inc - loc;
        // target in fixed point: u * total (the bins hold unnormalised mass in residual mode)
        const unsigned long long tgt = (unsigned long long)(dec.job.u * (double)total);
        if (loc > 0) atomicMax(&s_last_bin, tid * 64 + 63);
        if (excl <= tgt && tgt < excl + loc) {
            // the one thread whose 64 bins hold the target: first bin at which the running sum passes it.  Only the
            // run of sixteen the target falls into is fetched again, all of it at once (a loop over the 64 bins that
            // stops at the hit waits out one L2 round trip per bin)
            unsigned long long c = excl;
            int b = 0;
#pragma unroll
            for (int t = 0; t < 3; t++)
                if (b == t && !(tgt < c + quarter[t])) {
                    c += quarter[t];
                    b = t + 1;
                }
            unsigned long long hv[16];
#pragma unroll
            for (int i = 0; i < 16; i++) hv[i] = hmine[(b * 16 + i) * 64];
            unsigned long long before = c;
            int hit = -1;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                if (hit < 0 && tgt < c + hv[i]) {
                    hit = b * 16 + i;
                    before = c;
                }
                c += hv[i];
            }
            s_bin = tid * 64 + hit;
            s_before = before;
        }
        if (tid == 0) s_total = total;
        __syncthreads();
        int bin = s_bin;
        if (bin < 0) {
            // rounding at the tail: the reference falls back to the LAST surviving candidate
            // (choose.rs:333-338).  Last occupied bin, last matching index.
            const int lb = s_last_bin;  // upper end of the last occupied 64-bin group
            if (tid * 64 + 63 == lb) {
                int bb = lb;
                while (bb > tid * 64 && hsel[bin_addr(bb)] == 0) bb--;
                s_bin = bb;
                s_before = total;
                s_fallback = 1;
            }
            __syncthreads();
            bin = s_bin;
        }
        const bool fallback = s_fallback != 0;
        const double norm = (double)s_total;  // fixed-point total <-> 1.0 (p mode) or R (residual)
        const double cum0 = (double)s_before / norm;  // cumulative mass before this bin
        double side_sum = 0.0;
        if constexpr (PEN) {
            // the bin's candidates above its own value come first: few, walked by one thread
            const int ns = collect_side(ap, dec.job.row_p, lp, bin, s_raw, s_sorted, &s_nside, err);
            if (tid == 0) {
                double c = cum0;
                int last = -1;
                bool found = false;
                for (int i = 0; i < ns; i++) {
                    const int v = s_sorted[i].v;
                    const double wv = mode == 2 ? w[v] / R : w[v];
                    if (mode == 2 && !(wv > 0.0)) continue;
                    if (!fallback && !found && dec.job.u < c + wv) {
                        s_token = v;
                        s_cum_before = c;
                        s_cum_at = c + wv;
                        found = true;
                    }
                    c += wv;
                    last = v;
                }
                s_side_sum = c - cum0;
                s_side_last = last;
            }
            __syncthreads();
            side_sum = s_side_sum;
        }
        // walk the bin in index order: contiguous index chunk per thread
        const int per = ((vocab + 1023) / 1024 + 7) & ~7, v0 = min(tid * per, vocab), v1 = min(v0 + per, vocab);
        const bool vec = ((uintptr_t)lp & 15) == 0;
        // Without penalties a candidate of the bin is found by its fp16 bits.  The row is read ONCE, coalesced --
        // neighbouring lanes take neighbouring groups of eight entries, where a lane reading its own contiguous chunk
        // touches 64 cache lines per load -- and leaves one bit per entry in LDS; each thread then walks the bits of
        // its own chunk, here and again in the walk below, in the index order the sums are defined in.
        const int groups = per >> 3;
        const bool masked = !PEN && vec && groups <= PICK_MASK_GROUPS;
        if constexpr (!PEN) {
            if (masked) {
                uint8_t* mask8 = (uint8_t*)s_mask;
                const uint32_t want = key_bits(bin);
                const bool zero_bin = want == 0;
                // sixteen loads in flight per lane: a group past the row's last whole one reads group 0 and is discarded
                const int whole = vocab >> 3;  // groups of eight entries that lie wholly inside the row
                for (int g0 = 0; g0 < groups; g0 += 16) {
                    uint4 q[16];
#pragma unroll
                    for (int j = 0; j < 16; j++) {
                        const int g = (g0 + j) * 1024 + tid;
                        q[j] = *(const uint4*)(lp + (g0 + j < groups && g < whole ? (long)g * 8 : 0));
                    }
#pragma unroll
                    for (int j = 0; j < 16; j++) {
                        if (g0 + j >= groups) break;
                        const int g = (g0 + j) * 1024 + tid;
                        const uint32_t t[4] = {q[j].x, q[j].y, q[j].z, q[j].w};
                        uint32_t m = 0;
#pragma unroll
                        for (int h = 0; h < 8; h++) {
                            const uint32_t bits = (t[h >> 1] >> (16 * (h & 1))) & 0xFFFFu;
                            m |= (uint32_t)(bits == want || (zero_bin && bits == 0x8000u)) << h;
                        }
                        mask8[g] = g < whole ? (uint8_t)m : (uint8_t)0;
                    }
                }
                if ((vocab & 7) && whole < groups * 1024 && tid == (whole & 1023)) {  // the row's last, partial group
                    uint32_t m = 0;
                    for (int h = 0; h < (vocab & 7); h++) {
                        const uint32_t bits = lp[(long)whole * 8 + h];
                        m |= (uint32_t)(bits == want || (zero_bin && bits == 0x8000u)) << h;
                    }
                    mask8[whole] = (uint8_t)m;
                }
                __syncthreads();
            }
        }
        // on_match(v) for the candidates of this thread's chunk that sit on the bin's value, ascending
        auto for_matches = [&](auto&& on_match) {
            if constexpr (!PEN) {
                if (masked) {
                    const uint8_t* mine = (const uint8_t*)s_mask + tid * groups;
                    for (int k = 0; k < groups; k++)
                        for (uint32_t m = mine[k]; m; m &= m - 1) on_match(v0 + 8 * k + (__ffs(m) - 1));
                    return;
                }
            }
            scan_on<PEN>(ap, dec.job.row_p, lp, v0, v1, bin, vec, on_match);
        };
        double lsum = 0.0;
        int lastv = -1;
        for_matches([&](int v) {
            const double wv = mode == 2 ? w[v] / R : w[v];
            if (mode != 2 || wv > 0.0) {
                lsum += wv;
                lastv = v;
            }
        });
        double incd = lsum;
        for (int o = 1; o < 64; o <<= 1) {
            uint64_t u = __builtin_bit_cast(uint64_t, incd);
            uint32_t lo = __shfl_up((uint32_t)u, o), hi = __shfl_up((uint32_t)(u >> 32), o);
            const double up = __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
            if (lane >= o) incd += up;
        }
        if (lane == 63) dsum[wave] = incd;
        __syncthreads();
        double dbase = 0.0;
        for (int i = 0; i < wave; i++) dbase += dsum[i];
        const double before = PEN ? cum0 + side_sum + (dbase + incd - lsum) : cum0 + (dbase + incd - lsum);
        if (fallback) {
            if (lastv >= 0) atomicMax(&s_token, lastv);
        } else {
            const double u = dec.job.u;
            if (lsum > 0.0 && !(u < before) && u < before + lsum) {
                double c = before;
                bool found = false;
                for_matches([&](int v) {
                    if (found) return;
                    const double wv = mode == 2 ? w[v] / R : w[v];
                    if (mode == 2 && !(wv > 0.0)) return;
                    if (u < c + wv) {
                        s_token = v;
                        s_cum_before = c;
                        s_cum_at = c + wv;
                        found = true;
                        return;
                    }
                    c += wv;
                });
            }
        }
        __syncthreads();
        token = s_token;
        if (PEN && fallback && token < 0) token = s_side_last;  // no on-value candidate: the last of the others
        if (token < 0) {
            // the f64 walk and the fixed-point bin search disagreed by a rounding: the uniform
            // sits on a bin edge.  Take the bin's first (u below) or last candidate and report
            // a zero margin.
            if (lastv >= 0) atomicMax(&s_token, lastv);
            __syncthreads();
            token = s_token;
            if (PEN && token < 0) token = s_side_last;
            margin = 0.0;
        } else if (!fallback) {
            margin = fmin(margin, fmin(dec.job.u - s_cum_before, s_cum_at - dec.job.u));
        }
    }

    if (tid == 0) {
        if (kind == 1) {
            tokens_out[jobi] = token;
            if (jobi == 0) res->error = *err;
            // margins of the k draws are folded on the host side from res->min_margin
            atomicMin((unsigned long long*)&res->min_margin, __builtin_bit_cast(unsigned long long, margin));
        } else {
            res->accepted = dec.accepted;
            res->committed = dec.committed;
            res->stopped = dec.stopped;
            res->next = dec.stopped ? -1 : token;
            res->draw_step = dec.draw_step;
            res->path_len = dec.accepted + 1;
            for (int i = 0; i <= dec.accepted; i++) res->path[i] = kind == 2 ? tokens_out[i] : i;
            atomicMin((unsigned long long*)&res->min_margin, __builtin_bit_cast(unsigned long long, margin));
            res->error = *err;
        }
    }
}

// ---- sampled acceptance over a draft tree ---------------------------------------------------
// The reference has no multi-branch rejection sampler (speculative.rs:390-392 keeps tree rounds
// greedy); this follows the oracle's definition: at node `at`, with p the target distribution of
// row `at` and q the distribution its children were drawn from, the children are tried in slot
// order -- child x is accepted when r * q(x) <= p(x) for a fresh uniform r; a rejection replaces
// p by normalise(max(p - q, 0)) (kept as is when that mass is below 1e-12) -- and when no child
// survives the next token is drawn from the p that is left.  No stop / budget bookkeeping.
//
// First every node's p and q are written out as dense f64 rows by the whole chip (work slots
// 0..m-1 and m..2m-1); then the tree is walked one child test per launch.  A test is two lookups;
// only a rejection costs a pass over the vocabulary (slots 32 and 33 alternate as the residual,
// whose normalising division is applied when it is read, so a pass reads two rows and writes one).
constexpr int TREE_SCRATCH_SLOT = 2 * TSV_MAX_ROWS;  // two residual rows behind the 32 distribution rows

// The walk as a sequence of short chip-wide launches (one per child test there can be, then the
// finish): every workgroup re-derives the step's decision from the walk state (two lookups), a
// rejection's residual pass is spread over all of them, and the pass's total is folded by the next
// launch.  The state and the partial sums are double-buffered: launch k reads copy k & 1 and writes the
// other one, so a workgroup that starts late still sees what the previous launch left.
constexpr int TREE_WGS = 256;
struct TreeWalk {
    int32_t at, next_s, plen, which, done, pending, src_slot, pend_slot;
    double Z, margin;
    uint64_t ds;
    int32_t path[TSV_MAX_ROWS + 1];
    int32_t pad;
};
static_assert(sizeof(TreeWalk) % 8 == 0 && sizeof(TreeWalk) <= 32 * 8, "fits its slot of the statistics block");

// behind the decisions: two copies of the state (32 doubles each), then two sets of TREE_WGS partial sums
constexpr int STATS_DOUBLES = 4 * MAX_DIST_ROWS + 3 * MAX_DIST_ROWS * NSEG + MAX_JOBS * NSEG * NSUB + MAX_JOBS * 16;
constexpr int TREE_STATE_DOUBLES = 2 * 32 + 2 * TREE_WGS;
__device__ TreeWalk* tree_walk(double* scratch, int copy) { return (TreeWalk*)(scratch + STATS_DOUBLES + 32 * copy); }
__device__ double* tree_partials(double* scratch, int copy) { return scratch + STATS_DOUBLES + 64 + TREE_WGS * copy; }

template <bool PEN>
__global__ __launch_bounds__(256) void k_tree_probs(const uint16_t* target, const uint16_t* draft,
                                                    const AcceptParams* app, double* scratch, double* work) {
    __shared__ RowStat st;
    const AcceptParams& ap = *app;
    const int seg = blockIdx.x, row = blockIdx.y, vocab = ap.vocab;
    Layout L = layout(scratch);
    if (threadIdx.x < 64) {
        const RowStat s0 = load_stat(L, row);
        if (threadIdx.x == 0) st = s0;
    }
    __syncthreads();
    RowStat s0 = st;
    if (PEN && ap.has_min_p) s0.minp = ap.min_p;
    const double inv_t = 1.0 / ap.temperature;
    const uint16_t* lp = row_ptr(target, draft, ap.m, vocab, row);
    double* out = work + (long)row * vocab;
    if (seg == 0 && row == 0 && threadIdx.x == 0) {  // the walk starts at the root
        TreeWalk w;
        w.at = 0;
        w.next_s = 1;
        w.plen = 1;
        w.which = w.done = w.pending = w.src_slot = w.pend_slot = w.pad = 0;
        w.Z = 1.0;
        w.margin = 1.0;
        w.ds = ap.draw_step;
        w.path[0] = 0;
        *tree_walk(scratch, 0) = w;
    }
    const int per = (vocab + NSEG - 1) / NSEG, v0 = seg * per, v1 = min(v0 + per, vocab);
    for (int v = v0 + threadIdx.x; v < v1; v += 256) {
        const uint16_t b = lp[v];
        const float w = score_of<PEN>(ap, row, v, b);
        out[v] = prob_of_w<PEN>(w, (int)key_of<PEN>(w, b), v, s0, inv_t);
    }
}

// The state launch k starts from: copy k & 1 with the previous launch's residual pass resolved
// (its total decides whether the residual replaces the node's distribution: distribution.rs:96-126).
__device__ TreeWalk tree_state(double* scratch, int k, double* red) {
    TreeWalk w = *tree_walk(scratch, k & 1);
    if (w.pending) {
        const double part = (int)threadIdx.x < TREE_WGS ? tree_partials(scratch, k & 1)[threadIdx.x] : 0.0;
        const double total = block_sum_f64(part, red);
        if (total >= 1e-12) {
            w.src_slot = w.pend_slot;
            w.Z = total;
            w.which ^= 1;
        }
        w.pending = 0;
    }
    return w;
}

template <bool PEN>
__global__ __launch_bounds__(256) void k_tree_step(const AcceptParams* app, double* scratch, double* work, int k) {
    __shared__ double red[4];
    const AcceptParams& ap = *app;
    const int vocab = ap.vocab, m = ap.m;
    TreeWalk w = tree_state(scratch, k, red);
    TreeWalk* out = tree_walk(scratch, (k + 1) & 1);
    const bool writer = blockIdx.x == 0 && threadIdx.x == 0;
    int s = -1;
    if (!w.done)
        for (int c = w.next_s; c < m; c++)
            if (ap.parent[c] == w.at) {
                s = c;
                break;
            }
    if (s < 0) {  // nothing left to try below this node (or the walk had ended already)
        w.done = 1;
        if (writer) *out = w;
        return;
    }
    const double* src = work + (long)w.src_slot * vocab;  // the node's p; its values are src[v] / Z
    const double* q = work + (long)(m + w.at) * vocab;
    const int32_t x = ap.feed[s];
    const double r = unit_draw(ap.seed, w.ds);
    const double px = src[x] / w.Z, qx = q[x];
    fold_margin(w.margin, r * qx, px);
    w.ds += 1;
    w.next_s = s + 1;
    if (r * qx <= px) {
        w.path[w.plen] = s;
        w.plen += 1;
        w.at = s;
        w.src_slot = s;
        w.Z = 1.0;
        w.which = 0;
        if (writer) *out = w;
        return;
    }
    // residual max(p - q, 0) of this workgroup's slice; the next launch folds the totals
    double* dst = work + (long)(TREE_SCRATCH_SLOT + w.which) * vocab;
    const int per = (vocab + TREE_WGS - 1) / TREE_WGS, v0 = blockIdx.x * per, v1 = min(v0 + per, vocab);
    double acc = 0.0;
    for (int v = v0 + threadIdx.x; v < v1; v += 256) {
        const double mv = fmax(src[v] / w.Z - q[v], 0.0);
        dst[v] = mv;
        acc += mv;
    }
    acc = block_sum_f64(acc, red);
    if (threadIdx.x == 0) tree_partials(scratch, (k + 1) & 1)[blockIdx.x] = acc;
    w.pending = 1;
    w.pend_slot = TREE_SCRATCH_SLOT + w.which;
    if (writer) *out = w;
}

// After the last step: the rank histogram of what is left of p at the node the walk ended on, and the
// round's decision; the draw itself is k_pick's.
template <bool PEN>
__global__ __launch_bounds__(256) void k_tree_finish(const uint16_t* target, const AcceptParams* app, double* scratch,
                                                     double* work, unsigned long long* hist, Decision* dec_out,
                                                     int32_t* path_out, int k) {
    __shared__ double red[4];
    const AcceptParams& ap = *app;
    const int vocab = ap.vocab;
    const TreeWalk w = tree_state(scratch, k, red);
    Layout L = layout(scratch);
    unsigned long long* hr = hist + 65536;
    const double* src = work + (long)w.src_slot * vocab;
    const uint16_t* lpk = target + (long)w.at * vocab;
    const int per = (vocab + TREE_WGS - 1) / TREE_WGS, v0 = blockIdx.x * per, v1 = min(v0 + per, vocab);
    for (int v = v0 + threadIdx.x; v < v1; v += 256) {
        const double mv = src[v] / w.Z;
        if (mv > 0.0) {
            const uint16_t b = lpk[v];
            atomicAdd(hr + bin_addr(key_of<PEN>(score_of<PEN>(ap, w.at, v, b), b)), (unsigned long long)(mv * FIX));
        }
    }
    if (blockIdx.x != 0) return;
    // the draw divides the stored values by the fold of these pieces: Z, exactly
    if (threadIdx.x < NSEG * NSUB) L.segtot[threadIdx.x] = threadIdx.x == 0 ? w.Z : 0.0;
    if (threadIdx.x == 0) {
        for (int i = 0; i < w.plen; i++) path_out[i] = w.path[i];
        Decision d;
        d.job.mode = 2;
        d.job.row_p = w.at;
        d.job.row_q = 0;
        d.job.u = unit_draw(ap.seed, w.ds);
        d.accepted = w.plen - 1;
        d.committed = w.plen - 1;
        d.stopped = 0;
        d.pad = w.src_slot;  // the work slot the draw reads
        d.draw_step = w.ds + 1;
        d.margin = w.margin;
        dec_out[0] = d;
    }
}

// ---- greedy --------------------------------------------------------------------------------
// choose.rs:277-285: first maximum.  ARGMAX_SEG workgroups per target row, each over a contiguous
// run of the vocabulary: the best (value, index) of every run goes to a partial slot, and whoever
// needs the row's arg-max folds the runs in index order (a later run wins only with a strictly
// larger value, so ties go to the lower index whatever the split).
constexpr int ARGMAX_SEG = 16;

__global__ __launch_bounds__(256) void k_argmax_part(const uint16_t* target, int vocab, float* pv, int32_t* pi, int32_t* err) {
    __shared__ float bv[4];
    __shared__ int bi[4];
    const int row = blockIdx.y, seg = blockIdx.x;
    const uint16_t* p = target + (long)row * vocab;
    const int chunk = ((vocab + ARGMAX_SEG - 1) / ARGMAX_SEG + 7) & ~7;
    const int v0 = min(seg * chunk, vocab), v1 = min(v0 + chunk, vocab);
    float best = -INFINITY;
    int idx = 0x7FFFFFFF;
    bool bad = false;
    auto take = [&](uint16_t b, int v) {
        bad |= (b & 0x7C00u) == 0x7C00u;
        const float f = h2f(b);
        if (f > best || (f == best && v < idx)) {
            best = f;
            idx = v;
        }
    };
    if ((((uintptr_t)p) & 15) == 0) {  // eight logits per 16-byte load (v0 is a multiple of 8)
        const int i0 = v0 >> 3, i1 = v1 >> 3;
        for (int i = i0 + threadIdx.x; i < i1; i += 256) {
            const uint4 q = ((const uint4*)p)[i];
            const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int j = 0; j < 8; j++) take((uint16_t)(w[j >> 1] >> (16 * (j & 1))), 8 * i + j);
        }
        for (int v = max(i1 << 3, v0) + threadIdx.x; v < v1; v += 256) take(p[v], v);
    } else {
        for (int v = v0 + threadIdx.x; v < v1; v += 256) take(p[v], v);
    }
    if (bad) atomicOr(err, 1);
    for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o);
        const int oi = __shfl_xor(idx, o);
        if (ob > best || (ob == best && oi < idx)) {
            best = ob;
            idx = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        bv[threadIdx.x >> 6] = best;
        bi[threadIdx.x >> 6] = idx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 4; i++)
            if (bv[i] > best || (bv[i] == best && bi[i] < idx)) {
                best = bv[i];
                idx = bi[i];
            }
        pv[row * ARGMAX_SEG + seg] = best;
        pi[row * ARGMAX_SEG + seg] = idx;
    }
}

// the row's arg-max from its runs' partial results, read by one thread
__device__ __forceinline__ int32_t fold_argmax(const float* pv, const int32_t* pi, int row) {
    float v[ARGMAX_SEG];
    int32_t ix[ARGMAX_SEG];
#pragma unroll
    for (int s = 0; s < ARGMAX_SEG; s++) {
        v[s] = pv[row * ARGMAX_SEG + s];
        ix[s] = pi[row * ARGMAX_SEG + s];
    }
    float best = v[0];
    int32_t idx = ix[0];
#pragma unroll
    for (int s = 1; s < ARGMAX_SEG; s++)
        if (v[s] > best) {  // an empty run holds -inf and never wins
            best = v[s];
            idx = ix[s];
        }
    return idx;
}

__global__ void k_argmax_fold(const float* pv, const int32_t* pi, int rows, int32_t* out) {
    if ((int)threadIdx.x < rows) out[threadIdx.x] = fold_argmax(pv, pi, threadIdx.x);
}

// speculative.rs:736-754 (chain) and 494-550 (tree walk) at temperature 0, by one thread over the
// rows' arg-max tokens.
struct GreedyWalk {
    int32_t accepted, committed, stopped, next, path_len;
    int32_t path[TSV_MAX_ROWS + 1];
};
__device__ GreedyWalk walk_greedy(const AcceptParams& ap, const int32_t* amax) {
    GreedyWalk g;
    uint64_t gen = ap.generated;
    int32_t committed = 0, stopped = 0, next = -1;
    int at = 0, plen = 1;
    g.path[0] = 0;
    for (;;) {
        const int32_t want = amax[at];
        int hit = -1;
        if (ap.tree) {
            for (int s = 1; s < ap.m; s++)
                if (ap.parent[s] == at && ap.feed[s] == want) {
                    hit = s;
                    break;
                }
        } else if (at + 1 < ap.m && ap.feed[at + 1] == want) {
            hit = at + 1;
        }
        if (hit < 0) {
            next = want;
            break;
        }
        g.path[plen++] = hit;
        at = hit;
        if ((stopped = sink_commit(ap, want, gen, committed))) break;
    }
    g.accepted = plen - 1;
    g.committed = committed;
    g.stopped = stopped;
    g.next = stopped ? -1 : next;
    g.path_len = plen;
    return g;
}

__global__ void k_walk_greedy(const AcceptParams* app, const float* pv, const int32_t* pi, AcceptResult* res,
                              const int32_t* err) {
    __shared__ int32_t amax[TSV_MAX_ROWS];
    const AcceptParams& ap = *app;
    if ((int)threadIdx.x < ap.m) amax[threadIdx.x] = fold_argmax(pv, pi, threadIdx.x);
    __syncthreads();
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const GreedyWalk g = walk_greedy(ap, amax);
    for (int i = 0; i < g.path_len; i++) res->path[i] = g.path[i];
    res->accepted = g.accepted;
    res->committed = g.committed;
    res->stopped = g.stopped;
    res->next = g.next;
    res->draw_step = ap.draw_step;
    res->path_len = g.path_len;
    res->min_margin = 1.0;
    res->error = *err;
}

__global__ void k_clear_result(AcceptResult* res, int32_t* err) {
    if (threadIdx.x == 0) {
        *err = 0;
        res->error = 0;
        res->min_margin = 1.0;
    }
}

}  // namespace

// scratch.counters (ACCEPT_COUNTER_WORDS words): [0] error flag, [32..49) tree path, [64..) the greedy
// arg-max partials (value, then index, per row and run); decisions live after the
// statistics block; histograms and work arrays are separate allocations in AcceptScratch.
size_t accept_stats_doubles() { return STATS_DOUBLES + TREE_STATE_DOUBLES; }

static Decision* decisions(const AcceptScratch& sc) {
    return (Decision*)(sc.stats + 4 * MAX_DIST_ROWS + 3 * MAX_DIST_ROWS * NSEG + MAX_JOBS * NSEG * NSUB);
}

// Between the softmax sums and the reweighting totals: the truncation cut of every row.
template <bool PEN>
static void launch_trunc(hipStream_t s, const uint16_t* target, const uint16_t* draft, int m, int rows,
                         const AcceptParams* ap_dev, const AcceptParams& ap, const AcceptScratch& sc) {
    if (ap.top_k == 0 && !ap.has_top_p) {
        if (PEN || !ap.has_min_p) return;  // (penalised rounds test min-p per candidate)
    }
    unsigned long long* tm = (unsigned long long*)sc.tmass;
    if (ap.top_k != 0 || ap.has_top_p) {
        hipLaunchKernelGGL(k_trunc_clear, dim3(64 * rows), dim3(256), 0, s, tm, sc.tcount, rows);
        hipLaunchKernelGGL(k_trunc_hist<PEN>, dim3(NSEG, rows), dim3(256), 0, s, target, draft, m, ap.vocab, sc.stats, tm,
                           sc.tcount, ap.has_top_p, ap_dev);
    }
    hipLaunchKernelGGL(k_trunc_cut<PEN>, dim3(rows), dim3(1024), 0, s, target, draft, ap_dev, m, sc.stats, tm, sc.tcount,
                       sc.result, (int32_t*)sc.counters);
}

// The statistics of `rows` distribution rows, their truncation cuts and reweighting totals.
template <bool PEN>
static void launch_stats(hipStream_t s, const uint16_t* target, const uint16_t* draft, int m, int rows, int hist_words,
                         const AcceptParams* ap_dev, const AcceptParams& ap, const AcceptScratch& sc) {
    int32_t* err = (int32_t*)sc.counters;
    const double inv_t = 1.0 / ap.temperature;
    hipLaunchKernelGGL(k_row_max<PEN>, dim3(NSEG, rows), dim3(256), 0, s, target, draft, m, ap.vocab, sc.stats, err,
                       (unsigned long long*)sc.hist, hist_words, ap_dev);
    hipLaunchKernelGGL(k_row_sum<PEN>, dim3(NSEG, rows), dim3(256), 0, s, target, draft, m, ap.vocab, sc.stats, ap_dev);
    launch_trunc<PEN>(s, target, draft, m, rows, ap_dev, ap, sc);
    hipLaunchKernelGGL(k_row_total<PEN>, dim3(NSEG, rows), dim3(256), 0, s, target, draft, m, ap.vocab, sc.stats, inv_t,
                       ap_dev);
}

template <bool PEN>
static void launch_chain_sampled(hipStream_t s, const uint16_t* target, const uint16_t* draft,
                                 const AcceptParams* ap_dev, const AcceptParams& ap, const AcceptScratch& sc) {
    int32_t* err = (int32_t*)sc.counters;
    launch_stats<PEN>(s, target, draft, ap.m, ap.m + ap.k, 2 * 65536, ap_dev, ap, sc);
    hipLaunchKernelGGL(k_mass_hist<PEN>, dim3(NSEG, 1, NSUB), dim3(256), 0, s, target, draft, ap_dev, sc.stats, sc.work,
                       (unsigned long long*)sc.hist, decisions(sc), 0);
    hipLaunchKernelGGL(k_pick<PEN>, dim3(1), dim3(1024), 0, s, target, draft, ap_dev, sc.stats, sc.work,
                       (unsigned long long*)sc.hist, decisions(sc), sc.result, (int32_t*)nullptr, err, 0);
}

// The most child tests a walk can take before it stops.  At a node with children c_1 < ... < c_n (tested in slot
// order) the walk either rejects all n, or rejects j - 1, accepts c_j and goes on from there: worst(node) =
// max(n, max_j (j + worst(c_j))).  A parent's slot is below its children's, so one descending sweep fills the
// table.  Never more than m - 1 (every slot behind the root is tested at most once); 6 for the 16-node tree of a
// root with four chains, where m - 1 is 15.
int tree_walk_bound(const int32_t* parent, int m) {
    int worst[TSV_MAX_ROWS] = {0}, seen[TSV_MAX_ROWS] = {0};
    // children in descending slot order: the j of child c is known once all of its parent's children are counted
    int count[TSV_MAX_ROWS] = {0};
    for (int c = 1; c < m; c++) count[parent[c]]++;
    for (int c = m - 1; c >= 1; c--) {
        const int par = parent[c];
        const int j = count[par] - seen[par];  // c is the j-th child of its parent in ascending order
        seen[par]++;
        worst[par] = std::max(worst[par], std::max(count[par], j + worst[c]));
    }
    return std::min(worst[0], m - 1);
}

template <bool PEN>
static void launch_tree_sampled(hipStream_t s, const uint16_t* target, const uint16_t* draft, const AcceptParams* ap_dev,
                                const AcceptParams& ap, const AcceptScratch& sc) {
    int32_t* err = (int32_t*)sc.counters;
    int32_t* path = (int32_t*)sc.counters + 32;
    // statistics of the m target rows and the m rows the children were drawn from
    launch_stats<PEN>(s, target, draft, ap.m, 2 * ap.m, 2 * 65536, ap_dev, ap, sc);
    hipLaunchKernelGGL(k_tree_probs<PEN>, dim3(NSEG, 2 * ap.m), dim3(256), 0, s, target, draft, ap_dev, sc.stats, sc.work);
    // one child test per launch: as many launches as the longest walk through this tree can take
    const int steps = tree_walk_bound(ap.parent, ap.m);
    for (int k = 0; k < steps; k++)
        hipLaunchKernelGGL(k_tree_step<PEN>, dim3(TREE_WGS), dim3(256), 0, s, ap_dev, sc.stats, sc.work, k);
    hipLaunchKernelGGL(k_tree_finish<PEN>, dim3(TREE_WGS), dim3(256), 0, s, target, ap_dev, sc.stats, sc.work,
                       (unsigned long long*)sc.hist, decisions(sc), path, steps);
    hipLaunchKernelGGL(k_pick<PEN>, dim3(1), dim3(1024), 0, s, target, draft, ap_dev, sc.stats, sc.work,
                       (unsigned long long*)sc.hist, decisions(sc), sc.result, path, err, 2);
}

template <bool PEN>
static void launch_draft_sampled(hipStream_t s, const uint16_t* draft, const AcceptParams* ap_dev,
                                 const AcceptParams& ap, const AcceptScratch& sc, int32_t* proposals_dev) {
    int32_t* err = (int32_t*)sc.counters;
    launch_stats<PEN>(s, draft, draft, 0, ap.k, ap.k * 2 * 65536, ap_dev, ap, sc);
    hipLaunchKernelGGL(k_mass_hist<PEN>, dim3(NSEG, ap.k, NSUB), dim3(256), 0, s, draft, draft, ap_dev, sc.stats, sc.work,
                       (unsigned long long*)sc.hist, decisions(sc), 1);
    hipLaunchKernelGGL(k_pick<PEN>, dim3(ap.k), dim3(1024), 0, s, draft, draft, ap_dev, sc.stats, sc.work,
                       (unsigned long long*)sc.hist, decisions(sc), sc.result, proposals_dev, err, 1);
}

int launch_accept(hipStream_t s, const uint16_t* target, const uint16_t* draft, const AcceptParams* ap_dev,
                  const AcceptParams& ap, const AcceptScratch& sc) {
    int32_t* err = (int32_t*)sc.counters;
    float* pv = (float*)sc.counters + 64;
    int32_t* pi = (int32_t*)sc.counters + 64 + TSV_MAX_ROWS * ARGMAX_SEG;
    hipLaunchKernelGGL(k_clear_result, dim3(1), dim3(64), 0, s, sc.result, err);
    if (!ap.sampled) {  // (the arg-max ignores penalties and truncation: choose.rs:84-88)
        hipLaunchKernelGGL(k_argmax_part, dim3(ARGMAX_SEG, ap.m), dim3(256), 0, s, target, ap.vocab, pv, pi, err);
        hipLaunchKernelGGL(k_walk_greedy, dim3(1), dim3(64), 0, s, ap_dev, pv, pi, sc.result, err);
        TSV_HIP(hipGetLastError());
        return TSV_OK;
    }
    if (ap.tree) {
        if (ap.pen)
            launch_tree_sampled<true>(s, target, draft, ap_dev, ap, sc);
        else
            launch_tree_sampled<false>(s, target, draft, ap_dev, ap, sc);
        TSV_HIP(hipGetLastError());
        return TSV_OK;
    }
    if (ap.pen)
        launch_chain_sampled<true>(s, target, draft, ap_dev, ap, sc);
    else
        launch_chain_sampled<false>(s, target, draft, ap_dev, ap, sc);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// Draft half of a chain round: proposals[j] = q_j.draw(seed, draw_step + j) (speculative.rs:636-648),
// or the arg-max at temperature 0.  ap_dev: m = 0, k = rows, draw_step = first position.
int launch_draft_chain(hipStream_t s, const uint16_t* draft, const AcceptParams* ap_dev, const AcceptParams& ap,
                       const AcceptScratch& sc, int32_t* proposals_dev) {
    int32_t* err = (int32_t*)sc.counters;
    hipLaunchKernelGGL(k_clear_result, dim3(1), dim3(64), 0, s, sc.result, err);
    if (!ap.sampled) {
        float* pv = (float*)sc.counters + 64;
        int32_t* pi = (int32_t*)sc.counters + 64 + TSV_MAX_ROWS * ARGMAX_SEG;
        hipLaunchKernelGGL(k_argmax_part, dim3(ARGMAX_SEG, ap.k), dim3(256), 0, s, draft, ap.vocab, pv, pi, err);
        hipLaunchKernelGGL(k_argmax_fold, dim3(1), dim3(64), 0, s, pv, pi, ap.k, proposals_dev);
        TSV_HIP(hipGetLastError());
        return TSV_OK;
    }
    if (ap.pen)
        launch_draft_sampled<true>(s, draft, ap_dev, ap, sc, proposals_dev);
    else
        launch_draft_sampled<false>(s, draft, ap_dev, ap, sc, proposals_dev);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// The arg-max of `rows` logit rows (select() at temperature 0, crates/selection/src/choose.rs:61-98: the
// lowest index among equals, penalties and truncation ignored) into out[0, rows), nothing else touched but the error word, which is cleared only when
// `clear_error` says so: a chain of such calls keeps the first non-finite row's flag until the host reads it.
int launch_argmax_rows(hipStream_t s, const uint16_t* logits, int rows, int vocab, const AcceptScratch& sc, int32_t* out,
                       bool clear_error) {
    int32_t* err = (int32_t*)sc.counters;
    if (clear_error) hipLaunchKernelGGL(k_clear_result, dim3(1), dim3(64), 0, s, sc.result, err);
    float* pv = (float*)sc.counters + 64;
    int32_t* pi = (int32_t*)sc.counters + 64 + TSV_MAX_ROWS * ARGMAX_SEG;
    hipLaunchKernelGGL(k_argmax_part, dim3(ARGMAX_SEG, rows), dim3(256), 0, s, logits, vocab, pv, pi, err);
    hipLaunchKernelGGL(k_argmax_fold, dim3(1), dim3(64), 0, s, pv, pi, rows, out);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// The history's token statistics for a penalised round: cnt[v] bit 31 = v occurs in history[0, n),
// low bits = occurrences in history[suffix_start, n).  Token ids outside [0, vocab) are skipped
// (penalty.rs:27-33,73-78).
namespace {
__global__ void k_pen_clear(uint32_t* cnt, int vocab) {
    const int v = blockIdx.x * 256 + threadIdx.x;
    if (v < vocab) cnt[v] = 0;
}
__global__ void k_pen_count(const int32_t* history, long n, long suffix_start, int vocab, uint32_t* cnt) {
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        const int32_t t = history[i];
        if (t < 0 || t >= vocab) continue;
        atomicOr(cnt + t, 0x80000000u);
        if (i >= suffix_start) atomicAdd(cnt + t, 1u);
    }
}
}  // namespace

int launch_pen_counts(hipStream_t s, const int32_t* history_dev, long n, long suffix_start, int vocab, uint32_t* cnt) {
    hipLaunchKernelGGL(k_pen_clear, dim3((vocab + 255) / 256), dim3(256), 0, s, cnt, vocab);
    if (n > 0) {
        const int blocks = (int)std::min<long>((n + 255) / 256, 256);
        hipLaunchKernelGGL(k_pen_count, dim3(blocks), dim3(256), 0, s, history_dev, n, suffix_start, vocab, cnt);
    }
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

}  // namespace tsv

// ---- greedy acceptance for callers that cannot allocate ----------------------------------------
// The greedy round of tsv_accept (arg-max per row, the walk, the stop ladder and budget) over logits
// the caller holds on the device, writing the result to device memory of the caller's, on the
// caller's stream, with no handle behind it: nothing is allocated, copied from the host or waited
// for.  The partial results of the arg-max (one value / index pair per row and vocabulary run) and
// the error flag live in a static device array; every GPU the library runs on holds its own copy
// until the process ends, and every call on a GPU shares that GPU's copy, so two calls that overlap
// on one GPU race.
static __device__ __align__(256) unsigned char scratch[4096];

namespace tsv {
namespace {

struct NoAllocScratch {
    int32_t err;
    int32_t pad[63];
    float pv[TSV_MAX_ROWS * ARGMAX_SEG];
    int32_t pi[TSV_MAX_ROWS * ARGMAX_SEG];
};
static_assert(sizeof(NoAllocScratch) <= sizeof(scratch), "the static array holds the greedy round's partial results");

// the flag must start at zero; a fill kernel rather than a memset node, so a caller may capture the call
// (on a stream of its own, with the scratch address already resolved on the device: noalloc_prepare_device)
__global__ void k_noalloc_clear(int32_t* err) {
    if (threadIdx.x == 0) *err = 0;
}

__global__ void k_walk_greedy_value(AcceptParams ap, int64_t base, const float* pv, const int32_t* pi, const int32_t* err,
                                    tsv_round_result* out) {
    __shared__ int32_t amax[TSV_MAX_ROWS];
    if ((int)threadIdx.x < ap.m) amax[threadIdx.x] = fold_argmax(pv, pi, threadIdx.x);
    __syncthreads();
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    for (int i = 0; i <= TSV_MAX_ROWS; i++) out->path[i] = 0;
    if (*err) {  // a non-finite logit (choose.rs:122-132 refuses the row): no round was judged
        out->accepted = out->committed = 0;
        out->next = -1;
        out->stopped = -1;
        out->draw_step = ap.draw_step;
        out->path_len = 0;
        out->kv_position = base;
        out->min_margin = 0.0;
        return;
    }
    const GreedyWalk g = walk_greedy(ap, amax);
    for (int i = 0; i < g.path_len; i++) out->path[i] = g.path[i];
    out->accepted = g.accepted;
    out->committed = g.committed;
    out->next = g.next;
    out->stopped = g.stopped;
    out->draw_step = ap.draw_step;
    out->path_len = g.path_len;
    out->kv_position = base + g.committed + 1;
    out->min_margin = 1.0;
}

constexpr int NOALLOC_MAX_DEVICES = 64;
// device address of `scratch` on each GPU (the array's name is only a host-side handle of the symbol)
NoAllocScratch* g_noalloc_scratch[NOALLOC_MAX_DEVICES];

int noalloc_scratch(NoAllocScratch** out) {
    int dev = -1;
    TSV_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) {
        set_error("accept_greedy_noalloc: device ordinal outside 0..63");
        return TSV_ERR_UNSUPPORTED;
    }
    NoAllocScratch* p = __atomic_load_n(&g_noalloc_scratch[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        void* sym = nullptr;
        TSV_HIP(hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)));
        if (!sym) {
            set_error("accept_greedy_noalloc: the scratch symbol has no device address");
            return TSV_ERR_DEVICE;
        }
        p = (NoAllocScratch*)sym;
        __atomic_store_n(&g_noalloc_scratch[dev], p, __ATOMIC_RELEASE);
    }
    *out = p;
    return TSV_OK;
}

}  // namespace

// Resolves the scratch array's address on the current device, so that a later tsv_accept_greedy_noalloc makes no
// runtime query (tsv_open calls this: after any handle was opened on a device the entry point can be captured).
int noalloc_prepare_device() {
    NoAllocScratch* sc = nullptr;
    return noalloc_scratch(&sc);
}
}  // namespace tsv

extern "C" int32_t tsv_accept_greedy_noalloc(void* stream, const uint16_t* logits_dev, int32_t vocab, const int32_t* feed,
                                             const int32_t* parent, int32_t m, int64_t base, const int32_t* stop_tokens,
                                             int32_t n_stop, uint64_t generated, uint64_t max_new_tokens,
                                             tsv_round_result* result_dev) {
    using namespace tsv;
    if (!logits_dev || !feed || !result_dev || (n_stop > 0 && !stop_tokens)) {
        set_error("accept_greedy_noalloc: null argument");
        return TSV_ERR_INVALID;
    }
    if (m < 1 || m > TSV_MAX_ROWS) {
        set_error("accept_greedy_noalloc: 1..16 rows (the static scratch holds the partial results of 16 rows)");
        return TSV_ERR_INVALID;
    }
    if (vocab < 1 || base < 0 || n_stop < 0 || n_stop > 16) {
        set_error("accept_greedy_noalloc: vocabulary and base must be positive / non-negative, at most 16 stop tokens");
        return TSV_ERR_INVALID;
    }
    AcceptParams ap;
    std::memset(&ap, 0, sizeof ap);
    ap.m = m;
    ap.k = m - 1;
    ap.vocab = vocab;
    ap.tree = parent != nullptr;
    ap.n_stop = n_stop;
    for (int i = 0; i < m; i++) {
        if (parent && (i == 0 ? parent[0] != -1 : (parent[i] < 0 || parent[i] >= i))) {
            set_error("accept_greedy_noalloc: parent[0] must be -1 and parent[s] in [0, s)");
            return TSV_ERR_INVALID;
        }
        ap.feed[i] = feed[i];
        ap.parent[i] = parent ? parent[i] : i - 1;
    }
    for (int i = 0; i < n_stop; i++) ap.stop_tokens[i] = stop_tokens[i];
    ap.generated = generated;
    ap.max_new_tokens = max_new_tokens;
    NoAllocScratch* sc = nullptr;
    int rc = noalloc_scratch(&sc);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(k_noalloc_clear, dim3(1), dim3(64), 0, s, &sc->err);
    hipLaunchKernelGGL(k_argmax_part, dim3(ARGMAX_SEG, m), dim3(256), 0, s, logits_dev, vocab, sc->pv, sc->pi, &sc->err);
    hipLaunchKernelGGL(k_walk_greedy_value, dim3(1), dim3(64), 0, s, ap, base, sc->pv, sc->pi, &sc->err, result_dev);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// Test hook: the number of walk launches a sampled tree round of this shape gets (host arithmetic only).
extern "C" int32_t tsv_tree_walk_bound(const int32_t* parent, int32_t m) {
    using namespace tsv;
    if (!parent || m < 1 || m > TSV_MAX_ROWS || parent[0] != -1) {
        set_error("tree_walk_bound: 1..16 slots, parent[0] == -1");
        return -1;
    }
    for (int i = 1; i < m; i++)
        if (parent[i] < 0 || parent[i] >= i) {
            set_error("tree_walk_bound: parent[s] must lie in [0, s)");
            return -1;
        }
    return tree_walk_bound(parent, m);
}
