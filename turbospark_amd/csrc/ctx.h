// The handle behind the C ABI and what the translation units of the host runtime share: runtime.hip (open / close, the launch
// sequences, the producer entry points, acceptance), mtp.hip (the drafter head) and testing.hip (test and measurement hooks).
#pragma once
#include <cmath>
#include <cstring>
#include <new>
#include <string>
#include <vector>

#include "tsv_internal.h"
#include "kv_prefix.h"

namespace tsv {

struct LayerW {
    // the fused q/k/v projection; when the value projection has a format of its own (Q4_K_M files
    // keep attn_v in Q6_K) `qkv` holds q and k only and `v_only` the rest, written to the same
    // partial buffer at its column offset
    TiledW qkv, v_only, wo, gate_up, down;
    int n_experts = 0, top_k = 0;     // routed experts: gate_up / down hold every expert's tiles
    TiledW router;
    float *attn_norm = nullptr, *ffn_norm = nullptr, *q_norm = nullptr, *k_norm = nullptr;
    // gpt-oss additions, all optional: fused q/k/v bias, output bias, sinks, router bias, expert biases
    float *bqkv = nullptr, *bo = nullptr, *sinks = nullptr, *router_bias = nullptr;
    float *be_gate = nullptr, *be_up = nullptr, *be_down = nullptr;
    int window = 0;
    int cap = 0;        // positions the layer's cache holds: the context, or a ring of window + slack
    bool rope_fused = false;  // the q/k/v projection rotates and stores its own rows
    uint16_t *kc = nullptr, *vc = nullptr;
    // a quantized layer (TurboQuant): kc / vc are then the small fp16 staging cache all such layers
    // share (kv_slots positions instead of cap), and tq the layer's own stores
    int kv_slots = 0;
    TqKv tq{};
};

int dtype_fmt(int dtype);  // the tile format of a ggml storage type, -1: none

enum { PC_EMBED = 0, PC_NORM, PC_QKV, PC_ROPE, PC_ATTN, PC_WO, PC_GATEUP, PC_DOWN, PC_HEAD, PC_ACCEPT, PC_EVENTPAIR, PC_COUNT };
static_assert(PC_COUNT == TSV_PROFILE_CLASSES, "profile classes");

}  // namespace tsv

using namespace tsv;  // (this header is private to the host runtime's translation units)

struct tsv_ctx {
    int n_layers = 0, hidden = 0, nq = 0, nkv = 0, hd = 0, ffn = 0, vocab = 0, max_context = 0, ctx_alloc = 0;
    float eps = 0, attn_scale = 0, rope_mscale = 1.0f, act_alpha = 0, act_limit = 0;
    hipStream_t stream = nullptr;
    bool rope_fused_ok = true;     // TSV_ROPE_FUSED=0 keeps the projection and the rotation apart
    bool rope_fused_force = false;  // TSV_ROPE_FUSED=1 fuses them whatever a tile weighs
    std::vector<LayerW> layers;
    TiledW head;
    uint8_t* embed_raw = nullptr;
    int embed_dtype = 0;
    float* final_norm = nullptr;
    float* freqs = nullptr;
    float2* rope_cs = nullptr;  // [16][hd / 2] rotation table of the step's rows (fused q/k/v projection)
    // scratch
    float* x = nullptr;
    uint4 *xf_a = nullptr, *xf_b = nullptr, *xf_c = nullptr;
    float* partial = nullptr;
    size_t partial_floats = 0;
    // routed experts: routing tables, per-expert activation fragments, per-slot outputs
    int max_experts = 0;
    float* route_w = nullptr;
    int32_t* route_sel = nullptr;
    int32_t* route_forced = nullptr;  // test hook (tsv_force_route): [n_layers][16][8], negative = route freely
    uint8_t* frag_e = nullptr;
    size_t frag_e_stride = 0;
    float* moe_out = nullptr;
    // scaled-MFMA expert matmuls (moe_fp4.hip): activation terms (0 = the fp16 path), the pass's rows
    // and the groups' gate/up outputs as block-scaled fp8
    int moe_fp4_terms = 0;
    X8 x8_h{}, x8_e{};
    size_t x8_e_q_stride = 0, x8_e_s_stride = 0;
    // prompt passes of 64 rows (four blocks of sixteen): every block's rows, fragments, partial sums,
    // q rows, parameters and rotation table, block after block; allocated at the first such pass
    struct Wide {
        bool ok = false, ready = false;
        bool keep_epilogue = false;  // TSV_WIDE_ROPE_FUSED=1: the 64-row q/k/v launch rotates its own rows (one workgroup per tile)
        float* x = nullptr;
        uint8_t *xf_a = nullptr, *xf_b = nullptr, *xf_c = nullptr;
        size_t xfb = 0;
        float* partial = nullptr;
        uint16_t* q16 = nullptr;
        VerifyParams* vp = nullptr;
        float2* rope_cs = nullptr;
        float *part_o = nullptr, *part_ml = nullptr;  // attention partials of every block
        size_t part_o_stride = 0, part_ml_stride = 0;
        // routed layers: the 64 rows' factors and selections, every expert's members, the experts' gate/up outputs
        // (four 16-member sub-buffers per expert) and the blocks' per-slot down outputs
        float* route_w = nullptr;
        int32_t* route_sel = nullptr;
        MoeGroupW* groups = nullptr;
        uint8_t* frag_e = nullptr;
        size_t frag_e_sub = 0;
        float* moe_out = nullptr;
    } wide;
    bool route_forced_set = false;  // tsv_force_route holds selections: prompt passes stay at sixteen rows
    uint16_t* q16 = nullptr;
    float *part_o = nullptr, *part_ml = nullptr;
    int nch = 0;
    uint16_t* logits = nullptr;       // [16][vocab] fp16, device
    uint16_t* draft_stage = nullptr;  // [16][vocab] fp16, device
    VerifyParams *vp_dev = nullptr, *vp_host = nullptr;
    // Pinned staging slots of the per-pass parameters (four 16-row blocks each), used round robin: a slot is
    // rewritten only once the copy that last read it has completed (its event), so consecutive passes queue
    // without the host waiting for the stream.
    struct ParamRing {
        static constexpr int SLOTS = 8, PER_SLOT = 4;
        VerifyParams* host = nullptr;
        hipEvent_t ev[SLOTS] = {};
        bool used[SLOTS] = {};
        int next = 0;
    } ring;
    AcceptParams *ap_dev = nullptr, *ap_host = nullptr;
    uint16_t** kv_ptrs = nullptr;  // device: [2 * layer] = K buffer, [2 * layer + 1] = V buffer (tree compaction)
    int32_t* hist_dev = nullptr;  // the token history of a penalised round (grows on demand)
    size_t hist_cap = 0;
    uint32_t* pen_cnt = nullptr;  // [vocab] seen flag + generated-suffix count per token
    AcceptResult* res_host = nullptr;
    int32_t *tok_dev = nullptr, *tok_host = nullptr;
    AcceptScratch sc{};
    std::vector<void*> allocs;
    // TurboQuant KV rows (crates/model-io/src/kv_quant.rs): widths (0 = every layer fp16), the tables of the two
    // sides and the fp16 staging rows of the pass in flight (crates/runtime/src/kv_write.rs:36-60)
    int kv_k_bits = 0, kv_v_bits = 0;
    TqSide tq_k{}, tq_v{};
    uint16_t *tq_kc = nullptr, *tq_vc = nullptr;
    TqKv* tq_stores = nullptr;  // device: every layer's stores (tree compaction)
    int64_t position = 0;
    int64_t high_water = 0;     // one past the last position any pass has written since the last reset
    int64_t rewind_budget = INT64_MAX;  // KvCacheManager::max_safe_rewind: min over ring layers of capacity - window
    int32_t* kv_caps = nullptr;  // device: positions each layer's cache holds (tree compaction)
    tsv_prefix prefix;          // the ids behind rows [0, prefix length): kv_prefix.rs
    // Parked sessions (crates/runtime/src/session_pool.rs): each one a full set of per-layer KV buffers of its own
    // with its cursor and its record; the live session is the fields above and in `layers`.  A swap exchanges
    // pointers, never rows.
    struct Session {
        std::vector<uint16_t*> kc, vc;  // per layer (a quantized layer: unused, its rows are in `tq`)
        std::vector<TqKv> tq;
        uint16_t** kv_ptrs = nullptr;   // device copies of the pointer tables tree compaction reads
        TqKv* tq_stores = nullptr;
        int64_t position = 0, high_water = 0;
        tsv_prefix prefix;
        uint64_t last_used = 0;         // the pool's tick at parking (session_pool.rs:110-114)
    };
    std::vector<Session> parked;
    uint64_t session_clock = 0;
    bool session_slot_evicted = false;  // the last reset overwrote a parked conversation (real_forward_traits.rs:20-31)
    bool session_swapped = false;       // the last try_reuse_prefix swapped a parked conversation in
    bool prefix_reuse = false;  // RealForwardRunner::set_prefix_reuse: off unless the host opts in
    bool headless = false;      // the pass in flight is a prefill pass nobody reads the logits of
    int last_m = 0;
    int64_t last_base = -1;
    bool last_shape_known = false;  // vp_host holds the ancestor sets of the rows tsv_accept is about to judge
    // The launch sequence of a pass depends on the row count only (positions, tokens and the
    // tree shape are read from device memory), so it can be captured once per row count into a
    // HIP graph and replayed (environment TSV_GRAPH=1).  Off by default: the pass is bound by
    // the GPU-side cost of ~290 dependent kernels, not by host launch time, and replay measured
    // the same step time as plain stream launches.
    bool use_graph = false;
    hipGraphExec_t pass_graph[TSV_MAX_ROWS + 1] = {};
    // per-kernel-class timing (tsv_set_profile): one event pair per launch
    bool profile = false;
    int repeat[TSV_PROFILE_CLASSES] = {1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1};  // tsv_set_repeat
    std::vector<hipEvent_t> ev;
    std::vector<int> ev_class;
    size_t ev_used = 0;
    // A drafter head (tsv_mtp_open; docs/MTP.md:53-60): a one-layer handle on the target's stream whose rows
    // enter the layer as fc over [norm_e(embedding of the row's NEXT token) ; norm_h(target_final_norm(h))], h
    // the residual row of the row's position.  Embedding table and output head are the target's buffers.
    struct Mtp {
        bool on = false;
        tsv_ctx* target = nullptr;
        TiledW fc;
        float *norm_e = nullptr, *norm_h = nullptr;
        uint4* xf_cat = nullptr;                  // fc's input rows as matmul fragments (K = 2 hidden)
        const float* h_src = nullptr;             // the pass in flight: its residual rows, hidden floats apart
        bool own_valid = false;  // x row 0 is this head's own residual of the step at position - 1 (a chained step)
        const int32_t* feed_dev = nullptr;  // the pass in flight takes row 0's token from device memory
        bool params_staged = false;         // ... and finds its parameter block on the device already (vp_dev)
        VerifyParams *vp_block = nullptr, *vp_block_host = nullptr;  // [16] the parameter blocks of a block draft's steps
        int32_t *chain = nullptr, *chain_host = nullptr;  // the tokens of a block draft and the error word
        AcceptParams *draw_dev = nullptr, *draw_host = nullptr;  // [16] the draw parameters of a sampled block's steps
    } mtp;
    int64_t x_base = -1;  // rows [0, x_rows) of x are the finished residual rows of positions x_base ..
    int x_rows = 0;
    tsv_ctx* mtp_head = nullptr;  // target side: the attached head; prompt passes then finish their residual rows
    bool owns_stream = true;
};

namespace tsv {

template <class T>
int dev_alloc(tsv_ctx* c, T** p, size_t bytes, bool zero = false) {
    void* q = nullptr;
    TSV_HIP(hipMalloc(&q, bytes ? bytes : 16));
    c->allocs.push_back(q);
    if (zero) TSV_HIP(hipMemsetAsync(q, 0, bytes, c->stream));
    *p = (T*)q;
    return TSV_OK;
}

// the staging buffer weight tensors pass through on their way to the re-tiling kernels
struct Stager {
    uint8_t* dev = nullptr;
    size_t cap = 0;
};

int check_matrix(const tsv_tensor& t, int64_t rows, int64_t cols, const char* what);
int make_tiled(tsv_ctx* c, Stager& st, const tsv_tensor* const* parts, int n_parts, bool interleave, TiledW* out, int pair_parts = 0);
int check_shaping(const tsv_shaping& s, bool sampled_supported_only);
int fill_params(VerifyParams& vp, const int32_t* feed, const int32_t* parent, int m, int64_t base, int vocab);
// One verify pass: everything enqueued on the handle's stream, no synchronisation; then the optional copy of the rows' logits.
int enqueue_verify(tsv_ctx* c, const int32_t* feed, const int32_t* parent, int m, int64_t base);
int finish_verify(tsv_ctx* c, int m, uint16_t* logits_out);
// `share` / `md`: a drafter head opened on a target handle (its stream, embedding table and output head are the target's)
int open_impl(const tsv_model_desc* d, tsv_ctx* share, const tsv_mtp_desc* md, tsv_ctx** out);
// `head` (nullable): the drafter head primed after each pass over every row whose next token is known; next_token: the
// token after ids[n - 1], or -1
int prefill_passes(tsv_ctx* c, const int32_t* ids, int64_t n, int64_t pos0, uint16_t* logits, tsv_ctx* head = nullptr,
                   int32_t next_token = -1);
// one pass of a drafter head over m rows at position ..: row r pairs next_tokens[r] with row r of h_rows (mtp.hip)
int mtp_pass(tsv_ctx* c, const int32_t* next_tokens, int m, int64_t position, const float* h_rows, bool want_logits);
void fill_truncation(AcceptParams* ap, const tsv_shaping& sh);
int setup_penalties(tsv_ctx* c, const tsv_shaping& sh, const int32_t* history, int64_t n, uint64_t generated, AcceptParams* ap);
const char* accept_error_text(int bits);

}  // namespace tsv
