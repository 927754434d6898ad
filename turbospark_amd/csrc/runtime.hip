// Host runtime of libtsverify: the handle, weight upload / re-tiling, the KV arena, the launch
// sequence of one verify pass, and the C ABI.
//
// The pass composes the reference's Llama-family decode graph row-wise
// (crates/runtime/src/families/llama/mod.rs:197-316, attn.rs:152-369, dense.rs:45-120) under the
// batched-verify contract of crates/runtime/src/families/qwen/batched.rs:92-456.  Residual
// stream and all intermediates are fp32; fp16 appears where the engine's storage dtype is
// fixed (KV cache, logits) and as the MFMA operand type of the matmuls.
#include "ctx.h"

using namespace tsv;

namespace tsv {

int dtype_fmt(int dtype) {
    return dtype == TSV_Q4_K    ? FMT_Q4K
           : dtype == TSV_Q8_0  ? FMT_Q80
           : dtype == TSV_MXFP4 ? FMT_MX4
           : dtype == TSV_BF16  ? FMT_BF16
           : dtype == TSV_Q6_K  ? FMT_Q6K
           : dtype == TSV_Q5_K  ? FMT_Q5K
                                : -1;
}

float to_f32(const tsv_tensor& t, int64_t i) {
    switch (t.dtype) {
        case TSV_F32: return ((const float*)t.data)[i];
        case TSV_F16: {
            _Float16 h;
            std::memcpy(&h, (const uint16_t*)t.data + i, 2);
            return (float)h;
        }
        case TSV_BF16: {
            uint32_t u = (uint32_t)((const uint16_t*)t.data)[i] << 16;
            float f;
            std::memcpy(&f, &u, 4);
            return f;
        }
    }
    return 0.f;
}

int upload_vector(tsv_ctx* c, const tsv_tensor& t, int64_t n, float** out, const char* what) {
    if (!t.data || t.rows * t.cols != n || (t.dtype != TSV_F32 && t.dtype != TSV_F16 && t.dtype != TSV_BF16)) {
        set_error(std::string(what) + ": expected an f32/f16/bf16 vector of the model's width");
        return TSV_ERR_INVALID;
    }
    std::vector<float> h((size_t)n);
    for (int64_t i = 0; i < n; i++) h[i] = to_f32(t, i);
    int rc = dev_alloc(c, out, (size_t)n * 4);
    if (rc) return rc;
    TSV_HIP(hipMemcpy(*out, h.data(), (size_t)n * 4, hipMemcpyHostToDevice));
    return TSV_OK;
}

int stage_raw(tsv_ctx* c, Stager& st, const tsv_tensor& t) {
    const int64_t rb = row_bytes(t.dtype, t.cols);
    const size_t bytes = (size_t)(rb * t.rows);
    if (bytes > st.cap) {
        if (st.dev) TSV_HIP(hipFree(st.dev));
        st.dev = nullptr;
        TSV_HIP(hipMalloc((void**)&st.dev, bytes));
        st.cap = bytes;
    }
    TSV_HIP(hipMemcpyAsync(st.dev, t.data, bytes, hipMemcpyHostToDevice, c->stream));
    return TSV_OK;
}

int check_matrix(const tsv_tensor& t, int64_t rows, int64_t cols, const char* what) {
    const int fmt = dtype_fmt(t.dtype);
    if (!t.data || t.rows != rows || t.cols != cols) {
        set_error(std::string(what) + ": shape does not match the model description");
        return TSV_ERR_INVALID;
    }
    if (fmt < 0) {
        set_error(std::string(what) + ": matmul weights must be Q4_K, Q5_K, Q6_K, Q8_0, MXFP4 or bf16 in this build");
        return TSV_ERR_UNSUPPORTED;
    }
    // MXFP4 rows may end inside a 256-element chunk (the tile is padded with zero blocks)
    const int gran = fmt == FMT_MX4 ? 32 : fmt_chunk_elems(fmt);
    if (cols % gran || rows < 1) {
        set_error(std::string(what) + ": K must be whole 256 (Q4_K, Q5_K, Q6_K) / 128 (Q8_0) / 64 (bf16) / 32 (MXFP4) element runs");
        return TSV_ERR_UNSUPPORTED;
    }
    return TSV_OK;
}

// Allocates a tiled matrix of `total_rows` rows and re-tiles `parts` into it: concatenated row
// by row (interleave == false) or alternating in runs of 32 rows (gate / up: each 64-row tile
// holds 32 gate rows in its low lanes and the matching 32 up rows in its high lanes).
// pair_parts > 0 (128-wide heads feeding the rotating epilogue): inside every head of the first
// `pair_parts` parts the rows are reordered so that a 64-row tile holds dims 32t..32t+31 in its low
// lanes and their rotation partners, dims 64+32t.., in its high lanes.
int make_tiled(tsv_ctx* c, Stager& st, const tsv_tensor* const* parts, int n_parts, bool interleave, TiledW* out, int pair_parts) {
    const int fmt = dtype_fmt(parts[0]->dtype);
    int64_t total_rows = 0;
    for (int i = 0; i < n_parts; i++) {
        if (dtype_fmt(parts[i]->dtype) != fmt || parts[i]->cols != parts[0]->cols) {
            set_error("fused projection parts must share dtype and K");
            return TSV_ERR_INVALID;
        }
        if (interleave && (parts[i]->rows != parts[0]->rows || parts[i]->rows % 32)) {
            set_error("gate / up projections must have the same row count, a multiple of 32");
            return TSV_ERR_UNSUPPORTED;
        }
        total_rows += parts[i]->rows;
    }
    out->fmt = fmt;
    out->k = (int)parts[0]->cols;
    out->kchunks = (out->k + fmt_chunk_elems(fmt) - 1) / fmt_chunk_elems(fmt);
    out->n_rows = (int)total_rows;
    out->n_tiles = (int)((total_rows + TILE_ROWS - 1) / TILE_ROWS);
    out->bytes = (size_t)out->n_tiles * out->kchunks * fmt_tile_bytes(fmt);
    int rc = dev_alloc(c, &out->tiles, out->bytes, true);  // rows past the last one stay zero blocks
    if (rc) return rc;
    int row_off = 0;
    for (int i = 0; i < n_parts; i++) {
        if ((rc = stage_raw(c, st, *parts[i]))) return rc;
        const int rows = (int)parts[i]->rows;
        if (i < pair_parts) {
            if (interleave || rows % 128) {
                set_error("paired row order needs whole 128-wide heads");
                return TSV_ERR_INVALID;
            }
            std::vector<int32_t> map((size_t)rows);
            for (int r = 0; r < rows; r++) {
                const int hl = r & 127, half = hl >> 6, w = hl & 63, t = w >> 5, j = w & 31;
                map[(size_t)r] = row_off + (r & ~127) + t * 64 + half * 32 + j;
            }
            int32_t* map_dev = nullptr;
            TSV_HIP(hipMalloc((void**)&map_dev, map.size() * 4));
            hipError_t e = hipMemcpyAsync(map_dev, map.data(), map.size() * 4, hipMemcpyHostToDevice, c->stream);
            if (e == hipSuccess) {
                rc = launch_repack(c->stream, fmt, st.dev, rows, out->k, out->tiles, out->kchunks, rows, 0, row_off, map_dev);
                e = hipStreamSynchronize(c->stream);
            }
            (void)hipFree(map_dev);
            TSV_HIP(e);
            if (rc) return rc;
            row_off += rows;
            continue;
        }
        rc = interleave ? launch_repack(c->stream, fmt, st.dev, rows, out->k, out->tiles, out->kchunks, 32, 32 * n_parts, 32 * i)
                        : launch_repack(c->stream, fmt, st.dev, rows, out->k, out->tiles, out->kchunks, rows, 0, row_off);
        if (rc) return rc;
        TSV_HIP(hipStreamSynchronize(c->stream));  // the stager is reused by the next part
        row_off += rows;
    }
    return TSV_OK;
}

int splits_for(const TiledW& w, int m, int epi) { return epi == EPI_PARTIAL ? gemm_default_splits(w, m) : 1; }

size_t partial_need(const TiledW& w) {
    size_t need = 0;
    for (int m : {4, 8, 16}) {
        size_t s = (size_t)splits_for(w, m, EPI_PARTIAL) * 16 * (size_t)w.n_tiles * TILE_ROWS;
        if (s > need) need = s;
    }
    return need;
}

int is_device_pointer(const void* p) {
    hipPointerAttribute_t a;
    hipError_t e = hipPointerGetAttributes(&a, p);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return a.type == hipMemoryTypeDevice;
}

int check_shaping(const tsv_shaping& s, bool sampled_supported_only) {
    if (!(s.temperature >= 0.0) || !std::isfinite(s.temperature)) {
        set_error("temperature must be finite and non-negative");
        return TSV_ERR_INVALID;
    }
    if (s.temperature == 0.0) return TSV_OK;
    if (!s.has_seed) {
        set_error("a sampled round needs an explicit seed");
        return TSV_ERR_INVALID;
    }
    (void)sampled_supported_only;
    if (!(s.repetition_penalty > 0.0) || !std::isfinite(s.repetition_penalty) || !std::isfinite(s.presence_penalty) ||
        !std::isfinite(s.frequency_penalty)) {
        set_error("penalties must be finite, the repetition penalty positive");
        return TSV_ERR_INVALID;
    }
    return TSV_OK;
}

bool has_penalties(const tsv_shaping& s) {
    return s.temperature != 0.0 && (s.repetition_penalty != 1.0 || s.presence_penalty != 0.0 || s.frequency_penalty != 0.0);
}

struct ProfScope {
    tsv_ctx* c;
    ProfScope(tsv_ctx* c_, int cls) : c(c_) {
        if (!c->profile) return;
        if (c->ev_used + 2 > c->ev.size()) {
            for (int i = 0; i < 2; i++) {
                hipEvent_t e;
                (void)hipEventCreate(&e);
                c->ev.push_back(e);
                c->ev_class.push_back(0);
            }
        }
        c->ev_class[c->ev_used] = cls;
        (void)hipEventRecord(c->ev[c->ev_used], c->stream);
    }
    ~ProfScope() {
        if (!c->profile) return;
        (void)hipEventRecord(c->ev[c->ev_used + 1], c->stream);
        c->ev_used += 2;
    }
};
#define PROF(cls) ProfScope prof_scope_(c, cls)

int fill_params(VerifyParams& vp, const int32_t* feed, const int32_t* parent, int m, int64_t base, int vocab) {
    std::memset(&vp, 0, sizeof vp);
    vp.m = m;
    vp.base = (int32_t)base;
    int depth[TSV_MAX_ROWS] = {0};
    for (int i = 0; i < m; i++) {
        if (feed) {
            if (feed[i] < 0 || feed[i] >= vocab) {
                set_error("verify: token id outside the vocabulary");
                return TSV_ERR_INVALID;
            }
            vp.feed[i] = feed[i];
        }
        if (parent) {
            if (i == 0 ? parent[0] != -1 : (parent[i] < 0 || parent[i] >= i)) {
                set_error("verify_tree: parent[0] must be -1 and parent[s] in [0, s)");
                return TSV_ERR_INVALID;
            }
            depth[i] = i == 0 ? 0 : depth[parent[i]] + 1;
            vp.anc[i] = (i == 0 ? 0u : vp.anc[parent[i]]) | (1u << i);
        } else {
            depth[i] = i;
            vp.anc[i] = (2u << i) - 1u;
        }
        vp.pos[i] = (int32_t)base + depth[i];
    }
    return TSV_OK;
}

int run_pass(tsv_ctx* c, int m);

// n parameter blocks to `dev` through the next pinned staging slot, on the handle's stream.
int stage_params(tsv_ctx* c, const VerifyParams* vp, int n, VerifyParams* dev) {
    auto& r = c->ring;
    const int i = r.next;
    r.next = (i + 1) % tsv_ctx::ParamRing::SLOTS;
    if (r.used[i]) TSV_HIP(hipEventSynchronize(r.ev[i]));
    VerifyParams* slot = r.host + (size_t)i * tsv_ctx::ParamRing::PER_SLOT;
    std::memcpy(slot, vp, (size_t)n * sizeof(VerifyParams));
    TSV_HIP(hipMemcpyAsync(dev, slot, (size_t)n * sizeof(VerifyParams), hipMemcpyHostToDevice, c->stream));
    TSV_HIP(hipEventRecord(r.ev[i], c->stream));
    r.used[i] = true;
    return TSV_OK;
}

// One verify pass: enqueue everything on the handle's stream; no synchronisation.
int enqueue_verify(tsv_ctx* c, const int32_t* feed, const int32_t* parent, int m, int64_t base) {
    TSV_NEED(c, "verify: null handle");
    // batched.rs:106-185 refusals
    if (!feed || m < 1) {
        set_error("verify: empty feed");
        return TSV_ERR_INVALID;
    }
    if (m > TSV_MAX_ROWS) {
        set_error("verify: more rows than one pass takes (16)");
        return TSV_ERR_INVALID;
    }
    if (base != c->position) {
        set_error("verify: start position does not match the KV cursor");
        return TSV_ERR_INVALID;
    }
    if (base + m > c->max_context) {
        set_error("verify: block would write past the KV capacity");
        return TSV_ERR_INVALID;
    }
    VerifyParams vp;
    int prc = fill_params(vp, feed, parent, m, base, c->vocab);
    if (prc) return prc;
    *c->vp_host = vp;  // the host's own copy of the pass in flight
    // (a block draft has put the parameter blocks of all its steps on the device in one copy: vp_dev names this step's)
    if (!c->mtp.params_staged)
        if (int prc2 = stage_params(c, &vp, 1, c->vp_dev)) return prc2;
    int rc = run_pass(c, m);
    if (rc) return rc;
    c->position = base + m;
    c->high_water = std::max(c->high_water, c->position);
    c->last_m = m;
    c->last_base = base;
    c->last_shape_known = true;
    // whose residual rows x holds now: a chain pass that ran its last residual add leaves row r = position base + r
    c->x_base = base;
    c->x_rows = parent || (c->headless && !c->mtp_head) ? 0 : m;
    if (c->mtp_head) c->mtp_head->mtp.own_valid = false;  // the head's next step reads the target's rows again
    return TSV_OK;
}

// kv_cache_rewind.rs:46-55: a cursor may move back only as far as every ring layer still holds the
// window of the position it lands on.  Rows are overwritten up to the high-water mark, so the test
// is made against it (the reference tests each rewind's own count, which is the same thing in a
// loop that never rolls back past its last checkpoint).
int check_rewind(tsv_ctx* c, int64_t new_position, const char* who) {
    if (c->rewind_budget == INT64_MAX || c->high_water - new_position <= c->rewind_budget) return TSV_OK;
    set_error(std::string(who) + ": rewind of " + std::to_string((long long)(c->high_water - new_position)) +
              " rows exceeds the ring slack of " + std::to_string((long long)c->rewind_budget) +
              ": a sliding-window layer would read rows that have already been overwritten");
    return TSV_ERR_INVALID;
}

// The kernels of one pass over m rows, in order, on the handle's stream.
int launch_pass(tsv_ctx* c, int m) {
    hipStream_t s = c->stream;
    int rc;
    { PROF(PC_EVENTPAIR); }  // calibration: an event pair around nothing
    int prev_splits = 0;
    if (c->mtp.on) {
        // the head's rows: fc over the normed embedding of each row's next token and the normed state of its
        // position; fc's split-K partial sums are added onto the cleared rows by the layer's first residual kernel
        tsv_ctx::Mtp& h = c->mtp;
        PROF(PC_EMBED);
        if ((rc = launch_mtp_input(s, c->embed_raw, c->embed_dtype, c->vp_dev, h.feed_dev, c->vocab, h.h_src, h.norm_e,
                                   h.target->final_norm, h.norm_h, c->eps, c->hidden, h.xf_cat, c->x, c->freqs, c->rope_mscale,
                                   c->hd / 2, c->rope_cs, m)))
            return rc;
        prev_splits = splits_for(h.fc, m, EPI_PARTIAL);
        rc = launch_gemm(s, h.fc, h.xf_cat, c->partial, c->vp_dev, m, prev_splits, EPI_PARTIAL, c->hidden, c->hidden);
    } else {
        PROF(PC_EMBED);
        rc = launch_embed(s, c->embed_raw, c->embed_dtype, c->hidden, c->x, c->vp_dev, m, c->freqs, c->rope_mscale,
                          c->hd / 2, c->rope_cs);
    }
    if (rc) return rc;
    const float* prev_partial = c->partial;
    const float* prev_weights = nullptr;  // routed experts: the factors of the per-slot outputs
    float* x = c->x;
    const int qkv_n = (c->nq + 2 * c->nkv) * c->hd;
    for (int l = 0; l < c->n_layers; l++) {
        LayerW& L = c->layers[l];
        {
            PROF(PC_NORM);
            rc = launch_addnorm(s, x, prev_partial, prev_splits, c->hidden, L.attn_norm, c->eps, c->hidden, c->xf_a, m,
                                prev_weights);
            prev_weights = nullptr;
        }
        if (rc) return rc;
        int sp = splits_for(L.qkv, m, EPI_PARTIAL);
        if (L.v_only.tiles) {  // one split count for both pieces: the consumer adds `sp` partials per column
            auto fits = [](const TiledW& w, int n) {
                const int kslice = (w.kchunks + n - 1) / n;
                return (w.kchunks + kslice - 1) / kslice == n;
            };
            while (sp > 1 && !(fits(L.qkv, sp) && fits(L.v_only, sp))) sp--;
        }
        if (L.rope_fused) {
            RopeEpi re{};
            re.cs = c->rope_cs;
            re.bias = L.bqkv;
            re.q16 = c->q16;
            re.kc = L.kc;
            re.vc = L.vc;
            re.nq = c->nq;
            re.nkv = c->nkv;
            re.hd = c->hd;
            re.max_ctx = L.kv_slots;
            PROF(PC_QKV);
            rc = 0;
            for (int rep = 0; rep < c->repeat[PC_QKV] && !rc; rep++)
                rc = launch_gemm(s, L.qkv, c->xf_a, nullptr, c->vp_dev, m, 1, EPI_ROPE, qkv_n, L.qkv.n_rows, &re);
        } else {
            PROF(PC_QKV);
            rc = 0;
            for (int rep = 0; rep < c->repeat[PC_QKV] && !rc; rep++) {
                rc = launch_gemm(s, L.qkv, c->xf_a, c->partial, c->vp_dev, m, sp, EPI_PARTIAL, qkv_n, L.qkv.n_rows);
                if (!rc && L.v_only.tiles)
                    rc = launch_gemm(s, L.v_only, c->xf_a, c->partial + L.qkv.n_rows, c->vp_dev, m, sp, EPI_PARTIAL, qkv_n,
                                     L.v_only.n_rows);
            }
        }
        if (rc) return rc;
        RopeKvArgs ra{};
        ra.qkv = c->partial;
        ra.splits = sp;
        ra.ldq = qkv_n;
        ra.freqs = c->freqs;
        ra.mscale = c->rope_mscale;
        ra.bias = L.bqkv;
        ra.q_norm = L.q_norm;
        ra.k_norm = L.k_norm;
        ra.eps = c->eps;
        ra.q16 = c->q16;
        ra.kc = L.kc;
        ra.vc = L.vc;
        ra.nq = c->nq;
        ra.nkv = c->nkv;
        ra.hd = c->hd;
        ra.max_ctx = L.kv_slots;
        ra.vp = c->vp_dev;
        if (!L.rope_fused) {
            PROF(PC_ROPE);
            rc = 0;
            for (int rep = 0; rep < c->repeat[PC_ROPE] && !rc; rep++) rc = launch_rope_kv(s, ra, m);
        }
        if (rc) return rc;
        if (L.tq.k_bits) {
            // the pass's K / V rows sit in the staging cache (crates/runtime/src/kv_write.rs:66-118): quantize them
            // into the layer's stores and rotate q -- attention then runs in the rotated space, over the stores
            // (kv_quant_attention.rs:58-136)
            TqArgs ta{};
            ta.q16 = c->q16;
            ta.kc = L.kc;
            ta.vc = L.vc;
            ta.stage_cap = L.kv_slots;
            ta.store = L.tq;
            ta.k = c->tq_k;
            ta.v = c->tq_v;
            ta.nq = c->nq;
            ta.nkv = c->nkv;
            ta.hd = c->hd;
            ta.cap = L.cap;
            ta.vp = c->vp_dev;
            ta.m_hint = m;
            ta.base_hint = c->use_graph ? -1 : c->vp_host->base;
            PROF(PC_ROPE);
            rc = launch_tq_prepare(s, ta);
            if (rc) return rc;
        }
        AttnArgs aa{};
        aa.q16 = c->q16;
        aa.kc = L.kc;
        aa.vc = L.vc;
        aa.unrot = L.tq.k_bits ? c->tq_v.signs : nullptr;
        aa.tq = L.tq;
        aa.part_o = c->part_o;
        aa.part_ml = c->part_ml;
        aa.xfrag = c->xf_b;
        aa.nq = c->nq;
        aa.nkv = c->nkv;
        aa.hd = c->hd;
        aa.max_ctx = L.cap;
        aa.ring = L.cap < c->ctx_alloc;
        aa.nch = c->nch;
        aa.scale = c->attn_scale;
        aa.window = L.window;
        aa.sinks = L.sinks;
        aa.vp = c->vp_dev;
        aa.m_hint = m;
        aa.base_hint = c->use_graph ? -1 : c->vp_host->base;  // a captured launch must read the position at replay
        {
            PROF(PC_ATTN);
            rc = 0;
            for (int rep = 0; rep < c->repeat[PC_ATTN] && !rc; rep++) rc = launch_attention(s, aa, m);
        }
        if (rc) return rc;
        sp = splits_for(L.wo, m, EPI_PARTIAL);
        {
            PROF(PC_WO);
            rc = 0;
            for (int rep = 0; rep < c->repeat[PC_WO] && !rc; rep++) rc = launch_gemm(s, L.wo, c->xf_b, c->partial, c->vp_dev, m, sp, EPI_PARTIAL, c->hidden, c->hidden);
        }
        if (rc) return rc;
        {
            PROF(PC_NORM);
            const bool fp4 = L.n_experts && c->moe_fp4_terms;
            rc = launch_addnorm(s, x, c->partial, sp, c->hidden, L.ffn_norm, c->eps, c->hidden, c->xf_a, m, nullptr, L.bo,
                                fp4 ? &c->x8_h : nullptr, c->moe_fp4_terms);
        }
        if (rc) return rc;
        if (L.n_experts) {
            // router -> top-k -> grouped expert matmuls; the per-slot outputs are added, weighted
            // and in slot order, by the next residual kernel
            MoeRouteArgs ra2{};
            const int rsp = splits_for(L.router, m, EPI_PARTIAL);
            ra2.logits = c->partial;
            ra2.splits = rsp;
            ra2.ld = L.n_experts;
            ra2.n_experts = L.n_experts;
            ra2.top_k = L.top_k;
            ra2.m = m;
            ra2.weights = c->route_w;
            ra2.selected = c->route_sel + (size_t)l * 16 * 8;  // kept per layer: tsv_route_selected reads them back
            ra2.bias = L.router_bias;
            ra2.forced = c->route_forced + (size_t)l * 16 * 8;
            MoeGemmArgs g1{}, g2{};
            g1.w = L.gate_up.tiles;
            g1.tiles_per_expert = c->ffn / 32;
            g1.kchunks = L.gate_up.kchunks;
            g1.k = c->hidden;
            g1.rows = m;
            g1.xfrag = c->xf_a;
            g1.x_stride = 0;
            g1.out = c->frag_e;
            g1.out_stride = c->frag_e_stride;
            g1.n_out = c->ffn;
            g1.selected = ra2.selected;
            g1.top_k = L.top_k;
            g1.bias = L.be_gate;
            g1.bias2 = L.be_up;
            g1.alpha = c->act_alpha;
            g1.limit = c->act_limit;
            const int n_groups = m * L.top_k;
            g2 = g1;
            g2.bias = L.be_down;
            g2.bias2 = nullptr;
            g2.w = L.down.tiles;
            g2.tiles_per_expert = c->hidden / 64;
            g2.kchunks = L.down.kchunks;
            g2.k = c->ffn;
            g2.xfrag = c->frag_e;
            g2.x_stride = c->frag_e_stride;
            g2.out = c->moe_out;
            g2.out_stride = 0;
            g2.n_out = c->hidden;
            const bool fp4 = c->moe_fp4_terms != 0;
            if (fp4) {
                g1.x8_terms = g2.x8_terms = c->moe_fp4_terms;
                g1.x8 = c->x8_h;
                g1.o8 = c->x8_e;
                g1.o8_q_stride = c->x8_e_q_stride;
                g1.o8_s_stride = c->x8_e_s_stride;
                g2.x8 = c->x8_e;
                g2.x8_q_stride = c->x8_e_q_stride;
                g2.x8_s_stride = c->x8_e_s_stride;
                g2.o8 = X8{};
            }
            {
                PROF(PC_GATEUP);
                rc = 0;
                for (int rep = 0; rep < c->repeat[PC_GATEUP] && !rc; rep++) {
                    rc = launch_gemm(s, L.router, c->xf_a, c->partial, c->vp_dev, m, rsp, EPI_PARTIAL, L.n_experts, L.n_experts);
                    if (!rc) rc = launch_route(s, ra2);
                    if (!rc) rc = fp4 ? launch_moe_fp4_gate_up(s, g1, n_groups) : launch_moe_gate_up(s, L.gate_up.fmt, g1, n_groups);
                }
            }
            if (rc) return rc;
            {
                PROF(PC_DOWN);
                rc = 0;
                for (int rep = 0; rep < c->repeat[PC_DOWN] && !rc; rep++)
                    rc = fp4 ? launch_moe_fp4_down(s, g2, n_groups) : launch_moe_down(s, L.down.fmt, g2, n_groups);
            }
            if (rc) return rc;
            prev_partial = c->moe_out;
            prev_splits = L.top_k;
            prev_weights = c->route_w;
            continue;
        }
        {
            PROF(PC_GATEUP);
            rc = 0;
            for (int rep = 0; rep < c->repeat[PC_GATEUP] && !rc; rep++)
                rc = launch_gemm(s, L.gate_up, c->xf_a, c->xf_c, c->vp_dev, m, 1, EPI_SILU, 0, 0);
        }
        if (rc) return rc;
        sp = splits_for(L.down, m, EPI_PARTIAL);
        {
            PROF(PC_DOWN);
            rc = 0;
            for (int rep = 0; rep < c->repeat[PC_DOWN] && !rc; rep++)
                rc = launch_gemm(s, L.down, c->xf_c, c->partial, c->vp_dev, m, sp, EPI_PARTIAL, c->hidden, c->hidden);
        }
        if (rc) return rc;
        prev_partial = c->partial;
        prev_splits = sp;
    }
    // produce_prefill (producer.rs:92-103, real_forward_traits.rs:291-300): a prompt token whose
    // logits nobody reads skips the final norm and the output head; every other side effect of
    // the pass (the rows in the cache, the cursor) is that of a full pass.
    // (With a drafter head attached the rows' last residual add still happens: the head reads them.)
    if (c->headless && !c->mtp_head) return TSV_OK;
    {
        PROF(PC_NORM);
        rc = launch_addnorm(s, x, prev_partial, prev_splits, c->hidden, c->final_norm, c->eps, c->hidden, c->xf_a, m,
                            prev_weights);
    }
    if (rc || c->headless) return rc;
    {
        PROF(PC_HEAD);
        rc = 0;
        for (int rep = 0; rep < c->repeat[PC_HEAD] && !rc; rep++)
            rc = launch_gemm(s, c->head, c->xf_a, c->logits, c->vp_dev, m, 1, EPI_LOGITS, c->vocab, c->vocab);
    }
    return rc;
}

// ---- prompt passes of 64 rows -------------------------------------------------------------
// producer.rs:122-150 (ChunkedPrefillRunner) feeds a prompt in blocks; here a block of 64 tokens is
// one pass whose matmuls read every weight tile once for all 64 rows (k_gemm_wide).  The rows are
// kept as four blocks of sixteen so that everything else -- embedding, norms, the rotating epilogue's
// cache stores, attention -- is the 16-row pass's own code on block-strided buffers: block b is
// rows base + 16 b .. base + 16 b + 15, its attention sees the cache up to its own rows, which the
// q/k/v projection of the same pass has already stored for every block before any block attends.
// Only for headless passes (no logits wanted), in any of the storage types the 64-row matmuls read
// (wide_fmt; the q/k/v projection with the rotating epilogue, or followed by the rotation kernel over
// the four blocks; routed layers through the experts' member lists).  A ring layer stores and attends
// the four blocks one after the other (below).
constexpr int WIDE_B = 4;
static bool wide_fmt(int fmt) { return fmt == FMT_Q4K || fmt == FMT_Q5K || fmt == FMT_Q6K || fmt == FMT_Q80 || fmt == FMT_BF16; }

int wide_prepare(tsv_ctx* c) {
    tsv_ctx::Wide& w = c->wide;
    if (w.ready) return TSV_OK;
    const int qd = c->nq * c->hd;
    const int kmax = std::max(std::max(c->hidden, qd), c->ffn);
    w.xfb = xfrag_bytes(kmax);
    int rc;
    if ((rc = dev_alloc(c, &w.x, (size_t)WIDE_B * 16 * c->hidden * 4, true)) || (rc = dev_alloc(c, &w.xf_a, WIDE_B * w.xfb, true)) ||
        (rc = dev_alloc(c, &w.xf_b, WIDE_B * w.xfb, true)) || (rc = dev_alloc(c, &w.xf_c, WIDE_B * w.xfb, true)) ||
        (rc = dev_alloc(c, &w.partial, (size_t)WIDE_B * c->partial_floats * 4, true)) ||
        (rc = dev_alloc(c, &w.q16, (size_t)WIDE_B * 16 * qd * 2, true)) || (rc = dev_alloc(c, &w.vp, WIDE_B * sizeof(VerifyParams), true)) ||
        (rc = dev_alloc(c, &w.rope_cs, (size_t)WIDE_B * 16 * (c->hd / 2) * sizeof(float2), true)))
        return rc;
    const size_t rows_max = (size_t)TSV_MAX_ROWS * (c->nq / c->nkv);
    w.part_o_stride = (size_t)c->nkv * c->nch * rows_max * c->hd;
    w.part_ml_stride = (size_t)c->nkv * c->nch * rows_max * 2;
    if ((rc = dev_alloc(c, &w.part_o, WIDE_B * w.part_o_stride * 4, true)) || (rc = dev_alloc(c, &w.part_ml, WIDE_B * w.part_ml_stride * 4, true)))
        return rc;
    int ne_max = 0;
    for (const LayerW& L : c->layers) ne_max = std::max(ne_max, L.n_experts);
    if (ne_max) {
        w.frag_e_sub = (xfrag_bytes(c->ffn) + 255) & ~(size_t)255;
        if ((rc = dev_alloc(c, &w.route_w, (size_t)WIDE_B * 16 * 8 * 4, true)) || (rc = dev_alloc(c, &w.route_sel, (size_t)WIDE_B * 16 * 8 * 4, true)) ||
            (rc = dev_alloc(c, &w.groups, (size_t)ne_max * sizeof(MoeGroupW), true)) ||
            (rc = dev_alloc(c, &w.frag_e, (size_t)ne_max * WIDE_B * w.frag_e_sub, true)) ||
            (rc = dev_alloc(c, &w.moe_out, (size_t)WIDE_B * 8 * 16 * c->hidden * 4, true)))
            return rc;
    }
    w.ready = true;
    return TSV_OK;
}

int launch_wide_pass(tsv_ctx* c, int64_t base) {
    hipStream_t s = c->stream;
    tsv_ctx::Wide& w = c->wide;
    int rc;
    const int qd = c->nq * c->hd, half = c->hd / 2;
    for (int b = 0; b < WIDE_B; b++)
        if ((rc = launch_embed(s, c->embed_raw, c->embed_dtype, c->hidden, w.x + (size_t)b * 16 * c->hidden, w.vp + b, 16, c->freqs,
                               c->rope_mscale, half, w.rope_cs + (size_t)b * 16 * half)))
            return rc;
    const NormBlocks nb{(long)16 * c->hidden, (long)c->partial_floats, (long)w.xfb, 1, nullptr};
    // after a routed layer the partial sums are the blocks' per-slot expert outputs and come with the rows' factors
    const long moe_block = (long)8 * 16 * c->hidden;
    const NormBlocks nb_moe{nb.x, moe_block, nb.frag, 1, nullptr};
    const size_t pstride = c->partial_floats * 4;
    const int qkv_n = (c->nq + 2 * c->nkv) * c->hd;
    int prev_splits = 0;
    const float* prev_partial = w.partial;
    const float* prev_weights = nullptr;
    for (int l = 0; l < c->n_layers; l++) {
        LayerW& L = c->layers[l];
        if ((rc = launch_addnorm(s, w.x, prev_partial, prev_splits, c->hidden, L.attn_norm, c->eps, c->hidden, (uint4*)w.xf_a, 16, prev_weights,
                                 nullptr, nullptr, 0, WIDE_B, prev_weights ? &nb_moe : &nb)))
            return rc;
        prev_partial = w.partial;
        prev_weights = nullptr;
        RopeEpi re{};
        re.cs = w.rope_cs;
        re.bias = L.bqkv;
        re.q16 = w.q16;
        re.kc = L.kc;
        re.vc = L.vc;
        re.nq = c->nq;
        re.nkv = c->nkv;
        re.hd = c->hd;
        re.max_ctx = L.kv_slots;
        // A ring layer (kv_cache.rs:360-378) holds window + 32 positions, fewer than a 64-row pass would write ahead of
        // its first block's window: there the rows are stored and attended one block of sixteen after the other,
        // exactly the cache states four 16-row passes go through; everywhere else all 64 rows are stored (and, where
        // the layer keeps quantized rows, quantized) before any block attends, and the four blocks are one launch.
        const bool ring = L.cap < c->ctx_alloc;
        // The rotating epilogue needs whole sums, so its launch has one workgroup per tile (96 at the 8B shape, for 256
        // compute units: 29.7 us); split along K it fills the chip and the rotation kernel finishes all four blocks in
        // one launch.  TSV_WIDE_ROPE_FUSED=1 keeps the epilogue (not on ring layers: it stores all 64 rows at once).
        const bool epilogue = L.rope_fused && w.keep_epilogue && !ring;
        int spq = 1;
        if (epilogue) {
            if ((rc = launch_gemm_wide(s, L.qkv, (const uint4*)w.xf_a, w.xfb, nullptr, 0, w.vp, 1, EPI_ROPE, qkv_n, L.qkv.n_rows, &re))) return rc;
        } else {
            // the projection's partial sums; the 16-row pass's own norm / rotation / cache stores follow
            spq = splits_for(L.qkv, 16, EPI_PARTIAL);
            if (L.v_only.tiles) {  // (the value projection in a storage type of its own: one split count for both pieces)
                auto fits = [](const TiledW& t, int n) {
                    const int kslice = (t.kchunks + n - 1) / n;
                    return (t.kchunks + kslice - 1) / kslice == n;
                };
                while (spq > 1 && !(fits(L.qkv, spq) && fits(L.v_only, spq))) spq--;
            }
            if ((rc = launch_gemm_wide(s, L.qkv, (const uint4*)w.xf_a, w.xfb, w.partial, pstride, w.vp, spq, EPI_PARTIAL, qkv_n, L.qkv.n_rows)))
                return rc;
            if (L.v_only.tiles && (rc = launch_gemm_wide(s, L.v_only, (const uint4*)w.xf_a, w.xfb, w.partial + L.qkv.n_rows, pstride, w.vp, spq,
                                                         EPI_PARTIAL, qkv_n, L.v_only.n_rows)))
                return rc;
        }
        // rotation + cache stores, quantization and attention of blocks b0 .. b0 + nb - 1 (one launch each)
        auto store_rows = [&](int b0, int nb) -> int {
            if (epilogue) return TSV_OK;
            RopeKvArgs ra{};
            ra.qkv = w.partial + (size_t)b0 * c->partial_floats;
            ra.blocks = nb;
            ra.qkv_block_stride = (long)c->partial_floats;
            ra.paired = L.rope_fused && c->hd == 128;
            ra.splits = spq;
            ra.ldq = qkv_n;
            ra.freqs = c->freqs;
            ra.mscale = c->rope_mscale;
            ra.bias = L.bqkv;
            ra.q_norm = L.q_norm;
            ra.k_norm = L.k_norm;
            ra.eps = c->eps;
            ra.q16 = w.q16 + (size_t)b0 * 16 * qd;
            ra.kc = L.kc;
            ra.vc = L.vc;
            ra.nq = c->nq;
            ra.nkv = c->nkv;
            ra.hd = c->hd;
            ra.max_ctx = L.kv_slots;
            ra.vp = w.vp + b0;
            return launch_rope_kv(s, ra, 16);
        };
        auto attend = [&](int b0, int nb) -> int {
            if (L.tq.k_bits) {  // the rows are quantized (and their q rows rotated) before they are attended
                TqArgs ta{};
                ta.q16 = w.q16 + (size_t)b0 * 16 * qd;
                ta.kc = L.kc;
                ta.vc = L.vc;
                ta.stage_cap = L.kv_slots;
                ta.store = L.tq;
                ta.k = c->tq_k;
                ta.v = c->tq_v;
                ta.nq = c->nq;
                ta.nkv = c->nkv;
                ta.hd = c->hd;
                ta.cap = L.cap;
                ta.vp = w.vp + b0;
                ta.m_hint = 16 * nb;
                ta.base_hint = (int)base + 16 * b0;
                if (int trc = launch_tq_prepare(s, ta)) return trc;
            }
            // the blocks in one launch: block b attends with its own base position base + 16 b
            AttnArgs aa{};
            aa.q16 = w.q16 + (size_t)b0 * 16 * qd;
            aa.kc = L.kc;
            aa.vc = L.vc;
            aa.unrot = L.tq.k_bits ? c->tq_v.signs : nullptr;
            aa.tq = L.tq;
            aa.part_o = w.part_o + (size_t)b0 * w.part_o_stride;
            aa.part_ml = w.part_ml + (size_t)b0 * w.part_ml_stride;
            aa.xfrag = (uint4*)(w.xf_b + (size_t)b0 * w.xfb);
            aa.nq = c->nq;
            aa.nkv = c->nkv;
            aa.hd = c->hd;
            aa.max_ctx = L.cap;
            aa.ring = ring;
            aa.nch = c->nch;
            aa.scale = c->attn_scale;
            aa.window = L.window;
            aa.sinks = L.sinks;
            aa.vp = w.vp + b0;
            aa.m_hint = 16;
            aa.base_hint = (int)base + 16 * b0;
            aa.frag16 = 1;
            aa.blocks = nb;
            aa.q_stride = (size_t)16 * qd;
            aa.part_o_stride = w.part_o_stride;
            aa.part_ml_stride = w.part_ml_stride;
            aa.frag_stride = w.xfb;
            return launch_attention(s, aa, 16);
        };
        if (ring) {
            for (int b = 0; b < WIDE_B; b++)
                if ((rc = store_rows(b, 1)) || (rc = attend(b, 1))) return rc;
        } else if ((rc = store_rows(0, WIDE_B)) || (rc = attend(0, WIDE_B))) {
            return rc;
        }
        int sp = splits_for(L.wo, 16, EPI_PARTIAL);
        if ((rc = launch_gemm_wide(s, L.wo, (const uint4*)w.xf_b, w.xfb, w.partial, pstride, w.vp, sp, EPI_PARTIAL, c->hidden, c->hidden)))
            return rc;
        if (L.n_experts) {
            // routed experts over the 64 rows: the router and the expert matmuls read the 16-row kernels' fragment
            // layout; the router runs block by block (its matrix is small), its ranking as one launch of four
            // workgroups; then every expert is multiplied once against all of the pass's rows that chose it
            // (where the router's format has a 64-row matmul the norm leaves its rows in that kernel's layout as well,
            //  in the buffer the dense FFN would use, and the router is one launch; else one launch per block)
            const bool wide_router = wide_fmt(L.router.fmt);
            const NormBlocks nb4{nb.x, nb.partial, nb.frag, 0, wide_router ? (void*)w.xf_c : nullptr};
            if ((rc = launch_addnorm(s, w.x, w.partial, sp, c->hidden, L.ffn_norm, c->eps, c->hidden, (uint4*)w.xf_a, 16, nullptr, L.bo,
                                     nullptr, 0, WIDE_B, &nb4)))
                return rc;
            const int rsp = splits_for(L.router, 16, EPI_PARTIAL);
            if (wide_router) {
                if ((rc = launch_gemm_wide(s, L.router, (const uint4*)w.xf_c, w.xfb, w.partial, pstride, w.vp, rsp, EPI_PARTIAL, L.n_experts,
                                           L.n_experts)))
                    return rc;
            } else {
                for (int b = 0; b < WIDE_B; b++)
                    if ((rc = launch_gemm(s, L.router, (const uint4*)(w.xf_a + (size_t)b * w.xfb), w.partial + (size_t)b * c->partial_floats,
                                          w.vp + b, 16, rsp, EPI_PARTIAL, L.n_experts, L.n_experts)))
                        return rc;
            }
            MoeRouteArgs ra{};
            ra.logits = w.partial;
            ra.splits = rsp;
            ra.ld = L.n_experts;
            ra.n_experts = L.n_experts;
            ra.top_k = L.top_k;
            ra.m = 16;
            ra.weights = w.route_w;
            ra.selected = w.route_sel;
            ra.bias = L.router_bias;
            ra.forced = nullptr;
            ra.blocks = WIDE_B;
            ra.logits_block_stride = (long)c->partial_floats;
            if ((rc = launch_route(s, ra)) || (rc = launch_moe_groups(s, w.route_sel, 16 * WIDE_B, L.top_k, L.n_experts, w.groups))) return rc;
            MoeGemmArgs g1{};
            g1.w = L.gate_up.tiles;
            g1.tiles_per_expert = c->ffn / 32;
            g1.kchunks = L.gate_up.kchunks;
            g1.k = c->hidden;
            g1.rows = 16 * WIDE_B;
            g1.xfrag = w.xf_a;
            g1.x_stride = 0;
            g1.x_block_stride = w.xfb;
            g1.out = w.frag_e;
            g1.out_stride = WIDE_B * w.frag_e_sub;
            g1.sub_stride = w.frag_e_sub;
            g1.n_out = c->ffn;
            g1.selected = w.route_sel;
            g1.top_k = L.top_k;
            g1.bias = L.be_gate;
            g1.bias2 = L.be_up;
            g1.alpha = c->act_alpha;
            g1.limit = c->act_limit;
            g1.groups = w.groups;
            g1.n_experts = L.n_experts;
            MoeGemmArgs g2 = g1;
            g2.bias = L.be_down;
            g2.bias2 = nullptr;
            g2.w = L.down.tiles;
            g2.tiles_per_expert = c->hidden / 64;
            g2.kchunks = L.down.kchunks;
            g2.k = c->ffn;
            g2.xfrag = w.frag_e;
            g2.x_stride = WIDE_B * w.frag_e_sub;
            g2.out = w.moe_out;
            g2.out_stride = 0;
            g2.out_block_stride = (size_t)moe_block;
            g2.n_out = c->hidden;
            if ((rc = launch_moe_wide_gate_up(s, L.gate_up.fmt, g1)) || (rc = launch_moe_wide_down(s, L.down.fmt, g2))) return rc;
            prev_partial = w.moe_out;
            prev_splits = L.top_k;
            prev_weights = w.route_w;
            continue;
        }
        if ((rc = launch_addnorm(s, w.x, w.partial, sp, c->hidden, L.ffn_norm, c->eps, c->hidden, (uint4*)w.xf_a, 16, nullptr, L.bo, nullptr,
                                 0, WIDE_B, &nb)))
            return rc;
        if ((rc = launch_gemm_wide(s, L.gate_up, (const uint4*)w.xf_a, w.xfb, w.xf_c, w.xfb, w.vp, 1, EPI_SILU, 0, 0))) return rc;
        sp = splits_for(L.down, 16, EPI_PARTIAL);
        if ((rc = launch_gemm_wide(s, L.down, (const uint4*)w.xf_c, w.xfb, w.partial, pstride, w.vp, sp, EPI_PARTIAL, c->hidden, c->hidden)))
            return rc;
        prev_splits = sp;
    }
    // headless: nobody reads these rows' logits, and the last layer's sums are added only for a drafter head,
    // which reads the finished rows (64 consecutive rows of w.x)
    if (c->mtp_head)
        return launch_addnorm(s, w.x, prev_partial, prev_splits, c->hidden, c->final_norm, c->eps, c->hidden, (uint4*)w.xf_a, 16, prev_weights,
                              nullptr, nullptr, 0, WIDE_B, prev_weights ? &nb_moe : &nb);
    return TSV_OK;
}

// One 64-row prompt pass at the cursor: parameters of the four blocks, then the kernels.
int enqueue_wide_prefill(tsv_ctx* c, const int32_t* ids, int64_t base) {
    const int rows = 16 * WIDE_B;
    if (base != c->position) {
        set_error("prefill: start position does not match the KV cursor");
        return TSV_ERR_INVALID;
    }
    if (base + rows > c->max_context) {
        set_error("prefill: block would write past the KV capacity");
        return TSV_ERR_INVALID;
    }
    int rc = wide_prepare(c);
    if (rc) return rc;
    VerifyParams vp[WIDE_B];
    for (int b = 0; b < WIDE_B; b++)
        if ((rc = fill_params(vp[b], ids + 16 * b, nullptr, 16, base + 16 * b, c->vocab))) return rc;
    static_assert(WIDE_B <= tsv_ctx::ParamRing::PER_SLOT, "a staging slot holds a prompt pass's blocks");
    if ((rc = stage_params(c, vp, WIDE_B, c->wide.vp))) return rc;
    if ((rc = launch_wide_pass(c, base))) return rc;
    c->position = base + rows;
    c->high_water = std::max(c->high_water, c->position);
    c->last_m = 0;  // no logits on the device for tsv_accept to judge
    c->x_rows = 0;  // (the pass's rows are in the wide buffers, not in x)
    if (c->mtp_head) c->mtp_head->mtp.own_valid = false;
    return TSV_OK;
}

int run_pass(tsv_ctx* c, int m) {
    if (!c->use_graph || c->profile || c->headless || c->mtp.on) return launch_pass(c, m);
    if (!c->pass_graph[m]) {
        hipGraph_t g = nullptr;
        TSV_HIP(hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal));
        const int rc = launch_pass(c, m);
        const hipError_t e = hipStreamEndCapture(c->stream, &g);
        if (rc || e != hipSuccess) {
            if (g) (void)hipGraphDestroy(g);
            if (!rc) set_error(std::string("verify: graph capture failed: ") + hipGetErrorString(e));
            return rc ? rc : TSV_ERR_DEVICE;
        }
        const hipError_t ei = hipGraphInstantiate(&c->pass_graph[m], g, nullptr, nullptr, 0);
        (void)hipGraphDestroy(g);
        if (ei != hipSuccess) {
            c->pass_graph[m] = nullptr;
            set_error(std::string("verify: graph instantiation failed: ") + hipGetErrorString(ei));
            return TSV_ERR_DEVICE;
        }
    }
    TSV_HIP(hipGraphLaunch(c->pass_graph[m], c->stream));
    return TSV_OK;
}

int finish_verify(tsv_ctx* c, int m, uint16_t* logits_out) {
    if (logits_out) {
        TSV_HIP(hipMemcpyAsync(logits_out, c->logits, (size_t)m * c->vocab * 2, hipMemcpyDeviceToHost, c->stream));
        TSV_HIP(hipStreamSynchronize(c->stream));
    }
    return TSV_OK;
}

}  // namespace tsv

// `share` / `md`: a drafter head opened on a target handle -- its stream, embedding table and output head are
// the target's, and md names fc and the norms of fc's two halves.
int tsv::open_impl(const tsv_model_desc* d, tsv_ctx* share, const tsv_mtp_desc* md, tsv_ctx** out) {
    if (!d || !out || !d->layers) {
        set_error("open: null argument");
        return TSV_ERR_INVALID;
    }
    if (d->n_layers < 1 || !d->layers || d->hidden < 1 || d->n_q_heads < 1 || d->n_kv_heads < 1 || d->ffn < 1 ||
        d->vocab < 1 || d->max_context < 1) {
        set_error("open: layer count, widths, head counts, vocabulary and context must all be positive");
        return TSV_ERR_INVALID;
    }
    if (d->head_dim != 64 && d->head_dim != 128) {
        set_error("open: head_dim must be 64 or 128");
        return TSV_ERR_UNSUPPORTED;
    }
    if (d->n_q_heads % d->n_kv_heads || d->n_q_heads / d->n_kv_heads > 8 || d->hidden % 32 || d->ffn % 32) {
        set_error("open: unsupported head grouping or widths");
        return TSV_ERR_UNSUPPORTED;
    }
    tsv_ctx* c = new tsv_ctx();
    auto fail = [&](int rc) {
        tsv_close(c);
        return rc;
    };
    c->n_layers = d->n_layers;
    c->hidden = d->hidden;
    c->nq = d->n_q_heads;
    c->nkv = d->n_kv_heads;
    c->hd = d->head_dim;
    c->ffn = d->ffn;
    c->vocab = d->vocab;
    c->max_context = d->max_context;
    c->ctx_alloc = ((d->max_context + 15) / 16) * 16;
    c->eps = d->rms_eps;
    c->attn_scale = d->attn_scale > 0.f ? d->attn_scale : 1.0f / std::sqrt((float)d->head_dim);
    c->rope_mscale = d->rope_mscale > 0.f ? d->rope_mscale : 1.0f;
    c->act_alpha = d->act_alpha;
    c->act_limit = d->act_limit;
    if (const char* e = getenv("TSV_GRAPH")) c->use_graph = e[0] == '1';
    if (const char* e = getenv("TSV_ROPE_FUSED")) {
        c->rope_fused_ok = e[0] != '0';
        c->rope_fused_force = e[0] == '1';
    }
    // MXFP4 experts on the block-scaled matrix instruction: activation terms, 0 = the fp16 path
    c->moe_fp4_terms = MOE_FP4_DEFAULT_TERMS;
    if (const char* e = getenv("TSV_MOE_FP4")) c->moe_fp4_terms = e[0] == '2' ? 2 : e[0] == '3' ? 3 : 0;
    if (share) {
        c->stream = share->stream;
        c->owns_stream = false;
    } else if (hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking) != hipSuccess) {
        set_error("open: cannot create a HIP stream (no GPU?)");
        delete c;
        return TSV_ERR_DEVICE;
    }
    int rc;
    if (d->kv_k_bits || d->kv_v_bits) {
        // crates/model-io/src/kv_quant.rs:48-72: the widths --kv-bits can name (2, 3, 3.5 = K3/V4, 4);
        // crates/runtime/src/real_forward_init.rs:170-199: refused by name when no layer would be quantized
        const int kb = d->kv_k_bits, vb = d->kv_v_bits;
        if (!((kb == 2 && vb == 2) || (kb == 3 && vb == 3) || (kb == 3 && vb == 4) || (kb == 4 && vb == 4))) {
            set_error("open: KV quantization widths must be one of K2/V2, K3/V3, K3/V4, K4/V4");
            return fail(TSV_ERR_INVALID);
        }
        bool any = false;
        for (int l = 0; l < d->n_layers; l++)
            any = any || (d->layers[l].window == 0 && (d->n_layers <= 2 || l + 1 < d->n_layers));
        if (!any) {
            set_error("open: KV quantization has nothing to quantize here: every full-attention layer is excluded by "
                      "the last-layer rule, or there are no full-attention layers at all");
            return fail(TSV_ERR_UNSUPPORTED);
        }
        float* tables = nullptr;
        if ((rc = dev_alloc(c, &tables, (size_t)2 * TQ_TABLE_FLOATS * 4)) ||
            (rc = tq_upload_side(c->hd, kb, 0, tables, &c->tq_k)) ||
            (rc = tq_upload_side(c->hd, vb, 1, tables + TQ_TABLE_FLOATS, &c->tq_v)))
            return fail(rc);
        c->kv_k_bits = kb;
        c->kv_v_bits = vb;
    }
    Stager st;
    const int qd = c->nq * c->hd, kvd = c->nkv * c->hd;
    c->layers.resize(c->n_layers);
    size_t pneed = 0;
    for (int l = 0; l < c->n_layers; l++) {
        const tsv_layer& s = d->layers[l];
        LayerW& L = c->layers[l];
        if ((rc = check_matrix(s.wq, qd, c->hidden, "wq")) || (rc = check_matrix(s.wk, kvd, c->hidden, "wk")) ||
            (rc = check_matrix(s.wv, kvd, c->hidden, "wv")) || (rc = check_matrix(s.wo, c->hidden, qd, "wo")))
            return fail(rc);
        const tsv_tensor* qkv[3] = {&s.wq, &s.wk, &s.wv};
        const tsv_tensor* wo[1] = {&s.wo};
        if (s.wq.dtype != s.wk.dtype) {
            set_error("open: the q and k projections must share a storage type");
            return fail(TSV_ERR_UNSUPPORTED);
        }
        // One launch that projects, rotates and stores (no split-K partials, no separate rotation
        // kernel) where the head needs no per-head norm in between and q/k/v share a storage type.
        // The fused launch has one workgroup per 64-row tile and no K split, and one compute unit draws only so much:
        // it is taken while a tile's weights stay under 256 KiB (8B Q4_K: 147 KB per tile, a tie with the two
        // launches; gpt-oss-120B bf16: 369 KB, 15.3 us fused against 7.9 + 3.1 us apart).
        const bool light_tiles = 64 * row_bytes(s.wq.dtype, s.wq.cols) <= 256 * 1024;
        L.rope_fused = c->rope_fused_ok && (light_tiles || c->rope_fused_force) && s.wv.dtype == s.wq.dtype &&
                       !s.q_norm.data && !s.k_norm.data && (c->hd == 64 || c->hd == 128);
        if (s.wv.dtype == s.wq.dtype) {
            if ((rc = make_tiled(c, st, qkv, 3, false, &L.qkv, L.rope_fused && c->hd == 128 ? 2 : 0))) return fail(rc);
        } else {
            const tsv_tensor* vonly[1] = {&s.wv};
            if ((rc = make_tiled(c, st, qkv, 2, false, &L.qkv)) || (rc = make_tiled(c, st, vonly, 1, false, &L.v_only)))
                return fail(rc);
        }
        if ((rc = make_tiled(c, st, wo, 1, false, &L.wo))) return fail(rc);
        const int ne = s.n_experts;
        if (ne > 0) {
            // every expert's gate/up rows interleave in runs of 32 inside the stacked matrix, so an
            // expert owns ffn / 32 consecutive tiles; its down projection owns hidden / 64 tiles
            if (ne > 256 || s.top_k < 1 || s.top_k > 8 || s.top_k > ne || c->ffn % 32 || c->hidden % 64) {
                set_error("open: routed experts need <= 256 experts, top-k in 1..8, ffn % 32 == 0, hidden % 64 == 0");
                return fail(TSV_ERR_UNSUPPORTED);
            }
            if ((rc = check_matrix(s.router, ne, c->hidden, "router")) ||
                (rc = check_matrix(s.we_gate, (int64_t)ne * c->ffn, c->hidden, "we_gate")) ||
                (rc = check_matrix(s.we_up, (int64_t)ne * c->ffn, c->hidden, "we_up")) ||
                (rc = check_matrix(s.we_down, (int64_t)ne * c->hidden, c->ffn, "we_down")))
                return fail(rc);
            const tsv_tensor* rt[1] = {&s.router};
            const tsv_tensor* gu[2] = {&s.we_gate, &s.we_up};
            const tsv_tensor* dn[1] = {&s.we_down};
            if ((rc = make_tiled(c, st, rt, 1, false, &L.router)) || (rc = make_tiled(c, st, gu, 2, true, &L.gate_up)) ||
                (rc = make_tiled(c, st, dn, 1, false, &L.down)))
                return fail(rc);
            pneed = std::max(pneed, partial_need(L.router));
            L.n_experts = ne;
            L.top_k = s.top_k;
            if (L.gate_up.fmt != FMT_MX4 || L.down.fmt != FMT_MX4) c->moe_fp4_terms = 0;
            c->max_experts = std::max(c->max_experts, ne);
        } else {
            if ((rc = check_matrix(s.w_gate, c->ffn, c->hidden, "w_gate")) ||
                (rc = check_matrix(s.w_up, c->ffn, c->hidden, "w_up")) ||
                (rc = check_matrix(s.w_down, c->hidden, c->ffn, "w_down")))
                return fail(rc);
            const tsv_tensor* gu[2] = {&s.w_gate, &s.w_up};
            const tsv_tensor* dn[1] = {&s.w_down};
            if ((rc = make_tiled(c, st, gu, 2, true, &L.gate_up)) || (rc = make_tiled(c, st, dn, 1, false, &L.down)))
                return fail(rc);
            pneed = std::max(pneed, partial_need(L.down));
        }
        if ((rc = upload_vector(c, s.attn_norm, c->hidden, &L.attn_norm, "attn_norm")) ||
            (rc = upload_vector(c, s.ffn_norm, c->hidden, &L.ffn_norm, "ffn_norm")))
            return fail(rc);
        if (s.q_norm.data) {
            if ((rc = upload_vector(c, s.q_norm, c->hd, &L.q_norm, "q_norm")) ||
                (rc = upload_vector(c, s.k_norm, c->hd, &L.k_norm, "k_norm")))
                return fail(rc);
        }
        // gpt-oss additions (families/gptoss/mod.rs:11-23)
        if (s.bq.data || s.bk.data || s.bv.data) {
            if (!s.bq.data || !s.bk.data || !s.bv.data) {
                set_error("open: q, k and v projection biases come together");
                return fail(TSV_ERR_INVALID);
            }
            float *bq = nullptr, *bk = nullptr, *bv = nullptr;  // one device vector in the fused row order
            if ((rc = dev_alloc(c, &L.bqkv, (size_t)(qd + 2 * kvd) * 4))) return fail(rc);
            if ((rc = upload_vector(c, s.bq, qd, &bq, "bq")) || (rc = upload_vector(c, s.bk, kvd, &bk, "bk")) ||
                (rc = upload_vector(c, s.bv, kvd, &bv, "bv")))
                return fail(rc);
            if (hipMemcpy(L.bqkv, bq, (size_t)qd * 4, hipMemcpyDeviceToDevice) != hipSuccess ||
                hipMemcpy(L.bqkv + qd, bk, (size_t)kvd * 4, hipMemcpyDeviceToDevice) != hipSuccess ||
                hipMemcpy(L.bqkv + qd + kvd, bv, (size_t)kvd * 4, hipMemcpyDeviceToDevice) != hipSuccess)
                return fail(TSV_ERR_DEVICE);
        }
        if (s.bo.data && (rc = upload_vector(c, s.bo, c->hidden, &L.bo, "bo"))) return fail(rc);
        if (s.sinks.data && (rc = upload_vector(c, s.sinks, c->nq, &L.sinks, "sinks"))) return fail(rc);
        if (s.window < 0 || (s.window > 0 && s.window <= TSV_MAX_ROWS)) {
            set_error("open: a sliding window must be wider than one verify pass (16 rows)");
            return fail(TSV_ERR_UNSUPPORTED);
        }
        L.window = s.window;
        if (ne > 0) {
            if (s.router_bias.data && (rc = upload_vector(c, s.router_bias, ne, &L.router_bias, "router_bias")))
                return fail(rc);
            if (s.be_gate.data || s.be_up.data) {
                if (!s.be_gate.data || !s.be_up.data) {
                    set_error("open: expert gate and up biases come together");
                    return fail(TSV_ERR_INVALID);
                }
                if ((rc = upload_vector(c, s.be_gate, (int64_t)ne * c->ffn, &L.be_gate, "be_gate")) ||
                    (rc = upload_vector(c, s.be_up, (int64_t)ne * c->ffn, &L.be_up, "be_up")))
                    return fail(rc);
            }
            if (s.be_down.data && (rc = upload_vector(c, s.be_down, (int64_t)ne * c->hidden, &L.be_down, "be_down")))
                return fail(rc);
        }
        // kv_cache.rs:122-131,194-198: a windowed layer may keep a ring of window + chunk positions
        // instead of the whole context (position p in slot p % capacity); the slack beyond the window
        // is what a rollback may take back (kv_cache_rewind.rs:26-35).  Here the chunk is two passes
        // wide so that a pass can follow a rollback of a whole pass.
        L.cap = c->ctx_alloc;
        if (s.ring) {
            if (s.window <= 0) {
                set_error("open: only a layer with a sliding window can keep its cache as a ring");
                return fail(TSV_ERR_INVALID);
            }
            const int ring_cap = ((s.window + 15) / 16) * 16 + 2 * TSV_MAX_ROWS;
            if (ring_cap < c->ctx_alloc) {
                L.cap = ring_cap;
                c->rewind_budget = std::min<int64_t>(c->rewind_budget, ring_cap - s.window);
            }
        }
        const size_t kvb = (size_t)c->nkv * L.cap * c->hd * 2;
        // crates/model-io/src/kv_quant.rs:102-107: every full-attention layer of a stack of at most two, else
        // every one but the last; windowed layers keep fp16 rows
        L.kv_slots = L.cap;
        if (c->kv_k_bits && s.window == 0 && (c->n_layers <= 2 || l + 1 < c->n_layers)) {
            L.kv_slots = 4 * TSV_MAX_ROWS;  // a prompt pass of four 16-row blocks stages all of its rows
            const size_t stage = (size_t)c->nkv * L.kv_slots * c->hd * 2;
            if (!c->tq_kc && ((rc = dev_alloc(c, &c->tq_kc, stage, true)) || (rc = dev_alloc(c, &c->tq_vc, stage, true)))) return fail(rc);
            L.kc = c->tq_kc;
            L.vc = c->tq_vc;
            L.tq.k_bits = c->kv_k_bits;
            L.tq.v_bits = c->kv_v_bits;
            L.tq.k_cb = c->tq_k.cb;
            L.tq.v_cb = c->tq_v.cb;
            const size_t norms = (size_t)c->nkv * L.cap * 4;
            if ((rc = dev_alloc(c, &L.tq.kq, tq_kq_bytes(c->nkv, L.cap, c->hd, c->kv_k_bits), true)) ||
                (rc = dev_alloc(c, &L.tq.vq, tq_vq_bytes(c->nkv, L.cap, c->hd, c->kv_v_bits), true)) ||
                (rc = dev_alloc(c, &L.tq.kn, norms, true)) || (rc = dev_alloc(c, &L.tq.vn, norms, true)))
                return fail(rc);
        } else if ((rc = dev_alloc(c, &L.kc, kvb, true)) || (rc = dev_alloc(c, &L.vc, kvb, true))) {
            return fail(rc);
        }
        pneed = std::max(pneed, std::max(partial_need(L.qkv), partial_need(L.wo)));
        pneed = std::max(pneed, (size_t)8 * 16 * ((size_t)(qd + 2 * kvd) + TILE_ROWS));
    }
    {
        std::vector<uint16_t*> ptrs;
        for (auto& L : c->layers) {
            ptrs.push_back(L.kc);
            ptrs.push_back(L.vc);
        }
        if ((rc = dev_alloc(c, &c->kv_ptrs, ptrs.size() * sizeof(uint16_t*)))) return fail(rc);
        if (hipMemcpy(c->kv_ptrs, ptrs.data(), ptrs.size() * sizeof(uint16_t*), hipMemcpyHostToDevice) != hipSuccess)
            return fail(TSV_ERR_DEVICE);
        std::vector<int32_t> caps;
        // a quantized layer holds no fp16 rows to move (its staging slots are shared by all such layers and are dead
        // once the pass has quantized them; launch_tq_gather moves its stored rows): capacity 0, the gather skips it
        for (auto& L : c->layers) caps.push_back(L.tq.k_bits ? 0 : L.kv_slots);
        if ((rc = dev_alloc(c, &c->kv_caps, caps.size() * 4))) return fail(rc);
        if (hipMemcpy(c->kv_caps, caps.data(), caps.size() * 4, hipMemcpyHostToDevice) != hipSuccess) return fail(TSV_ERR_DEVICE);
    }
    if (c->kv_k_bits) {
        std::vector<TqKv> stores;
        for (auto& L : c->layers) stores.push_back(L.tq);
        if ((rc = dev_alloc(c, &c->tq_stores, stores.size() * sizeof(TqKv)))) return fail(rc);
        if (hipMemcpy(c->tq_stores, stores.data(), stores.size() * sizeof(TqKv), hipMemcpyHostToDevice) != hipSuccess)
            return fail(TSV_ERR_DEVICE);
    }
    // --session-slots (crates/runtime/src/real_forward_api.rs:526-556, real_forward_open.rs:674-716): slots - 1 parked
    // sessions, every one with KV buffers of its own, allocated here and never again
    if (d->session_slots > 1) {
        if (c->use_graph) {
            set_error("open: captured passes (TSV_GRAPH=1) hold the live session's buffers and cannot be used with a session pool");
            return fail(TSV_ERR_UNSUPPORTED);
        }
        if (d->session_slots > 64) {
            set_error("open: at most 64 session slots");
            return fail(TSV_ERR_INVALID);
        }
        for (int slot = 1; slot < d->session_slots; slot++) {
            tsv_ctx::Session ses;
            std::vector<uint16_t*> ptrs;
            for (auto& L : c->layers) {
                uint16_t *kc = L.kc, *vc = L.vc;  // a quantized layer: the shared staging slots
                TqKv tq = L.tq;
                if (L.tq.k_bits) {
                    const size_t norms = (size_t)c->nkv * L.cap * 4;
                    if ((rc = dev_alloc(c, &tq.kq, tq_kq_bytes(c->nkv, L.cap, c->hd, c->kv_k_bits), true)) ||
                        (rc = dev_alloc(c, &tq.vq, tq_vq_bytes(c->nkv, L.cap, c->hd, c->kv_v_bits), true)) ||
                        (rc = dev_alloc(c, &tq.kn, norms, true)) || (rc = dev_alloc(c, &tq.vn, norms, true)))
                        return fail(rc);
                } else {
                    const size_t kvb = (size_t)c->nkv * L.cap * c->hd * 2;
                    if ((rc = dev_alloc(c, &kc, kvb, true)) || (rc = dev_alloc(c, &vc, kvb, true))) return fail(rc);
                }
                ses.kc.push_back(kc);
                ses.vc.push_back(vc);
                ses.tq.push_back(tq);
                ptrs.push_back(kc);
                ptrs.push_back(vc);
            }
            if ((rc = dev_alloc(c, &ses.kv_ptrs, ptrs.size() * sizeof(uint16_t*)))) return fail(rc);
            if (hipMemcpy(ses.kv_ptrs, ptrs.data(), ptrs.size() * sizeof(uint16_t*), hipMemcpyHostToDevice) != hipSuccess)
                return fail(TSV_ERR_DEVICE);
            if (c->kv_k_bits) {
                if ((rc = dev_alloc(c, &ses.tq_stores, ses.tq.size() * sizeof(TqKv)))) return fail(rc);
                if (hipMemcpy(ses.tq_stores, ses.tq.data(), ses.tq.size() * sizeof(TqKv), hipMemcpyHostToDevice) != hipSuccess)
                    return fail(TSV_ERR_DEVICE);
            }
            c->parked.push_back(std::move(ses));
        }
    }
    // embedding table (raw GGUF rows for the lookup) and output head (tiled)
    const int64_t erb = row_bytes(d->embed.dtype, c->hidden);
    if (share) {
        if (d->embed.data || d->lm_head.data) {
            set_error("mtp_open: the head takes the target's embedding table and output head; leave both empty");
            return fail(TSV_ERR_INVALID);
        }
        c->embed_raw = share->embed_raw;
        c->embed_dtype = share->embed_dtype;
        c->head = share->head;
        const tsv_tensor* fp[1] = {&md->fc};
        if ((rc = check_matrix(md->fc, c->hidden, 2 * (int64_t)c->hidden, "fc")) || (rc = make_tiled(c, st, fp, 1, false, &c->mtp.fc)) ||
            (rc = upload_vector(c, md->norm_embedding, c->hidden, &c->mtp.norm_e, "norm_embedding")) ||
            (rc = upload_vector(c, md->norm_hidden, c->hidden, &c->mtp.norm_h, "norm_hidden")))
            return fail(rc);
        pneed = std::max(pneed, partial_need(c->mtp.fc));
    } else if (!d->embed.data || d->embed.rows != c->vocab || d->embed.cols != c->hidden || erb < 0) {
        set_error("open: embedding table shape / dtype");
        return fail(TSV_ERR_INVALID);
    } else {
        c->embed_dtype = d->embed.dtype;
        if ((rc = dev_alloc(c, &c->embed_raw, (size_t)(erb * c->vocab)))) return fail(rc);
        if (hipMemcpy(c->embed_raw, d->embed.data, (size_t)(erb * c->vocab), hipMemcpyHostToDevice) != hipSuccess) {
            set_error("open: embedding upload failed");
            return fail(TSV_ERR_DEVICE);
        }
    }
    if (!share) {
        tsv_tensor head = d->lm_head.data ? d->lm_head : d->embed;
        // the head's row count need not be a multiple of 16: the last tile is zero padded
        if ((rc = check_matrix(head, c->vocab, c->hidden, "output head"))) return fail(rc);
        const tsv_tensor* hp[1] = {&head};
        if ((rc = make_tiled(c, st, hp, 1, false, &c->head))) return fail(rc);
    }
    if (st.dev) (void)hipFree(st.dev);
    if ((rc = upload_vector(c, d->final_norm, c->hidden, &c->final_norm, "final_norm"))) return fail(rc);
    {
        // rope.rs:208-256 (scalar theta: exp(-(2i/hd) * ln theta)) or rope.rs:447-460 (per-pair divisors)
        std::vector<float> f((size_t)c->hd / 2);
        for (int i = 0; i < c->hd / 2; i++) {
            if (d->rope_freqs)
                f[i] = d->rope_freqs[i];  // an explicit table (YaRN)
            else if (d->rope_factors)
                f[i] = std::pow(d->rope_theta, -((float)(2 * i)) / (float)c->hd) / d->rope_factors[i];
            else
                f[i] = std::exp((-((float)(2 * i)) / (float)c->hd) * std::log(d->rope_theta));
        }
        if ((rc = dev_alloc(c, &c->freqs, f.size() * 4))) return fail(rc);
        if (hipMemcpy(c->freqs, f.data(), f.size() * 4, hipMemcpyHostToDevice) != hipSuccess) return fail(TSV_ERR_DEVICE);
        if ((rc = dev_alloc(c, &c->rope_cs, (size_t)TSV_MAX_ROWS * f.size() * sizeof(float2), true))) return fail(rc);
    }
    // scratch
    const int kmax = std::max(std::max(c->hidden, qd), c->ffn);
    const size_t xfb = xfrag_bytes(kmax);
    c->nch = attn_chunks(c->nkv);
    const size_t rows_max = (size_t)TSV_MAX_ROWS * (c->nq / c->nkv);
    c->partial_floats = pneed;
    c->x8_h.kpad = (c->hidden + 255) / 256 * 256;
    c->x8_e.kpad = (c->ffn + 255) / 256 * 256;
    if ((rc = dev_alloc(c, &c->x, (size_t)16 * c->hidden * 4, true)) || (rc = dev_alloc(c, &c->xf_a, xfb, true)) ||
        (rc = dev_alloc(c, &c->xf_b, xfb, true)) || (rc = dev_alloc(c, &c->xf_c, xfb, true)) ||
        (rc = dev_alloc(c, &c->partial, pneed * 4, true)) ||
        (c->max_experts &&
         ((rc = dev_alloc(c, &c->route_w, 16 * 8 * 4, true)) || (rc = dev_alloc(c, &c->route_sel, (size_t)c->n_layers * 16 * 8 * 4, true)) ||
          (rc = dev_alloc(c, &c->route_forced, (size_t)c->n_layers * 16 * 8 * 4)) ||
          (rc = dev_alloc(c, &c->frag_e, (size_t)TSV_MAX_ROWS * 8 * (c->frag_e_stride = (xfrag_bytes(c->ffn) + 255) & ~(size_t)255), true)) ||
          (rc = dev_alloc(c, &c->moe_out, (size_t)8 * 16 * c->hidden * 4, true)) ||
          (c->moe_fp4_terms &&
           ((rc = dev_alloc(c, &c->x8_h.q, x8_q_bytes(c->hidden), true)) || (rc = dev_alloc(c, &c->x8_h.s, x8_s_bytes(c->hidden), true)) ||
            (rc = dev_alloc(c, &c->x8_e.q, (size_t)TSV_MAX_ROWS * 8 * (c->x8_e_q_stride = x8_q_bytes(c->ffn)), true)) ||
            (rc = dev_alloc(c, &c->x8_e.s, (size_t)TSV_MAX_ROWS * 8 * (c->x8_e_s_stride = x8_s_bytes(c->ffn)), true)))))) ||
        (rc = dev_alloc(c, &c->q16, (size_t)16 * qd * 2, true)) ||
        (rc = dev_alloc(c, &c->part_o, (size_t)c->nkv * c->nch * rows_max * c->hd * 4, true)) ||
        (rc = dev_alloc(c, &c->part_ml, (size_t)c->nkv * c->nch * rows_max * 2 * 4, true)) ||
        (rc = dev_alloc(c, &c->logits, (size_t)16 * c->vocab * 2, true)) ||
        (rc = dev_alloc(c, &c->draft_stage, (size_t)16 * c->vocab * 2, true)) ||
        (rc = dev_alloc(c, &c->vp_dev, sizeof(VerifyParams), true)) ||
        (rc = dev_alloc(c, &c->ap_dev, sizeof(AcceptParams), true)) ||
        (rc = dev_alloc(c, &c->pen_cnt, (size_t)c->vocab * 4, true)) ||
        (rc = dev_alloc(c, &c->tok_dev, 64 * 4, true)) ||
        (rc = dev_alloc(c, &c->sc.stats, accept_stats_doubles() * 8, true)) ||
        (rc = dev_alloc(c, &c->sc.work, (size_t)(16 * 2 + 2) * c->vocab * 8, true)) ||
        (rc = dev_alloc(c, &c->sc.hist, (size_t)16 * 2 * 65536 * 8, true)) ||
        (rc = dev_alloc(c, &c->sc.counters, ACCEPT_COUNTER_WORDS * 4, true)) ||
        (rc = dev_alloc(c, &c->sc.tmass, (size_t)32 * 65536 * 8, true)) ||
        (rc = dev_alloc(c, &c->sc.tcount, (size_t)32 * 65536 * 4, true)) ||
        (rc = dev_alloc(c, &c->sc.result, sizeof(AcceptResult), true)))
        return fail(rc);
    if (c->route_forced && hipMemsetAsync(c->route_forced, 0xFF, (size_t)c->n_layers * 16 * 8 * 4, c->stream) != hipSuccess)
        return fail(TSV_ERR_DEVICE);  // every entry -1: rows route freely until tsv_force_route says otherwise
    for (hipEvent_t& e : c->ring.ev)
        if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) {
            set_error("open: event creation failed");
            return fail(TSV_ERR_DEVICE);
        }
    if (hipHostMalloc((void**)&c->ring.host, sizeof(VerifyParams) * tsv_ctx::ParamRing::SLOTS * tsv_ctx::ParamRing::PER_SLOT) != hipSuccess ||
        hipHostMalloc((void**)&c->vp_host, sizeof(VerifyParams)) != hipSuccess ||
        hipHostMalloc((void**)&c->ap_host, sizeof(AcceptParams)) != hipSuccess ||
        hipHostMalloc((void**)&c->res_host, sizeof(AcceptResult)) != hipSuccess ||
        hipHostMalloc((void**)&c->tok_host, 64 * 4) != hipSuccess) {
        set_error("open: pinned host allocation failed");
        return fail(TSV_ERR_DEVICE);
    }
    if (share) {
        tsv_ctx::Mtp& h = c->mtp;
        if ((rc = dev_alloc(c, &h.xf_cat, xfrag_bytes(2 * c->hidden), true)) || (rc = dev_alloc(c, &h.chain, 32 * 4, true)) ||
            (rc = dev_alloc(c, &h.vp_block, TSV_MAX_ROWS * sizeof(VerifyParams), true)) ||
            (rc = dev_alloc(c, &h.draw_dev, TSV_MAX_ROWS * sizeof(AcceptParams), true)))
            return fail(rc);
        if (hipHostMalloc((void**)&h.chain_host, 32 * 4) != hipSuccess ||
            hipHostMalloc((void**)&h.draw_host, TSV_MAX_ROWS * sizeof(AcceptParams)) != hipSuccess ||
            hipHostMalloc((void**)&h.vp_block_host, TSV_MAX_ROWS * sizeof(VerifyParams)) != hipSuccess) {
            set_error("mtp_open: pinned host allocation failed");
            return fail(TSV_ERR_DEVICE);
        }
        h.on = true;
        h.target = share;
    }
    if (int nrc = noalloc_prepare_device()) return fail(nrc);  // tsv_accept_greedy_noalloc is capturable from here on
    if (hipStreamSynchronize(c->stream) != hipSuccess) {
        set_error("open: device initialisation failed");
        return fail(TSV_ERR_DEVICE);
    }
    // 64-row prompt passes (TSV_WIDE_PREFILL=0 keeps every pass at sixteen rows)
    c->wide.ok = true;
    for (const LayerW& L : c->layers)
        if (L.n_experts) {  // routed layers: the attention projections as below, the experts in any format, fp16 activations
            if (c->moe_fp4_terms || !wide_fmt(L.qkv.fmt) || !wide_fmt(L.wo.fmt) || (L.v_only.tiles && !wide_fmt(L.v_only.fmt))) c->wide.ok = false;
        } else if (!wide_fmt(L.qkv.fmt) || !wide_fmt(L.wo.fmt) || (L.v_only.tiles && !wide_fmt(L.v_only.fmt)) ||
                   !wide_fmt(L.gate_up.fmt) || !wide_fmt(L.down.fmt))
            c->wide.ok = false;
    if (const char* e = getenv("TSV_WIDE_PREFILL")) c->wide.ok = c->wide.ok && e[0] != '0';
    if (const char* e = getenv("TSV_WIDE_ROPE_FUSED")) c->wide.keep_epilogue = e[0] == '1';
    if (share) c->wide.ok = false;  // the head's rows come sixteen at a time
    *out = c;
    return TSV_OK;
}

extern "C" int32_t tsv_open(const tsv_model_desc* d, tsv_ctx** out) { return open_impl(d, nullptr, nullptr, out); }

extern "C" void tsv_close(tsv_ctx* c) {
    if (!c) return;
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    for (void* p : c->allocs) (void)hipFree(p);
    if (c->hist_dev) (void)hipFree(c->hist_dev);
    if (c->vp_host) (void)hipHostFree(c->vp_host);
    if (c->ring.host) (void)hipHostFree(c->ring.host);
    for (hipEvent_t e : c->ring.ev)
        if (e) (void)hipEventDestroy(e);
    if (c->ap_host) (void)hipHostFree(c->ap_host);
    if (c->res_host) (void)hipHostFree(c->res_host);
    if (c->tok_host) (void)hipHostFree(c->tok_host);
    if (c->mtp.chain_host) (void)hipHostFree(c->mtp.chain_host);
    if (c->mtp.draw_host) (void)hipHostFree(c->mtp.draw_host);
    if (c->mtp.vp_block_host) (void)hipHostFree(c->mtp.vp_block_host);
    if (c->mtp.on && c->mtp.target && c->mtp.target->mtp_head == c) c->mtp.target->mtp_head = nullptr;
    for (hipGraphExec_t g : c->pass_graph)
        if (g) (void)hipGraphExecDestroy(g);
    for (hipEvent_t e : c->ev) (void)hipEventDestroy(e);
    if (c->stream && c->owns_stream) (void)hipStreamDestroy(c->stream);
    delete c;
}

extern "C" void* tsv_stream(tsv_ctx* c) { return c ? (void*)c->stream : nullptr; }

// session_pool.rs:116-121 best_scoring_index: the index of the highest score (the last one among equals, as
// Iterator::max_by_key returns), none when the pool is empty or every score is zero
extern "C" int64_t tsv_session_best_match(const int64_t* scores, int64_t n, int64_t* score_out) {
    int64_t best = 0, idx = -1;
    for (int64_t i = 0; scores && i < n; i++)
        if (scores[i] > 0 && scores[i] >= best) {
            best = scores[i];
            idx = i;
        }
    if (score_out) *score_out = idx < 0 ? 0 : best;
    return idx;
}
// session_pool.rs:124-129 lru_index: the index of the smallest tick (the first one among equals, as
// Iterator::min_by_key returns), -1 on an empty pool
extern "C" int64_t tsv_session_lru(const uint64_t* ticks, int64_t n) {
    int64_t idx = -1;
    for (int64_t i = 0; ticks && i < n; i++)
        if (idx < 0 || ticks[i] < ticks[idx]) idx = i;
    return idx;
}

namespace {
// real_forward_traits.rs:686-724 swap_live_session: the incoming session's buffers, cursor and record become the
// live ones; what was live is left in `s` for the caller to park.
void swap_live_session(tsv_ctx* c, tsv_ctx::Session& s) {
    for (int l = 0; l < c->n_layers; l++) {
        LayerW& L = c->layers[l];
        if (L.tq.k_bits) {
            std::swap(L.tq, s.tq[l]);
        } else {
            std::swap(L.kc, s.kc[l]);
            std::swap(L.vc, s.vc[l]);
        }
    }
    std::swap(c->kv_ptrs, s.kv_ptrs);
    std::swap(c->tq_stores, s.tq_stores);
    std::swap(c->position, s.position);
    std::swap(c->high_water, s.high_water);
    std::swap(c->prefix, s.prefix);
    c->last_m = 0;  // the logits on the device describe the outgoing conversation
}
void park_session(tsv_ctx* c, tsv_ctx::Session&& s) {  // session_pool.rs:110-114
    s.last_used = ++c->session_clock;
    c->parked.push_back(std::move(s));
}
// real_forward_traits.rs:655-673 select_session: the parked session that continues the prompt furthest, if it beats
// the live one (a tie stays live, an all-zero pool offers nothing: session_pool.rs:78-85,116-121)
bool select_session(tsv_ctx* c, const int32_t* prompt, int64_t n) {
    if (c->parked.empty()) return false;
    const int64_t live = c->prefix.common_prefix(prompt, n);
    std::vector<int64_t> scores;
    for (auto& ses : c->parked) scores.push_back(ses.prefix.common_prefix(prompt, n));
    int64_t best = 0;
    const int64_t idx = tsv_session_best_match(scores.data(), (int64_t)scores.size(), &best);
    if (idx < 0 || best <= live) return false;
    tsv_ctx::Session incoming = std::move(c->parked[idx]);
    c->parked.erase(c->parked.begin() + (long)idx);
    swap_live_session(c, incoming);
    park_session(c, std::move(incoming));
    return true;
}
}  // namespace

extern "C" int32_t tsv_reset(tsv_ctx* c) {
    TSV_NEED(c, "reset: null handle");
    // real_forward_traits.rs:12-31: with a pool, the live conversation is parked rather than overwritten and the
    // least recently used parked one takes its place (an eviction if that one held a conversation)
    c->session_slot_evicted = false;
    if (!c->parked.empty() && c->position > 0) {
        std::vector<uint64_t> ticks;
        for (auto& ses : c->parked) ticks.push_back(ses.last_used);
        const size_t lru = (size_t)tsv_session_lru(ticks.data(), (int64_t)ticks.size());
        tsv_ctx::Session promoted = std::move(c->parked[lru]);
        c->parked.erase(c->parked.begin() + (long)lru);
        c->session_slot_evicted = promoted.position > 0;
        swap_live_session(c, promoted);
        park_session(c, std::move(promoted));
    }
    c->position = 0;
    c->high_water = 0;
    c->last_m = 0;
    c->prefix.clear();  // cleared beside the cache it describes (real_forward_traits.rs:33-35)
    return TSV_OK;
}

extern "C" int32_t tsv_session_pool_size(const tsv_ctx* c) { return c ? (int32_t)c->parked.size() + 1 : -1; }
extern "C" int32_t tsv_session_swapped(const tsv_ctx* c) { return c ? (c->session_swapped ? 1 : 0) : -1; }
extern "C" int32_t tsv_session_slot_evicted(const tsv_ctx* c) { return c ? (c->session_slot_evicted ? 1 : 0) : -1; }
extern "C" int64_t tsv_kv_position(const tsv_ctx* c) { return c ? c->position : -1; }
extern "C" int64_t tsv_max_safe_rewind(const tsv_ctx* c) { return c ? c->rewind_budget : -1; }
extern "C" const uint16_t* tsv_device_logits(tsv_ctx* c) { return c ? c->logits : nullptr; }
extern "C" int64_t tsv_max_context(const tsv_ctx* c) { return c ? c->max_context : -1; }
extern "C" int64_t tsv_vocab(const tsv_ctx* c) { return c ? c->vocab : -1; }

extern "C" int32_t tsv_verify(tsv_ctx* c, const int32_t* feed, int32_t m, int64_t base, uint16_t* logits) {
    int rc = enqueue_verify(c, feed, nullptr, m, base);
    return rc ? rc : finish_verify(c, m, logits);
}

extern "C" int32_t tsv_verify_tree(tsv_ctx* c, const int32_t* feed, const int32_t* parent, int32_t m, int64_t base,
                                   uint16_t* logits) {
    if (!parent) {
        set_error("verify_tree: null parent array");
        return TSV_ERR_INVALID;
    }
    int rc = enqueue_verify(c, feed, parent, m, base);
    return rc ? rc : finish_verify(c, m, logits);
}

// The one recording point of the token-by-token walk (real_forward_traits.rs:135-152): recorded
// after the call and on success only; a failed pass may have left rows half written.
extern "C" int32_t tsv_produce(tsv_ctx* c, int32_t token, int64_t position, uint16_t* logits) {
    const int rc = tsv_verify(c, &token, 1, position, logits);
    if (c) {
        if (rc == TSV_OK) c->prefix.record(&token, 1, position);
        else c->prefix.taint();
    }
    return rc;
}

// `head` (nullable): the drafter head primed after each pass over every row whose next token is known
// (mtp_prime_rows_batched, families/qwen/mtp.rs:146-400); next_token: the token after ids[n - 1], or -1.
int tsv::prefill_passes(tsv_ctx* c, const int32_t* ids, int64_t n, int64_t pos0, uint16_t* logits, tsv_ctx* head, int32_t next_token) {
    const int wide_rows = 16 * WIDE_B;
    for (int64_t i = 0; i < n;) {
        // 64 rows at a time while that many remain and nobody wants their logits
        // (with a drafter head the last pass is a sixteen-row one: the first draft step reads its rows)
        if (c->wide.ok && !c->profile && !c->route_forced_set && n - i >= wide_rows && (i + wide_rows < n || (!logits && !head))) {
            if (int rc = enqueue_wide_prefill(c, ids + i, pos0 + i)) return rc;
            if (head) {
                for (int b = 0; b < WIDE_B; b++) {
                    int32_t nt[TSV_MAX_ROWS];
                    for (int r = 0; r < 16; r++) nt[r] = ids[i + 16 * b + r + 1];  // (i + 64 < n: every row has a next token)
                    if (int rc = mtp_pass(head, nt, 16, pos0 + i + 16 * b, c->wide.x + (size_t)b * 16 * c->hidden, false)) return rc;
                }
            }
            i += wide_rows;
            continue;
        }
        const int m = (int)std::min<int64_t>(TSV_MAX_ROWS, n - i);
        // only the last row's logits are ever handed out: every earlier pass is headless, and so
        // is the last one when the caller takes no logits
        c->headless = i + m < n || !logits;
        int rc = enqueue_verify(c, ids + i, nullptr, m, pos0 + i);
        const bool skipped = c->headless;
        c->headless = false;
        if (skipped) c->last_m = 0;  // no rows on the device for tsv_accept to judge
        if (rc) return rc;
        if (i + m >= n && logits) {
            TSV_HIP(hipMemcpyAsync(logits, c->logits + (size_t)(m - 1) * c->vocab, (size_t)c->vocab * 2,
                                   hipMemcpyDeviceToHost, c->stream));
        }
        if (head) {
            int32_t nt[TSV_MAX_ROWS];
            int rows = 0;
            for (; rows < m; rows++) {
                const int64_t j = i + rows + 1;
                if (j < n) nt[rows] = ids[j];
                else if (next_token >= 0) nt[rows] = next_token;
                else break;
            }
            if (rows && (rc = mtp_pass(head, nt, rows, pos0 + i, c->x, false))) return rc;
        }
        i += m;
    }
    TSV_HIP(hipStreamSynchronize(c->stream));
    return TSV_OK;
}

extern "C" int32_t tsv_prefill(tsv_ctx* c, const int32_t* ids, int64_t n, int64_t pos0, uint16_t* logits) {
    TSV_NEED(c && ids, "prefill: null handle or token list");
    if (n < 1) {
        set_error("prefill: empty token list");
        return TSV_ERR_INVALID;
    }
    // the chunk is recorded once it has run to completion, and taints the record when it has
    // not (real_forward_traits.rs:395-402)
    int rc = prefill_passes(c, ids, n, pos0, logits);
    if (rc == TSV_OK) c->prefix.record(ids, n, pos0);
    else c->prefix.taint();
    return rc;
}

extern "C" int32_t tsv_checkpoint(tsv_ctx* c, tsv_point* out) {
    TSV_NEED(c && out, "checkpoint: null handle or output");
    out->position = c->position;
    return TSV_OK;
}

// real_forward_rollback.rs:153-209 for a target without recurrent state: kv.rewind_by, a
// cursor move (kv_cache_rewind.rs:46-55); rows past the cursor become unreachable.
extern "C" int32_t tsv_rollback(tsv_ctx* c, const tsv_point* p) {
    TSV_NEED(c && p, "rollback: null handle or point");
    if (p->position < 0 || p->position > c->position) {
        set_error("rollback: point is ahead of the KV cursor");
        return TSV_ERR_INVALID;
    }
    if (int rrc = check_rewind(c, p->position, "rollback")) return rrc;
    c->position = p->position;
    c->last_m = 0;  // the logits on the device no longer describe rows behind the cursor
    c->prefix.rewind_to(p->position);  // real_forward_rollback.rs:203
    return TSV_OK;
}

extern "C" int32_t tsv_rollback_retaining(tsv_ctx* c, const tsv_point* p, int32_t keep_rows) {
    TSV_NEED(c && p, "rollback_retaining: null handle or point");
    if (keep_rows < 0 || p->position < 0 || p->position + keep_rows > c->position) {
        set_error("rollback_retaining: keep_rows exceeds the rows the last verify wrote");
        return TSV_ERR_INVALID;
    }
    if (int rrc = check_rewind(c, p->position + keep_rows, "rollback_retaining")) return rrc;
    c->position = p->position + keep_rows;
    c->last_m = 0;
    c->prefix.rewind_to(c->position);  // real_forward_rollback.rs:406
    return TSV_OK;
}

extern "C" int32_t tsv_commit_pending(tsv_ctx*, int32_t) { return TSV_OK; }
extern "C" int32_t tsv_discard_pending(tsv_ctx*) { return TSV_OK; }

// ---- the record of what the rows were built from, on its own and behind the handle ----
extern "C" tsv_prefix* tsv_prefix_new(void) { return new (std::nothrow) tsv_prefix(); }
extern "C" void tsv_prefix_free(tsv_prefix* p) { delete p; }
extern "C" void tsv_prefix_clear(tsv_prefix* p) {
    if (p) p->clear();
}
extern "C" void tsv_prefix_taint(tsv_prefix* p) {
    if (p) p->taint();
}
extern "C" void tsv_prefix_record(tsv_prefix* p, const int32_t* tokens, int64_t n, int64_t pos0) {
    if (p && (tokens || n <= 0)) p->record(tokens, n, pos0);
}
extern "C" void tsv_prefix_rewind_to(tsv_prefix* p, int64_t position) {
    if (p) p->rewind_to(position);
}
extern "C" int64_t tsv_prefix_untainted_len(const tsv_prefix* p) { return p ? p->untainted_len() : -1; }
extern "C" int64_t tsv_prefix_common(const tsv_prefix* p, const int32_t* prompt, int64_t n) {
    return p && prompt ? p->common_prefix(prompt, n) : 0;
}

extern "C" int32_t tsv_set_prefix_reuse(tsv_ctx* c, int32_t on) {
    TSV_NEED(c, "set_prefix_reuse: null handle");
    c->prefix_reuse = on != 0;
    return TSV_OK;
}

// real_forward_traits.rs:173-289 for a target without recurrent state, session pool or drafter of
// its own: the longest common prefix of the record and the prompt; a state that runs past it is
// moved back there (kv.rewind_by + kv_prefix.rewind_to), as far as the cache can go back.
extern "C" int64_t tsv_try_reuse_prefix(tsv_ctx* c, const int32_t* prompt, int64_t n) {
    if (!c || (!prompt && n > 0)) {
        set_error("try_reuse_prefix: null handle or prompt");
        return -1;
    }
    c->session_swapped = false;
    if (!c->prefix_reuse) return 0;
    const bool swapped = c->session_swapped = select_session(c, prompt, n);  // real_forward_traits.rs:184
    const int64_t keep = c->prefix.common_prefix(prompt, n);
    if (keep == 0 || keep > c->position) return 0;
    const int64_t back = c->position - keep;
    if (back > 0) {
        // real_forward_traits.rs:247-285: with a pool, a shallow match against a live session nobody compared with
        // anything would overwrite that conversation in place instead of parking it; the caller's reset parks it
        if (!c->parked.empty() && !swapped && back > keep) return 0;
        if (c->rewind_budget != INT64_MAX && c->high_water - keep > c->rewind_budget) return 0;  // real_forward_traits.rs:241-262: as far as the cache can go back
        c->position = keep;
        c->prefix.rewind_to(keep);
    }
    return keep;
}

// record_committed(tokens, pos0) (real_forward_traits.rs:567-569): a verify feeds a block and only
// the caller knows how much of it survived, so the loop reports the surviving rows after the round.
extern "C" int32_t tsv_record_committed(tsv_ctx* c, const int32_t* tokens, int64_t n, int64_t pos0) {
    TSV_NEED(c && (tokens || n <= 0), "record_committed: null handle or token list");
    c->prefix.record(tokens, n, pos0);
    return TSV_OK;
}

extern "C" int64_t tsv_prefix_len(const tsv_ctx* c) { return c ? c->prefix.untainted_len() : -1; }

extern "C" int32_t tsv_compact_tree(tsv_ctx* c, int64_t base, const uint32_t* path, int32_t n) {
    TSV_NEED(c && path, "compact_tree: null handle or path");
    if (n < 1 || n > TSV_MAX_ROWS || path[0] != 0) {
        set_error("compact_tree: path must start at slot 0 and hold 1..16 slots");
        return TSV_ERR_INVALID;
    }
    for (int i = 1; i < n; i++)
        if (path[i] <= path[i - 1] || path[i] >= TSV_MAX_ROWS) {
            set_error("compact_tree: path must be strictly increasing");
            return TSV_ERR_INVALID;
        }
    if (base < 0 || base + (int64_t)path[n - 1] >= c->ctx_alloc) {
        set_error("compact_tree: the block at `base` lies outside the KV cache");
        return TSV_ERR_INVALID;
    }
    TSV_HIP(hipStreamSynchronize(c->stream));
    for (int i = 0; i < n; i++) c->tok_host[32 + i] = (int32_t)path[i];
    TSV_HIP(hipMemcpyAsync(c->tok_dev + 32, c->tok_host + 32, (size_t)n * 4, hipMemcpyHostToDevice, c->stream));
    int rc = launch_kv_gather(c->stream, c->kv_ptrs, c->kv_caps, c->n_layers, c->nkv, c->hd, c->tok_dev + 32, n, (int)base);
    if (!rc && c->kv_k_bits)
        rc = launch_tq_gather(c->stream, c->tq_stores, c->n_layers, c->nkv, c->hd, c->ctx_alloc, c->tok_dev + 32, n, (int)base);
    return rc;
}

namespace tsv {

void fill_truncation(AcceptParams* ap, const tsv_shaping& sh) {
    ap->top_k = (int32_t)sh.top_k;
    ap->has_top_p = sh.has_top_p != 0;
    ap->top_p = sh.top_p;
    ap->has_min_p = sh.has_min_p != 0;
    ap->min_p = sh.min_p;
}

int fill_accept(tsv_ctx* c, const tsv_round* r, AcceptParams* ap) {
    std::memset(ap, 0, sizeof *ap);
    ap->m = r->m;
    ap->k = r->m - 1;
    ap->vocab = c->vocab;
    ap->tree = r->parent != nullptr;
    ap->sampled = r->shaping.temperature != 0.0;
    if (r->n_stop < 0 || r->n_stop > 16) {
        set_error("accept: at most 16 stop tokens");
        return TSV_ERR_INVALID;
    }
    ap->n_stop = r->n_stop;
    for (int i = 0; i < r->m; i++) {
        ap->feed[i] = r->feed[i];
        ap->parent[i] = r->parent ? r->parent[i] : i - 1;
    }
    for (int i = 0; i < r->n_stop; i++) ap->stop_tokens[i] = r->stop_tokens[i];
    ap->temperature = r->shaping.temperature;
    ap->seed = r->shaping.seed;
    fill_truncation(ap, r->shaping);
    ap->draw_step = r->draw_step;
    ap->generated = r->generated;
    ap->max_new_tokens = r->max_new_tokens;
    return TSV_OK;
}

// Penalised sampled rounds (choose.rs:138-154): uploads the history, counts its tokens on the device
// and fills the penalty fields of the parameter block.  `generated` is the sink's count of reported
// tokens: the last min(generated, n) tokens of the history are the generated suffix.
int setup_penalties(tsv_ctx* c, const tsv_shaping& sh, const int32_t* history, int64_t n, uint64_t generated,
                    AcceptParams* ap) {
    ap->pen = 0;
    if (!has_penalties(sh)) return TSV_OK;
    if (n < 0 || (n > 0 && !history)) {
        set_error("penalties: the round carries no token history");
        return TSV_ERR_INVALID;
    }
    if ((size_t)n > c->hist_cap) {
        if (c->hist_dev) TSV_HIP(hipFree(c->hist_dev));
        c->hist_dev = nullptr;
        c->hist_cap = 0;
        const size_t cap = ((size_t)n + 4095) & ~(size_t)4095;
        TSV_HIP(hipMalloc((void**)&c->hist_dev, cap * 4));
        c->hist_cap = cap;
    }
    if (n > 0) TSV_HIP(hipMemcpyAsync(c->hist_dev, history, (size_t)n * 4, hipMemcpyHostToDevice, c->stream));
    const int64_t suffix = (int64_t)std::min<uint64_t>(generated, (uint64_t)n);
    int rc = launch_pen_counts(c->stream, c->hist_dev, (long)n, (long)(n - suffix), c->vocab, c->pen_cnt);
    if (rc) return rc;
    if (n > 0) TSV_HIP(hipStreamSynchronize(c->stream));  // the caller's history buffer is free again
    ap->pen = 1;
    ap->pen_has_rep = sh.repetition_penalty != 1.0;
    // penalty.rs:20-25: the f64 setting as an f32 kept inside the normal range
    ap->pen_rep = std::min(std::max((float)sh.repetition_penalty, 1.17549435e-38f), 3.40282347e+38f);
    ap->pen_has_pf = sh.presence_penalty != 0.0 || sh.frequency_penalty != 0.0;
    ap->pen_presence = sh.presence_penalty;
    ap->pen_frequency = sh.frequency_penalty;
    ap->pen_cnt = c->pen_cnt;
    return TSV_OK;
}

const char* accept_error_text(int bits) {
    if (bits & 1) return "score vector must not contain a non-finite entry";
    if (bits & 4) return "a penalised score lies below every fp16 value (not built)";
    return "too many penalised candidates between two neighbouring fp16 values (not built)";
}

int stage_draft(tsv_ctx* c, const uint16_t* draft, int rows, const uint16_t** dev) {
    if (is_device_pointer(draft)) {
        *dev = draft;
        return TSV_OK;
    }
    TSV_HIP(hipMemcpyAsync(c->draft_stage, draft, (size_t)rows * c->vocab * 2, hipMemcpyHostToDevice, c->stream));
    *dev = c->draft_stage;
    return TSV_OK;
}

int check_round(const tsv_round* r) {
    int rc = check_shaping(r->shaping, true);
    if (rc) return rc;
    return TSV_OK;
}

int accept_impl(tsv_ctx* c, const tsv_round* r, tsv_round_result* out) {
    int rc = check_round(r);
    if (rc) return rc;
    if (r->m != c->last_m || r->base != c->last_base) {
        set_error("accept: the round does not describe the last verify pass");
        return TSV_ERR_INVALID;
    }
    // the tree the round names: well formed (the walks on both sides follow parent links towards slot 0), and the
    // one the pass attended by -- a chain pass judged as a tree, or the other way round, would accept rows that never
    // saw their supposed ancestors
    uint32_t anc[TSV_MAX_ROWS];
    for (int i = 0; i < r->m; i++) {
        if (r->parent && (i == 0 ? r->parent[0] != -1 : (r->parent[i] < 0 || r->parent[i] >= i))) {
            set_error("accept: parent[0] must be -1 and parent[s] in [0, s)");
            return TSV_ERR_INVALID;
        }
        anc[i] = r->parent ? (i == 0 ? 0u : anc[r->parent[i]]) | (1u << i) : (2u << i) - 1u;
        if (c->last_shape_known && anc[i] != c->vp_host->anc[i]) {
            set_error("accept: the round's tree is not the one the last verify pass attended by");
            return TSV_ERR_INVALID;
        }
    }
    const bool sampled = r->shaping.temperature != 0.0;
    const uint16_t* draft = nullptr;
    if (sampled) {
        if (!r->draft_logits) {
            set_error("accept: a sampled round needs the drafter's logits");
            return TSV_ERR_INVALID;
        }
        if (r->parent && (r->n_stop > 0 || r->max_new_tokens > 0)) {
            set_error("accept: sampled acceptance over a tree takes no stop tokens or budget");
            return TSV_ERR_UNSUPPORTED;
        }
        if ((rc = stage_draft(c, r->draft_logits, r->parent ? r->m : r->m - 1, &draft))) return rc;
    }
    TSV_HIP(hipStreamSynchronize(c->stream));  // pinned parameter block is about to be rewritten
    if ((rc = fill_accept(c, r, c->ap_host))) return rc;
    if ((rc = setup_penalties(c, r->shaping, r->history, r->n_history, r->generated, c->ap_host))) return rc;
    TSV_HIP(hipMemcpyAsync(c->ap_dev, c->ap_host, sizeof(AcceptParams), hipMemcpyHostToDevice, c->stream));
    {
        PROF(PC_ACCEPT);
        rc = launch_accept(c->stream, c->logits, draft, c->ap_dev, *c->ap_host, c->sc);
    }
    if (rc) return rc;
    TSV_HIP(hipMemcpyAsync(c->res_host, c->sc.result, sizeof(AcceptResult), hipMemcpyDeviceToHost, c->stream));
    if (r->logits_out)
        TSV_HIP(hipMemcpyAsync(r->logits_out, c->logits, (size_t)r->m * c->vocab * 2, hipMemcpyDeviceToHost, c->stream));
    TSV_HIP(hipStreamSynchronize(c->stream));
    const AcceptResult& a = *c->res_host;
    if (a.error) {
        set_error(std::string("accept: ") + accept_error_text(a.error));
        return (a.error & 1) ? TSV_ERR_INVALID : TSV_ERR_UNSUPPORTED;
    }
    std::memset(out, 0, sizeof *out);
    out->accepted = a.accepted;
    out->committed = a.committed;
    out->next = a.next;
    out->stopped = a.stopped;
    out->draw_step = a.draw_step;
    out->path_len = a.path_len;
    for (int i = 0; i < a.path_len; i++) out->path[i] = a.path[i];
    out->min_margin = a.min_margin;
    // KV truncation.  Rows base..base+committed hold the confirmed token and every committed
    // proposal; everything after becomes unreachable (speculative.rs:791-814).
    const int keep = a.committed + 1;
    if (r->parent && keep > 1) {
        uint32_t path[TSV_MAX_ROWS + 1];
        for (int i = 0; i < keep; i++) path[i] = (uint32_t)a.path[i];
        if ((rc = tsv_compact_tree(c, r->base, path, keep))) return rc;
    }
    c->position = r->base + keep;
    c->prefix.rewind_to(c->position);
    out->kv_position = c->position;
    return TSV_OK;
}

}  // namespace tsv

extern "C" int32_t tsv_accept(tsv_ctx* c, const tsv_round* r, tsv_round_result* out) {
    if (!c || !r || !out || !r->feed) {
        set_error("accept: null argument");
        return TSV_ERR_INVALID;
    }
    return accept_impl(c, r, out);
}

extern "C" int32_t tsv_verify_accept(tsv_ctx* c, const tsv_round* r, tsv_round_result* out) {
    if (!c || !r || !out || !r->feed) {
        set_error("verify_accept: null argument");
        return TSV_ERR_INVALID;
    }
    int rc = check_round(r);
    if (rc) return rc;
    if ((rc = enqueue_verify(c, r->feed, r->parent, r->m, r->base))) return rc;
    return accept_impl(c, r, out);
}

extern "C" int32_t tsv_draft_chain(tsv_ctx* c, const uint16_t* draft_logits, int32_t k, const tsv_shaping* sh,
                                   uint64_t* draw_step, int32_t* proposals, const int32_t* history,
                                   int64_t n_history, uint64_t generated) {
    if (!c || !draft_logits || !sh || !draw_step || !proposals || k < 1 || k > TSV_MAX_ROWS - 1) {
        set_error("draft_chain: bad argument");
        return TSV_ERR_INVALID;
    }
    int rc = check_shaping(*sh, true);
    if (rc) return rc;
    const uint16_t* draft = nullptr;
    if ((rc = stage_draft(c, draft_logits, k, &draft))) return rc;
    TSV_HIP(hipStreamSynchronize(c->stream));
    AcceptParams* ap = c->ap_host;
    std::memset(ap, 0, sizeof *ap);
    ap->m = 0;
    ap->k = k;
    ap->vocab = c->vocab;
    ap->sampled = sh->temperature != 0.0;
    ap->temperature = sh->temperature;
    ap->seed = sh->seed;
    fill_truncation(ap, *sh);
    ap->draw_step = *draw_step;
    if ((rc = setup_penalties(c, *sh, history, n_history, generated, ap))) return rc;
    TSV_HIP(hipMemcpyAsync(c->ap_dev, ap, sizeof *ap, hipMemcpyHostToDevice, c->stream));
    if ((rc = launch_draft_chain(c->stream, draft, c->ap_dev, *ap, c->sc, c->tok_dev))) return rc;
    TSV_HIP(hipMemcpyAsync(c->tok_host, c->tok_dev, (size_t)k * 4, hipMemcpyDeviceToHost, c->stream));
    TSV_HIP(hipMemcpyAsync(c->res_host, c->sc.result, sizeof(AcceptResult), hipMemcpyDeviceToHost, c->stream));
    TSV_HIP(hipStreamSynchronize(c->stream));
    if (c->res_host->error) {
        set_error(std::string("draft_chain: ") + accept_error_text(c->res_host->error));
        return (c->res_host->error & 1) ? TSV_ERR_INVALID : TSV_ERR_UNSUPPORTED;
    }
    for (int i = 0; i < k; i++) proposals[i] = c->tok_host[i];
    if (ap->sampled) *draw_step += (uint64_t)k + 1;  // k draws + the row-only step (speculative.rs:618-624)
    return TSV_OK;
}

// crates/model-io/src/kv_quant.rs:146-205 kv_layer_strides, for the layer kinds of this path and as this library
// lays the rows out: bytes one position costs in layer `layer`, K side and V side
extern "C" int32_t tsv_kv_row_bytes(const tsv_model_desc* d, int32_t layer, int64_t* k_bytes, int64_t* v_bytes) {
    if (!d || !d->layers || layer < 0 || layer >= d->n_layers || !k_bytes || !v_bytes || d->n_kv_heads < 1 || d->head_dim < 1) {
        set_error("kv_row_bytes: null argument or layer outside the model");
        return TSV_ERR_INVALID;
    }
    const bool quantized = d->kv_k_bits > 0 && d->layers[layer].window == 0 && (d->n_layers <= 2 || layer + 1 < d->n_layers);
    if (!quantized) {
        *k_bytes = *v_bytes = (int64_t)d->n_kv_heads * d->head_dim * 2;
        return TSV_OK;
    }
    // one f32 norm and the packed indices per kv head (kv_quant.rs:141-144); the V indices are kept sixteen positions to
    // a group of 32 or 64 bits per dimension, which at three bits is a third more than the packed row
    *k_bytes = (int64_t)d->n_kv_heads * (4 + 4 * tq_words(d->head_dim, d->kv_k_bits));
    *v_bytes = (int64_t)d->n_kv_heads * (4 + (int64_t)d->head_dim * tq_v_group_words(d->kv_v_bits) * 4 / 16);
    return TSV_OK;
}

// crates/model-io/src/context_policy.rs:294-333 kv_bytes_for_context_with: what one conversation's KV state costs at
// `context` positions (rounded up to whole blocks of sixteen, as allocated): a ring layer stops growing at its capacity
extern "C" int64_t tsv_kv_bytes_for_context(const tsv_model_desc* d, int64_t context) {
    if (!d || !d->layers || context < 1) {
        set_error("kv_bytes_for_context: null description or empty context");
        return -1;
    }
    const int64_t alloc = (context + 15) / 16 * 16;
    int64_t total = 0;
    for (int l = 0; l < d->n_layers; l++) {
        int64_t k, v;
        if (tsv_kv_row_bytes(d, l, &k, &v)) return -1;
        int64_t cap = alloc;
        if (d->layers[l].ring && d->layers[l].window > 0)
            cap = std::min<int64_t>(alloc, (int64_t)((d->layers[l].window + 15) / 16) * 16 + 2 * TSV_MAX_ROWS);
        total += cap * (k + v);
    }
    return total;
}
