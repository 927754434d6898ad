// Test and measurement hooks of include/tsverify_testing.h: cache and logits I/O, the kernels one at a time, routing
// read-back and forcing, per-class timing, the timing loops.  Nothing a producer needs.
#include "ctx.h"

using namespace tsv;

// The measurement hooks (per-class event pairs, repeated launches, the timing loops) answer only in a process
// whose environment carries TSV_MEASUREMENT_HOOKS=1: a serving process cannot be put into a measuring mode by
// a stray call.
static int measurement_hooks_on(const char* who) {
    const char* e = getenv("TSV_MEASUREMENT_HOOKS");
    if (e && e[0] == '1') return TSV_OK;
    set_error(std::string(who) + ": measurement hooks are off (set TSV_MEASUREMENT_HOOKS=1 in the process environment)");
    return TSV_ERR_UNSUPPORTED;
}

extern "C" int32_t tsv_set_profile(tsv_ctx* c, int32_t on) {
    TSV_NEED(c, "set_profile: null handle");
    if (on)
        if (int rc = measurement_hooks_on("set_profile")) return rc;
    TSV_HIP(hipStreamSynchronize(c->stream));
    c->profile = on != 0;
    c->ev_used = 0;
    return TSV_OK;
}

extern "C" int32_t tsv_set_repeat(tsv_ctx* c, int32_t cls, int32_t times) {
    TSV_NEED(c, "set_repeat: null handle");
    if (times != 1)
        if (int rc = measurement_hooks_on("set_repeat")) return rc;
    if (cls != PC_QKV && cls != PC_ROPE && cls != PC_ATTN && cls != PC_WO && cls != PC_GATEUP && cls != PC_DOWN &&
        cls != PC_HEAD) {
        set_error("set_repeat: only the matmul, rope and attention classes can be repeated");
        return TSV_ERR_INVALID;
    }
    if (times < 1 || times > 8) {
        set_error("set_repeat: times must be 1..8");
        return TSV_ERR_INVALID;
    }
    TSV_HIP(hipStreamSynchronize(c->stream));
    c->repeat[cls] = times;
    return TSV_OK;
}

extern "C" int32_t tsv_get_profile(tsv_ctx* c, float* ms, int32_t* counts, int32_t n_classes) {
    TSV_NEED(c && ms && counts && n_classes >= 0, "get_profile: null handle or output");
    TSV_HIP(hipStreamSynchronize(c->stream));
    for (int i = 0; i < n_classes; i++) {
        ms[i] = 0.f;
        counts[i] = 0;
    }
    for (size_t i = 0; i + 1 < c->ev_used; i += 2) {
        float t = 0.f;
        TSV_HIP(hipEventElapsedTime(&t, c->ev[i], c->ev[i + 1]));
        const int cls = c->ev_class[i];
        if (cls < n_classes) {
            ms[cls] += t;
            counts[cls] += 1;
        }
    }
    c->ev_used = 0;
    return TSV_OK;
}


extern "C" int32_t tsv_read_kv(tsv_ctx* c, int32_t layer, int64_t pos0, int64_t n, uint16_t* k, uint16_t* v) {
    if (!c || !k || !v || layer < 0 || layer >= c->n_layers || pos0 < 0 || n < 1 || pos0 + n > c->ctx_alloc) {
        set_error("read_kv: null argument or range outside the cache");
        return TSV_ERR_INVALID;
    }
    if (c->layers[layer].tq.k_bits) {
        set_error("read_kv: this layer keeps quantized rows (tsv_read_kv_quantized reads them)");
        return TSV_ERR_UNSUPPORTED;
    }
    const size_t bytes = (size_t)n * c->nkv * c->hd * 2;
    uint16_t *kd = nullptr, *vd = nullptr;
    TSV_HIP(hipMalloc((void**)&kd, bytes));
    if (hipMalloc((void**)&vd, bytes) != hipSuccess) {
        (void)hipFree(kd);
        set_error("KV staging buffer: out of device memory");
        return TSV_ERR_DEVICE;
    }
    if (c->layers[layer].cap < c->ctx_alloc && pos0 < c->high_water - c->layers[layer].cap) {
        (void)hipFree(kd);
        (void)hipFree(vd);
        set_error("read_kv: the ring of this layer no longer holds the first rows asked for");
        return TSV_ERR_INVALID;
    }
    int rc = launch_kv_read(c->stream, c->layers[layer].kc, c->layers[layer].vc, c->nkv, c->hd, c->layers[layer].cap,
                            (int)pos0, (int)n, kd, vd);
    if (!rc) {
        hipError_t e1 = hipMemcpyAsync(k, kd, bytes, hipMemcpyDeviceToHost, c->stream);
        hipError_t e2 = hipMemcpyAsync(v, vd, bytes, hipMemcpyDeviceToHost, c->stream);
        hipError_t e3 = hipStreamSynchronize(c->stream);
        if (e1 != hipSuccess || e2 != hipSuccess || e3 != hipSuccess) {
            set_error("read_kv: copy failed");
            rc = TSV_ERR_DEVICE;
        }
    }
    (void)hipFree(kd);
    (void)hipFree(vd);
    return rc;
}

extern "C" int32_t tsv_route_selected(tsv_ctx* c, int32_t* out, int32_t n_layers) {
    if (!c || !out || n_layers != c->n_layers) {
        set_error("route_selected: null argument or layer count mismatch");
        return TSV_ERR_INVALID;
    }
    if (!c->route_sel) {
        set_error("route_selected: the model has no routed layers");
        return TSV_ERR_INVALID;
    }
    TSV_HIP(hipMemcpyAsync(out, c->route_sel, (size_t)c->n_layers * 16 * 8 * 4, hipMemcpyDeviceToHost, c->stream));
    TSV_HIP(hipStreamSynchronize(c->stream));
    return TSV_OK;
}

extern "C" int32_t tsv_force_route(tsv_ctx* c, const int32_t* sel, int32_t n_layers) {
    if (!c || (sel && n_layers != c->n_layers)) {
        set_error("force_route: null handle or layer count mismatch");
        return TSV_ERR_INVALID;
    }
    if (!c->route_forced) {
        set_error("force_route: the model has no routed layers");
        return TSV_ERR_INVALID;
    }
    const size_t bytes = (size_t)c->n_layers * 16 * 8 * 4;
    TSV_HIP(hipStreamSynchronize(c->stream));
    c->route_forced_set = sel != nullptr;
    if (sel) {
        TSV_HIP(hipMemcpy(c->route_forced, sel, bytes, hipMemcpyHostToDevice));
    } else {
        TSV_HIP(hipMemset(c->route_forced, 0xFF, bytes));  // every entry -1: every row routes freely
    }
    return TSV_OK;
}

extern "C" int32_t tsv_write_logits(tsv_ctx* c, const uint16_t* logits, int32_t m, int64_t base) {
    if (!c || !logits || m < 1 || m > TSV_MAX_ROWS || base < 0) {
        set_error("write_logits: bad argument");
        return TSV_ERR_INVALID;
    }
    TSV_HIP(hipMemcpyAsync(c->logits, logits, (size_t)m * c->vocab * 2, hipMemcpyHostToDevice, c->stream));
    TSV_HIP(hipStreamSynchronize(c->stream));
    c->last_m = m;
    c->last_base = base;
    c->last_shape_known = false;  // rows from the host: whatever tree the round names is taken at its word
    return TSV_OK;
}

extern "C" int32_t tsv_write_kv(tsv_ctx* c, int32_t layer, int64_t pos0, int64_t n, const uint16_t* k,
                                const uint16_t* v) {
    if (!c || !k || !v || layer < 0 || layer >= c->n_layers || pos0 < 0 || n < 1 || pos0 + n > c->max_context) {
        set_error("write_kv: range outside the cache");
        return TSV_ERR_INVALID;
    }
    const size_t bytes = (size_t)n * c->nkv * c->hd * 2;
    uint16_t *kd = nullptr, *vd = nullptr;
    TSV_HIP(hipMalloc((void**)&kd, bytes));
    if (hipMalloc((void**)&vd, bytes) != hipSuccess) {
        (void)hipFree(kd);
        set_error("KV staging buffer: out of device memory");
        return TSV_ERR_DEVICE;
    }
    int rc = TSV_OK;
    if (hipMemcpyAsync(kd, k, bytes, hipMemcpyHostToDevice, c->stream) != hipSuccess ||
        hipMemcpyAsync(vd, v, bytes, hipMemcpyHostToDevice, c->stream) != hipSuccess) {
        set_error("write_kv: copy failed");
        rc = TSV_ERR_DEVICE;
    }
    if (!rc && c->layers[layer].tq.k_bits) {
        // a quantized layer: the rows go through the staging slots and the quantizer sixteen at a time, as the
        // forward's own rows do (crates/runtime/src/kv_write.rs:66-118)
        const LayerW& L = c->layers[layer];
        TqArgs ta{};
        ta.kc = L.kc;
        ta.vc = L.vc;
        ta.stage_cap = L.kv_slots;
        ta.store = L.tq;
        ta.k = c->tq_k;
        ta.v = c->tq_v;
        ta.nkv = c->nkv;
        ta.hd = c->hd;
        ta.cap = L.cap;
        ta.vp = c->vp_dev;
        const size_t row = (size_t)c->nkv * c->hd;
        for (int64_t p = 0; !rc && p < n; p += L.kv_slots) {
            const int cnt = (int)std::min<int64_t>(L.kv_slots, n - p);
            rc = launch_kv_fill(c->stream, L.kc, L.vc, c->nkv, c->hd, L.kv_slots, (int)(pos0 + p), cnt, kd + p * row, vd + p * row);
            ta.m_hint = cnt;
            ta.base_hint = (int)(pos0 + p);
            if (!rc) rc = launch_tq_prepare(c->stream, ta);
        }
    } else if (!rc) {
        // a ring layer keeps the last `cap` of the rows (earlier ones would only be overwritten, by
        // rows of the same launch)
        const int64_t cap = c->layers[layer].cap, skip = n > cap ? n - cap : 0;
        const size_t off = (size_t)skip * c->nkv * c->hd;
        rc = launch_kv_fill(c->stream, c->layers[layer].kc, c->layers[layer].vc, c->nkv, c->hd, (int)cap,
                            (int)(pos0 + skip), (int)(n - skip), kd + off, vd + off);
    }
    if (hipStreamSynchronize(c->stream) != hipSuccess && !rc) {
        set_error("write_kv: device execution failed");
        rc = TSV_ERR_DEVICE;
    }
    (void)hipFree(kd);
    (void)hipFree(vd);
    if (!rc && pos0 + n > c->position) c->position = pos0 + n;
    if (!rc) c->high_water = std::max(c->high_water, pos0 + n);
    c->prefix.taint();  // rows no token ids describe
    return rc;
}

extern "C" int32_t tsv_matmul(const tsv_tensor* w, const float* x, int32_t m, float* y, int32_t splits) {
    if (!w || !x || !y || m < 1 || m > TSV_MAX_ROWS) {
        set_error("matmul: bad argument");
        return TSV_ERR_INVALID;
    }
    int rc = check_matrix(*w, w->rows, w->cols, "matmul weight");
    if (rc) return rc;
    tsv_ctx tmp;
    tsv_ctx* c = &tmp;
    TSV_HIP(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
    Stager st;
    TiledW tw;
    const tsv_tensor* parts[1] = {w};
    VerifyParams vp;
    std::memset(&vp, 0, sizeof vp);
    vp.m = m;
    float *xd = nullptr, *pd = nullptr;
    uint4* xf = nullptr;
    VerifyParams* vpd = nullptr;
    const int k = (int)w->cols, n = (int)w->rows;
    std::vector<float> part;
    int sp = 1;
    rc = make_tiled(c, st, parts, 1, false, &tw);
    if (!rc) {
        sp = splits > 0 ? std::min(splits, tw.kchunks) : gemm_default_splits(tw, m);
        const int kslice = (tw.kchunks + sp - 1) / sp;
        sp = (tw.kchunks + kslice - 1) / kslice;
    }
    if (!rc) rc = dev_alloc(c, &xd, (size_t)m * k * 4);
    if (!rc) rc = dev_alloc(c, &xf, xfrag_bytes(k), true);
    if (!rc) rc = dev_alloc(c, &pd, (size_t)sp * 16 * n * 4, true);
    if (!rc) rc = dev_alloc(c, &vpd, sizeof vp);
    if (!rc && hipMemcpyAsync(xd, x, (size_t)m * k * 4, hipMemcpyHostToDevice, c->stream) != hipSuccess) rc = TSV_ERR_DEVICE;
    if (!rc && hipMemcpyAsync(vpd, &vp, sizeof vp, hipMemcpyHostToDevice, c->stream) != hipSuccess) rc = TSV_ERR_DEVICE;
    if (!rc) rc = launch_f32_to_xfrag(c->stream, xd, k, xf, m);
    if (!rc) rc = launch_gemm(c->stream, tw, xf, pd, vpd, m, sp, EPI_PARTIAL, n, n);
    if (!rc) {
        part.resize((size_t)sp * 16 * n);
        if (hipMemcpyAsync(part.data(), pd, part.size() * 4, hipMemcpyDeviceToHost, c->stream) != hipSuccess ||
            hipStreamSynchronize(c->stream) != hipSuccess) {
            set_error("matmul: device execution failed");
            rc = TSV_ERR_DEVICE;
        }
    }
    if (!rc)
        for (int b = 0; b < m; b++)
            for (int j = 0; j < n; j++) {
                float acc = 0.f;
                for (int s = 0; s < sp; s++) acc += part[((size_t)s * 16 + b) * n + j];
                y[(size_t)b * n + j] = acc;
            }
    if (st.dev) (void)hipFree(st.dev);
    (void)hipStreamSynchronize(c->stream);
    for (void* p : c->allocs) (void)hipFree(p);
    (void)hipStreamDestroy(c->stream);
    return rc;
}

extern "C" int32_t tsv_attention(const uint16_t* q, const uint16_t* k, const uint16_t* v, int32_t m, int32_t nq,
                                 int32_t nkv, int32_t hd, int64_t base, const int32_t* parent, float scale,
                                 int32_t window, const float* sinks, uint16_t* out) {
    if (!q || !k || !v || !out || m < 1 || m > TSV_MAX_ROWS || nq % nkv || nq / nkv > 8 || base < 0 || window < 0 ||
        (window > 0 && window <= TSV_MAX_ROWS)) {
        set_error("attention: bad argument");
        return TSV_ERR_INVALID;
    }
    tsv_ctx tmp;
    tsv_ctx* c = &tmp;
    TSV_HIP(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
    VerifyParams vp;
    int rc = fill_params(vp, nullptr, parent, m, base, 0);
    const int seq = (int)base + m, ctx = (seq + 15) / 16 * 16, nch = attn_chunks(nkv), G = nq / nkv;
    const size_t kvb = (size_t)nkv * ctx * hd * 2, inb = (size_t)seq * nkv * hd * 2, qb = (size_t)m * nq * hd * 2;
    uint16_t *kc = nullptr, *vc = nullptr, *kin = nullptr, *vin = nullptr, *q16 = nullptr;
    float *po = nullptr, *pml = nullptr, *sinks_dev = nullptr;
    uint4* xf = nullptr;
    VerifyParams* vpd = nullptr;
    const size_t xfb = xfrag_bytes(nq * hd);
    if (!rc && sinks) {
        rc = dev_alloc(c, &sinks_dev, (size_t)nq * 4);
        if (!rc && hipMemcpyAsync(sinks_dev, sinks, (size_t)nq * 4, hipMemcpyHostToDevice, c->stream) != hipSuccess)
            rc = TSV_ERR_DEVICE;
    }
    if (!rc) rc = dev_alloc(c, &kc, kvb, true);
    if (!rc) rc = dev_alloc(c, &vc, kvb, true);
    if (!rc) rc = dev_alloc(c, &kin, inb);
    if (!rc) rc = dev_alloc(c, &vin, inb);
    if (!rc) rc = dev_alloc(c, &q16, qb);
    if (!rc) rc = dev_alloc(c, &po, (size_t)nkv * nch * m * G * hd * 4, true);
    if (!rc) rc = dev_alloc(c, &pml, (size_t)nkv * nch * m * G * 2 * 4, true);
    if (!rc) rc = dev_alloc(c, &xf, xfb, true);
    if (!rc) rc = dev_alloc(c, &vpd, sizeof vp);
    if (!rc && (hipMemcpyAsync(kin, k, inb, hipMemcpyHostToDevice, c->stream) != hipSuccess ||
                hipMemcpyAsync(vin, v, inb, hipMemcpyHostToDevice, c->stream) != hipSuccess ||
                hipMemcpyAsync(q16, q, qb, hipMemcpyHostToDevice, c->stream) != hipSuccess ||
                hipMemcpyAsync(vpd, &vp, sizeof vp, hipMemcpyHostToDevice, c->stream) != hipSuccess))
        rc = TSV_ERR_DEVICE;
    if (!rc) rc = launch_kv_fill(c->stream, kc, vc, nkv, hd, ctx, 0, seq, kin, vin);
    if (!rc) {
        AttnArgs aa{};
        aa.q16 = q16;
        aa.kc = kc;
        aa.vc = vc;
        aa.part_o = po;
        aa.part_ml = pml;
        aa.xfrag = xf;
        aa.nq = nq;
        aa.nkv = nkv;
        aa.hd = hd;
        aa.max_ctx = ctx;
        aa.nch = nch;
        aa.scale = scale > 0.f ? scale : 1.0f / std::sqrt((float)hd);
        aa.window = window;
        aa.sinks = sinks_dev;
        aa.vp = vpd;
        aa.m_hint = m;
        aa.base_hint = (int)base;
        rc = launch_attention(c->stream, aa, m);
    }
    std::vector<uint16_t> frag(xfb / 2);
    if (!rc && (hipMemcpyAsync(frag.data(), xf, xfb, hipMemcpyDeviceToHost, c->stream) != hipSuccess ||
                hipStreamSynchronize(c->stream) != hipSuccess)) {
        set_error("attention: device execution failed");
        rc = TSV_ERR_DEVICE;
    }
    if (!rc)
        for (int b = 0; b < m; b++)
            for (int kk = 0; kk < nq * hd; kk++) out[(size_t)b * nq * hd + kk] = frag[(size_t)frag_index(kk, b)];
    (void)hipStreamSynchronize(c->stream);
    for (void* p : c->allocs) (void)hipFree(p);
    (void)hipStreamDestroy(c->stream);
    return rc;
}

extern "C" int32_t tsv_kv_quant_tables(int32_t head_dim, int32_t bits, int32_t value_side, float* signs, float* codebook,
                                       float* midpoints) {
    if (head_dim < 32 || head_dim > 512 || (head_dim & (head_dim - 1)) || bits < 1 || bits > 4 || !signs || !codebook ||
        !midpoints) {
        set_error("kv_quant_tables: head_dim must be a power of two in 32..512 and bits in 1..4");
        return TSV_ERR_INVALID;
    }
    tq_sign_vector(head_dim, value_side ? 1 : 0, signs);
    const std::vector<float> cb = tq_codebook(head_dim, bits);
    for (size_t i = 0; i < cb.size(); i++) codebook[i] = cb[i];
    for (size_t i = 0; i + 1 < cb.size(); i++) midpoints[i] = 0.5f * (cb[i] + cb[i + 1]);
    return TSV_OK;
}

namespace {
// The stores of positions [pos0, pos0 + n) as the rows the reference keeps, [position][kv head][norm, words]
// (crates/gpu/tests/kv_quantize_parity.rs:22-38): K rows are stored that way but for the norm; V indices are
// stored transposed per block of sixteen positions and are packed back LSB first (kv_quant.rs:289-312) here.
int tq_rows_to_host(hipStream_t stream, const TqKv& t, int nkv, int hd, int cap, int64_t pos0, int64_t n, uint32_t* k_rows,
                    uint32_t* v_rows) {
    const int kw = tq_words(hd, t.k_bits), vw = tq_words(hd, t.v_bits), gw = t.v_bits == 2 ? 1 : 2;
    std::vector<uint32_t> kq((size_t)nkv * cap * kw), vq(tq_vq_bytes(nkv, cap, hd, t.v_bits) / 4);
    std::vector<float> kn((size_t)nkv * cap), vn((size_t)nkv * cap);
    TSV_HIP(hipStreamSynchronize(stream));
    TSV_HIP(hipMemcpy(kq.data(), t.kq, kq.size() * 4, hipMemcpyDeviceToHost));
    TSV_HIP(hipMemcpy(vq.data(), t.vq, vq.size() * 4, hipMemcpyDeviceToHost));
    TSV_HIP(hipMemcpy(kn.data(), t.kn, kn.size() * 4, hipMemcpyDeviceToHost));
    TSV_HIP(hipMemcpy(vn.data(), t.vn, vn.size() * 4, hipMemcpyDeviceToHost));
    for (int64_t i = 0; i < n; i++) {
        const int64_t pos = pos0 + i;
        for (int h = 0; h < nkv; h++) {
            uint32_t* kr = k_rows + ((size_t)i * nkv + h) * (1 + kw);
            std::memcpy(kr, &kn[(size_t)h * cap + pos], 4);
            std::memcpy(kr + 1, &kq[((size_t)h * cap + pos) * kw], (size_t)kw * 4);
            uint32_t* vr = v_rows + ((size_t)i * nkv + h) * (1 + vw);
            std::memcpy(vr, &vn[(size_t)h * cap + pos], 4);
            std::fill(vr + 1, vr + 1 + vw, 0u);
            for (int d = 0; d < hd; d++) {
                const uint32_t* g = &vq[(((size_t)h * (cap / 16) + pos / 16) * hd + d) * gw];
                const uint64_t group = gw == 2 ? ((uint64_t)g[1] << 32) | g[0] : g[0];
                const uint32_t idx = (uint32_t)(group >> ((pos & 15) * t.v_bits)) & ((1u << t.v_bits) - 1u);
                const uint32_t bit = (uint32_t)d * t.v_bits, w = bit >> 5, off = bit & 31;
                vr[1 + w] |= idx << off;
                if (off + t.v_bits > 32) vr[1 + w + 1] |= idx >> (32 - off);
            }
        }
    }
    return TSV_OK;
}
}  // namespace

extern "C" int32_t tsv_read_kv_quantized(tsv_ctx* c, int32_t layer, int64_t pos0, int64_t n, uint32_t* k_rows,
                                         uint32_t* v_rows) {
    if (!c || !k_rows || !v_rows || layer < 0 || layer >= c->n_layers || pos0 < 0 || n < 1 || pos0 + n > c->ctx_alloc) {
        set_error("read_kv_quantized: null argument or range outside the cache");
        return TSV_ERR_INVALID;
    }
    const LayerW& L = c->layers[layer];
    if (!L.tq.k_bits) {
        set_error("read_kv_quantized: this layer keeps fp16 rows");
        return TSV_ERR_INVALID;
    }
    return tq_rows_to_host(c->stream, L.tq, c->nkv, c->hd, L.cap, pos0, n, k_rows, v_rows);
}

extern "C" int32_t tsv_attention_quantized(const uint16_t* q, const uint16_t* k, const uint16_t* v, int32_t m, int32_t nq,
                                           int32_t nkv, int32_t hd, int64_t base, int32_t k_bits, int32_t v_bits,
                                           float scale, const float* sinks, uint16_t* out, uint32_t* k_rows,
                                           uint32_t* v_rows) {
    if (!q || !k || !v || !out || !k_rows || !v_rows || m < 1 || m > TSV_MAX_ROWS || nq % nkv || nq / nkv > 8 || base < 0 ||
        k_bits < 2 || k_bits > 4 || v_bits < 2 || v_bits > 4 || (hd != 64 && hd != 128)) {
        set_error("attention_quantized: bad argument");
        return TSV_ERR_INVALID;
    }
    tsv_ctx tmp;
    tsv_ctx* c = &tmp;
    TSV_HIP(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
    VerifyParams vp;
    int rc = fill_params(vp, nullptr, nullptr, m, base, 0);
    const int seq = (int)base + m, ctx = (seq + 15) / 16 * 16, nch = attn_chunks(nkv), G = nq / nkv, slots = TSV_MAX_ROWS;
    const size_t stb = (size_t)nkv * slots * hd * 2, inb = (size_t)seq * nkv * hd * 2, qb = (size_t)m * nq * hd * 2;
    uint16_t *kc = nullptr, *vc = nullptr, *kin = nullptr, *vin = nullptr, *q16 = nullptr;
    float *po = nullptr, *pml = nullptr, *sinks_dev = nullptr, *tables = nullptr;
    uint4* xf = nullptr;
    VerifyParams* vpd = nullptr;
    const size_t xfb = xfrag_bytes(nq * hd);
    TqArgs ta{};
    TqKv st{};
    st.k_bits = k_bits;
    st.v_bits = v_bits;
    if (!rc && sinks) {
        rc = dev_alloc(c, &sinks_dev, (size_t)nq * 4);
        if (!rc && hipMemcpyAsync(sinks_dev, sinks, (size_t)nq * 4, hipMemcpyHostToDevice, c->stream) != hipSuccess)
            rc = TSV_ERR_DEVICE;
    }
    if (!rc) rc = dev_alloc(c, &kc, stb, true);
    if (!rc) rc = dev_alloc(c, &vc, stb, true);
    if (!rc) rc = dev_alloc(c, &st.kq, tq_kq_bytes(nkv, ctx, hd, k_bits), true);
    if (!rc) rc = dev_alloc(c, &st.vq, tq_vq_bytes(nkv, ctx, hd, v_bits), true);
    if (!rc) rc = dev_alloc(c, &st.kn, (size_t)nkv * ctx * 4, true);
    if (!rc) rc = dev_alloc(c, &st.vn, (size_t)nkv * ctx * 4, true);
    if (!rc) rc = dev_alloc(c, &kin, inb);
    if (!rc) rc = dev_alloc(c, &vin, inb);
    if (!rc) rc = dev_alloc(c, &q16, qb);
    if (!rc) rc = dev_alloc(c, &po, (size_t)nkv * nch * m * G * hd * 4, true);
    if (!rc) rc = dev_alloc(c, &pml, (size_t)nkv * nch * m * G * 2 * 4, true);
    if (!rc) rc = dev_alloc(c, &xf, xfb, true);
    if (!rc) rc = dev_alloc(c, &vpd, sizeof vp);
    if (!rc) rc = dev_alloc(c, &tables, (size_t)2 * TQ_TABLE_FLOATS * 4);
    if (!rc) rc = tq_upload_side(hd, k_bits, 0, tables, &ta.k);
    if (!rc) rc = tq_upload_side(hd, v_bits, 1, tables + TQ_TABLE_FLOATS, &ta.v);
    if (!rc && (hipMemcpyAsync(kin, k, inb, hipMemcpyHostToDevice, c->stream) != hipSuccess ||
                hipMemcpyAsync(vin, v, inb, hipMemcpyHostToDevice, c->stream) != hipSuccess ||
                hipMemcpyAsync(q16, q, qb, hipMemcpyHostToDevice, c->stream) != hipSuccess ||
                hipMemcpyAsync(vpd, &vp, sizeof vp, hipMemcpyHostToDevice, c->stream) != hipSuccess))
        rc = TSV_ERR_DEVICE;
    st.k_cb = ta.k.cb;
    st.v_cb = ta.v.cb;
    ta.q16 = q16;
    ta.kc = kc;
    ta.vc = vc;
    ta.stage_cap = slots;
    ta.store = st;
    ta.nkv = nkv;
    ta.hd = hd;
    ta.cap = ctx;
    ta.vp = vpd;
    // every row goes through the staging slots and the quantizer, sixteen at a time as passes do; the last
    // group is the pass itself, whose q rows are rotated with it
    const size_t row = (size_t)nkv * hd;
    for (int64_t p = 0; !rc && p < seq;) {
        const bool last = p >= base;
        const int n = last ? m : (int)std::min<int64_t>(slots, base - p);
        rc = launch_kv_fill(c->stream, kc, vc, nkv, hd, slots, (int)p, n, kin + (size_t)p * row, vin + (size_t)p * row);
        ta.nq = last ? nq : 0;
        ta.m_hint = n;
        ta.base_hint = (int)p;
        if (!rc) rc = launch_tq_prepare(c->stream, ta);
        p += n;
    }
    if (!rc) {
        AttnArgs aa{};
        aa.q16 = q16;
        aa.unrot = ta.v.signs;
        aa.tq = st;
        aa.part_o = po;
        aa.part_ml = pml;
        aa.xfrag = xf;
        aa.nq = nq;
        aa.nkv = nkv;
        aa.hd = hd;
        aa.max_ctx = ctx;
        aa.nch = nch;
        aa.scale = scale > 0.f ? scale : 1.0f / std::sqrt((float)hd);
        aa.sinks = sinks_dev;
        aa.vp = vpd;
        aa.m_hint = m;
        aa.base_hint = (int)base;
        rc = launch_attention(c->stream, aa, m);
    }
    std::vector<uint16_t> frag(xfb / 2);
    if (!rc && (hipMemcpyAsync(frag.data(), xf, xfb, hipMemcpyDeviceToHost, c->stream) != hipSuccess ||
                hipStreamSynchronize(c->stream) != hipSuccess)) {
        set_error("attention_quantized: device execution failed");
        rc = TSV_ERR_DEVICE;
    }
    if (!rc) rc = tq_rows_to_host(c->stream, st, nkv, hd, ctx, 0, seq, k_rows, v_rows);
    if (!rc)
        for (int b = 0; b < m; b++)
            for (int kk = 0; kk < nq * hd; kk++) out[(size_t)b * nq * hd + kk] = frag[(size_t)frag_index(kk, b)];
    (void)hipStreamSynchronize(c->stream);
    for (void* p : c->allocs) (void)hipFree(p);
    (void)hipStreamDestroy(c->stream);
    return rc;
}

namespace {
__global__ __launch_bounds__(256) void k_copy_probe(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}
}  // namespace

extern "C" int32_t tsv_copy_time(int64_t bytes, int32_t iters, float* avg_us) {
    if (int hrc = measurement_hooks_on("copy_time")) return hrc;
    if (bytes < 16 || bytes % 16 || iters < 1 || !avg_us) {
        set_error("copy_time: bad argument");
        return TSV_ERR_INVALID;
    }
    hipStream_t s;
    TSV_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    uint4 *a = nullptr, *b = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = TSV_OK;
    if (hipMalloc((void**)&a, (size_t)bytes) != hipSuccess || hipMalloc((void**)&b, (size_t)bytes) != hipSuccess ||
        hipMemsetAsync(a, 1, (size_t)bytes, s) != hipSuccess || hipEventCreate(&e0) != hipSuccess ||
        hipEventCreate(&e1) != hipSuccess) {
        set_error("copy_time: allocation failed");
        rc = TSV_ERR_DEVICE;
    }
    for (int pass = 0; pass < 2 && !rc; pass++) {
        if (pass) (void)hipEventRecord(e0, s);
        for (int i = 0; i < (pass ? iters : 2); i++)
            hipLaunchKernelGGL(k_copy_probe, dim3(256 * 16), dim3(256), 0, s, a, b, (size_t)bytes / 16);
        if (pass) (void)hipEventRecord(e1, s);
    }
    if (!rc) {
        if (hipStreamSynchronize(s) != hipSuccess) {
            set_error("copy_time: device execution failed");
            rc = TSV_ERR_DEVICE;
        } else {
            float ms = 0.f;
            (void)hipEventElapsedTime(&ms, e0, e1);
            *avg_us = ms * 1000.f / (float)iters;
        }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (a) (void)hipFree(a);
    if (b) (void)hipFree(b);
    (void)hipStreamDestroy(s);
    return rc;
}

// Measurement hook: average duration (HIP events on a private stream) of `iters` back-to-back
// launches of the verify pass's matmul over a rows x cols weight of the given dtype filled with
// pseudo-random block bytes, m activation rows, epilogue `epi` (0 split-K partials, 1 silu-mul over
// interleaved gate/up tiles, 2 fp16 logits).  `rotate` distinct weight copies are cycled so the
// kernel streams from HBM rather than from cache.
extern "C" int32_t tsv_matmul_time(int32_t dtype, int64_t rows, int64_t cols, int32_t m, int32_t epi, int32_t splits,
                                   int32_t iters, int32_t rotate, float* avg_us) {
    if (int hrc = measurement_hooks_on("matmul_time")) return hrc;
    const int fmt = dtype_fmt(dtype);
    if (fmt < 0 || rows % TILE_ROWS || cols % fmt_chunk_elems(fmt) || m < 1 || m > TSV_MAX_ROWS || iters < 1 || rotate < 1) {
        set_error("matmul_time: bad argument");
        return TSV_ERR_INVALID;
    }
    tsv_ctx tmp;
    tsv_ctx* c = &tmp;
    TSV_HIP(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
    TiledW w;
    w.fmt = fmt;
    w.k = (int)cols;
    w.kchunks = w.k / fmt_chunk_elems(fmt);
    w.n_rows = (int)rows;
    w.n_tiles = (int)(rows / TILE_ROWS);
    w.bytes = (size_t)w.n_tiles * w.kchunks * fmt_tile_bytes(fmt);
    std::vector<uint8_t*> copies((size_t)rotate);
    int rc = TSV_OK;
    {
        // block bytes: small fp16 scales (0x2xxx) and arbitrary quants
        std::vector<uint8_t> host(w.bytes);
        uint64_t sd = 88172645463325252ull;
        for (size_t i = 0; i < host.size(); i += 8) {
            sd ^= sd << 13;
            sd ^= sd >> 7;
            sd ^= sd << 17;
            std::memcpy(&host[i], &sd, std::min<size_t>(8, host.size() - i));
        }
        const int tb = fmt_tile_bytes(fmt);
        for (size_t t = 0; t < w.bytes / tb; t++) {
            uint8_t* sc = &host[t * tb + 8192];
            if (fmt == FMT_Q4K || fmt == FMT_Q5K)
                for (int r = 0; r < 64; r++) {
                    sc[r * 16 + 1] = 0x20;
                    sc[r * 16 + 3] = 0x20;
                }
            else if (fmt == FMT_Q80)
                for (int i = 0; i < 256; i++) sc[2 * i + 1] = 0x20;
            else if (fmt == FMT_MX4)
                for (int i = 0; i < 512; i++) sc[i] = 0x70 + (sc[i] & 7);  // e8m0 scales around 2^-12
            else if (fmt == FMT_Q6K)
                for (int r = 0; r < 64; r++) host[t * tb + 13312 + r * 4 + 1] = 0x20;  // f16 d
            else  // bf16: every value a small finite number
                for (int i = 0; i < 4096; i++) host[t * tb + 2 * i + 1] = (uint8_t)(0x3C | (host[t * tb + 2 * i + 1] & 0x80));
        }
        for (int i = 0; i < rotate && !rc; i++) {
            rc = dev_alloc(c, &copies[i], w.bytes);
            if (!rc && hipMemcpy(copies[i], host.data(), w.bytes, hipMemcpyHostToDevice) != hipSuccess) rc = TSV_ERR_DEVICE;
        }
    }
    VerifyParams vp;
    std::memset(&vp, 0, sizeof vp);
    vp.m = m;
    uint4* xf = nullptr;
    float* out = nullptr;
    VerifyParams* vpd = nullptr;
    int sp = 1;
    if (!rc) {
        w.tiles = copies[0];
        sp = epi == EPI_PARTIAL ? (splits > 0 ? splits : gemm_default_splits(w, m)) : 1;
        const int kslice = (w.kchunks + sp - 1) / sp;
        sp = (w.kchunks + kslice - 1) / kslice;
    }
    if (!rc) rc = dev_alloc(c, &xf, xfrag_bytes((int)cols), true);
    if (!rc) rc = dev_alloc(c, &out, (size_t)sp * 16 * rows * 4 + xfrag_bytes((int)rows), true);
    if (!rc) rc = dev_alloc(c, &vpd, sizeof vp);
    if (!rc && hipMemcpy(vpd, &vp, sizeof vp, hipMemcpyHostToDevice) != hipSuccess) rc = TSV_ERR_DEVICE;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (!rc && (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)) rc = TSV_ERR_DEVICE;
    for (int pass = 0; pass < 2 && !rc; pass++) {  // pass 0 warms up
        if (pass == 1) (void)hipEventRecord(e0, c->stream);
        for (int i = 0; i < (pass ? iters : std::min(iters, 3)) && !rc; i++) {
            w.tiles = copies[(size_t)(i % rotate)];
            rc = launch_gemm(c->stream, w, xf, (void*)out, vpd, m, sp, epi, (int)rows, (int)rows);
        }
        if (pass == 1) (void)hipEventRecord(e1, c->stream);
    }
    if (!rc) {
        if (hipStreamSynchronize(c->stream) != hipSuccess) {
            set_error("matmul_time: device execution failed");
            rc = TSV_ERR_DEVICE;
        } else {
            float ms = 0.f;
            (void)hipEventElapsedTime(&ms, e0, e1);
            *avg_us = ms * 1000.f / (float)iters;
        }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipStreamSynchronize(c->stream);
    for (void* p : c->allocs) (void)hipFree(p);
    (void)hipStreamDestroy(c->stream);
    return rc;
}
