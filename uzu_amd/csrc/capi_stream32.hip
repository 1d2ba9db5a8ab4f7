// capi_stream32.hip -- the kernels of the f32-stream designs behind plain C entries (include/uzu_hip_engine.h): host arrays in, host arrays out, ONE sequence.
// They exist so that every mechanism can be held to an independent statement of its equations on its own (tests/test_gpu_lazolix_kernels.py) and so that two
// forms of one kernel can be compared on the same inputs; the engine calls the kernels directly (engine_stream32.hip).
#include <algorithm>
#include <vector>

#include "device_utils.h"
#include "kernels_stream32.h"

using namespace uzu;

namespace {

struct Scratch { // device allocations of one call
    std::vector<void*> ptrs;
    ~Scratch() {
        for (void* p : ptrs) (void)hipFree(p);
    }
    template <class T> uzu_status up(const T* host, size_t count, T** out) {
        *out = nullptr;
        if (!count) return UZU_OK;
        void* p = nullptr;
        UZU_HIP_TRY(hipMalloc(&p, count * sizeof(T) + 256));
        ptrs.push_back(p);
        if (host) UZU_HIP_TRY(hipMemcpy(p, host, count * sizeof(T), hipMemcpyHostToDevice));
        else UZU_HIP_TRY(hipMemset(p, 0xFF, count * sizeof(T))); // an output: what the kernel does not write reads as NaN
        *out = (T*)p;
        return UZU_OK;
    }
};

uzu_status one_sequence(Scratch& S, uint32_t rows, uint32_t start, k::SeqSpan** spans, uint32_t** row_seq) {
    const k::SeqSpan sp{0, rows, start};
    std::vector<uint32_t> zeros(rows, 0u);
    UZU_PROPAGATE(S.up(&sp, 1, spans));
    return S.up(zeros.data(), rows, row_seq);
}

uzu_status finish(uzu_hip_context* ctx) {
    UZU_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return UZU_OK;
}

} // namespace

extern "C" {

uzu_status uzu_hip_s32_linear(uzu_hip_context* ctx, const float* x, const uint16_t* w, const uint16_t* bias, const float* residual, float* y, uint32_t rows, uint32_t n, uint32_t kk,
                              uint32_t batch, uint32_t act, uint32_t bf16_products, uint32_t form) {
    UZU_REQUIRE(ctx && x && w && y && batch, "s32_linear: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    k::LinearF32Params p{};
    float *dx, *dy, *dr = nullptr;
    uint16_t *dw, *db = nullptr;
    // batch > 1: x [rows][batch * k], w [batch][n][k], y [rows][batch * n] (the per-head products of the attention)
    UZU_PROPAGATE(S.up(x, (size_t)rows * kk * batch, &dx));
    UZU_PROPAGATE(S.up(w, (size_t)n * kk * batch, &dw));
    if (bias) UZU_PROPAGATE(S.up(bias, n, &db));
    if (residual) UZU_PROPAGATE(S.up(residual, (size_t)rows * n, &dr));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * n * batch, &dy));
    p.x = dx, p.w = dw, p.bias = db, p.residual = dr, p.y = dy, p.rows = rows, p.n = n, p.k = kk, p.ldx = kk * batch, p.ldy = n * batch, p.ldr = n, p.batch = batch;
    p.x_batch = kk, p.w_batch = (size_t)n * kk, p.y_batch = n, p.act = act, p.bf16_products = bf16_products;
    if (form == 1) { // the matrix-core form or nothing
        UZU_UNSUPPORTED(!k::linear_mfma_supported(p), "s32_linear: the matrix-core form does not take this shape");
        UZU_PROPAGATE(k::linear_mfma(ctx->stream, p));
    } else if (form == 2) { // without the matrix cores
        k::LinearF32Params q = p;
        q.bf16_products = 0; // (the dispatcher only offers the matrix cores to bf16 products)
        if (bf16_products) { // round the operand here, then true f32 products: the same numbers as bf16 products
            std::vector<float> xr((size_t)rows * kk * batch);
            for (size_t i = 0; i < xr.size(); ++i) xr[i] = round_bf16(x[i]);
            UZU_HIP_TRY(hipMemcpy(dx, xr.data(), xr.size() * 4, hipMemcpyHostToDevice));
        }
        UZU_PROPAGATE(k::linear_f32(ctx->stream, q));
    } else {
        UZU_PROPAGATE(k::linear_f32(ctx->stream, p));
    }
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(y, dy, (size_t)rows * n * batch * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

// prev_inout [d]: the sequence's last normalised row before the call / after it (token shift only)
uzu_status uzu_hip_s32_dyn_tanh(uzu_hip_context* ctx, const float* x, const float* scales, const float* biases, float alpha, const float* shift, float* prev_inout, uint32_t start,
                                float* out, uint32_t rows, uint32_t d) {
    UZU_REQUIRE(ctx && x && scales && out && (!shift || prev_inout), "s32_dyn_tanh: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    k::DynTanhParams p{};
    float *dx, *ds, *db = nullptr, *dsh = nullptr, *dprev = nullptr, *dout;
    float** dpp = nullptr;
    UZU_PROPAGATE(S.up(x, (size_t)rows * d, &dx));
    UZU_PROPAGATE(S.up(scales, d, &ds));
    if (biases) UZU_PROPAGATE(S.up(biases, d, &db));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * d, &dout));
    p.x = dx, p.out = dout, p.scales = ds, p.biases = db, p.alpha = alpha, p.rows = rows, p.d = d;
    if (shift) {
        k::SeqSpan* spans;
        uint32_t* row_seq;
        UZU_PROPAGATE(S.up(shift, d, &dsh));
        UZU_PROPAGATE(S.up((const float*)prev_inout, d, &dprev));
        UZU_PROPAGATE(S.up((float* const*)&dprev, 1, &dpp));
        UZU_PROPAGATE(one_sequence(S, rows, start, &spans, &row_seq));
        p.shift = dsh, p.prev = dpp, p.spans = spans, p.row_seq = row_seq;
    }
    UZU_PROPAGATE(k::dyn_tanh_norm(ctx->stream, p));
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(out, dout, (size_t)rows * d * 4, hipMemcpyDeviceToHost));
    if (shift) UZU_HIP_TRY(hipMemcpy(prev_inout, dprev, (size_t)d * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

uzu_status uzu_hip_s32_depth_mix(uzu_hip_context* ctx, const float* slots, const float* w, uint32_t count, float* out, uint32_t rows, uint32_t d) {
    UZU_REQUIRE(ctx && slots && w && out, "s32_depth_mix: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    float *ds, *dw, *dout;
    UZU_PROPAGATE(S.up(slots, (size_t)count * rows * d, &ds));
    UZU_PROPAGATE(S.up(w, count, &dw));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * d, &dout));
    UZU_PROPAGATE(k::depth_mix(ctx->stream, ds, (size_t)rows * d, dw, count, dout, rows, d));
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(out, dout, (size_t)rows * d * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

// x [rows][rank] raw latents of positions start ..; cache_out [(start + rows)][rank] f32: rows below `start` come back as given in cache_inout
uzu_status uzu_hip_s32_latent_norm_append(uzu_hip_context* ctx, const float* x, const float* scales, float eps, float* cache_inout, uint32_t cache_bf16, uint32_t start, uint32_t rows,
                                          uint32_t rank) {
    UZU_REQUIRE(ctx && x && scales && cache_inout, "s32_latent_norm_append: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    const size_t total = (size_t)(start + rows) * rank;
    float *dx, *ds, *dc32 = nullptr;
    uint16_t* dc16 = nullptr;
    void** dcp;
    k::SeqSpan* spans;
    uint32_t* row_seq;
    UZU_PROPAGATE(S.up(x, (size_t)rows * rank, &dx));
    UZU_PROPAGATE(S.up(scales, rank, &ds));
    std::vector<uint16_t> bits(total);
    if (cache_bf16) {
        for (size_t i = 0; i < total; ++i) bits[i] = f32_to_bf16(cache_inout[i]);
        UZU_PROPAGATE(S.up(bits.data(), total, &dc16));
    } else {
        UZU_PROPAGATE(S.up((const float*)cache_inout, total, &dc32));
    }
    void* cache = cache_bf16 ? (void*)dc16 : (void*)dc32;
    UZU_PROPAGATE(S.up((void* const*)&cache, 1, &dcp));
    UZU_PROPAGATE(one_sequence(S, rows, start, &spans, &row_seq));
    UZU_PROPAGATE(k::latent_norm_append(ctx->stream, dx, ds, eps, dcp, cache_bf16, spans, row_seq, rows, rank));
    UZU_PROPAGATE(finish(ctx));
    if (cache_bf16) {
        UZU_HIP_TRY(hipMemcpy(bits.data(), dc16, total * 2, hipMemcpyDeviceToHost));
        for (size_t i = 0; i < total; ++i) cache_inout[i] = bf16_to_f32(bits[i]);
    } else {
        UZU_HIP_TRY(hipMemcpy(cache_inout, dc32, total * 4, hipMemcpyDeviceToHost));
    }
    return UZU_OK;
}

// qlat / out [rows][heads * rank] for positions start .. start + rows - 1; cache f32 [(start + rows)][rank] (rounded to bf16 here when cache_bf16).
// form 0: the engine's choice for the shape; 1: the simple form (a wave per row and head); 2: the tiled form; 3: the tiled form with split keys + merge
uzu_status uzu_hip_s32_latent_attention(uzu_hip_context* ctx, const float* qlat, const float* cache, const float* sinks, float* out, uint32_t rows, uint32_t start, uint32_t heads,
                                        uint32_t rank, uint32_t window, float scale, uint32_t cache_bf16, uint32_t form) {
    UZU_REQUIRE(ctx && qlat && cache && out, "s32_latent_attention: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    const size_t total = (size_t)(start + rows) * rank;
    float *dq, *dout, *dsink = nullptr, *dc32 = nullptr;
    uint16_t* dc16 = nullptr;
    void** dcp;
    k::SeqSpan* spans;
    uint32_t* row_seq;
    UZU_PROPAGATE(S.up(qlat, (size_t)rows * heads * rank, &dq));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * heads * rank, &dout));
    if (sinks) UZU_PROPAGATE(S.up(sinks, heads, &dsink));
    if (cache_bf16) {
        std::vector<uint16_t> bits(total);
        for (size_t i = 0; i < total; ++i) bits[i] = f32_to_bf16(cache[i]);
        UZU_PROPAGATE(S.up(bits.data(), total, &dc16));
    } else {
        UZU_PROPAGATE(S.up(cache, total, &dc32));
    }
    void* cp = cache_bf16 ? (void*)dc16 : (void*)dc32;
    UZU_PROPAGATE(S.up((void* const*)&cp, 1, &dcp));
    UZU_PROPAGATE(one_sequence(S, rows, start, &spans, &row_seq));
    k::LatentAttentionParams p{};
    p.qlat = dq, p.out = dout, p.caches = dcp, p.cache_bf16 = cache_bf16, p.sinks = dsink, p.spans = spans, p.row_seq = row_seq;
    p.rows = rows, p.heads = heads, p.rank = rank, p.window = window, p.scale = scale, p.form = form, p.nseq = 1, p.tiles = (rows * heads + 127) / 128;
    float* ws = nullptr;
    if (form == 3) { // the tiled form with its key blocks split over workgroups + the merge launch
        p.form = 2, p.splits = 5;
        p.split_ws_bytes = k::latent_attention_split_ws_bytes(rows, heads, rank, p.splits);
        UZU_PROPAGATE(S.up((const float*)nullptr, p.split_ws_bytes / 4, &ws));
        p.split_ws = ws;
    }
    UZU_PROPAGATE(k::latent_attention(ctx->stream, p));
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(out, dout, (size_t)rows * heads * rank * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

// the whole score-routed block on rows x: ids / weights [rows][top] and y = residual + sum of the winners' outputs
uzu_status uzu_hip_s32_moe(uzu_hip_context* ctx, const float* x, const uint16_t* router, const float* selection_bias, const uint16_t* w13, const uint16_t* w2, const float* residual,
                           float* y, int32_t* ids_out, float* weights_out, uint32_t rows, uint32_t d, uint32_t ff, uint32_t routed, uint32_t identity, uint32_t top,
                           uint32_t bf16_products) {
    UZU_REQUIRE(ctx && x && router && y && (!routed || (w13 && w2)), "s32_moe: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    float *dx, *dsb = nullptr, *dres = nullptr, *dy, *dwt, *dh;
    uint16_t *dr, *d13 = nullptr, *d2 = nullptr;
    int32_t* dids;
    UZU_PROPAGATE(S.up(x, (size_t)rows * d, &dx));
    UZU_PROPAGATE(S.up(router, (size_t)(routed + identity) * d, &dr));
    if (selection_bias) UZU_PROPAGATE(S.up(selection_bias, routed + identity, &dsb));
    if (routed) {
        UZU_PROPAGATE(S.up(w13, (size_t)routed * 2 * ff * d, &d13));
        UZU_PROPAGATE(S.up(w2, (size_t)routed * d * ff, &d2));
    }
    if (residual) UZU_PROPAGATE(S.up(residual, (size_t)rows * d, &dres));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * d, &dy));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * top, &dwt));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * top * (ff ? ff : 1), &dh));
    UZU_PROPAGATE(S.up((const int32_t*)nullptr, (size_t)rows * top, &dids));
    UZU_PROPAGATE(k::moe_route_scores(ctx->stream, dx, dr, dsb, dids, dwt, rows, d, routed + identity, top));
    if (bf16_products == 2) { // bf16 products through the grouped matrix-core form
        k::MoeGroupedParams gp{};
        uint32_t *perm, *slot_pos, *offsets, *cursor;
        float *y1, *y2;
        UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * top * 2 * ff, &y1));
        UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * top * d, &y2));
        UZU_PROPAGATE(S.up((const uint32_t*)nullptr, (size_t)rows * top, &perm));
        UZU_PROPAGATE(S.up((const uint32_t*)nullptr, (size_t)rows * top, &slot_pos));
        UZU_PROPAGATE(S.up((const uint32_t*)nullptr, (size_t)routed + 1, &offsets));
        UZU_PROPAGATE(S.up((const uint32_t*)nullptr, (size_t)routed + 1, &cursor));
        gp.x = dx, gp.ids = dids, gp.weights = dwt, gp.w13 = d13, gp.w2 = d2, gp.residual = dres, gp.y = dy, gp.y1 = y1, gp.hidden = dh, gp.y2 = y2;
        gp.perm = perm, gp.slot_pos = slot_pos, gp.offsets = offsets, gp.cursor = cursor, gp.rows = rows, gp.d = d, gp.ff = ff, gp.routed = routed, gp.top = top;
        UZU_UNSUPPORTED(!k::moe_experts_grouped_supported(gp), "s32_moe: the grouped form does not take this shape");
        UZU_PROPAGATE(k::moe_experts_grouped(ctx->stream, gp));
    } else {
        UZU_PROPAGATE(k::moe_experts_gate_up(ctx->stream, dx, dids, d13, dh, rows, d, ff, routed, top, bf16_products));
        UZU_PROPAGATE(k::moe_experts_down_combine(ctx->stream, dh, dx, dids, dwt, d2, dres, dy, rows, d, ff, routed, top, bf16_products));
    }
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(y, dy, (size_t)rows * d * 4, hipMemcpyDeviceToHost));
    if (ids_out) UZU_HIP_TRY(hipMemcpy(ids_out, dids, (size_t)rows * top * 4, hipMemcpyDeviceToHost));
    if (weights_out) UZU_HIP_TRY(hipMemcpy(weights_out, dwt, (size_t)rows * top * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

// Rotation + key scaling in place on packed rows [rows][heads * dim (queries) + kv_heads * dim (keys)] at positions start ..; tables [start + rows][rope_dim]
uzu_status uzu_hip_s32_rotate(uzu_hip_context* ctx, float* qk_inout, const float* cosines, const float* sines, uint32_t rows, uint32_t start, uint32_t heads, uint32_t kv_heads,
                              uint32_t dim, uint32_t rope_dim, float key_scale) {
    UZU_REQUIRE(ctx && qk_inout && cosines && sines, "s32_rotate: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    const uint32_t ld = (heads + kv_heads) * dim;
    float *dx, *dc, *ds;
    k::SeqSpan* spans;
    uint32_t* row_seq;
    UZU_PROPAGATE(S.up((const float*)qk_inout, (size_t)rows * ld, &dx));
    UZU_PROPAGATE(S.up(cosines, (size_t)(start + rows) * rope_dim, &dc));
    UZU_PROPAGATE(S.up(sines, (size_t)(start + rows) * rope_dim, &ds));
    UZU_PROPAGATE(one_sequence(S, rows, start, &spans, &row_seq));
    k::RopeAppendParams p{};
    p.qkv = dx, p.ld = ld, p.k_col = heads * dim, p.v_col = ld, p.heads = heads, p.kv_heads = kv_heads, p.dim = dim, p.vdim = 0, p.rope_dim = rope_dim, p.cosines = dc, p.sines = ds;
    p.key_scale = key_scale, p.spans = spans, p.row_seq = row_seq, p.rows = rows;
    UZU_PROPAGATE(k::rope_append(ctx->stream, p));
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(qk_inout, dx, (size_t)rows * ld * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

// Attention of rows at positions start .. over keys [start + rows][kv_heads * dim] and values [start + rows][kv_heads * vdim] (f32 in; rounded to bf16 for a bf16
// cache); q [rows][heads * dim] rotated already; sinks f32 [heads] or null.  form 0 dispatch, 1 simple, 2 matrix cores, 3 matrix cores with split keys.
uzu_status uzu_hip_s32_window_attention(uzu_hip_context* ctx, const float* q, const float* keys, const float* values, const float* sinks, float* out, uint32_t rows, uint32_t start,
                                        uint32_t heads, uint32_t kv_heads, uint32_t dim, uint32_t vdim, uint32_t window, float scale, float soft_cap, uint32_t cache_bf16, uint32_t form) {
    UZU_REQUIRE(ctx && q && keys && values && out && kv_heads, "s32_window_attention: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    float *dq, *dout, *dsink = nullptr;
    void *dk = nullptr, *dv = nullptr;
    void **dkp, **dvp;
    k::SeqSpan* spans;
    uint32_t* row_seq;
    UZU_PROPAGATE(S.up(q, (size_t)rows * heads * dim, &dq));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * heads * vdim, &dout));
    if (sinks) UZU_PROPAGATE(S.up(sinks, heads, &dsink));
    auto cache = [&](const float* host, size_t total, void** dev) -> uzu_status {
        if (cache_bf16) {
            std::vector<uint16_t> bits(total);
            for (size_t i = 0; i < total; ++i) bits[i] = f32_to_bf16(host[i]);
            uint16_t* d16;
            UZU_PROPAGATE(S.up(bits.data(), total, &d16));
            *dev = d16;
        } else {
            float* d32;
            UZU_PROPAGATE(S.up(host, total, &d32));
            *dev = d32;
        }
        return UZU_OK;
    };
    UZU_PROPAGATE(cache(keys, (size_t)(start + rows) * kv_heads * dim, &dk));
    UZU_PROPAGATE(cache(values, (size_t)(start + rows) * kv_heads * vdim, &dv));
    UZU_PROPAGATE(S.up((void* const*)&dk, 1, &dkp));
    UZU_PROPAGATE(S.up((void* const*)&dv, 1, &dvp));
    UZU_PROPAGATE(one_sequence(S, rows, start, &spans, &row_seq));
    k::WindowAttentionParams p{};
    p.q = dq, p.ldq = heads * dim, p.out = dout, p.key_caches = dkp, p.value_caches = dvp, p.cache_bf16 = cache_bf16, p.sinks = dsink, p.spans = spans, p.row_seq = row_seq;
    p.rows = rows, p.heads = heads, p.kv_heads = kv_heads, p.dim = dim, p.vdim = vdim, p.window = window, p.scale = scale, p.soft_cap = soft_cap, p.form = form, p.nseq = 1;
    p.tiles = heads % kv_heads == 0 ? (rows * (heads / kv_heads) + 127) / 128 : 0;
    if (form == 3) { // the matrix-core form with its key blocks split over workgroups + the merge launch
        float* ws = nullptr;
        p.form = 2, p.splits = 5;
        p.split_ws_bytes = k::window_attention_split_ws_bytes(rows, heads, p.splits);
        UZU_PROPAGATE(S.up((const float*)nullptr, p.split_ws_bytes / 4, &ws));
        p.split_ws = ws;
    }
    UZU_PROPAGATE(k::window_attention(ctx->stream, p));
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(out, dout, (size_t)rows * heads * vdim * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

// Retention of rows at positions start ..: q, k [rows][heads * dim] (rotated, scaled), v [rows][heads * vdim], decay [heads]; state_inout [heads][dim][vdim] is the
// state in front of the rows (ignored when start == 0) and behind them.  form 0 dispatch, 1 token by token, 2 in chunks.
uzu_status uzu_hip_s32_retention(uzu_hip_context* ctx, const float* q, const float* kk, const float* v, const float* decay, float* state_inout, float* out, uint32_t rows, uint32_t start,
                                 uint32_t heads, uint32_t dim, uint32_t vdim, uint32_t form) {
    UZU_REQUIRE(ctx && q && kk && v && decay && state_inout && out, "s32_retention: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    const uint32_t ld = heads * (2 * dim + vdim);
    std::vector<float> packed((size_t)rows * ld);
    for (uint32_t r = 0; r < rows; ++r) {
        std::copy(q + (size_t)r * heads * dim, q + (size_t)(r + 1) * heads * dim, packed.begin() + (size_t)r * ld);
        std::copy(kk + (size_t)r * heads * dim, kk + (size_t)(r + 1) * heads * dim, packed.begin() + (size_t)r * ld + heads * dim);
        std::copy(v + (size_t)r * heads * vdim, v + (size_t)(r + 1) * heads * vdim, packed.begin() + (size_t)r * ld + 2 * heads * dim);
    }
    float *dx, *dd, *dst, *dout, *dws = nullptr;
    float** dsp;
    k::SeqSpan* spans;
    uint32_t* row_seq;
    UZU_PROPAGATE(S.up(packed.data(), packed.size(), &dx));
    UZU_PROPAGATE(S.up(decay, heads, &dd));
    UZU_PROPAGATE(S.up((const float*)state_inout, (size_t)heads * dim * vdim, &dst));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * heads * vdim, &dout));
    UZU_PROPAGATE(S.up((float* const*)&dst, 1, &dsp));
    UZU_PROPAGATE(one_sequence(S, rows, start, &spans, &row_seq));
    k::RetentionParams p{};
    p.qkv = dx, p.ld = ld, p.q_col = 0, p.k_col = heads * dim, p.v_col = 2 * heads * dim, p.out = dout, p.states = dsp, p.decay = dd, p.spans = spans, p.nseq = 1, p.rows = rows;
    p.heads = heads, p.dim = dim, p.vdim = vdim, p.form = form, p.chunks = (rows + 63) / 64;
    p.chunk_ws_bytes = k::retention_chunk_ws_bytes(p.chunks, heads, dim, vdim);
    UZU_PROPAGATE(S.up((const float*)nullptr, p.chunk_ws_bytes / 4, &dws));
    p.chunk_ws = dws;
    UZU_PROPAGATE(k::retention(ctx->stream, p));
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(out, dout, (size_t)rows * heads * vdim * 4, hipMemcpyDeviceToHost));
    UZU_HIP_TRY(hipMemcpy(state_inout, dst, (size_t)heads * dim * vdim * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

// Weight-vector RMS norm of a sublayer's result joined to the stream: out = residual + rms(y) (scales + offset) layer_scale (layer_scale optional), and with
// next_out the norm of the new rows for the sublayer that follows (next_scales + next_offset, next_eps).  Host arrays [rows][d].
uzu_status uzu_hip_s32_rms_norm_add(uzu_hip_context* ctx, const float* y, const float* residual, float* out, const float* scales, float offset, const float* layer_scale, float eps,
                                    uint32_t rows, uint32_t d, float* next_out, const float* next_scales, float next_offset, float next_eps) {
    UZU_REQUIRE(ctx && y && residual && out && scales && (!next_out || next_scales), "s32_rms_norm_add: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    float *dy, *dr, *ds, *dl = nullptr, *dn = nullptr, *dns = nullptr;
    UZU_PROPAGATE(S.up(y, (size_t)rows * d, &dy));
    UZU_PROPAGATE(S.up(residual, (size_t)rows * d, &dr)); // in place, as the engine runs it behind a dense block
    UZU_PROPAGATE(S.up(scales, d, &ds));
    if (layer_scale) UZU_PROPAGATE(S.up(layer_scale, d, &dl));
    if (next_out) {
        UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * d, &dn));
        UZU_PROPAGATE(S.up(next_scales, d, &dns));
    }
    UZU_PROPAGATE(k::rms_norm_add_rows(ctx->stream, dy, dr, dr, ds, offset, dl, eps, rows, d, dn, dns, next_offset, next_eps));
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(out, dr, (size_t)rows * d * 4, hipMemcpyDeviceToHost));
    if (next_out) UZU_HIP_TRY(hipMemcpy(next_out, dn, (size_t)rows * d * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

// uzu_hip_s32_rotate with a per-head RMS norm of queries (q_norm [dim] or NULL) and keys (k_norm) in front of the rotation
uzu_status uzu_hip_s32_rotate_normed(uzu_hip_context* ctx, float* qk_inout, const float* cosines, const float* sines, const float* q_norm, const float* k_norm, float norm_eps,
                                     uint32_t rows, uint32_t start, uint32_t heads, uint32_t kv_heads, uint32_t dim, uint32_t rope_dim) {
    UZU_REQUIRE(ctx && qk_inout && (!rope_dim || (cosines && sines)), "s32_rotate_normed: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    const uint32_t ld = (heads + kv_heads) * dim;
    float *dx, *dc = nullptr, *ds = nullptr, *dqn = nullptr, *dkn = nullptr;
    k::SeqSpan* spans;
    uint32_t* row_seq;
    UZU_PROPAGATE(S.up((const float*)qk_inout, (size_t)rows * ld, &dx));
    if (rope_dim) {
        UZU_PROPAGATE(S.up(cosines, (size_t)(start + rows) * rope_dim, &dc));
        UZU_PROPAGATE(S.up(sines, (size_t)(start + rows) * rope_dim, &ds));
    }
    if (q_norm) UZU_PROPAGATE(S.up(q_norm, dim, &dqn));
    if (k_norm) UZU_PROPAGATE(S.up(k_norm, dim, &dkn));
    UZU_PROPAGATE(one_sequence(S, rows, start, &spans, &row_seq));
    k::RopeAppendParams p{};
    p.qkv = dx, p.ld = ld, p.k_col = heads * dim, p.v_col = ld, p.heads = heads, p.kv_heads = kv_heads, p.dim = dim, p.vdim = 0, p.rope_dim = rope_dim, p.cosines = dc, p.sines = ds;
    p.key_scale = 1.0f, p.q_norm = dqn, p.k_norm = dkn, p.norm_eps = norm_eps, p.spans = spans, p.row_seq = row_seq, p.rows = rows;
    UZU_PROPAGATE(k::rope_append(ctx->stream, p));
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(qk_inout, dx, (size_t)rows * ld * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

// x [rows][heads * q_width + rank + rope_dim]: query heads (the last rope_dim coordinates of each turn), then the down projection's row.  cache_inout
// [(start + rows)][rank + rope_dim] f32 (rows below `start` come back as given); qlat_out [rows][heads][rank + rope_dim]: only the rotated columns are written
// (the others come back as NaN).  Tables [start + rows][rope_dim].
uzu_status uzu_hip_s32_latent_rope_append(uzu_hip_context* ctx, const float* x, const float* scales, float eps, const float* cosines, const float* sines, float* cache_inout,
                                          float* qlat_out, uint32_t cache_bf16, uint32_t interleaved, uint32_t start, uint32_t rows, uint32_t heads, uint32_t q_width, uint32_t rank,
                                          uint32_t rope_dim) {
    UZU_REQUIRE(ctx && x && scales && cache_inout && qlat_out && (!rope_dim || (cosines && sines)), "s32_latent_rope_append: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    const uint32_t kw = rank + rope_dim, ldx = heads * q_width + kw;
    const size_t total = (size_t)(start + rows) * kw;
    float *dx, *dsc, *dc = nullptr, *dsn = nullptr, *dc32 = nullptr, *dq;
    uint16_t* dc16 = nullptr;
    void** dcp;
    k::SeqSpan* spans;
    uint32_t* row_seq;
    UZU_PROPAGATE(S.up(x, (size_t)rows * ldx, &dx));
    UZU_PROPAGATE(S.up(scales, rank, &dsc));
    if (rope_dim) {
        UZU_PROPAGATE(S.up(cosines, (size_t)(start + rows) * rope_dim, &dc));
        UZU_PROPAGATE(S.up(sines, (size_t)(start + rows) * rope_dim, &dsn));
    }
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * heads * kw, &dq));
    std::vector<uint16_t> bits(total);
    if (cache_bf16) {
        for (size_t i = 0; i < total; ++i) bits[i] = f32_to_bf16(cache_inout[i]);
        UZU_PROPAGATE(S.up(bits.data(), total, &dc16));
    } else {
        UZU_PROPAGATE(S.up((const float*)cache_inout, total, &dc32));
    }
    void* cache = cache_bf16 ? (void*)dc16 : (void*)dc32;
    UZU_PROPAGATE(S.up((void* const*)&cache, 1, &dcp));
    UZU_PROPAGATE(one_sequence(S, rows, start, &spans, &row_seq));
    k::LatentRopeAppendParams p{};
    p.x = dx, p.ldx = ldx, p.c_col = heads * q_width, p.rank = rank, p.rope_dim = rope_dim, p.scales = dsc, p.eps = eps, p.caches = dcp, p.cache_bf16 = cache_bf16, p.heads = heads;
    p.q_width = q_width, p.qlat = rope_dim ? dq : nullptr, p.cosines = dc, p.sines = dsn, p.interleaved = interleaved, p.spans = spans, p.row_seq = row_seq, p.rows = rows;
    UZU_PROPAGATE(k::latent_rope_append(ctx->stream, p));
    UZU_PROPAGATE(finish(ctx));
    if (cache_bf16) {
        UZU_HIP_TRY(hipMemcpy(bits.data(), dc16, total * 2, hipMemcpyDeviceToHost));
        for (size_t i = 0; i < total; ++i) cache_inout[i] = bf16_to_f32(bits[i]);
    } else {
        UZU_HIP_TRY(hipMemcpy(cache_inout, dc32, total * 4, hipMemcpyDeviceToHost));
    }
    UZU_HIP_TRY(hipMemcpy(qlat_out, dq, (size_t)rows * heads * kw * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

// The gated linear recurrent unit on rows at positions start ..: branches [rows][2 width] (gate branch | recurrent branch, biases added), conv_w [width][taps],
// conv_b [width], gate_w bf16 [blocks][2 bw][bw], gate_b [blocks][2 bw], lambda [width]; state_inout [width] and conv_state_inout [taps - 1][width] (at least one
// row) are the state in front of the rows (ignored where positions lie in front of 0) and behind them; out [rows][width] = S * gelu(gate branch).
// form 0 dispatch, 1 position by position, 2 in pieces.
uzu_status uzu_hip_s32_gated_lru(uzu_hip_context* ctx, const float* branches, const float* conv_w, const float* conv_b, const uint16_t* gate_w, const float* gate_b,
                                 const float* lambda, float rate, float* state_inout, float* conv_state_inout, float* out, uint32_t rows, uint32_t start, uint32_t width,
                                 uint32_t blocks, uint32_t taps, uint32_t form) {
    UZU_REQUIRE(ctx && branches && conv_w && gate_w && lambda && state_inout && conv_state_inout && out && blocks && width % blocks == 0 && taps, "s32_gated_lru: null argument");
    (void)hipSetDevice(ctx->device);
    Scratch S;
    const uint32_t bw = width / blocks, keep = taps > 1 ? taps - 1 : 1;
    float *dx, *dcw, *dcb = nullptr, *dgb = nullptr, *dl, *dst, *dcs, *du, *dg, *dout, *dws;
    uint16_t* dgw;
    float **dsp, **dcsp;
    k::SeqSpan* spans;
    uint32_t* row_seq;
    UZU_PROPAGATE(S.up(branches, (size_t)rows * 2 * width, &dx));
    UZU_PROPAGATE(S.up(conv_w, (size_t)width * taps, &dcw));
    if (conv_b) UZU_PROPAGATE(S.up(conv_b, width, &dcb));
    UZU_PROPAGATE(S.up(gate_w, (size_t)2 * width * bw, &dgw));
    if (gate_b) UZU_PROPAGATE(S.up(gate_b, (size_t)2 * width, &dgb));
    UZU_PROPAGATE(S.up(lambda, width, &dl));
    UZU_PROPAGATE(S.up((const float*)state_inout, width, &dst));
    UZU_PROPAGATE(S.up((const float*)conv_state_inout, (size_t)keep * width, &dcs));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * width, &du));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * 2 * width, &dg));
    UZU_PROPAGATE(S.up((const float*)nullptr, (size_t)rows * width, &dout));
    UZU_PROPAGATE(S.up((float* const*)&dst, 1, &dsp));
    UZU_PROPAGATE(S.up((float* const*)&dcs, 1, &dcsp));
    UZU_PROPAGATE(one_sequence(S, rows, start, &spans, &row_seq));
    k::GatedLruParams p{};
    p.branches = dx, p.ld = 2 * width, p.x_col = width, p.u = du, p.gates = dg, p.out = dout, p.conv_w = dcw, p.conv_b = dcb, p.gate_b = dgb, p.lambda = dl, p.rate = rate;
    p.states = dsp, p.conv_states = dcsp, p.spans = spans, p.row_seq = row_seq, p.nseq = 1, p.rows = rows, p.width = width, p.blocks = blocks, p.taps = taps, p.form = form;
    p.max_count = rows, p.pieces = (rows + 31) / 32, p.piece_ws_bytes = k::lru_piece_ws_bytes(p.pieces, width);
    UZU_PROPAGATE(S.up((const float*)nullptr, p.piece_ws_bytes / 4, &dws));
    p.piece_ws = dws;
    UZU_PROPAGATE(k::lru_conv(ctx->stream, p));
    k::LinearF32Params g{};
    g.x = du, g.w = dgw, g.y = dg, g.rows = rows, g.n = 2 * bw, g.k = bw, g.ldx = width, g.ldy = 2 * width, g.batch = blocks, g.x_batch = bw, g.w_batch = (size_t)2 * bw * bw;
    g.y_batch = 2 * bw, g.bf16_products = 0;
    UZU_PROPAGATE(k::linear_f32(ctx->stream, g));
    UZU_PROPAGATE(k::lru_scan(ctx->stream, p));
    UZU_PROPAGATE(finish(ctx));
    UZU_HIP_TRY(hipMemcpy(out, dout, (size_t)rows * width * 4, hipMemcpyDeviceToHost));
    UZU_HIP_TRY(hipMemcpy(state_inout, dst, (size_t)width * 4, hipMemcpyDeviceToHost));
    UZU_HIP_TRY(hipMemcpy(conv_state_inout, dcs, (size_t)keep * width * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

} // extern "C"
