// engine_stream32.hip -- the forward encoder of the f32-stream designs (uzu_model_desc::f32_stream; first family: Lazolix).
//
// What differs from the reference's models (engine_forward.hip): the residual stream stays f32 from the embedding to the read-out (nothing is re-rounded to
// bf16 between layers), norms are dynamic-tanh norms, a layer's mixer reads token-shifted rows, the mixer is attention over a cached low-rank latent
// (k_latent_attention.hip), the MLP is a plain dense block or score-routed experts with identity experts, every layer ends in a depth mix over the results of
// all layers before it, and logits are f32.  What is shared: the model / state objects and their memory accounting (engine_build.hip), the sampling kernels,
// the device-resident control block (context length, next token, sampled history) and the C ABI above (engine_api.hip).
//
// A pass carries rows of SEVERAL sequences of unequal length (struct k::SeqSpan): linears, norms and experts see one matrix of all rows; the token shift, the
// latent cache and the attention core address each row's own sequence through pointer tables built per pass.  A prompt longer than one pass (m->chunk rows)
// continues in the next pass from the state the previous one left: the cache rows and the last normalised row per layer.
//
// Next to those the encoder carries the mechanisms of designs with rotated attention and recurrent layers (second family: Relulix): RMS norms with one gain,
// parallel blocks (mixer and MLP read the same normalised rows, one residual add), attention over a per-position cache of rotated keys and values (grouped
// heads, biases, partial rotation with scaled frequencies, soft-capped scores, sliding window, a unit sink; k_window_attention.hip), retention layers with an
// f32 state per sequence (k_retention.hip), top-k routed experts with clamped gates, a scaled embedding and an untied read-out.  Each is chosen per layer by the
// description's fields, so a model may mix them.
//
// A third family (Begasun) adds: RMS norms with a weight vector stored around zero in front of AND behind every sublayer, a layer scale on each sublayer's result, a
// per-layer token input (a slice of a second token table, gated by the stream), a gated dense block with clamps, layer runs that share an earlier run's tensors with
// a re-entry projection of [stream ; embedding rows] (a looped stack; every run keeps its own sequence state), latent attention whose cache row carries one rotated
// key part for all heads (interleaved pairs, scaled frequencies) with a sigmoid gate per head, per-head query / key norms on the cached-key attention, and a
// gated linear recurrent unit behind a short convolution (k_gated_lru.hip).
//
// A fourth family (Zovolorn) adds: sublayers WITHOUT a norm in front that read the stream through a short causal convolution (rows + convolution, the window is
// sequence state; k_causal_conv.hip) and join it behind an RMS norm taken in equal parts of the row, a hashed (previous token, token) table beside the embedding, a
// capped read-out, a gelu-gated dense block with biases; on the cached-key attention one RMS norm over the whole query / key projection, interleaved pairs, a sigmoid
// gate per head, causal chunks, values that are the key rows, a temperature per head and a learned bias per distance bucket; and a SECOND mixer beside the first in one
// layer -- a gated delta rule with a decay per head and key channel (k_channel_delta.hip) -- whose result is summed with the first's through their own out projections.
//
// Precisions: `bf16_products` (default) rounds the activation operand of every matrix product to bf16 and keeps the latent cache in bf16; UZU_MODEL_FULL_F32
// makes every product a true f32 product and the cache f32.  Everything else is f32 either way.
#include <algorithm>

#include "engine_types.h"
#include "kernels_stream32.h"
#include "uzu_math.h"

using namespace uzu;
using namespace uzu::eng;

namespace uzu {
namespace eng {

struct Stream32 {
    bool full_f32 = false;
    uint32_t max_rows = 0, max_seqs = 1;
    float *slots = nullptr, *xin = nullptr, *normed = nullptr, *q = nullptr, *ckv = nullptr, *qlat = nullptr, *ctx = nullptr, *attn = nullptr, *hid = nullptr;
    int32_t* moe_ids = nullptr;
    float* moe_w = nullptr;
    float *tmp = nullptr, *y1 = nullptr, *lru_u = nullptr, *lru_g = nullptr, *side_g = nullptr; // a sublayer's result in front of its post norm; [up | gate] of a gated dense block; LRU input / gates; token-input gate
    float *moe_y1 = nullptr, *moe_y2 = nullptr; // grouped expert form: [max_rows * top][2 ff] and [max_rows * top][d]
    uint32_t *moe_perm = nullptr, *moe_slot_pos = nullptr, *moe_offsets = nullptr, *moe_cursor = nullptr;
    float *out_normed = nullptr, *logits = nullptr;
    size_t logit_rows = 0;
    k::SeqSpan* d_spans = nullptr;
    uint32_t *d_row_seq = nullptr, *d_out_rows = nullptr;
    void** d_cache_ptrs = nullptr;  // [layers][max_seqs]: latent rows / key rows / the retention state
    void** d_cache2_ptrs = nullptr; // [layers][max_seqs]: value rows
    float** d_shift_ptrs = nullptr; // [layers][max_seqs]
    float** d_pair_state_ptrs = nullptr; // [layers][max_seqs]: the second mixer's recurrent state
    float** d_pair_conv_ptrs = nullptr;  // [layers][max_seqs]: ... and its convolution window
    float** d_inconv_ptrs = nullptr;     // [layers][max_seqs]: the windows of the sublayers' input convolutions (mixer's, then MLP's)
    uint32_t** d_prev_tok_ptrs = nullptr; // [max_seqs]: the previous token (hashed token-pair table)
    float *dn_in = nullptr, *dn_cv = nullptr, *dn_decay = nullptr, *dn_gate = nullptr, *dn_o = nullptr; // the delta rule: packed projection, convolved q | k | v, decays, gate, result
    uint16_t* pair_table = nullptr; // bf16 [buckets + 1][d]
    // a pair of mixers in a prompt-sized pass: the first mixer's launches run on a stream of their own beside the second's (its recurrence is a chain of dependent
    // steps on few workgroups and leaves most of the chip idle); default priority, joined again in front of the out projections
    hipStream_t side = nullptr;
    hipEvent_t side_fork = nullptr, side_join = nullptr;
    struct Layer {
        uint16_t* up_keys_t = nullptr; // bf16 [heads][rank][head_dim]: W_up_k of a head transposed, so that folding it into the query is an ordinary product
        float* sinks = nullptr;        // f32 [heads]
        float *token_shift = nullptr, *depth_weights = nullptr, *selection_bias = nullptr;
        float alpha1 = 0.f, alpha2 = 0.f;
        float* decay = nullptr; // retention: f32 [heads]
        float *ls1 = nullptr, *ls2 = nullptr; // layer scales f32 [d]
        uint16_t* lru_gate_w = nullptr;       // gated LRU: bf16 [blocks][2 bw][bw]
        float *lru_gate_b = nullptr, *lru_lambda = nullptr;
        DLinear reentry_a, reentry_b; // the re-entry projection's halves: on the stream, on the embedding rows
        float *in_conv_mixer = nullptr, *in_conv_mlp = nullptr; // input convolutions f32 [d][taps]
        float* dist_bias = nullptr;   // f32 [dist_rows][heads]: the distance bias by distance (the bucket rule applied on the host)
        uint32_t dist_rows = 0;
        float* head_temp = nullptr;   // f32 [heads]
        DLinear decay_up, gate_up;    // the delta rule's low-rank second factors
    };
    std::vector<Layer> layers;
    float alpha_out = 0.f;
    float* ret_ws = nullptr; // retention in chunks: one state block per (chunk of the pass, head)
    size_t ret_ws_bytes = 0;
    float* lru_ws = nullptr; // the recurrent unit in pieces: local state, decay product and carry per (piece of the pass, channel)
    size_t lru_ws_bytes = 0;
    float* att_ws = nullptr; // partial sums of the key-split attention of decode-sized passes
    size_t att_ws_bytes = 0;
    float* taps = nullptr; // UZU_MODEL_DEBUG_TAPS: f32 [layers][max_rows][d], what each layer handed on in the last pass
    uint32_t tap_rows = 0;
    uint32_t last_logit_rows = 0; // rows of `logits` the last pass produced
};

namespace {

uint32_t state_length(const uzu_hip_model* m, const uzu_hip_state* st) { return m->bound == st ? m->context_length : st->context_length; }
void state_set_length(uzu_hip_model* m, uzu_hip_state* st, uint32_t len) {
    st->context_length = len;
    if (m->bound == st) m->context_length = len;
}

// `span` (optional): the device-side span of a one-sequence decode step moves on with the context, so the next step needs nothing from the host
__global__ void s32_commit_kernel(uint32_t* ctx_len, uint32_t* tokens, const uint32_t* out_token, uint32_t* sampled, uint32_t count, uint32_t has_token, k::SeqSpan* span) {
    const uint32_t len = *ctx_len;
    if (has_token) {
        const uint32_t t = *out_token;
        sampled[len + count - 1] = t;
        tokens[0] = t;
    }
    *ctx_len = len + count;
    if (span) span->start = len + count;
}

uzu_status need_f32(uzu_hip_model* m, size_t floats, float** out) {
    void* p = nullptr;
    UZU_PROPAGATE(dev_alloc(m, floats * 4, &p)); // scratch: every row a kernel reads was written earlier in the same pass (poison mode hands it out as NaNs)
    *out = (float*)p;
    return UZU_OK;
}

struct PassSeq {
    uzu_hip_state* st;
    uint32_t count, start;
};

k::LinearF32Params lin(const Stream32& S, const DLinear& L, const float* x, float* y, uint32_t rows) {
    k::LinearF32Params p{};
    p.x = x, p.w = (const uint16_t*)L.w, p.bias = (const uint16_t*)L.out_biases, p.y = y;
    p.rows = rows, p.n = L.n, p.k = L.k, p.ldx = L.k, p.ldy = L.n, p.ldr = L.n, p.batch = 1;
    p.bf16_products = S.full_f32 ? 0u : 1u;
    return p;
}

void run_linear(Enc& e, const k::LinearF32Params& p) {
    const char* variant = "linear_f32";
    e.begin();
    const uzu_status r = k::linear_f32(e.s, p, &variant);
    e.run(r, variant, k::linear_f32_bytes(p));
}

// a norm of the stream's rows by its kind; row_index: a gather of the rows (the read-out)
void run_norm(Enc& e, const DNorm& N, uint32_t kind, float alpha, const float* x, float* out, uint32_t rows, uint32_t d, const uint32_t* row_index) {
    hipStream_t s = e.s;
    if (kind == UZU_NORM_RMS_SCALAR) {
        RUN("rms_norm_rows", (size_t)rows * d * 8, k::rms_norm_rows(s, x, out, nullptr, alpha, N.eps, row_index, rows, d));
        return;
    }
    if (kind == UZU_NORM_STATISTICS) { // RMS with a weight vector (+ offset)
        RUN("rms_norm_rows", (size_t)rows * d * 8, k::rms_norm_rows(s, x, out, N.scales, 1.0f, N.eps, row_index, rows, d, N.offset, N.groups));
        return;
    }
    k::DynTanhParams np{};
    np.x = x, np.out = out, np.scales = N.scales, np.biases = N.biases, np.alpha = alpha, np.row_index = row_index, np.rows = rows, np.d = d;
    RUN("dyn_tanh_norm", (size_t)rows * d * 8, k::dyn_tanh_norm(s, np));
}

k::ExpertAct expert_act(const uzu_moe_desc& M) {
    k::ExpertAct a;
    a.alpha = M.silu_alpha != 0.0f ? M.silu_alpha : 1.0f;
    if (M.gate_clip_min != 0.0f || M.gate_clip_max != 0.0f) a.gate_min = M.gate_clip_min, a.gate_max = M.gate_clip_max; // (all zero: a description that never set them)
    if (M.up_clip_min != 0.0f || M.up_clip_max != 0.0f) a.up_min = M.up_clip_min, a.up_max = M.up_clip_max;
    a.up_offset = M.up_offset;
    return a;
}

// The tables of a pass over `seqs`: spans, row -> sequence, per-layer cache / shift-state pointers, the rows whose logits are wanted.
uzu_status s32_upload_tables(uzu_hip_model* m, const std::vector<PassSeq>& seqs, const std::vector<uint32_t>& out_rows) {
    Stream32& S = *m->s32;
    hipStream_t s = m->ctx->stream;
    const uint32_t nl = m->d.num_layers, nseq = (uint32_t)seqs.size();
    UZU_REQUIRE(nseq > 0 && nseq <= S.max_seqs, "engine: a pass of %u sequences (the model carries at most %u)", nseq, S.max_seqs);
    std::vector<k::SeqSpan> spans(nseq);
    std::vector<uint32_t> row_seq;
    uint32_t rows = 0;
    for (uint32_t i = 0; i < nseq; ++i) {
        spans[i] = {rows, seqs[i].count, seqs[i].start};
        UZU_REQUIRE(seqs[i].count > 0 && seqs[i].start + seqs[i].count <= m->max_positions, "engine: sequence %u leaves its state's capacity", i);
        for (uint32_t j = 0; j < seqs[i].count; ++j) row_seq.push_back(i);
        rows += seqs[i].count;
    }
    UZU_REQUIRE(rows <= S.max_rows, "engine: a pass of %u rows (at most %u)", rows, S.max_rows);
    std::vector<void*> cache_ptrs((size_t)nl * S.max_seqs, nullptr), cache2_ptrs((size_t)nl * S.max_seqs, nullptr);
    std::vector<float*> shift_ptrs((size_t)nl * S.max_seqs, nullptr), pair_state((size_t)nl * S.max_seqs, nullptr), pair_conv((size_t)nl * S.max_seqs, nullptr);
    std::vector<float*> inconv((size_t)nl * S.max_seqs, nullptr);
    std::vector<uint32_t*> prev_tok(S.max_seqs, nullptr);
    for (uint32_t i = 0; i < nseq; ++i) prev_tok[i] = seqs[i].st->prev_token;
    for (uint32_t l = 0; l < nl; ++l) {
        const uzu_layer_desc& h = m->layers[l].d;
        const uint32_t src = h.is_kv_sharing ? h.kv_source_layer_index : l;
        for (uint32_t i = 0; i < nseq; ++i) {
            const uzu_hip_state::Layer& own = seqs[i].st->layers[src];
            const size_t at = (size_t)l * S.max_seqs + i;
            if (h.mixer_kind == UZU_MIXER_ATTENTION) cache_ptrs[at] = own.cache_k, cache2_ptrs[at] = own.cache_v;
            else if (h.mixer_kind == UZU_MIXER_GATED_LRU) cache_ptrs[at] = own.ssm_state, cache2_ptrs[at] = own.conv_state;
            else if (h.mixer_kind == UZU_MIXER_RETENTION) cache_ptrs[at] = own.ret_state;
            else cache_ptrs[at] = own.latent;
            shift_ptrs[at] = seqs[i].st->layers[l].shift_prev;
            inconv[at] = seqs[i].st->layers[l].in_conv;
            if (h.pair_mixer) pair_state[at] = seqs[i].st->layers[l].ssm_state, pair_conv[at] = seqs[i].st->layers[l].conv_state;
        }
    }
    // (pageable sources: the copies have left the host buffers when the calls return)
    HIPCHK(hipMemcpyAsync(S.d_spans, spans.data(), spans.size() * sizeof(k::SeqSpan), hipMemcpyHostToDevice, s));
    HIPCHK(hipMemcpyAsync(S.d_row_seq, row_seq.data(), row_seq.size() * 4, hipMemcpyHostToDevice, s));
    HIPCHK(hipMemcpyAsync(S.d_cache_ptrs, cache_ptrs.data(), cache_ptrs.size() * sizeof(void*), hipMemcpyHostToDevice, s));
    HIPCHK(hipMemcpyAsync(S.d_cache2_ptrs, cache2_ptrs.data(), cache2_ptrs.size() * sizeof(void*), hipMemcpyHostToDevice, s));
    HIPCHK(hipMemcpyAsync(S.d_shift_ptrs, shift_ptrs.data(), shift_ptrs.size() * sizeof(float*), hipMemcpyHostToDevice, s));
    if (S.d_pair_state_ptrs) {
        HIPCHK(hipMemcpyAsync(S.d_pair_state_ptrs, pair_state.data(), pair_state.size() * sizeof(float*), hipMemcpyHostToDevice, s));
        HIPCHK(hipMemcpyAsync(S.d_pair_conv_ptrs, pair_conv.data(), pair_conv.size() * sizeof(float*), hipMemcpyHostToDevice, s));
    }
    if (S.d_inconv_ptrs) HIPCHK(hipMemcpyAsync(S.d_inconv_ptrs, inconv.data(), inconv.size() * sizeof(float*), hipMemcpyHostToDevice, s));
    if (S.d_prev_tok_ptrs) HIPCHK(hipMemcpyAsync(S.d_prev_tok_ptrs, prev_tok.data(), prev_tok.size() * sizeof(uint32_t*), hipMemcpyHostToDevice, s));
    if (!out_rows.empty()) HIPCHK(hipMemcpyAsync(S.d_out_rows, out_rows.data(), out_rows.size() * 4, hipMemcpyHostToDevice, s));
    return UZU_OK;
}

// The launches of one pass (tables uploaded before): rows = sum of the sequences' counts (<= max_rows), token ids on the device, row-major in sequence order;
// n_out rows (S.d_out_rows) get logits in S.logits [n_out][vocab] f32.  Nothing here depends on the sequences' positions -- the kernels read them from the
// device-side spans -- so a one-token step can be captured once and replayed.  Does not move the sequences' context lengths.
uzu_status s32_encode(uzu_hip_model* m, const std::vector<uint32_t>& counts, const uint32_t* d_tokens, uint32_t n_out) {
    Stream32& S = *m->s32;
    hipStream_t s = m->ctx->stream; // (the stream the next launch goes to: a pair's first mixer switches it to S.side and back)
    const hipStream_t main_stream = s;
    Enc e{m, s};
    e.prof = (std::vector<ProfEntry>*)m->prof_sink;
    m->launches = 0;
    const uint32_t d = m->d.model_dim, nl = m->d.num_layers, nseq = (uint32_t)counts.size();
    uint32_t rows = 0;
    for (uint32_t c : counts) rows += c;
    const size_t slot_stride = (size_t)S.max_rows * d;
    const uint32_t bf = S.full_f32 ? 0u : 1u;
    uint32_t max_count = 0;
    for (uint32_t c : counts) max_count = std::max(max_count, c);
    if (S.pair_table) { // + the hashed (previous token, token) row; two launches: the rows, then the sequences' new previous tokens
        k::EmbedPairParams ep{};
        ep.tokens = d_tokens, ep.table = (const uint16_t*)m->embedding.w, ep.pair_table = S.pair_table, ep.out = S.slots, ep.rows = rows, ep.vocab = m->d.vocab_size, ep.d = d;
        ep.scale = m->d.input_scale, ep.buckets = m->d.bigram_buckets, ep.mul_prev = m->d.bigram_mul_prev, ep.mul_cur = m->d.bigram_mul_cur, ep.spans = S.d_spans;
        ep.row_seq = S.d_row_seq, ep.prev = S.d_prev_tok_ptrs, ep.nseq = nseq, ep.max_count = max_count;
        RUN("embed_pair_rows_f32", (size_t)rows * d * 8, k::embed_pair_rows_f32(s, ep));
        if (max_count > 1) ++m->launches;
    } else {
        RUN("embed_rows_f32", (size_t)rows * d * 6, k::embed_rows_f32(s, d_tokens, (const uint16_t*)m->embedding.w, S.slots, rows, m->d.vocab_size, d, m->d.input_scale));
    }
    const float* cur = S.slots; // what the layer about to run reads: X_0, then the depth mix of the layer before
    // A sublayer's result joins the stream behind its post norm; the same launch leaves the norm of the new rows for the sublayer that follows where that is an
    // RMS norm with a weight vector (`next`), so that norm needs no launch of its own.
    auto add_normed = [&](const float* y, const float* residual, float* out, const DNorm& N, const float* layer_scale, const DNorm* next) {
        RUN("rms_norm_add_rows", (size_t)rows * d * (next ? 16 : 12),
            k::rms_norm_add_rows(s, y, residual, out, N.scales, N.offset, layer_scale, N.eps, rows, d, next ? S.normed : nullptr, next ? next->scales : nullptr,
                                 next ? next->offset : 0.0f, next ? next->eps : 0.0f, N.groups));
    };
    // what a sublayer without a pre norm reads: the stream rows themselves, or (with an input convolution) rows + conv(rows) in S.normed; `which` = 0 the mixer's
    // window of the layer's state, 1 the MLP's.  The window is replaced right away: `x` still holds the pass's inputs here.
    auto conv_input = [&](uint32_t l, const float* x, const float* w, uint32_t taps, uint32_t which) -> const float* {
        if (!w) return x;
        k::CausalConvParams cp{};
        cp.x = x, cp.ldx = d, cp.out = S.normed, cp.ldo = d, cp.w = w, cp.channels = d, cp.taps = taps, cp.add_input = 1;
        cp.states = S.d_inconv_ptrs + (size_t)l * S.max_seqs, cp.state_offset = (size_t)which * (taps - 1) * d, cp.spans = S.d_spans, cp.row_seq = S.d_row_seq, cp.nseq = nseq, cp.rows = rows;
        cp.max_count = max_count;
        RUN("causal_conv_rows", (size_t)rows * d * 4 * (taps + 1), k::causal_conv_rows(s, cp));
        if (taps > 1 && max_count > 1) RUN("causal_conv_commit", (size_t)nseq * d * 8 * (taps - 1), k::causal_conv_commit(s, cp));
        return S.normed;
    };
    bool normed_ready = false; // S.normed already holds this run's pre-mixer norm (left by the run before)
    for (uint32_t l = 0; l < nl; ++l) {
        DLayer& L = m->layers[l];
        const Stream32::Layer& X = S.layers[l];
        const uzu_layer_desc& h = L.d;
        float* slot = S.slots + (size_t)(l + 1) * slot_stride; // X_(l+1): the layer's own result
        void* const* caches = S.d_cache_ptrs + (size_t)l * S.max_seqs;
        if (X.reentry_a.w) { // x <- W [x ; x0]: the two halves of W on the stream and on the embedding rows, summed
            run_linear(e, lin(S, X.reentry_a, cur, S.xin, rows));
            k::LinearF32Params b = lin(S, X.reentry_b, S.slots, S.xin, rows);
            b.residual = S.xin, b.ldr = d;
            run_linear(e, b);
            cur = S.xin;
        }
        // which launch ends this run, and whether it can leave the next run's pre-mixer norm
        const DNorm* next_pre = nullptr;
        if (l + 1 < nl && !X.depth_weights && !S.layers[l + 1].reentry_a.w && m->layers[l + 1].pre_mixer.present && m->layers[l + 1].d.pre_mixer_norm.kind == UZU_NORM_STATISTICS &&
            m->layers[l + 1].pre_mixer.groups <= 1)
            next_pre = &m->layers[l + 1].pre_mixer;
        const bool pre_mlp_fused = !h.no_mlp && !h.parallel_block && L.post_mixer.present && L.post_mixer.groups <= 1 && L.pre_mlp.present && h.pre_mlp_norm.kind == UZU_NORM_STATISTICS &&
                                   L.pre_mlp.groups <= 1;
        if (next_pre && ((L.post_mixer.present && L.post_mixer.groups > 1) || (L.post_mlp.present && L.post_mlp.groups > 1) || (h.has_ple && L.ple_norm.groups > 1))) next_pre = nullptr;
        const bool have_normed = normed_ready;
        normed_ready = false;
        const float* mix_in = S.normed; // the rows the mixer reads
        if (have_normed) {
        } else if (!L.pre_mixer.present) {
            mix_in = conv_input(l, cur, X.in_conv_mixer, h.input_conv_taps, 0);
        } else if (h.pre_mixer_norm.kind != UZU_NORM_DYNAMIC_TANH) {
            run_norm(e, L.pre_mixer, h.pre_mixer_norm.kind, X.alpha1, cur, S.normed, rows, d, nullptr);
        } else { // dynamic-tanh norm + token shift
            k::DynTanhParams np{};
            np.x = cur, np.out = S.normed, np.scales = L.pre_mixer.scales, np.biases = L.pre_mixer.biases, np.alpha = X.alpha1, np.shift = X.token_shift;
            np.spans = S.d_spans, np.row_seq = S.d_row_seq, np.prev = S.d_shift_ptrs + (size_t)l * S.max_seqs, np.rows = rows, np.d = d;
            RUN("dyn_tanh_norm+shift", (size_t)rows * d * 8, k::dyn_tanh_norm(s, np));
        }
        const uint32_t H = h.num_heads, hd = h.head_dim, vd = h.value_head_dim, rank = h.latent_rank;
        // prompt-sized pass over a pair of mixers: the first one's projection, rotation / append and attention core go to the side stream (they touch S.q, S.attn and
        // the caches; the second mixer touches its own rows); not while a launch is being timed or captured
        bool forked = false;
        if (h.pair_mixer && S.side && rows >= 256 && !e.prof) {
            hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(main_stream, &cap) == hipSuccess && cap == hipStreamCaptureStatusNone && hipEventRecord(S.side_fork, main_stream) == hipSuccess &&
                hipStreamWaitEvent(S.side, S.side_fork, 0) == hipSuccess)
                forked = true, s = S.side, e.s = S.side;
        }
        run_linear(e, lin(S, L.qkv, mix_in, S.q, rows)); // the packed projection of the mixer (queries first)
        if (h.mixer_kind == UZU_MIXER_GATED_LRU) {
            const uint32_t w = h.lru_width, bw = w / h.lru_blocks;
            k::GatedLruParams gp{};
            gp.branches = S.q, gp.ld = L.qkv.n, gp.x_col = w, gp.u = S.lru_u, gp.gates = S.lru_g, gp.out = S.attn, gp.conv_w = L.conv_w, gp.conv_b = L.conv_b, gp.gate_b = X.lru_gate_b;
            gp.lambda = X.lru_lambda, gp.rate = h.lru_decay_rate, gp.states = (float* const*)caches, gp.conv_states = (float* const*)(S.d_cache2_ptrs + (size_t)l * S.max_seqs);
            gp.spans = S.d_spans, gp.row_seq = S.d_row_seq, gp.nseq = nseq, gp.rows = rows, gp.width = w, gp.blocks = h.lru_blocks, gp.taps = h.dn_kernel_size, gp.max_count = max_count;
            for (uint32_t i = 0; i < nseq; ++i) gp.pieces += (counts[i] + 31) / 32;
            gp.piece_ws = S.lru_ws, gp.piece_ws_bytes = S.lru_ws_bytes;
            RUN("lru_conv", (size_t)rows * w * 4 * (gp.taps + 1), k::lru_conv(s, gp));
            {   // both gates of every block in one batched product; what enters the recurrence is never rounded: true f32 products in both precisions
                k::LinearF32Params p{};
                p.x = S.lru_u, p.w = X.lru_gate_w, p.y = S.lru_g, p.rows = rows, p.n = 2 * bw, p.k = bw, p.ldx = w, p.ldy = 2 * w, p.batch = h.lru_blocks;
                p.x_batch = bw, p.w_batch = (size_t)2 * bw * bw, p.y_batch = 2 * bw, p.bf16_products = 0;
                run_linear(e, p);
            }
            RUN("lru_scan", (size_t)rows * w * 20, k::lru_scan(s, gp));
        } else if (h.mixer_kind == UZU_MIXER_ATTENTION) {
            const uint32_t G = h.num_groups, ldq = L.qkv.n;
            void* const* vcaches = S.d_cache2_ptrs + (size_t)l * S.max_seqs;
            k::RopeAppendParams rp{};
            rp.qkv = S.q, rp.ld = ldq, rp.k_col = H * hd, rp.v_col = h.values_are_keys ? H * hd : H * hd + G * hd, rp.heads = H, rp.kv_heads = h.is_kv_sharing ? 0u : G, rp.dim = hd, rp.vdim = vd;
            rp.rope_dim = h.use_rope ? L.rope_dim : 0u, rp.cosines = L.rope_cos, rp.sines = L.rope_sin, rp.key_scale = h.key_scale != 0.0f ? h.key_scale : 1.0f;
            rp.norm_whole = h.qk_norm_whole, rp.interleaved = h.rope_interleaved;
            rp.key_caches = caches, rp.value_caches = vcaches, rp.cache_bf16 = bf, rp.spans = S.d_spans, rp.row_seq = S.d_row_seq, rp.rows = rows;
            rp.q_norm = L.qn.present ? L.qn.scales : nullptr, rp.k_norm = L.kn.present && !h.is_kv_sharing ? L.kn.scales : nullptr, rp.norm_eps = L.qn.present ? L.qn.eps : L.kn.eps;
            RUN("rope_append", (size_t)rows * ldq * 8, k::rope_append(s, rp));
            k::WindowAttentionParams ap{};
            ap.q = S.q, ap.ldq = ldq, ap.out = S.attn, ap.key_caches = caches, ap.value_caches = vcaches, ap.cache_bf16 = bf, ap.sinks = X.sinks, ap.spans = S.d_spans;
            ap.row_seq = S.d_row_seq, ap.rows = rows, ap.heads = H, ap.kv_heads = G, ap.dim = hd, ap.vdim = vd, ap.window = h.sliding_window_size;
            ap.scale = h.attention_scale != 0.0f ? h.attention_scale : 1.0f / sqrtf((float)hd), ap.soft_cap = h.score_soft_cap, ap.nseq = nseq;
            ap.chunk = h.attention_chunk_size, ap.head_scale = X.head_temp, ap.dist_bias = X.dist_bias, ap.dist_rows = X.dist_rows;
            if (h.has_gate) ap.gate = S.q + H * hd + (h.is_kv_sharing ? 0u : G * hd + (h.values_are_keys ? 0u : G * vd)), ap.ldgate = ldq; // the gate rows stand behind the values
            for (uint32_t i = 0; i < nseq; ++i) ap.tiles += (counts[i] * (H / G) + 127) / 128;
            // decode-sized passes: spread a tile's key blocks over workgroups (a constant of the layer, so that a captured step stays valid as the context grows)
            uint32_t keys = h.sliding_window_size ? h.sliding_window_size : m->d.max_context_length;
            if (h.attention_chunk_size) keys = std::min(keys, h.attention_chunk_size);
            if (rows <= 4 * S.max_seqs && rows * H <= 4096) ap.splits = std::min<uint32_t>(16, (keys + 31) / 32), ap.split_ws = S.att_ws, ap.split_ws_bytes = S.att_ws_bytes;
            RUN("window_attention", (size_t)rows * H * (hd + vd) * 4, k::window_attention(s, ap));
        } else if (h.mixer_kind == UZU_MIXER_RETENTION) {
            const uint32_t ldq = L.qkv.n; // queries | keys | values | gate
            k::RopeAppendParams rp{};
            rp.qkv = S.q, rp.ld = ldq, rp.k_col = H * hd, rp.v_col = 2 * H * hd, rp.heads = H, rp.kv_heads = H, rp.dim = hd, rp.vdim = vd;
            rp.rope_dim = h.use_rope ? L.rope_dim : 0u, rp.cosines = L.rope_cos, rp.sines = L.rope_sin, rp.key_scale = h.key_scale != 0.0f ? h.key_scale : 1.0f;
            rp.spans = S.d_spans, rp.row_seq = S.d_row_seq, rp.rows = rows;
            RUN("rope_append", (size_t)rows * 2 * H * hd * 8, k::rope_append(s, rp));
            k::RetentionParams tp{};
            tp.qkv = S.q, tp.ld = ldq, tp.q_col = 0, tp.k_col = H * hd, tp.v_col = 2 * H * hd, tp.out = S.attn, tp.states = (float* const*)caches, tp.decay = X.decay;
            tp.spans = S.d_spans, tp.nseq = nseq, tp.rows = rows, tp.heads = H, tp.dim = hd, tp.vdim = vd;
            for (uint32_t i = 0; i < nseq; ++i) tp.chunks += (counts[i] + 63) / 64;
            tp.chunk_ws = S.ret_ws, tp.chunk_ws_bytes = S.ret_ws_bytes;
            RUN("retention", (size_t)rows * ldq * 4 + (size_t)nseq * H * hd * vd * 8, k::retention(s, tp));
            RUN("head_rms_gate", (size_t)rows * H * vd * 12, k::head_rms_gate(s, S.attn, S.q + 2 * H * hd + H * vd, ldq, h.head_norm_epsilon, rows, H, vd));
        } else {
        // rd: the rotated key part every head shares; the cache row is [latent | rotated part] (kw wide), a query head [plain | rotated] (qw wide)
        const uint32_t rd = h.latent_rope_dim, kw = rank + rd, qw = hd + rd, ldq = L.qkv.n;
        if (!h.is_kv_sharing && !h.latent_packed) run_linear(e, lin(S, L.lat_down, mix_in, S.ckv, rows));
        if (!rd && !h.latent_packed) {
            if (!h.is_kv_sharing)
                RUN("latent_norm_append", (size_t)rows * rank * 6,
                    k::latent_norm_append(s, S.ckv, L.lat_norm.scales, L.lat_norm.eps, caches, bf, S.d_spans, S.d_row_seq, rows, rank));
        } else {
            k::LatentRopeAppendParams lp{};
            lp.x = h.latent_packed ? S.q : S.ckv, lp.ldx = h.latent_packed ? ldq : L.lat_down.n, lp.c_col = h.latent_packed ? H * qw : 0, lp.rank = rank, lp.rope_dim = rd;
            lp.scales = L.lat_norm.scales, lp.eps = L.lat_norm.eps, lp.caches = h.is_kv_sharing ? nullptr : caches, lp.cache_bf16 = bf, lp.heads = H, lp.q_width = qw;
            lp.qlat = rd ? S.qlat : nullptr, lp.cosines = L.rope_cos, lp.sines = L.rope_sin, lp.interleaved = h.rope_interleaved, lp.spans = S.d_spans, lp.row_seq = S.d_row_seq, lp.rows = rows;
            if (h.latent_packed) { // the rotated query parts are read from the packed rows; a separate down projection leaves them in S.q as well
                RUN("latent_rope_append", (size_t)rows * (kw * 6 + H * rd * 8), k::latent_rope_append(s, lp));
            } else {
                k::LatentRopeAppendParams cp = lp; // cache rows from the down projection's rows, query parts from the query rows
                cp.qlat = nullptr;
                if (!h.is_kv_sharing) RUN("latent_rope_append", (size_t)rows * kw * 6, k::latent_rope_append(s, cp));
                if (rd) {
                    k::LatentRopeAppendParams qp = lp;
                    qp.x = S.q, qp.ldx = ldq, qp.c_col = 0, qp.caches = nullptr;
                    RUN("latent_rope_append", (size_t)rows * H * rd * 8, k::latent_rope_append(s, qp));
                }
            }
        }
        {   // the head's key projection folded into the query: qlat[r, h, :rank] = W_up_k[h]^T q[r, h, :hd]
            k::LinearF32Params p{};
            p.x = S.q, p.w = X.up_keys_t, p.y = S.qlat, p.rows = rows, p.n = rank, p.k = hd, p.ldx = ldq, p.ldy = H * kw, p.batch = H;
            p.x_batch = qw, p.w_batch = (size_t)rank * hd, p.y_batch = kw, p.bf16_products = bf;
            run_linear(e, p);
        }
        {
            k::LatentAttentionParams ap{};
            ap.qlat = S.qlat, ap.out = S.ctx, ap.caches = caches, ap.cache_bf16 = bf, ap.sinks = X.sinks, ap.spans = S.d_spans, ap.row_seq = S.d_row_seq;
            ap.rows = rows, ap.heads = H, ap.rank = kw, ap.window = h.sliding_window_size;
            if (rd && rank % 4 == 0) ap.value_rank = rank; // the rotated columns score and carry no value
            ap.scale = h.attention_scale != 0.0f ? h.attention_scale : 1.0f / sqrtf((float)hd);
            ap.nseq = nseq;
            // decode-sized passes: spread a tile's key blocks over workgroups (a constant of the layer, so that a captured step stays valid as the context grows)
            const uint32_t keys = h.sliding_window_size ? h.sliding_window_size : m->d.max_context_length;
            if (rows <= 4 * S.max_seqs && rows * H <= 4096) ap.splits = std::min<uint32_t>(32, (keys + 31) / 32), ap.split_ws = S.att_ws, ap.split_ws_bytes = S.att_ws_bytes;
            for (uint32_t i = 0; i < nseq; ++i) ap.tiles += (counts[i] * H + 127) / 128;
            RUN("latent_attention", (size_t)rows * H * kw * 8, k::latent_attention(s, ap));
        }
        {   // the head's value projection on the weighted latent sum (the rotated columns of the sum are not read): attn[r, h, :] = W_up_v[h] ctx[r, h, :rank],
            // times the head's sigmoid gate where the layer has one
            k::LinearF32Params p{};
            p.x = S.ctx, p.w = (const uint16_t*)L.lat_up_v.w, p.y = S.attn, p.rows = rows, p.n = vd, p.k = rank, p.ldx = H * kw, p.ldy = H * vd, p.batch = H;
            p.x_batch = kw, p.w_batch = (size_t)vd * rank, p.y_batch = vd, p.bf16_products = bf;
            if (h.has_gate) p.gate = S.q + H * qw + (h.latent_packed ? kw : 0), p.ldgate = ldq;
            run_linear(e, p);
        }
        } // latent attention
        if (forked) { // the first mixer is on its way: the main stream goes on with the second and meets it in front of the out projections
            if (hipEventRecord(S.side_join, S.side) != hipSuccess && e.st == UZU_OK) set_error("engine: recording the side stream's join failed"), e.st = UZU_ERR_HIP;
            s = main_stream, e.s = main_stream;
        }
        if (h.pair_mixer) { // the second mixer beside the first: a delta rule with a decay per head and key channel, reading the same rows
            const uint32_t Hd = h.dn_num_heads, Gd = h.dn_num_groups, dk = h.dn_head_dim, dv = h.dn_value_head_dim, taps = h.dn_kernel_size, ldi = L.in_proj.n;
            const uint32_t conv_dim = 2 * Gd * dk + Hd * dv, b_col = conv_dim, a_col = b_col + Hd, g_col = a_col + h.dn_decay_rank;
            run_linear(e, lin(S, L.in_proj, mix_in, S.dn_in, rows)); // q | k | v | beta | decay down | gate down
            k::CausalConvParams cp{};
            cp.x = S.dn_in, cp.ldx = ldi, cp.out = S.dn_cv, cp.ldo = conv_dim, cp.w = L.conv_w, cp.bias = L.conv_b, cp.channels = conv_dim, cp.taps = taps, cp.act = 1;
            cp.states = S.d_pair_conv_ptrs + (size_t)l * S.max_seqs, cp.spans = S.d_spans, cp.row_seq = S.d_row_seq, cp.nseq = nseq, cp.rows = rows, cp.max_count = max_count;
            RUN("causal_conv_rows", (size_t)rows * conv_dim * 4 * (taps + 1), k::causal_conv_rows(s, cp));
            if (taps > 1 && max_count > 1) RUN("causal_conv_commit", (size_t)nseq * conv_dim * 8 * (taps - 1), k::causal_conv_commit(s, cp));
            {   // the low-rank factors' second halves: what enters the recurrence is never rounded, true f32 products in both precisions
                k::LinearF32Params up = lin(S, X.decay_up, S.dn_in + a_col, S.dn_decay, rows);
                up.ldx = ldi, up.bf16_products = 0;
                run_linear(e, up);
                k::LinearF32Params gu = lin(S, X.gate_up, S.dn_in + g_col, S.dn_gate, rows);
                gu.ldx = ldi, gu.bf16_products = 0;
                run_linear(e, gu);
            }
            k::ChannelDeltaParams dp{};
            dp.qkv = S.dn_cv, dp.ld = conv_dim, dp.q_col = 0, dp.k_col = Gd * dk, dp.v_col = 2 * Gd * dk, dp.decay = S.dn_decay, dp.beta = S.dn_in + b_col, dp.ldbeta = ldi;
            dp.a_log = L.a_log, dp.dt_bias = L.dt_bias, dp.unit_eps = 1e-6f, dp.out = S.dn_o, dp.states = S.d_pair_state_ptrs + (size_t)l * S.max_seqs, dp.spans = S.d_spans;
            dp.nseq = nseq, dp.rows = rows, dp.heads = Hd, dp.groups = Gd, dp.dim = dk, dp.vdim = dv;
            RUN("channel_delta_prep", (size_t)rows * (conv_dim + Hd * dk) * 8, k::channel_delta_prep(s, dp));
            RUN("channel_delta", (size_t)rows * (conv_dim + Hd * (dk + dv)) * 4 + (size_t)nseq * Hd * dk * dv * 8, k::channel_delta(s, dp));
            k::HeadNormGateParams np{};
            np.x = S.dn_o, np.ldx = Hd * dv, np.weight = L.dn_norm, np.gate = S.dn_gate, np.ldgate = Hd * dv, np.gate_sigmoid = 1, np.eps = h.dn_norm_epsilon, np.rows = rows, np.heads = Hd, np.width = dv;
            RUN("head_norm_gate_rows", (size_t)rows * Hd * dv * 12, k::head_norm_gate_rows(s, np));
            if (forked && hipStreamWaitEvent(main_stream, S.side_join, 0) != hipSuccess && e.st == UZU_OK) set_error("engine: waiting for the side stream failed"), e.st = UZU_ERR_HIP;
            // tmp = scale_main * out(main) + scale_second * out(second)
            // (a scale of exactly zero takes its mixer's product out; both zero: a product that vanishes)
            const bool main_on = h.pair_scale_main != 0.0f, second_on = h.pair_scale_second != 0.0f;
            if (main_on || !second_on) {
                k::LinearF32Params o1 = lin(S, L.out, S.attn, S.tmp, rows);
                o1.y_scale = main_on ? h.pair_scale_main : 1.0e-37f;
                run_linear(e, o1);
            }
            if (second_on) {
                k::LinearF32Params o2 = lin(S, L.out_proj, S.dn_o, S.tmp, rows);
                o2.y_scale = h.pair_scale_second;
                if (main_on) o2.residual = S.tmp, o2.ldr = d;
                run_linear(e, o2);
            }
            add_normed(S.tmp, cur, slot, L.post_mixer, X.ls1, nullptr);
        } else if (L.post_mixer.present) { // the mixer's result joins the stream behind its own norm (and the layer scale)
            run_linear(e, lin(S, L.out, S.attn, S.tmp, rows));
            add_normed(S.tmp, cur, slot, L.post_mixer, X.ls1, pre_mlp_fused ? &L.pre_mlp : (h.no_mlp && !h.has_ple) ? next_pre : nullptr);
            normed_ready = h.no_mlp && !h.has_ple && next_pre;
        } else { // X_(l+1) = input + out projection
            k::LinearF32Params p = lin(S, L.out, S.attn, slot, rows);
            p.residual = cur, p.ldr = d;
            run_linear(e, p);
        }
        if (!h.no_mlp) {
            // a parallel block's MLP reads the rows the mixer read (still in S.normed) and adds to the same sum; otherwise the MLP has its own norm of the sum so far
            const float* mlp_in = h.parallel_block ? mix_in : S.normed;
            if (!h.parallel_block && !L.pre_mlp.present) mlp_in = conv_input(l, slot, X.in_conv_mlp, h.input_conv_taps, 1); // no pre norm: the stream itself (+ its convolution)
            else if (!h.parallel_block && !pre_mlp_fused) run_norm(e, L.pre_mlp, h.pre_mlp_norm.kind, X.alpha2, slot, S.normed, rows, d, nullptr);
            if (h.mlp_kind == UZU_MLP_MOE) {
                const uzu_moe_desc& M = h.moe;
                const uint32_t E = M.num_routed_experts, top = M.num_active_experts, ff = M.expert_hidden_dim;
                const k::ExpertAct act = expert_act(M);
                if (M.routing == UZU_MOE_ROUTE_SCORES) {
                    RUN("moe_route_scores", (size_t)(E + M.num_identity_experts) * d * 2,
                        k::moe_route_scores(s, mlp_in, L.moe.router_weights, X.selection_bias, S.moe_ids, S.moe_w, rows, d, E + M.num_identity_experts, top));
                } else {
                    RUN("moe_route_topk", (size_t)E * d * 2, k::moe_route_topk(s, mlp_in, L.moe.router_weights, L.moe.router_biases, S.moe_ids, S.moe_w, rows, d, E, top, M.router_renorm));
                }
                k::MoeGroupedParams gp{};
                gp.x = mlp_in, gp.ids = S.moe_ids, gp.weights = S.moe_w, gp.w13 = L.moe.w13, gp.w2 = L.moe.w2, gp.residual = slot, gp.y = slot, gp.y1 = S.moe_y1, gp.hidden = S.hid;
                gp.y2 = S.moe_y2, gp.perm = S.moe_perm, gp.slot_pos = S.moe_slot_pos, gp.offsets = S.moe_offsets, gp.cursor = S.moe_cursor;
                gp.rows = rows, gp.d = d, gp.ff = ff, gp.routed = E, gp.top = top, gp.act = act;
                if (bf && k::moe_experts_grouped_supported(gp)) { // prefill-sized: buckets per expert through the matrix-core linear
                    RUN("moe_experts_grouped", (size_t)E * 3 * ff * d * 2 + (size_t)rows * top * (3 * ff + 2 * d) * 4, k::moe_experts_grouped(s, gp));
                } else {
                    RUN("moe_experts_gate_up", (size_t)rows * top * 2 * ff * d * 2, k::moe_experts_gate_up(s, mlp_in, S.moe_ids, L.moe.w13, S.hid, rows, d, ff, E, top, bf, act));
                    RUN("moe_experts_down_combine", (size_t)rows * top * ff * d * 2,
                        k::moe_experts_down_combine(s, S.hid, mlp_in, S.moe_ids, S.moe_w, L.moe.w2, slot, slot, rows, d, ff, E, top, bf));
                }
            } else {
                if (h.mlp_plain) {
                    k::LinearF32Params up = lin(S, L.up, mlp_in, S.hid, rows);
                    up.act = 1;
                    run_linear(e, up);
                } else { // gated: [up ; gate] rows of one projection, then the clamped gate product
                    run_linear(e, lin(S, L.up, mlp_in, S.y1, rows));
                    k::ExpertAct ga = expert_act(h.moe);
                    ga.gelu = h.activation == UZU_ACT_GELU_APPROX ? 1u : 0u;
                    RUN("gated_act_rows", (size_t)rows * h.hidden_dim * 12, k::gated_act_rows(s, S.y1, S.hid, rows, h.hidden_dim, ga));
                }
                if (L.post_mlp.present) {
                    run_linear(e, lin(S, L.down, S.hid, S.tmp, rows));
                    add_normed(S.tmp, slot, slot, L.post_mlp, X.ls2, h.has_ple ? nullptr : next_pre);
                    normed_ready = !h.has_ple && next_pre;
                } else {
                    k::LinearF32Params down = lin(S, L.down, S.hid, slot, rows);
                    down.residual = slot, down.ldr = d;
                    run_linear(e, down);
                }
            }
        }
        if (h.has_ple) { // the per-layer token input: x <- x + norm(projection(gelu(gate x) * the token's slice of the side table))
            k::LinearF32Params g = lin(S, L.ple_gate, slot, S.side_g, rows); // gelu and the token's slice in the product's epilogue
            g.act = 2, g.mul_table = (const uint16_t*)m->ple_token_embedding.w, g.mul_tokens = d_tokens, g.mul_ld = m->ple_token_embedding.k, g.mul_col0 = h.ple_slice * h.ple_dim;
            g.mul_vocab = m->ple_token_embedding.n;
            run_linear(e, g);
            run_linear(e, lin(S, L.ple_projection, S.side_g, S.tmp, rows));
            add_normed(S.tmp, slot, slot, L.ple_norm, nullptr, next_pre);
            normed_ready = next_pre != nullptr;
        }
        if (X.depth_weights) {
            RUN("depth_mix", (size_t)rows * d * 4 * (l + 3), k::depth_mix(s, S.slots, slot_stride, X.depth_weights, h.num_depth_weights, S.xin, rows, d));
            cur = S.xin;
        } else {
            cur = slot;
        }
        if (S.taps) HIPCHK(hipMemcpyAsync(S.taps + (size_t)l * slot_stride, cur, (size_t)rows * d * 4, hipMemcpyDeviceToDevice, s));
    }
    S.tap_rows = rows;
    S.last_logit_rows = 0;
    if (n_out) {
        run_norm(e, m->output_norm, m->d.output_norm.kind, S.alpha_out, cur, S.out_normed, n_out, d, S.d_out_rows);
        k::LinearF32Params head = lin(S, m->d.tied_embeddings ? m->embedding : m->output_embedding, S.out_normed, S.logits, n_out);
        if (m->d.logit_scale != 1.0f) head.y_scale = m->d.logit_scale; // (0 = a description that never set it)
        head.soft_cap = m->d.logit_soft_cap;
        run_linear(e, head);
        S.last_logit_rows = n_out;
    }
    if (e.st != UZU_OK) return e.st;
    const hipError_t herr = hipGetLastError();
    if (herr != hipSuccess) {
        set_error("engine: f32-stream pass launch failed: %s", hipGetErrorString(herr));
        return UZU_ERR_HIP;
    }
    return UZU_OK;
}

uzu_status s32_pass(uzu_hip_model* m, const std::vector<PassSeq>& seqs, const uint32_t* d_tokens, const std::vector<uint32_t>& out_rows) {
    UZU_PROPAGATE(s32_upload_tables(m, seqs, out_rows));
    std::vector<uint32_t> counts;
    for (const PassSeq& q : seqs) counts.push_back(q.count);
    return s32_encode(m, counts, d_tokens, (uint32_t)out_rows.size());
}

uzu_status ensure_logits(uzu_hip_model* m, size_t rows) {
    Stream32& S = *m->s32;
    if (rows <= S.logit_rows) return UZU_OK;
    HIPCHK(hipStreamSynchronize(m->ctx->stream));
    // captured decode steps carry the old block's address: every state's graph goes (it is rebuilt at that state's next decode)
    auto drop = [](hipGraphExec_t& g) {
        if (g) (void)hipGraphExecDestroy(g);
        g = nullptr;
    };
    drop(m->graph_single);
    if (m->state0 && m->state0 != m->bound) drop(m->state0->graph_single);
    for (uzu_hip_state* u : m->user_states)
        if (u != m->bound) drop(u->graph_single);
    if (m->bound) m->bound->graph_single = nullptr;
    if (S.logits) dev_free(m, S.logits);
    S.logits = nullptr, S.logit_rows = 0;
    size_t want = rows < 16 ? 16 : rows;
    void* p = nullptr;
    UZU_PROPAGATE(dev_alloc(m, want * m->d.vocab_size * 4, &p));
    S.logits = (float*)p, S.logit_rows = want;
    return UZU_OK;
}

// sample from row `logit_row` of the last pass's logits into st's control block and advance it by `count`
uzu_status sample_commit(uzu_hip_model* m, uzu_hip_state* st, uint32_t logit_row, uint32_t count, bool sample, k::SeqSpan* span = nullptr) {
    Stream32& S = *m->s32;
    hipStream_t s = m->ctx->stream;
    Enc e{m, s};
    if (sample) {
        const float* row = S.logits + (size_t)logit_row * m->d.vocab_size;
        if (m->sampling.on) { // the seed of the sampled row's position, as in the engine's other models
            RUN("derive_seed", 0, k::derive_seed(s, m->sampling.seed, st->d_ctx_len, count - 1, m->d_seed));
            k::UnifiedSamplingParams sp = m->sampling.p;
            sp.logits = row, sp.dt = UZU_F32, sp.output = st->d_out_token, sp.seeds = m->d_seed, sp.vocab_size = m->d.vocab_size, sp.batch_size = 1;
            RUN("unified_sampling", (size_t)sp.vocab_size * 4, k::unified_sampling(s, sp, m->sampling_scratch));
        } else {
            RUN("argmax", (size_t)m->d.vocab_size * 4, k::argmax(s, row, UZU_F32, st->d_out_token, m->d.vocab_size, 1, m->argmax_scratch));
        }
    }
    if (e.st != UZU_OK) return e.st;
    hipLaunchKernelGGL(s32_commit_kernel, dim3(1), dim3(1), 0, s, st->d_ctx_len, st->d_tokens, st->d_out_token, st->d_sampled, count, sample ? 1u : 0u, span);
    ++m->launches;
    return UZU_OK;
}

} // namespace

// ---------------------------------------------------------------------------------- construction

uzu_status s32_create(uzu_hip_context* ctx, const uzu_model_desc* desc, uint32_t flags, uzu_hip_model** out) {
    const uint32_t d = desc->model_dim, nl = desc->num_layers;
    UZU_REQUIRE(desc->embedding.method == UZU_QUANT_NONE && desc->embedding.weights && desc->embedding.n == desc->vocab_size && desc->embedding.k == d,
                "model_create: an f32-stream design embeds through a full-precision table [vocab, model_dim]");
    UZU_REQUIRE(desc->tied_embeddings || (desc->output_embedding.method == UZU_QUANT_NONE && desc->output_embedding.weights && desc->output_embedding.n == desc->vocab_size &&
                                          desc->output_embedding.k == d && !desc->output_embedding.out_biases),
                "model_create: an untied read-out of an f32-stream design is a full-precision matrix [vocab, model_dim]");
    auto rms_vec = [](const uzu_norm_desc& n) { return n.present && n.kind == UZU_NORM_STATISTICS && n.scales && !n.subtract_mean && !n.biases; };
    auto norm_ok = [&](const uzu_norm_desc& n) { return n.present && ((n.kind == UZU_NORM_DYNAMIC_TANH && n.scales) || n.kind == UZU_NORM_RMS_SCALAR || rms_vec(n)); };
    UZU_REQUIRE(norm_ok(desc->output_norm), "model_create: an f32-stream design ends in a dynamic-tanh norm or an RMS norm (one gain, or a weight vector)");
    UZU_UNSUPPORTED(desc->embedding_norm.present, "model_create: decoder options of the bf16-stream families on an f32-stream design");
    auto groups_ok = [&](const uzu_norm_desc& n, uint32_t dim) { return n.groups <= 1 || (rms_vec(n) && dim % n.groups == 0); };
    UZU_REQUIRE(groups_ok(desc->output_norm, d), "model_create: a norm in parts is an RMS norm with a weight vector over model_dim %% groups == 0 coordinates");
    if (desc->bigram_buckets)
        UZU_REQUIRE(desc->bigram_table.weights && desc->bigram_table.method == UZU_QUANT_NONE && desc->bigram_table.n == desc->bigram_buckets + 1 && desc->bigram_table.k == d,
                    "model_create: the hashed token-pair table is a full-precision matrix [buckets + 1, model_dim]");
    if (desc->has_ple) { // the side table alone: a layer's token input is its slice of the token's row
        UZU_UNSUPPORTED(desc->ple_model_projection.weights || desc->ple_projection_norm.present, "model_create: an f32-stream design's per-layer token input has no model projection");
        UZU_REQUIRE(desc->ple_dim && desc->ple_token_embedding.weights && desc->ple_token_embedding.method == UZU_QUANT_NONE && desc->ple_token_embedding.n == desc->ple_vocab_size &&
                    desc->ple_vocab_size >= desc->vocab_size && desc->ple_token_embedding.k % desc->ple_dim == 0,
                    "model_create: the side table is a full-precision matrix [>= vocab, slices * ple_dim]");
    }
    auto full = [](const uzu_linear_desc& L, uint32_t n, uint32_t kk) { return L.weights && L.method == UZU_QUANT_NONE && L.n == n && L.k == kk && !L.input_signs && !L.output_signs && !L.lora_rank; };
    for (uint32_t l = 0; l < nl; ++l) {
        const uzu_layer_desc& h = desc->layers[l];
        UZU_UNSUPPORTED(h.mixer_kind != UZU_MIXER_LATENT_ATTENTION && h.mixer_kind != UZU_MIXER_ATTENTION && h.mixer_kind != UZU_MIXER_RETENTION && h.mixer_kind != UZU_MIXER_GATED_LRU,
                        "model_create: layer %u: an f32-stream design's mixer is latent attention, attention over cached keys and values, retention, or a gated linear recurrent unit "
                        "(a channel-decay delta rule rides beside attention as the second mixer of a pair)", l);
        UZU_UNSUPPORTED(h.mixer_kind != UZU_MIXER_ATTENTION && (h.qk_norm_whole || h.attention_chunk_size || h.values_are_keys || h.rel_bias_rows || h.head_temperature || h.pair_mixer),
                        "model_create: layer %u: chunks, a distance bias, head temperatures, values that are keys, a whole-projection norm and a second mixer are options of attention", l);
        UZU_REQUIRE(!h.pre_mixer_norm.present || norm_ok(h.pre_mixer_norm), "model_create: layer %u: a pre-mixer norm is a dynamic-tanh or RMS norm (absent: the mixer reads the stream)", l);
        UZU_REQUIRE(groups_ok(h.pre_mixer_norm, d) && groups_ok(h.post_mixer_norm, d) && groups_ok(h.pre_mlp_norm, d) && groups_ok(h.post_mlp_norm, d),
                    "model_create: layer %u: a norm in parts is an RMS norm with a weight vector over model_dim %% groups == 0 coordinates", l);
        UZU_REQUIRE(!(h.input_conv_mixer || h.input_conv_mlp) || (h.input_conv_taps >= 1 && h.input_conv_taps <= 64), "model_create: layer %u: an input convolution of 1 .. 64 taps", l);
        UZU_UNSUPPORTED((h.input_conv_mixer && h.pre_mixer_norm.present) || (h.input_conv_mlp && (h.pre_mlp_norm.present || h.parallel_block || h.no_mlp)),
                        "model_create: layer %u: an input convolution feeds a sublayer that reads the stream itself (no pre norm)", l);
        UZU_UNSUPPORTED(!h.pre_mixer_norm.present && h.stream_reentry.weights, "model_create: layer %u: a re-entry projection in front of a mixer without a pre norm", l);
        UZU_UNSUPPORTED(h.token_shift && h.pre_mixer_norm.kind != UZU_NORM_DYNAMIC_TANH, "model_create: layer %u: the token shift follows a dynamic-tanh norm", l);
        UZU_REQUIRE(!h.post_mixer_norm.present || rms_vec(h.post_mixer_norm), "model_create: layer %u: a post-mixer norm is an RMS norm with a weight vector", l);
        UZU_REQUIRE(!h.post_mlp_norm.present || (rms_vec(h.post_mlp_norm) && !h.no_mlp && h.mlp_kind != UZU_MLP_MOE && !h.parallel_block),
                    "model_create: layer %u: a post-MLP norm is an RMS norm with a weight vector behind a dense block", l);
        UZU_REQUIRE((!h.layer_scale_mixer || h.post_mixer_norm.present) && (!h.layer_scale_mlp || h.post_mlp_norm.present), "model_create: layer %u: a layer scale follows a post norm", l);
        UZU_UNSUPPORTED(h.has_post_layer_scalar || h.normalize_values || h.is_non_causal, "model_create: layer %u: layer options of the bf16-stream families", l);
        if (h.weights_of_layer) {
            UZU_REQUIRE(h.weights_of_layer - 1 < l, "model_create: layer %u uses the tensors of run %u, which does not precede it", l, h.weights_of_layer - 1);
            const uzu_layer_desc& src = desc->layers[h.weights_of_layer - 1];
            UZU_REQUIRE(!src.weights_of_layer && src.mixer_kind == h.mixer_kind && src.qkv_projection.n == h.qkv_projection.n && src.out_projection.k == h.out_projection.k &&
                        src.hidden_dim == h.hidden_dim && src.no_mlp == h.no_mlp && src.mlp_kind == h.mlp_kind && src.has_ple == h.has_ple && !h.is_kv_sharing && !src.is_kv_sharing &&
                        (src.stream_reentry.weights != nullptr) == (h.stream_reentry.weights != nullptr),
                        "model_create: layer %u: a run that shares tensors has the shapes and options of the run that owns them", l);
        }
        if (h.stream_reentry.weights) {
            UZU_REQUIRE(full(h.stream_reentry, d, 2 * d), "model_create: layer %u: the re-entry projection is a full-precision matrix [model_dim, 2 model_dim]", l);
            UZU_UNSUPPORTED(l > 0 && desc->layers[l - 1].depth_weights, "model_create: layer %u: a re-entry projection behind a depth mix", l);
        }
        if (h.has_ple) {
            UZU_REQUIRE(desc->has_ple && h.ple_dim == desc->ple_dim && (h.ple_slice + 1) * h.ple_dim <= desc->ple_token_embedding.k && full(h.ple_gate, h.ple_dim, d) &&
                        full(h.ple_projection, d, h.ple_dim) && rms_vec(h.ple_norm) && h.ple_activation == UZU_ACT_GELU_APPROX,
                        "model_create: layer %u: the token input needs the model's side table, its slice, gate [ple_dim, model_dim], projection [model_dim, ple_dim], a weight-vector RMS norm and the tanh gelu", l);
        }
        if (h.mixer_kind == UZU_MIXER_GATED_LRU) {
            const uint32_t w = h.lru_width;
            UZU_REQUIRE(w && h.lru_blocks && w % h.lru_blocks == 0 && h.dn_kernel_size >= 1 && h.dn_kernel_size <= 64, "model_create: layer %u: lru_width in lru_blocks equal blocks, 1 .. 64 taps", l);
            UZU_REQUIRE(full(h.qkv_projection, 2 * w, d) && full(h.out_projection, d, w) && h.dn_conv_weights && h.lru_gate_weights && h.lru_lambda,
                        "model_create: layer %u: the recurrent unit's packed projection [2 lru_width, model_dim], out projection [model_dim, lru_width], convolution, gates and lambda", l);
            UZU_UNSUPPORTED(h.is_kv_sharing || h.sliding_window_size || h.has_sinks || h.unit_sink || h.score_soft_cap != 0.0f || h.use_rope || h.has_gate,
                            "model_create: layer %u: attention options on a recurrent layer", l);
        } else {
        UZU_REQUIRE(h.num_heads && h.head_dim && h.value_head_dim, "model_create: layer %u: heads / head_dim / value_head_dim", l);
        UZU_REQUIRE(full(h.out_projection, d, h.num_heads * h.value_head_dim), "model_create: layer %u: the out projection must be a full-precision matrix [model_dim, heads * value_head_dim]", l);
        }
        if (h.use_rope) {
            const uzu_rope_desc& R = desc->num_ropes ? desc->ropes[h.rope_index < desc->num_ropes ? h.rope_index : 0] : desc->rope;
            const bool latent = h.mixer_kind == UZU_MIXER_LATENT_ATTENTION;
            UZU_REQUIRE((!desc->num_ropes || h.rope_index < desc->num_ropes) && R.kind != UZU_ROPE_NONE && R.head_dim && R.head_dim % 2 == 0 &&
                        (latent ? R.head_dim == h.latent_rope_dim : R.head_dim <= h.head_dim),
                        "model_create: layer %u: its rotation must turn an even number of at most head_dim coordinates (latent attention: exactly the rotated key part)", l);
            UZU_UNSUPPORTED(h.rope_interleaved && !latent && h.mixer_kind != UZU_MIXER_ATTENTION, "model_create: layer %u: interleaved pairs are a rotation of latent attention and attention", l);
        }
        UZU_REQUIRE(h.mixer_kind != UZU_MIXER_LATENT_ATTENTION || (h.latent_rope_dim != 0) == (h.use_rope != 0), "model_create: layer %u: a rotated key part and its rotation come together", l);
        if (h.mixer_kind == UZU_MIXER_LATENT_ATTENTION) {
            const uint32_t rd = h.latent_rope_dim, kw = h.latent_rank + rd, qn = h.num_heads * (h.head_dim + rd);
            UZU_REQUIRE(h.latent_rank && kw <= k::kLatentMaxRank, "model_create: layer %u: latent_rank (+ the rotated part <= %u)", l, k::kLatentMaxRank);
            UZU_REQUIRE(full(h.latent_up_keys, h.num_heads * h.head_dim, h.latent_rank) && full(h.latent_up_values, h.num_heads * h.value_head_dim, h.latent_rank),
                        "model_create: layer %u: latent up projections must be full-precision matrices of the configured shapes", l);
            if (h.latent_packed) {
                UZU_REQUIRE(!h.is_kv_sharing && !h.latent_down.weights && full(h.qkv_projection, qn + kw + (h.has_gate ? h.num_heads : 0), d) && h.latent_norm.present && h.latent_norm.scales,
                            "model_create: layer %u: the packed projection is queries | down projection | gates [heads (head_dim + rope) + rank + rope (+ heads), model_dim], with the latent norm", l);
            } else {
                UZU_REQUIRE(full(h.qkv_projection, qn + (h.has_gate ? h.num_heads : 0), d), "model_create: layer %u: the query projection must be a full-precision matrix of the configured shape", l);
            }
            if (h.is_kv_sharing) {
                UZU_REQUIRE(h.kv_source_layer_index < l, "model_create: layer %u shares the latents of layer %u, which does not precede it", l, h.kv_source_layer_index);
                const uzu_layer_desc& src = desc->layers[h.kv_source_layer_index];
                UZU_REQUIRE(src.mixer_kind == UZU_MIXER_LATENT_ATTENTION && !src.is_kv_sharing && src.latent_rank == h.latent_rank && src.latent_rope_dim == rd,
                            "model_create: layer %u: the source layer %u must own latents of the same rank", l, h.kv_source_layer_index);
            } else if (!h.latent_packed) {
                UZU_REQUIRE(full(h.latent_down, kw, d) && h.latent_norm.present && h.latent_norm.scales, "model_create: layer %u owns its latents: down projection + latent norm required", l);
            }
        } else if (h.mixer_kind == UZU_MIXER_ATTENTION) {
            UZU_REQUIRE(h.num_groups && h.num_heads % h.num_groups == 0, "model_create: layer %u: %u query heads on %u key / value heads", l, h.num_heads, h.num_groups);
            UZU_REQUIRE((!h.query_norm.present || h.query_norm.scales) && (!h.key_norm.present || h.key_norm.scales) &&
                        (!h.query_norm.present || !h.key_norm.present || h.query_norm.epsilon == h.key_norm.epsilon),
                        "model_create: layer %u: query / key norms carry weights [head_dim] (or, over the whole projection, [heads head_dim] / [groups head_dim]) and one epsilon", l);
            UZU_REQUIRE(!h.values_are_keys || (h.value_head_dim == h.head_dim && !h.is_kv_sharing), "model_create: layer %u: values that are the key rows have the keys' width and a cache of their own", l);
            if (h.rel_bias_rows)
                UZU_REQUIRE(h.rel_bias && (h.rel_bias_rows == 1 || h.rel_bias_max > (float)(h.rel_bias_rows / 2)), "model_create: layer %u: a distance bias [rows, heads] whose last bucket starts beyond rows / 2", l);
            if (h.pair_mixer) {
                const uint32_t Hd = h.dn_num_heads, Gd = h.dn_num_groups, dk = h.dn_head_dim, dv = h.dn_value_head_dim;
                UZU_UNSUPPORTED(h.pair_mixer != 1 + UZU_MIXER_DELTA_NET || !h.dn_channel_decay, "model_create: layer %u: the second mixer of a pair is a delta rule with channel decays", l);
                UZU_REQUIRE(h.post_mixer_norm.present && !h.parallel_block, "model_create: layer %u: a pair of mixers joins the stream behind a post-mixer norm", l);
                UZU_REQUIRE(Hd && Gd && Hd % Gd == 0 && dk && dv && h.dn_kernel_size >= 1 && h.dn_kernel_size <= 64 && h.dn_decay_rank && h.dn_gate_rank,
                            "model_create: layer %u: the delta rule's %u value heads on %u query / key heads, 1 .. 64 taps, low-rank decay and gate", l, Hd, Gd);
                UZU_UNSUPPORTED(!k::channel_delta_supported(dk, dv), "model_create: layer %u: delta-rule heads of %u x %u (keys up to 256)", l, dk, dv);
                UZU_REQUIRE(full(h.dn_in_proj, 2 * Gd * dk + Hd * dv + Hd + h.dn_decay_rank + h.dn_gate_rank, d) && !h.dn_in_proj.out_biases && full(h.dn_out_proj, d, Hd * dv) &&
                            full(h.dn_decay_up, Hd * dk, h.dn_decay_rank) && full(h.dn_gate_up, Hd * dv, h.dn_gate_rank) && !h.dn_decay_up.out_biases && !h.dn_gate_up.out_biases &&
                            h.dn_conv_weights && h.dn_a_log && h.dn_dt_bias && h.dn_norm_scales,
                            "model_create: layer %u: the delta rule's packed projection q | k | v | beta | decay down | gate down, out projection, up factors, convolution, a_log, dt_bias and norm", l);
            }
            if (h.is_kv_sharing) {
                UZU_REQUIRE(h.kv_source_layer_index < l, "model_create: layer %u shares the cache of layer %u, which does not precede it", l, h.kv_source_layer_index);
                const uzu_layer_desc& src = desc->layers[h.kv_source_layer_index];
                UZU_REQUIRE(src.mixer_kind == UZU_MIXER_ATTENTION && !src.is_kv_sharing && src.num_groups == h.num_groups && src.head_dim == h.head_dim && src.value_head_dim == h.value_head_dim,
                            "model_create: layer %u: the source layer %u must own a cache of the same key / value heads and widths", l, h.kv_source_layer_index);
                UZU_REQUIRE(full(h.qkv_projection, h.num_heads * h.head_dim + (h.has_gate ? h.num_heads : 0), d), "model_create: layer %u reads another layer's cache: its projection yields queries only (+ gates)", l);
            } else {
                UZU_REQUIRE(full(h.qkv_projection, h.num_heads * h.head_dim + h.num_groups * (h.head_dim + (h.values_are_keys ? 0 : h.value_head_dim)) + (h.has_gate ? h.num_heads : 0), d),
                            "model_create: layer %u: the packed projection must be a full-precision matrix [heads head_dim + groups (head_dim + value_head_dim) (+ heads gate rows), model_dim]", l);
            }
        } else if (h.mixer_kind == UZU_MIXER_RETENTION) {
            UZU_REQUIRE(full(h.qkv_projection, 2 * h.num_heads * h.head_dim + 2 * h.num_heads * h.value_head_dim, d) && !h.qkv_projection.out_biases,
                        "model_create: layer %u: a retention layer's packed projection is queries | keys | values | gate without biases", l);
            UZU_REQUIRE(h.retention_decay, "model_create: layer %u: retention without its decays", l);
            UZU_UNSUPPORTED(!k::retention_supported(h.head_dim, h.value_head_dim), "model_create: layer %u: retention heads of %u x %u (keys up to 512, values up to 256)", l, h.head_dim,
                            h.value_head_dim);
            UZU_UNSUPPORTED(h.is_kv_sharing || h.sliding_window_size || h.has_sinks || h.unit_sink || h.score_soft_cap != 0.0f, "model_create: layer %u: attention options on a retention layer", l);
        }
        UZU_REQUIRE(!h.has_sinks || h.sinks, "model_create: layer %u: has_sinks without the tensor", l);
        UZU_REQUIRE(!(h.has_sinks && h.unit_sink), "model_create: layer %u: sink logits and a unit sink exclude each other", l);
        UZU_REQUIRE(!h.depth_weights || h.num_depth_weights == l + 2, "model_create: layer %u: a depth mix takes %u weights", l, l + 2);
        if (!h.no_mlp) {
            UZU_REQUIRE(h.parallel_block ? !h.pre_mlp_norm.present : (!h.pre_mlp_norm.present || norm_ok(h.pre_mlp_norm)),
                        "model_create: layer %u: a pre-MLP norm is a dynamic-tanh or RMS norm (absent: the MLP reads the stream), and none in a parallel block", l);
            if (h.mlp_kind == UZU_MLP_MOE) {
                const uzu_moe_desc& M = h.moe;
                UZU_REQUIRE((M.routing == UZU_MOE_ROUTE_SCORES || M.routing == UZU_MOE_ROUTE_TOPK_LOGITS) && M.num_active_experts &&
                            M.num_active_experts <= M.num_routed_experts + M.num_identity_experts && M.router_weights &&
                            (M.num_routed_experts == 0 || (M.expert_hidden_dim && M.w13 && M.w2)) && M.gating_sel == 2 && !M.up_biases && !M.down_biases,
                            "model_create: layer %u: routed SiLU-gated experts without biases, with their router and expert tensors", l);
                UZU_REQUIRE(M.routing == UZU_MOE_ROUTE_SCORES || (!M.num_identity_experts && !M.selection_bias), "model_create: layer %u: identity experts and selection biases belong to score routing", l);
            } else if (h.mlp_plain) {
                UZU_REQUIRE(h.activation == UZU_ACT_RELU_SQUARED && full(h.up_projection, h.hidden_dim, d) && full(h.down_projection, d, h.hidden_dim),
                            "model_create: layer %u: the plain dense block is down(relu(up x + b)^2) + b with full-precision matrices", l);
            } else {
                UZU_REQUIRE((h.activation == UZU_ACT_SILU || h.activation == UZU_ACT_GELU_APPROX) && h.hidden_dim && full(h.up_projection, 2 * h.hidden_dim, d) &&
                            full(h.down_projection, d, h.hidden_dim) && !h.parallel_block,
                            "model_create: layer %u: the gated dense block is down(act(gate) * (up + offset)), act = the sigmoid gate or the tanh gelu, with full-precision matrices [up ; gate] and [model_dim, hidden]", l);
            }
        }
    }
    (void)hipSetDevice(ctx->device);
    auto* m = new uzu_hip_model();
    m->ctx = ctx, m->flags = flags, m->d = *desc;
    m->d.layers = nullptr;
    auto* Sp = new Stream32();
    m->s32 = Sp;
    Stream32& S = *Sp;
    S.full_f32 = (flags & UZU_MODEL_FULL_F32) != 0;
    uzu_status st = UZU_OK;
    auto fail = [&](uzu_status r) {
        uzu_hip_model_destroy(m);
        return r;
    };
#define TRY(x) do { st = (x); if (st != UZU_OK) return fail(st); } while (0)
    TRY(upload_linear(m, desc->embedding, &m->embedding, true));
    TRY(upload_norm(m, desc->output_norm, d, &m->output_norm));
    S.alpha_out = desc->output_norm.alpha;
    m->chunk = prefill_chunk_rows();
    m->max_positions = desc->max_context_length + m->chunk;
    m->max_seqs = (flags >> 8) & 0xFF ? (flags >> 8) & 0xFF : 1;
    S.max_rows = m->chunk, S.max_seqs = m->max_seqs;
    m->layers.resize(nl);
    S.layers.resize(nl);
    uint32_t w_q = 0, w_rank = 0, w_lat = 0, w_attn = 0, w_hid = 0, w_top = 1, w_moe = 0, w_routed = 0, w_lru = 0, w_side = 0, w_y1 = 0;
    uint32_t w_dn_in = 0, w_dn_cv = 0, w_dn_k = 0, w_dn_v = 0;
    bool any_pair = false, any_inconv = false;
    for (uint32_t l = 0; l < nl; ++l) {
        const uzu_layer_desc& h = desc->layers[l];
        DLayer& L = m->layers[l];
        Stream32::Layer& X = S.layers[l];
        uint32_t kw_l = h.latent_rank + h.latent_rope_dim;
        w_q = std::max(w_q, h.qkv_projection.n), w_rank = std::max(w_rank, h.latent_down.n ? h.latent_down.n : kw_l), w_lat = std::max(w_lat, h.num_heads * kw_l);
        w_attn = std::max(w_attn, std::max(h.num_heads * h.value_head_dim, h.lru_width)), w_lru = std::max(w_lru, h.lru_width), w_side = std::max(w_side, h.has_ple ? h.ple_dim : 0u);
        if (!h.no_mlp && h.mlp_kind != UZU_MLP_MOE) w_hid = std::max(w_hid, h.hidden_dim), w_y1 = std::max(w_y1, h.mlp_plain ? 0u : 2 * h.hidden_dim);
        if (h.weights_of_layer) { // the tensors of an earlier run: its device pointers, this run's own scalars; nothing is uploaded twice
            L = m->layers[h.weights_of_layer - 1];
            X = S.layers[h.weights_of_layer - 1];
            L.d = h;
            L.last_reader = l;
            if (!h.no_mlp && h.mlp_kind == UZU_MLP_MOE) {
                const uzu_moe_desc& M = h.moe;
                w_hid = std::max<uint32_t>(w_hid, M.num_active_experts * M.expert_hidden_dim), w_top = std::max(w_top, M.num_active_experts);
                w_moe = std::max(w_moe, M.num_active_experts * 2 * M.expert_hidden_dim), w_routed = std::max(w_routed, M.num_routed_experts);
            }
            continue;
        }
        L.d = h;
        L.last_reader = l;
        TRY(upload_norm(m, h.pre_mixer_norm, d, &L.pre_mixer));
        TRY(upload_norm(m, h.post_mixer_norm, d, &L.post_mixer));
        if (h.layer_scale_mixer) TRY(upload(m, h.layer_scale_mixer, (size_t)d * 4, &X.ls1));
        if (h.layer_scale_mlp) TRY(upload(m, h.layer_scale_mlp, (size_t)d * 4, &X.ls2));
        if (h.stream_reentry.weights) { // [d, 2 d] -> the half on the stream and the half on the embedding rows (bf16 bits move)
            const uint16_t* src = (const uint16_t*)h.stream_reentry.weights;
            std::vector<uint16_t> a((size_t)d * d), b((size_t)d * d);
            for (uint32_t n = 0; n < d; ++n) {
                memcpy(&a[(size_t)n * d], src + (size_t)n * 2 * d, (size_t)d * 2);
                memcpy(&b[(size_t)n * d], src + (size_t)n * 2 * d + d, (size_t)d * 2);
            }
            X.reentry_a.n = X.reentry_b.n = d, X.reentry_a.k = X.reentry_b.k = d;
            TRY(upload(m, a.data(), a.size() * 2, &X.reentry_a.w));
            TRY(upload(m, b.data(), b.size() * 2, &X.reentry_b.w));
        }
        if (h.has_ple) {
            TRY(upload_linear(m, h.ple_gate, &L.ple_gate));
            TRY(upload_linear(m, h.ple_projection, &L.ple_projection));
            TRY(upload_norm(m, h.ple_norm, d, &L.ple_norm));
        }
        if (h.mixer_kind == UZU_MIXER_ATTENTION) {
            TRY(upload_norm(m, h.query_norm, h.qk_norm_whole ? h.num_heads * h.head_dim : h.head_dim, &L.qn));
            TRY(upload_norm(m, h.key_norm, h.qk_norm_whole ? h.num_groups * h.head_dim : h.head_dim, &L.kn));
            if (h.head_temperature) TRY(upload(m, h.head_temperature, (size_t)h.num_heads * 4, &X.head_temp));
            if (h.rel_bias_rows) { // the bias by distance: the bucket rule once, in double, for every distance up to the one the last bucket starts at
                const uint32_t B = h.rel_bias_rows, E = B / 2, H = h.num_heads;
                // (distances beyond the last bucket's start share its row; no distance reaches the cache's capacity)
                const uint32_t far = B == 1 ? 0u : (uint32_t)std::min<double>(ceil((double)h.rel_bias_max), (double)m->max_positions);
                std::vector<float> tab((size_t)(far + 1) * H);
                for (uint32_t n = 0; n <= far; ++n) {
                    uint32_t b = n;
                    if (n >= E) {
                        b = B - 1;
                        if (B > 1 && (double)n < (double)h.rel_bias_max) {
                            const double steps = floor(log((double)n / (double)E) / log((double)h.rel_bias_max / (double)E) * (double)(B - E));
                            b = std::min<uint32_t>(B - 1, E + (uint32_t)std::max(steps, 0.0));
                        }
                    }
                    for (uint32_t a = 0; a < H; ++a) tab[(size_t)n * H + a] = bf16_to_f32(h.rel_bias[(size_t)b * H + a]);
                }
                X.dist_rows = far + 1;
                TRY(upload(m, tab.data(), tab.size() * 4, &X.dist_bias));
            }
            if (h.pair_mixer) {
                const size_t conv_dim = 2 * (size_t)h.dn_num_groups * h.dn_head_dim + (size_t)h.dn_num_heads * h.dn_value_head_dim;
                TRY(upload_linear(m, h.dn_in_proj, &L.in_proj));
                TRY(upload_linear(m, h.dn_out_proj, &L.out_proj));
                TRY(upload_linear(m, h.dn_decay_up, &X.decay_up));
                TRY(upload_linear(m, h.dn_gate_up, &X.gate_up));
                TRY(upload(m, h.dn_conv_weights, conv_dim * h.dn_kernel_size * 4, &L.conv_w));
                if (h.dn_conv_biases) TRY(upload(m, h.dn_conv_biases, conv_dim * 4, &L.conv_b));
                TRY(upload(m, h.dn_a_log, (size_t)h.dn_num_heads * 4, &L.a_log));
                TRY(upload(m, h.dn_dt_bias, (size_t)h.dn_num_heads * h.dn_head_dim * 4, &L.dt_bias));
                TRY(upload(m, h.dn_norm_scales, (size_t)h.dn_value_head_dim * 4, &L.dn_norm));
                w_dn_in = std::max(w_dn_in, h.dn_in_proj.n), w_dn_cv = std::max<uint32_t>(w_dn_cv, (uint32_t)conv_dim);
                w_dn_k = std::max(w_dn_k, h.dn_num_heads * h.dn_head_dim), w_dn_v = std::max(w_dn_v, h.dn_num_heads * h.dn_value_head_dim);
            }
        }
        if (h.input_conv_mixer) TRY(upload(m, h.input_conv_mixer, (size_t)d * h.input_conv_taps * 4, &X.in_conv_mixer));
        if (h.input_conv_mlp) TRY(upload(m, h.input_conv_mlp, (size_t)d * h.input_conv_taps * 4, &X.in_conv_mlp));
        any_pair |= h.pair_mixer != 0, any_inconv |= h.input_conv_mixer || h.input_conv_mlp;
        if (h.mixer_kind == UZU_MIXER_GATED_LRU) {
            const size_t w = h.lru_width, bw = w / h.lru_blocks;
            TRY(upload(m, h.dn_conv_weights, w * h.dn_kernel_size * 4, &L.conv_w));
            if (h.dn_conv_biases) TRY(upload(m, h.dn_conv_biases, w * 4, &L.conv_b));
            TRY(upload(m, h.lru_gate_weights, 2 * w * bw * 2, &X.lru_gate_w));
            if (h.lru_gate_biases) TRY(upload(m, h.lru_gate_biases, 2 * w * 4, &X.lru_gate_b));
            TRY(upload(m, h.lru_lambda, w * 4, &X.lru_lambda));
        }
        X.alpha1 = h.pre_mixer_norm.alpha;
        TRY(upload_linear(m, h.qkv_projection, &L.qkv));
        TRY(upload_linear(m, h.out_projection, &L.out));
        if (h.mixer_kind == UZU_MIXER_RETENTION) TRY(upload(m, h.retention_decay, (size_t)h.num_heads * 4, &X.decay));
        if (h.unit_sink) { // a sink of logit 0 per head
            std::vector<float> f(h.num_heads, 0.0f);
            TRY(upload(m, f.data(), f.size() * 4, &X.sinks));
        }
        if (h.mixer_kind == UZU_MIXER_LATENT_ATTENTION) {
        TRY(upload_linear(m, h.latent_up_values, &L.lat_up_v));
        {   // W_up_k [heads * head_dim, rank] -> per head [rank, head_dim] (bf16 bits move, nothing is rounded)
            const uint32_t H = h.num_heads, hd = h.head_dim, rank = h.latent_rank;
            const uint16_t* src = (const uint16_t*)h.latent_up_keys.weights;
            std::vector<uint16_t> t((size_t)H * rank * hd);
            for (uint32_t hh = 0; hh < H; ++hh)
                for (uint32_t i = 0; i < hd; ++i)
                    for (uint32_t c = 0; c < rank; ++c) t[((size_t)hh * rank + c) * hd + i] = src[((size_t)hh * hd + i) * rank + c];
            TRY(upload(m, t.data(), t.size() * 2, &X.up_keys_t));
        }
        if (!h.is_kv_sharing) {
            if (!h.latent_packed) TRY(upload_linear(m, h.latent_down, &L.lat_down));
            TRY(upload_norm(m, h.latent_norm, h.latent_rank, &L.lat_norm));
        }
        } // latent attention
        if (h.has_sinks) {
            std::vector<float> f(h.num_heads);
            for (uint32_t i = 0; i < h.num_heads; ++i) f[i] = bf16_to_f32(((const uint16_t*)h.sinks)[i]);
            TRY(upload(m, f.data(), f.size() * 4, &X.sinks));
        }
        if (h.token_shift) TRY(upload(m, h.token_shift, (size_t)d * 4, &X.token_shift));
        if (h.depth_weights) TRY(upload(m, h.depth_weights, (size_t)h.num_depth_weights * 4, &X.depth_weights));
        if (!h.no_mlp) {
            if (!h.parallel_block) TRY(upload_norm(m, h.pre_mlp_norm, d, &L.pre_mlp));
            TRY(upload_norm(m, h.post_mlp_norm, d, &L.post_mlp));
            X.alpha2 = h.pre_mlp_norm.alpha;
            if (h.mlp_kind == UZU_MLP_MOE) {
                const uzu_moe_desc& M = h.moe;
                const size_t E = M.num_routed_experts, ff = M.expert_hidden_dim;
                TRY(upload(m, M.router_weights, (E + M.num_identity_experts) * d * 2, &L.moe.router_weights));
                if (M.router_biases) TRY(upload(m, M.router_biases, (E + M.num_identity_experts) * 2, &L.moe.router_biases));
                if (E) {
                    TRY(upload(m, M.w13, E * 2 * ff * d * 2, &L.moe.w13));
                    TRY(upload(m, M.w2, E * d * ff * 2, &L.moe.w2));
                }
                if (M.selection_bias) TRY(upload(m, M.selection_bias, (E + M.num_identity_experts) * 4, &X.selection_bias));
                w_hid = std::max<uint32_t>(w_hid, M.num_active_experts * M.expert_hidden_dim);
                w_top = std::max(w_top, M.num_active_experts);
                w_moe = std::max(w_moe, M.num_active_experts * 2 * M.expert_hidden_dim), w_routed = std::max(w_routed, M.num_routed_experts);
            } else {
                TRY(upload_linear(m, h.up_projection, &L.up));
                TRY(upload_linear(m, h.down_projection, &L.down));
            }
        }
    }
    if (desc->has_ple) TRY(upload_linear(m, desc->ple_token_embedding, &m->ple_token_embedding, true));
    if (desc->bigram_buckets) TRY(upload(m, desc->bigram_table.weights, ((size_t)desc->bigram_buckets + 1) * d * 2, &S.pair_table));
    if (!desc->tied_embeddings) TRY(upload_linear(m, desc->output_embedding, &m->output_embedding));
    {   // one table pair per distinct rotation; a layer points at its own
        const uint32_t n_ropes = desc->num_ropes ? desc->num_ropes : (desc->rope.kind != UZU_ROPE_NONE ? 1u : 0u);
        m->ropes.resize(n_ropes);
        const size_t saved = m->weight_bytes;
        for (uint32_t r = 0; r < n_ropes; ++r) {
            const uzu_rope_desc& Rd = desc->num_ropes ? desc->ropes[r] : desc->rope;
            if (Rd.kind == UZU_ROPE_NONE || !Rd.head_dim) {
                set_error("model_create: RoPE configuration %u is empty", r);
                return fail(UZU_ERR_INVALID_ARGUMENT);
            }
            std::vector<float> c, sn;
            rope_tables(Rd, m->max_positions, c, sn);
            TRY(upload(m, c.data(), c.size() * 4, &m->ropes[r].cos));
            TRY(upload(m, sn.data(), sn.size() * 4, &m->ropes[r].sin));
            m->ropes[r].dim = Rd.head_dim;
        }
        m->weight_bytes = saved;
        for (DLayer& L : m->layers)
            if (L.d.use_rope) {
                const uzu_hip_model::RopeTable& T = m->ropes[desc->num_ropes ? L.d.rope_index : 0];
                L.rope_cos = T.cos, L.rope_sin = T.sin, L.rope_dim = T.dim;
            }
    }
    const size_t R = S.max_rows;
    if (!w_lat) w_lat = 1;
    if (!w_rank) w_rank = 1;
    TRY(need_f32(m, (size_t)(nl + 1) * R * d, &S.slots));
    TRY(need_f32(m, R * d, &S.xin));
    TRY(need_f32(m, R * d, &S.normed));
    TRY(need_f32(m, R * d, &S.out_normed));
    TRY(need_f32(m, R * w_q, &S.q));
    TRY(need_f32(m, R * w_rank, &S.ckv));
    TRY(need_f32(m, R * w_lat, &S.qlat));
    TRY(need_f32(m, R * w_lat, &S.ctx));
    TRY(need_f32(m, R * w_attn, &S.attn));
    TRY(need_f32(m, R * (w_hid ? w_hid : 1), &S.hid));
    TRY(need_f32(m, R * d, &S.tmp));
    if (w_y1) TRY(need_f32(m, R * w_y1, &S.y1));
    if (w_lru) {
        TRY(need_f32(m, R * w_lru, &S.lru_u));
        TRY(need_f32(m, R * 2 * w_lru, &S.lru_g));
    }
    if (w_side) TRY(need_f32(m, R * w_side, &S.side_g));
    if (w_dn_in) {
        TRY(need_f32(m, R * w_dn_in, &S.dn_in));
        TRY(need_f32(m, R * w_dn_cv, &S.dn_cv));
        TRY(need_f32(m, R * w_dn_k, &S.dn_decay));
        TRY(need_f32(m, R * w_dn_v, &S.dn_gate));
        TRY(need_f32(m, R * w_dn_v, &S.dn_o));
    }
    TRY(need_f32(m, R * w_top, &S.moe_w));
    if (w_moe && !S.full_f32) { // workspaces of the grouped expert form (bf16 products only)
        void* q = nullptr;
        TRY(need_f32(m, R * w_moe, &S.moe_y1));
        TRY(need_f32(m, R * w_top * d, &S.moe_y2));
        TRY(dev_alloc(m, R * w_top * 4, &q)); S.moe_perm = (uint32_t*)q;
        TRY(dev_alloc(m, R * w_top * 4, &q)); S.moe_slot_pos = (uint32_t*)q;
        TRY(dev_alloc(m, ((size_t)w_routed + 1) * 4, &q)); S.moe_offsets = (uint32_t*)q;
        TRY(dev_alloc(m, ((size_t)w_routed + 1) * 4, &q)); S.moe_cursor = (uint32_t*)q;
    }
    void* p = nullptr;
    TRY(dev_alloc(m, R * w_top * 4, &p)); S.moe_ids = (int32_t*)p;
    TRY(dev_alloc(m, S.max_seqs * sizeof(k::SeqSpan), &p)); S.d_spans = (k::SeqSpan*)p;
    TRY(dev_alloc(m, R * 4, &p)); S.d_row_seq = (uint32_t*)p;
    TRY(dev_alloc(m, R * 4, &p)); S.d_out_rows = (uint32_t*)p;
    TRY(dev_alloc(m, (size_t)nl * S.max_seqs * sizeof(void*), &p)); S.d_cache_ptrs = (void**)p;
    TRY(dev_alloc(m, (size_t)nl * S.max_seqs * sizeof(void*), &p)); S.d_cache2_ptrs = (void**)p;
    TRY(dev_alloc(m, (size_t)nl * S.max_seqs * sizeof(float*), &p)); S.d_shift_ptrs = (float**)p;
    if (any_pair) {
        if (hipStreamCreateWithFlags(&S.side, hipStreamNonBlocking) != hipSuccess || hipEventCreateWithFlags(&S.side_fork, hipEventDisableTiming) != hipSuccess ||
            hipEventCreateWithFlags(&S.side_join, hipEventDisableTiming) != hipSuccess) {
            set_error("model_create: the side stream of a pair of mixers could not be created");
            return fail(UZU_ERR_HIP);
        }
        TRY(dev_alloc(m, (size_t)nl * S.max_seqs * sizeof(float*), &p)); S.d_pair_state_ptrs = (float**)p;
        TRY(dev_alloc(m, (size_t)nl * S.max_seqs * sizeof(float*), &p)); S.d_pair_conv_ptrs = (float**)p;
    }
    if (any_inconv) { TRY(dev_alloc(m, (size_t)nl * S.max_seqs * sizeof(float*), &p)); S.d_inconv_ptrs = (float**)p; }
    if (desc->bigram_buckets) { TRY(dev_alloc(m, S.max_seqs * sizeof(uint32_t*), &p)); S.d_prev_tok_ptrs = (uint32_t**)p; }
    TRY(dev_alloc(m, R * 4, &p)); m->batch_tokens = (uint32_t*)p;
    if (flags & UZU_MODEL_DEBUG_TAPS) TRY(need_f32(m, (size_t)nl * R * d, &S.taps));
    {
        uint32_t hmax = 0;
        for (uint32_t l = 0; l < nl; ++l) hmax = std::max(hmax, desc->layers[l].num_heads);
        if (!hmax) hmax = 1;
        const uint32_t few = std::min<uint32_t>(4 * S.max_seqs, 4096 / hmax ? 4096 / hmax : 1);
        S.att_ws_bytes = std::max(k::latent_attention_split_ws_bytes(few, hmax, 256, 32), k::window_attention_split_ws_bytes(few, hmax, 16));
        TRY(need_f32(m, S.att_ws_bytes / 4, &S.att_ws));
    }
    for (uint32_t l = 0; l < nl; ++l) {
        const uzu_layer_desc& h = desc->layers[l];
        if (h.mixer_kind == UZU_MIXER_RETENTION)
            S.ret_ws_bytes = std::max(S.ret_ws_bytes, k::retention_chunk_ws_bytes(S.max_rows / 64 + S.max_seqs, h.num_heads, h.head_dim, h.value_head_dim));
    }
    if (S.ret_ws_bytes) TRY(need_f32(m, S.ret_ws_bytes / 4, &S.ret_ws));
    if (w_lru) {
        S.lru_ws_bytes = k::lru_piece_ws_bytes(S.max_rows / 32 + S.max_seqs, w_lru);
        TRY(need_f32(m, S.lru_ws_bytes / 4, &S.lru_ws));
    }
    TRY(dev_alloc(m, k::argmax_scratch_bytes(1), &m->argmax_scratch));
    TRY(dev_alloc(m, k::unified_sampling_scratch_bytes(1), &m->sampling_scratch));
    TRY(dev_alloc(m, 8, &p, true)); m->d_seed = (uint64_t*)p;
    TRY(ensure_logits(m, 16));
    TRY(state_build(m, &m->state0));
    bind_state(m, m->state0);
    if (hipEventCreate(&m->ev0) != hipSuccess || hipEventCreate(&m->ev1) != hipSuccess) {
        set_error("model_create: hipEventCreate failed");
        return fail(UZU_ERR_HIP);
    }
    if (hipStreamSynchronize(ctx->stream) != hipSuccess) {
        set_error("model_create: synchronising the uploads failed");
        return fail(UZU_ERR_HIP);
    }
#undef TRY
    *out = m;
    return UZU_OK;
}

void s32_destroy(uzu_hip_model* m) {
    if (m->s32->side) {
        (void)hipStreamSynchronize(m->s32->side);
        (void)hipStreamDestroy(m->s32->side);
    }
    if (m->s32->side_fork) (void)hipEventDestroy(m->s32->side_fork);
    if (m->s32->side_join) (void)hipEventDestroy(m->s32->side_join);
    delete m->s32;
    m->s32 = nullptr;
}

// the state rows of one layer (state_build, engine_build.hip): the latent cache of a layer that owns one, the token shift's last row
uzu_status s32_state_layer(uzu_hip_model* m, uzu_hip_state* st, uint32_t l) {
    const uzu_layer_desc& h = m->layers[l].d;
    void* p = nullptr;
    const size_t elem = m->s32->full_f32 ? 4 : 2;
    if (h.mixer_kind == UZU_MIXER_RETENTION) { // read only behind position 0, where the kernel starts from zeros: no fill needed
        UZU_PROPAGATE(state_alloc(st, (size_t)h.num_heads * h.head_dim * h.value_head_dim * 4, &p, false));
        st->layers[l].ret_state = (float*)p;
    } else if (h.mixer_kind == UZU_MIXER_GATED_LRU) { // the state and the convolution's last taps - 1 inputs; both read only behind position 0
        UZU_PROPAGATE(state_alloc(st, (size_t)h.lru_width * 4, &p, false));
        st->layers[l].ssm_state = (float*)p;
        UZU_PROPAGATE(state_alloc(st, (size_t)h.lru_width * (h.dn_kernel_size > 1 ? h.dn_kernel_size - 1 : 1) * 4, &p, false));
        st->layers[l].conv_state = (float*)p;
    } else if (!h.is_kv_sharing) { // rows are written before they are read (the append precedes the core in every pass)
        if (h.mixer_kind == UZU_MIXER_ATTENTION) {
            UZU_PROPAGATE(state_alloc(st, (size_t)m->max_positions * h.num_groups * h.head_dim * elem, &p, false));
            st->layers[l].cache_k = p;
            UZU_PROPAGATE(state_alloc(st, (size_t)m->max_positions * h.num_groups * h.value_head_dim * elem, &p, false));
            st->layers[l].cache_v = p;
        } else {
            UZU_PROPAGATE(state_alloc(st, (size_t)m->max_positions * (h.latent_rank + h.latent_rope_dim) * elem, &p, false));
            st->layers[l].latent = p;
        }
    }
    if (h.token_shift) {
        UZU_PROPAGATE(state_alloc(st, (size_t)m->d.model_dim * 4, &p));
        st->layers[l].shift_prev = (float*)p;
    }
    if (h.pair_mixer) { // the second mixer's state and convolution window; both read only behind position 0
        UZU_PROPAGATE(state_alloc(st, (size_t)h.dn_num_heads * h.dn_head_dim * h.dn_value_head_dim * 4, &p, false));
        st->layers[l].ssm_state = (float*)p;
        const size_t conv_dim = 2 * (size_t)h.dn_num_groups * h.dn_head_dim + (size_t)h.dn_num_heads * h.dn_value_head_dim;
        UZU_PROPAGATE(state_alloc(st, conv_dim * (h.dn_kernel_size > 1 ? h.dn_kernel_size - 1 : 1) * 4, &p, false));
        st->layers[l].conv_state = (float*)p;
    }
    if ((h.input_conv_mixer || h.input_conv_mlp) && h.input_conv_taps > 1) { // the mixer's window, then the MLP's; read only behind position 0
        UZU_PROPAGATE(state_alloc(st, (size_t)2 * (h.input_conv_taps - 1) * m->d.model_dim * 4, &p, false));
        st->layers[l].in_conv = (float*)p;
    }
    return UZU_OK;
}

// ---------------------------------------------------------------------------------- the C ABI's f32-stream legs (engine_api.hip dispatches here)

// A batched step: sequence i appends counts[i] tokens.  want_rows index the concatenated token list; their logits go to logits_out [nwant][vocab] (host, f32).
// sampled_out (optional) [nseq]: the token sampled from every sequence's last row (greedy; the model's stochastic sampler when one sequence is stepped); the
// sampled token also becomes the sequence's next input token (uzu_hip_model_decode continues from it).
uzu_status s32_step_batch(uzu_hip_model* m, uzu_hip_state** states, uint32_t nseq, const uint32_t* token_ids, const uint32_t* counts, const uint32_t* want_rows, uint32_t nwant,
                          float* logits_out, uint32_t* sampled_out) {
    Stream32& S = *m->s32;
    hipStream_t s = m->ctx->stream;
    const uint32_t V = m->d.vocab_size;
    std::vector<uint32_t> offset(nseq + 1, 0), done(nseq, 0);
    for (uint32_t i = 0; i < nseq; ++i) {
        UZU_REQUIRE(states[i] && states[i]->m == m, "model_step_batch: state %u is null or belongs to another model", i);
        for (uint32_t j = 0; j < i; ++j) UZU_REQUIRE(states[i] != states[j], "model_step_batch: state %u listed twice", i);
        UZU_REQUIRE(counts[i] > 0, "model_step_batch: sequence %u brings no token", i);
        UZU_REQUIRE(state_length(m, states[i]) + counts[i] <= m->d.max_context_length, "model_step_batch: sequence %u exceeds max_context_length %u", i, m->d.max_context_length);
        offset[i + 1] = offset[i] + counts[i];
    }
    const uint32_t total = offset[nseq];
    for (uint32_t i = 0; i < total; ++i) UZU_REQUIRE(token_ids[i] < V, "model_step_batch: token id %u outside the vocabulary", token_ids[i]);
    for (uint32_t i = 0; i < nwant; ++i) UZU_REQUIRE(want_rows[i] < total && (i == 0 || want_rows[i] > want_rows[i - 1]), "model_step_batch: want_rows must be ascending rows of the step");
    UZU_REQUIRE(!nwant || logits_out, "model_step_batch: logits wanted without a buffer");
    const bool sample = sampled_out != nullptr;
    uint32_t seq_lo = 0;
    // passes: at most max_seqs sequences and max_rows rows each, sequences in order, a long prompt continues in the next pass
    while (seq_lo < nseq) {
        std::vector<PassSeq> pass;
        std::vector<uint32_t> pass_tok, out_rows, out_dst, sample_seq;
        uint32_t rows = 0, i = seq_lo;
        for (; i < nseq && pass.size() < S.max_seqs && rows < S.max_rows; ++i) {
            const uint32_t take = std::min(counts[i] - done[i], S.max_rows - rows);
            const uint32_t first = offset[i] + done[i];
            pass.push_back({states[i], take, state_length(m, states[i])});
            for (uint32_t j = 0; j < take; ++j) pass_tok.push_back(token_ids[first + j]);
            // wanted rows inside [first, first + take)
            const uint32_t* lo = std::lower_bound(want_rows, want_rows + nwant, first);
            for (const uint32_t* w = lo; w < want_rows + nwant && *w < first + take; ++w) out_rows.push_back(rows + (*w - first)), out_dst.push_back((uint32_t)(w - want_rows));
            rows += take;
            done[i] += take;
            if (done[i] < counts[i]) break; // the rest of this prompt opens the next pass
        }
        for (size_t a = 0; a < pass.size(); ++a) {
            const uint32_t qi = seq_lo + (uint32_t)a;
            if (sample && done[qi] == counts[qi]) sample_seq.push_back((uint32_t)a);
        }
        const size_t n_want_rows = out_rows.size();
        {
            uint32_t r0 = 0;
            std::vector<uint32_t> last_row(pass.size());
            for (size_t a = 0; a < pass.size(); ++a) r0 += pass[a].count, last_row[a] = r0 - 1;
            for (uint32_t a : sample_seq) out_rows.push_back(last_row[a]);
        }
        UZU_PROPAGATE(ensure_logits(m, out_rows.size()));
        HIPCHK(hipMemcpyAsync(m->batch_tokens, pass_tok.data(), pass_tok.size() * 4, hipMemcpyHostToDevice, s));
        UZU_PROPAGATE(s32_pass(m, pass, m->batch_tokens, out_rows));
        for (size_t a = 0; a < pass.size(); ++a) {
            size_t srow = 0;
            bool do_sample = false;
            for (size_t b = 0; b < sample_seq.size(); ++b)
                if (sample_seq[b] == a) srow = n_want_rows + b, do_sample = true;
            UZU_PROPAGATE(sample_commit(m, pass[a].st, (uint32_t)srow, pass[a].count, do_sample));
        }
        HIPCHK(hipStreamSynchronize(s));
        for (size_t a = 0; a < pass.size(); ++a) state_set_length(m, pass[a].st, pass[a].start + pass[a].count);
        // the wanted rows of a pass are consecutive entries of want_rows (both ascend): one copy
        if (n_want_rows) HIPCHK(hipMemcpy(logits_out + (size_t)out_dst[0] * V, S.logits, n_want_rows * (size_t)V * 4, hipMemcpyDeviceToHost));
        for (size_t b = 0; b < sample_seq.size(); ++b) {
            const uint32_t qi = seq_lo + sample_seq[b];
            HIPCHK(hipMemcpy(sampled_out + qi, states[qi]->d_out_token, 4, hipMemcpyDeviceToHost));
        }
        // sequences that are through leave the window; one that is not stays first
        while (seq_lo < nseq && done[seq_lo] == counts[seq_lo]) ++seq_lo;
    }
    m->hidden_ready = false;
    return UZU_OK;
}

uzu_status s32_prefill(uzu_hip_model* m, const uint32_t* token_ids, uint32_t count, uint32_t* first_token) {
    uzu_hip_state* st = m->bound;
    uint32_t sampled = 0;
    UZU_PROPAGATE(s32_step_batch(m, &st, 1, token_ids, &count, nullptr, 0, nullptr, &sampled));
    if (first_token) *first_token = sampled;
    return UZU_OK;
}

// `steps` chained decode steps of the bound sequence: the input token of a step is the one the step before left in the control block
uzu_status s32_decode_enqueue(uzu_hip_model* m, uint32_t steps) {
    uzu_hip_state* st = m->bound;
    UZU_REQUIRE(m->context_length + steps <= m->d.max_context_length, "model_decode: %u + %u tokens exceed max_context_length %u", m->context_length, steps, m->d.max_context_length);
    UZU_PROPAGATE(ensure_logits(m, 1));
    Stream32& S = *m->s32;
    hipStream_t s = m->ctx->stream;
    // the tables once (the model's table block serves whichever state steps; the span moves on the device with every commit)
    UZU_PROPAGATE(s32_upload_tables(m, {{st, 1, m->context_length}}, {0}));
    const std::vector<uint32_t> one{1};
    const bool graph = !(m->flags & (UZU_MODEL_NO_GRAPH | UZU_MODEL_DEBUG_TAPS));
    if (graph && m->graph_epoch != m->sampling_epoch) { // the captured step bakes the sampling kernels in
        if (m->graph_single) (void)hipGraphExecDestroy(m->graph_single);
        m->graph_single = nullptr, m->graph_epoch = m->sampling_epoch;
    }
    if (graph && !m->graph_single) { // one decode step of THIS state (its token / cache / control-block pointers) as a hipGraph
        HIPCHK(hipStreamSynchronize(s));
        HIPCHK(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
        uzu_status r = s32_encode(m, one, st->d_tokens, 1);
        if (r == UZU_OK) r = sample_commit(m, st, 0, 1, true, S.d_spans);
        hipGraph_t g = nullptr;
        const hipError_t ce = hipStreamEndCapture(s, &g);
        if (r != UZU_OK || ce != hipSuccess) {
            if (g) (void)hipGraphDestroy(g);
            if (r == UZU_OK) set_error("engine: decode graph capture failed: %s", hipGetErrorString(ce));
            return r != UZU_OK ? r : UZU_ERR_HIP;
        }
        HIPCHK(hipGraphInstantiate(&m->graph_single, g, nullptr, nullptr, 0));
        HIPCHK(hipGraphDestroy(g));
    }
    for (uint32_t i = 0; i < steps; ++i) {
        if (graph) {
            HIPCHK(hipGraphLaunch(m->graph_single, s));
        } else {
            UZU_PROPAGATE(s32_encode(m, one, st->d_tokens, 1));
            UZU_PROPAGATE(sample_commit(m, st, 0, 1, true, S.d_spans));
        }
        state_set_length(m, st, m->context_length + 1);
    }
    return UZU_OK;
}

uzu_status s32_read_logits_f32(uzu_hip_model* m, float* out, uint32_t row) {
    Stream32& S = *m->s32;
    UZU_REQUIRE(row < S.last_logit_rows, "model_read_logits: the last pass produced %u rows of logits", S.last_logit_rows);
    HIPCHK(hipStreamSynchronize(m->ctx->stream));
    HIPCHK(hipMemcpy(out, S.logits + (size_t)row * m->d.vocab_size, (size_t)m->d.vocab_size * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

uint32_t s32_last_logit_rows(const uzu_hip_model* m) { return m->s32->last_logit_rows; }

uzu_status s32_read_layer_output(uzu_hip_model* m, uint32_t layer, float* out, uint32_t* rows) {
    Stream32& S = *m->s32;
    UZU_REQUIRE(S.taps, "model_read_layer_output: create the model with UZU_MODEL_DEBUG_TAPS");
    UZU_REQUIRE(layer < m->d.num_layers, "model_read_layer_output: layer out of range");
    HIPCHK(hipStreamSynchronize(m->ctx->stream));
    if (rows) *rows = S.tap_rows;
    if (out) HIPCHK(hipMemcpy(out, S.taps + (size_t)layer * S.max_rows * m->d.model_dim, (size_t)S.tap_rows * m->d.model_dim * 4, hipMemcpyDeviceToHost));
    return UZU_OK;
}

} // namespace eng
} // namespace uzu
