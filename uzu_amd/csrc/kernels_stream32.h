// kernels_stream32.h -- kernels of the f32-stream designs (uzu_model_desc::f32_stream): the residual stream, norms, attention scores / weights and routers
// are f32; activations travel between kernels as f32 rows; weights are bf16 [n, k] in HBM.  `bf16_products` != 0: a matrix product rounds its activation
// operand to bf16 (weights are bf16 already) and accumulates in f32 -- the serving precision; 0: every product is a true f32 product.
//   k_stream32.hip           embedding rows, dynamic-tanh norm + token shift, depth mix, the full-precision linear, score-routed experts
//   k_linear_mfma.hip        the full-precision linear on the matrix cores (bf16 products, prefill-sized row counts)
//   k_latent_attention.hip   latent normalisation + cache append, the latent-space attention core (prompt rows and decode rows)
//   k_window_attention.hip   rotation + key / value cache append, attention over cached keys and values (grouped heads, score cap, window, sinks)
//   k_retention.hip          retention: the decayed outer-product state (token by token and in chunks), per-head RMS division + gate
//   k_gated_lru.hip          the gated linear recurrent unit: short causal convolution over a carried window, gates / decays / state update
//   k_causal_conv.hip        a causal per-channel convolution of row blocks over a carried window (sublayer inputs, the delta rule's q / k / v), per-head norm + gate
//   k_channel_delta.hip      the gated delta rule with a decay per head and key channel
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/uzu_hip.h"

namespace uzu {
namespace k {

// One sequence's share of a batched pass: its rows are row0 .. row0 + count - 1 of the pass, at positions start .. start + count - 1 of the sequence.
struct SeqSpan {
    uint32_t row0, count, start;
};

// out[r, :] = f32(table[token[r], :]) * scale   (table bf16 [vocab, d]; an id >= vocab reads row 0 and the host has refused it before)
uzu_status embed_rows_f32(hipStream_t s, const uint32_t* tokens, const uint16_t* table, float* out, uint32_t rows, uint32_t vocab, uint32_t d, float scale = 1.0f);

// RMS norm with one gain: out[r, :] = gain * x[src(r), :] / sqrt(mean(x[src(r), :]^2) + eps),   src(r) = row_index ? row_index[r] : r.
// scales (f32 [d], optional) multiplies per coordinate on top, as (scales[i] + offset): a weight stored around zero has offset 1.  The row's sum of squares is
// taken in a fixed order.
// groups > 1: the row is cut into that many equal consecutive parts and each part is divided by its own root mean square.
uzu_status rms_norm_rows(hipStream_t s, const float* x, float* out, const float* scales, float gain, float eps, const uint32_t* row_index, uint32_t rows, uint32_t d,
                         float offset = 0.0f, uint32_t groups = 1);

// out[r, :] = f32(table[token[r], :]) * scale + f32(pair_table[pair(r), :]): a second table indexed by a hash of (previous token, token),
//   pair(r) = (before * mul_prev + token * mul_cur) mod buckets, before = the token in front of r in its sequence -- of this pass, or (at the pass's first row)
//   the sequence's state *prev[z]; a sequence's position 0 reads row `buckets` (pair_table bf16 [buckets + 1, d]).  A second launch leaves every sequence's
//   last token of the pass in *prev[z].
struct EmbedPairParams {
    const uint32_t* tokens;
    const uint16_t *table, *pair_table;
    float* out;
    uint32_t rows, vocab, d;
    float scale;
    uint32_t buckets, mul_prev, mul_cur;
    const SeqSpan* spans;
    const uint32_t* row_seq;
    uint32_t* const* prev; // device array [nseq] of device pointers
    uint32_t nseq, max_count; // max_count (the longest share of the pass, 0 = unknown) == 1: no second launch, the row's own workgroup stores the token
};
uzu_status embed_pair_rows_f32(hipStream_t s, const EmbedPairParams& p);

// A sublayer's result joins the stream behind its own norm:  out[r, :] = residual[r, :] + y[r, :] / sqrt(mean(y[r, :]^2) + eps) * (scales + offset) * layer_scale
// (scales f32 [d]; layer_scale f32 [d] or null; out may alias residual).  The same fixed-order sum of squares as rms_norm_rows.  With `next` the launch also leaves
// the norm of the new row for the sublayer that follows: next[r, :] = out[r, :] / sqrt(mean(out[r, :]^2) + next_eps) * (next_scales + next_offset).
uzu_status rms_norm_add_rows(hipStream_t s, const float* y, const float* residual, float* out, const float* scales, float offset, const float* layer_scale, float eps,
                             uint32_t rows, uint32_t d, float* next = nullptr, const float* next_scales = nullptr, float next_offset = 0.0f, float next_eps = 0.0f,
                             uint32_t groups = 1); // groups > 1: y is normed in that many equal consecutive parts (no `next` then)

// Dynamic-tanh norm, optionally followed by the token shift:
//   h[r]   = tanh(alpha * x[src(r)]) * scales + biases          src(r) = row_index ? row_index[r] : r
//   out[r] = shift ? h[r] + (h[r - 1 of the same sequence] - h[r]) * shift : h[r]
// The predecessor of a sequence's first row of the pass is prev[seq] (f32 [d], the state; zeros are used instead at position 0); the launch leaves the
// sequence's last h there.  shift == nullptr: spans / row_seq / prev are unused.
struct DynTanhParams {
    const float* x;
    float* out;
    const float* scales;
    const float* biases;
    float alpha;
    const float* shift;
    const uint32_t* row_index;
    const SeqSpan* spans;
    const uint32_t* row_seq;
    float* const* prev; // device array [nseq] of device pointers
    uint32_t rows, d;
};
uzu_status dyn_tanh_norm(hipStream_t s, const DynTanhParams& p);

// out[r, :] = sum_{j < count} w[j] * slots[j * slot_stride + r * d ...]
uzu_status depth_mix(hipStream_t s, const float* slots, size_t slot_stride, const float* w, uint32_t count, float* out, uint32_t rows, uint32_t d);

// Y[z][r, n] = act(sum_k X[z][r, k] * W[z][n, k] + bias[n]) + residual[r, n]        z < batch (grid.z): a batch of independent products of one shape
//   X[z] = x + z * x_batch (row pitch ldx), W[z] = w + z * w_batch ([n, k] bf16), Y[z] = y + z * y_batch (row pitch ldy)
//   act: 0 none, 1 max(.,0)^2, 2 gelu (tanh form).  residual (pitch ldr, only with batch == 1) may alias y.
struct LinearF32Params {
    const float* x;
    const uint16_t* w;
    const uint16_t* bias; // bf16 [n] or null
    const float* residual;
    float* y;
    uint32_t rows, n, k;
    uint32_t ldx, ldy, ldr;
    uint32_t batch;
    size_t x_batch, w_batch, y_batch; // element strides
    uint32_t act;
    uint32_t bf16_products;
    float y_scale;     // != 0: the product (behind bias and act, before the residual) is multiplied by it
    float soft_cap;    // != 0: ... and then capped, cap * tanh(v / cap) (the read-out's logit cap)
    const float* gate; // batched products: product z of row r is multiplied by sigmoid(gate[r * ldgate + z]) (a scalar gate per head); null = none
    uint32_t ldgate;
    // a multiplier per (row's token, column) behind all of that: y[r, n] *= f32(mul_table[token[r] * mul_ld + mul_col0 + n])  (bf16 table, an id >= mul_vocab reads
    // row 0; one product per launch; null = none) -- the gate of a per-layer token input
    const uint16_t* mul_table;
    const uint32_t* mul_tokens;
    uint32_t mul_ld, mul_col0, mul_vocab;
    // Grouped form (matrix-core kernel only; the experts of a mixture, each with its own bucket of rows): product z covers rows row_offsets[z] ..
    // row_offsets[z + 1] - 1 of X and Y (device array [batch + 1]; x_batch / y_batch unused, `rows` = an upper bound of the total for the grid).
    const uint32_t* row_offsets;
    // row r of X is x[row_map[r]] (device array, or null): a gather folded into the operand load
    const uint32_t* row_map;
};
uzu_status linear_f32(hipStream_t s, const LinearF32Params& p, const char** variant = nullptr);
// the matrix-core form (k_linear_mfma.hip): bf16 products only; false = shape / mode not covered, nothing launched
bool linear_mfma_supported(const LinearF32Params& p);
uzu_status linear_mfma(hipStream_t s, const LinearF32Params& p);
size_t linear_f32_bytes(const LinearF32Params& p);

// Score routing: per row scores = softmax(router x) over all `outputs` (= routed + identity) in f32, the `top` largest (score + bias) win (ties: lower index),
// weights = score / (sum of the winners' scores + 1e-20).  ids [rows, top] (>= routed: an identity expert), weights f32 [rows, top].
uzu_status moe_route_scores(hipStream_t s, const float* x, const uint16_t* router, const float* selection_bias, int32_t* ids, float* weights, uint32_t rows, uint32_t d,
                            uint32_t outputs, uint32_t top);
// Top-k routing: per row logits z = router x + bias (f32; bias bf16 [outputs] or null), the `top` largest win (ties: lower index); weights = softmax over the
// winners' logits (renorm != 0) or the logits themselves.  ids / weights [rows, top], winners by falling logit.
uzu_status moe_route_topk(hipStream_t s, const float* x, const uint16_t* router, const uint16_t* router_bias, int32_t* ids, float* weights, uint32_t rows, uint32_t d,
                          uint32_t outputs, uint32_t top, uint32_t renorm);
// The gated product of an expert's hidden unit: g = clamp(gate, gate_min, gate_max), u = clamp(up, up_min, up_max), g * sigmoid(alpha * g) * (u + up_offset).
// The default is silu(gate) * up.
// gelu != 0: the gate's activation is the tanh form of gelu instead of g * sigmoid(alpha * g).
struct ExpertAct {
    float alpha = 1.0f, gate_min = -INFINITY, gate_max = INFINITY, up_min = -INFINITY, up_max = INFINITY, up_offset = 0.0f;
    uint32_t gelu = 0;
};
// The gated product of a dense block: hidden[r, f] = act(gate = y1[r, ff + f], up = y1[r, f])   (y1 f32 [rows][2 ff]: up rows first, as the packed projection yields them)
uzu_status gated_act_rows(hipStream_t s, const float* y1, float* hidden, uint32_t rows, uint32_t ff, const ExpertAct& act);

// hidden[r * top + j, f] = act(gate_e x_r, up_e x_r) for e = ids[r, j] < routed; w13 bf16 [routed][2 ff][d], rows [0, ff) of an expert = up, [ff, 2 ff) = gate
uzu_status moe_experts_gate_up(hipStream_t s, const float* x, const int32_t* ids, const uint16_t* w13, float* hidden, uint32_t rows, uint32_t d, uint32_t ff, uint32_t routed,
                               uint32_t top, uint32_t bf16_products, const ExpertAct& act = ExpertAct());
// y[r, :] = residual[r, :] + sum_j weights[r, j] * (ids[r, j] < routed ? down_e hidden[r * top + j] : x[r, :])   in slot order; w2 bf16 [routed][d][ff]; y may alias residual
uzu_status moe_experts_down_combine(hipStream_t s, const float* hidden, const float* x, const int32_t* ids, const float* weights, const uint16_t* w2, const float* residual,
                                    float* y, uint32_t rows, uint32_t d, uint32_t ff, uint32_t routed, uint32_t top, uint32_t bf16_products);

// The same block for prefill-sized row counts with bf16 products: the (row, slot) pairs are bucketed by expert (counts -> offsets -> positions), every expert runs
// its bucket through the matrix-core linear as one grouped launch (gate | up, then down), and the rows are combined in slot order.  Workspaces: y1
// [rows * top][2 ff], hidden [rows * top][ff], y2 [rows * top][d] f32; perm / slot_pos [rows * top], offsets [routed + 1], cursor [routed] u32.
struct MoeGroupedParams {
    const float* x;
    const int32_t* ids;
    const float* weights;
    const uint16_t *w13, *w2;
    const float* residual;
    float* y;
    float *y1, *hidden, *y2;
    uint32_t *perm, *slot_pos, *offsets, *cursor;
    uint32_t rows, d, ff, routed, top;
    ExpertAct act;
};
bool moe_experts_grouped_supported(const MoeGroupedParams& p);
uzu_status moe_experts_grouped(hipStream_t s, const MoeGroupedParams& p);

// RMS norm of the latent rows (x / sqrt(mean(x^2) + eps) * scales) and append to the sequences' caches: row r goes to cache[seq(r)] + (position of r) * rank,
// stored as bf16 (cache_bf16) or f32.
uzu_status latent_norm_append(hipStream_t s, const float* x, const float* scales, float eps, void* const* caches, uint32_t cache_bf16, const SeqSpan* spans,
                              const uint32_t* row_seq, uint32_t rows, uint32_t rank);

// Latent-space attention core.  Row r (sequence q, position t) and head h: keys j = max(0, t - window + 1) .. t (window 0: from 0),
//   s_j = scale * <qlat[r, h, :], c_j>,  weights = exp(s_j - m) / (sum_j exp(s_j - m) + exp(sink_h - m)),  out[r, h, :] = sum_j weights_j c_j
// qlat / out f32 [rows, heads * rank]; c_j = caches[q][j * rank ...] (bf16 or f32); sinks f32 [heads] or null (no sink term).
struct LatentAttentionParams {
    const float* qlat;
    float* out;
    void* const* caches;
    uint32_t cache_bf16;
    const float* sinks;
    const SeqSpan* spans;
    const uint32_t* row_seq;
    uint32_t rows, heads, rank, window;
    float scale;
    uint32_t form; // 0: chosen by shape; 1: the simple form (a wave per row and head, keys one after the other); 2: the tiled form
    // != 0: only the first value_rank columns of a cache row are values -- the rest (a rotated key part) takes part in the scores alone, and the matching columns of
    // `out` are left unwritten by the tiled form (a multiple of 4, at most rank); 0: the whole row
    uint32_t nseq;  // entries of `spans`
    uint32_t tiles; // sum over the sequences of ceil(count * heads / 128): the tiled form's workgroups (the caller knows the counts)
    uint32_t value_rank;
    // tiled form, few rows over many keys (decode): `splits` > 1 workgroups share the key blocks of an item tile, partial sums go through split_ws
    // (latent_attention_split_ws_bytes(rows, heads, rank, splits) bytes) and a merge launch.  0 / null: one workgroup walks all keys of its tile.
    uint32_t splits;
    float* split_ws;
    size_t split_ws_bytes;
};
size_t latent_attention_split_ws_bytes(uint32_t rows, uint32_t heads, uint32_t rank, uint32_t splits);
bool latent_attention_tiled_supported(const LatentAttentionParams& p);
uzu_status latent_attention(hipStream_t s, const LatentAttentionParams& p);
constexpr uint32_t kLatentMaxRank = 2048;

// What stands between the packed projection and the latent-space core when the cache row carries a rotated key part: row r of `x` (f32, pitch ldx) holds the down
// projection's rank + rope_dim numbers at column c_col and the queries [heads][q_width] at column 0, the last rope_dim coordinates of a query head being its
// rotated part.  The latent (first rank numbers) is RMS-normed with `scales`; the rope_dim numbers behind it turn by the row's position (tables f32
// [positions][rope_dim] as rope_append reads them; interleaved: pairs (2i, 2i + 1), else (i, i + rope_dim / 2)) and are NOT normed; [latent | rotated part] goes to
// row t of the sequence's cache (width rank + rope_dim, bf16 or f32).  Every query head's rotated part turns the same way and lands in
// qlat[r, head, rank .. rank + rope_dim) (qlat f32 [rows][heads][rank + rope_dim]; the first rank columns of a head are filled by the folded key projection).
// rope_dim == 0: normalisation + append alone.
struct LatentRopeAppendParams {
    const float* x;
    uint32_t ldx, c_col, rank, rope_dim;
    const float* scales;
    float eps;
    void* const* caches;
    uint32_t cache_bf16;
    uint32_t heads, q_width;
    float* qlat;
    const float *cosines, *sines;
    uint32_t interleaved;
    const SeqSpan* spans;
    const uint32_t* row_seq;
    uint32_t rows;
};
uzu_status latent_rope_append(hipStream_t s, const LatentRopeAppendParams& p);

// Rotation of queries and keys, key scaling, and the append of keys and values to the sequences' caches -- what stands between the packed projection and the
// mixer's core.  Row r of `qkv` (f32, pitch ld) holds queries [heads][dim] at column 0, keys [kv_heads][dim] at column k_col and values [kv_heads][vdim] at
// column v_col.  The first rope_dim coordinates of every query and key head turn by the angle of the row's position t: with half = rope_dim / 2,
//   (a_i, a_(i+half)) <- (a_i cos[t, i] - a_(i+half) sin[t, i], a_(i+half) cos[t, i] + a_i sin[t, i])      (tables f32 [positions][rope_dim])
// and keys are multiplied by key_scale afterwards.  Queries are replaced in place.  With caches (key_caches / value_caches: device arrays [nseq] of pointers to
// [positions][kv_heads * dim] and [positions][kv_heads * vdim], bf16 or f32) rotated keys and values go to row t of the sequence's caches; without (null) the
// keys are replaced in place and values stay where they are.  kv_heads == 0: the row carries queries only (a layer that reads another layer's cache).
// q_norm / k_norm (f32 [dim], optional): every query / key head is RMS-normed over its dim coordinates (norm_eps, plain weights) in front of the rotation.
// Values go to the cache first, as the projection left them: v_col == k_col (vdim == dim) makes the values the keys in front of their norm and rotation.
struct RopeAppendParams {
    float* qkv;
    uint32_t ld, k_col, v_col;
    uint32_t heads, kv_heads, dim, vdim, rope_dim;
    const float *cosines, *sines;
    float key_scale;
    const float *q_norm, *k_norm;
    float norm_eps;
    uint32_t norm_whole;  // q_norm / k_norm are f32 [heads * dim] / [kv_heads * dim]: ONE RMS norm over all of a row's query (key) coordinates instead of one per head
    uint32_t interleaved; // the rotation pairs coordinates (2i, 2i + 1) instead of (i, i + rope_dim / 2)
    void* const* key_caches;
    void* const* value_caches;
    uint32_t cache_bf16;
    const SeqSpan* spans;
    const uint32_t* row_seq;
    uint32_t rows;
};
uzu_status rope_append(hipStream_t s, const RopeAppendParams& p);

// Attention over cached keys and values.  Row r (sequence z, position t), query head a, key / value head g = a / (heads / kv_heads):
//   keys j = max(0, t - window + 1) .. t (window 0: from 0),  s_j = scale <q[r, a, :], K_z[j, g, :]>,  s_j <- cap tanh(s_j / cap) (cap != 0),
//   p_j = exp(s_j - m) / (sum_j exp(s_j - m) + exp(sink_a - m))   (sinks f32 [heads] or null: no sink term),   out[r, a, :] = sum_j p_j V_z[j, g, :]
// q f32 rows of pitch ldq (head a at column a * dim), out f32 [rows][heads * vdim]; caches as rope_append writes them.
struct WindowAttentionParams {
    const float* q;
    uint32_t ldq;
    float* out;
    void* const* key_caches;
    void* const* value_caches;
    uint32_t cache_bf16;
    const float* sinks;
    const SeqSpan* spans;
    const uint32_t* row_seq;
    uint32_t rows, heads, kv_heads, dim, vdim, window;
    float scale, soft_cap;
    // chunk != 0: the row at position t sees keys j <= t of its own chunk only, j >= floor(t / chunk) * chunk (chunks counted from position 0 of the sequence).
    // head_scale (f32 [heads] or null): the scaled score of head a is multiplied by head_scale[a].  dist_bias (f32 [dist_rows][heads] or null): dist_bias[min(t - j,
    // dist_rows - 1), a] is added behind scale, head_scale and cap.  gate (f32 rows of pitch ldgate or null): out[r, a, :] is multiplied by sigmoid(gate[r, a]).
    uint32_t chunk;
    const float* head_scale;
    const float* dist_bias;
    uint32_t dist_rows;
    const float* gate;
    uint32_t ldgate;
    uint32_t form;  // 0: chosen by shape; 1: the simple form (a wave per row and head); 2: the matrix-core form
    uint32_t nseq;  // entries of `spans`
    uint32_t tiles; // sum over the sequences of ceil(count * (heads / kv_heads) / 128): the matrix-core form's item tiles (the caller knows the counts)
    // matrix-core form, few rows over many keys (decode): `splits` > 1 workgroups share the key blocks of an item tile, partial sums go through split_ws
    // (window_attention_split_ws_bytes(rows, heads, splits) bytes) and a merge launch.  0 / null: one workgroup walks all keys of its tile.
    uint32_t splits;
    float* split_ws;
    size_t split_ws_bytes;
};
size_t window_attention_split_ws_bytes(uint32_t rows, uint32_t heads, uint32_t splits);
bool window_attention_mfma_supported(const WindowAttentionParams& p);
uzu_status window_attention(hipStream_t s, const WindowAttentionParams& p);

// Retention.  Row r (sequence z, position t), head a, with q, k [heads][dim] and v [heads][vdim] taken from the f32 rows `qkv` (pitch ld; columns q_col, k_col,
// v_col; q and k rotated and k scaled already):   S <- decay[a] S + k v^T,   out[r, a, :] = S^T q.
// states: device array [nseq] of pointers to f32 [heads][dim][vdim], the sequences' states, read at the pass's first row (zero instead when the span starts at
// position 0) and left behind its last.  Every sum runs in the same order whatever else the pass carries.  form 0: chosen by the sequence's row count; 1: token
// by token; 2: in chunks of 64 rows (scores of the chunk's own rows + the carried state, a decayed state update per chunk; head widths up to 128 on the matrix
// cores with f32 operands); 3: the chunks without the matrix cores.
struct RetentionParams {
    const float* qkv;
    uint32_t ld, q_col, k_col, v_col;
    float* out; // [rows][heads * vdim]
    float* const* states;
    const float* decay; // f32 [heads]
    const SeqSpan* spans;
    uint32_t nseq, rows, heads, dim, vdim;
    uint32_t form;
    // the chunked form: chunks = sum over the sequences of ceil(count / 64) (the caller knows the counts) and a workspace of
    // retention_chunk_ws_bytes(chunks, heads, dim, vdim) bytes; without one, form 0 goes token by token
    uint32_t chunks;
    float* chunk_ws;
    size_t chunk_ws_bytes;
};
size_t retention_chunk_ws_bytes(uint32_t chunks, uint32_t heads, uint32_t dim, uint32_t vdim);
bool retention_supported(uint32_t dim, uint32_t vdim);
uzu_status retention(hipStream_t s, const RetentionParams& p);

// Per head: x[r, a, :] <- x[r, a, :] / sqrt(mean(x[r, a, :]^2) + eps) * silu(gate[r, a * width ...])   (x f32 [rows][heads * width] in place; gate f32 rows of
// pitch ldg; gate == null: the division alone)
uzu_status head_rms_gate(hipStream_t s, float* x, const float* gate, uint32_t ldg, float eps, uint32_t rows, uint32_t heads, uint32_t width);

// Gated linear recurrent unit behind a short causal convolution (k_gated_lru.hip).  Row r (sequence z, position t) of `branches` (f32, pitch ld) holds the gate
// branch's `width` numbers at column 0 and the recurrent branch's at column x_col.
//   lru_conv:  u[r, c] = conv_b[c] + sum_j conv_w[c, j] * xin(t - (taps - 1) + j, c)     xin = the recurrent branch of the sequence's earlier rows: of this pass, or
//              (in front of the pass) the taps - 1 inputs the state keeps ([taps - 1][width] f32, oldest first), or zero in front of position 0.  u f32 [rows][width].
//   lru_scan:  with g = the gate pre-activations [rows][blocks][2 bw] (recurrence gate's bw numbers, then the input gate's) and their biases,
//              a = exp(-rate * sigmoid(g_r + b_r) * softplus(lambda)),  S <- a S + sqrt(1 - a^2) * sigmoid(g_i + b_i) * u,  out[r, c] = S * gelu_tanh(gate branch);
//              S starts from the sequence's state (zero at position 0) and is left there behind the pass's last row, and so are the last taps - 1 inputs.
//              All f32.  form 0: chosen by the row count; 1: position by position; 2: in pieces of 32 rows, each scanned from zero with its decay product,
//              the pieces' carries joined in order (differs from form 1 by f32 rounding only); needs `pieces` = sum over the sequences of ceil(count / 32) and a
//              workspace of lru_piece_ws_bytes(pieces, width) bytes, without which form 0 goes position by position.
struct GatedLruParams {
    const float* branches;
    uint32_t ld, x_col;
    float* u;            // [rows][width]
    const float* gates;  // [rows][2 width]
    float* out;          // [rows][width]
    const float *conv_w, *conv_b, *gate_b, *lambda;
    float rate;
    float* const* states;      // device array [nseq]: f32 [width]
    float* const* conv_states; // device array [nseq]: f32 [taps - 1][width]
    const SeqSpan* spans;
    const uint32_t* row_seq;
    uint32_t nseq, rows, width, blocks, taps;
    uint32_t form;
    uint32_t max_count; // the longest sequence share of the pass (the caller knows the counts)
    uint32_t pieces;
    float* piece_ws;
    size_t piece_ws_bytes;
};
size_t lru_piece_ws_bytes(uint32_t pieces, uint32_t width);
uzu_status lru_conv(hipStream_t s, const GatedLruParams& p);
uzu_status lru_scan(hipStream_t s, const GatedLruParams& p);

// A causal convolution over positions on every channel of a block of rows (k_causal_conv.hip).  Row r (sequence z, position t), channel c:
//   out[r, o_col + c] = act(bias[c] + sum_j w[c, j] * xin(t - (taps - 1) + j, c))  (+ x[r, x_col + c] with add_input: a sublayer that reads h + conv(h))
// xin = channel c of the sequence's input rows `x` (f32, pitch ldx, column x_col): of this pass, or (in front of the pass) the taps - 1 inputs the state keeps
// (states[z] + state_offset: f32 [taps - 1][channels], oldest first), or zero in front of position 0.  w f32 [channels][taps]: the last tap weighs the row itself.
// act: 0 none, 1 silu.  `out` is another block of rows than `x`.  causal_conv_commit leaves the last taps - 1 inputs behind the pass in the state; it reads the
// same `x`, which must still hold the pass's inputs.  A sequence that brings one row has its window replaced by causal_conv_rows itself; max_count (the longest
// share of the pass, 0 = unknown) == 1 makes causal_conv_commit a no-op.
struct CausalConvParams {
    const float* x;
    uint32_t ldx, x_col;
    float* out;
    uint32_t ldo, o_col;
    const float *w, *bias;
    uint32_t channels, taps, add_input, act;
    float* const* states; // device array [nseq]
    size_t state_offset;  // floats
    const SeqSpan* spans;
    const uint32_t* row_seq;
    uint32_t nseq, rows, max_count;
};
uzu_status causal_conv_rows(hipStream_t s, const CausalConvParams& p);
uzu_status causal_conv_commit(hipStream_t s, const CausalConvParams& p);

// Per head, in place: x[r, a, :] <- x[r, a, :] / sqrt(mean(x[r, a, :]^2) + eps) * weight[:] * gate(g[r, a, :])    (x f32 rows of pitch ldx, heads * width used;
// weight f32 [width] or null; g f32 rows of pitch ldgate or null; gate = sigmoid (gate_sigmoid) or silu)
struct HeadNormGateParams {
    float* x;
    uint32_t ldx;
    const float* weight;
    const float* gate;
    uint32_t ldgate, gate_sigmoid;
    float eps;
    uint32_t rows, heads, width;
};
uzu_status head_norm_gate_rows(hipStream_t s, const HeadNormGateParams& p);

// The gated delta rule with a decay per head and key channel (k_channel_delta.hip).  Row r (sequence z) of `qkv` (f32, pitch ld) holds queries [groups][dim] at
// q_col, keys [groups][dim] at k_col and values [heads][vdim] at v_col (behind their convolution and silu); value head a reads group a / (heads / groups).
//   channel_delta_prep (in place):  q <- q / sqrt(sum q^2 + unit_eps) * dim^(-1/2),  k <- k / sqrt(sum k^2 + unit_eps)  per head;
//                                   beta[r, a] <- sigmoid(beta[r, a]);   decay[r, a, c] <- exp(-exp(a_log[a]) * softplus(decay[r, a, c] + dt_bias[a, c]))
//   channel_delta:                  per head, row after row:  S <- decay * S (rows = key channels),  u = beta (v - S^T k),  S <- S + k u^T,  out[r, a, :] = S^T q
// states: device array [nseq] of pointers to f32 [heads][dim][vdim], read at the pass's first row (zeros instead when the span starts at position 0) and left
// behind its last.  decay f32 [rows][heads * dim], beta f32 rows of pitch ldbeta, out f32 [rows][heads * vdim].  All f32; every sum runs in the same order
// whatever else the pass carries and however the rows were cut into passes.
struct ChannelDeltaParams {
    float* qkv;
    uint32_t ld, q_col, k_col, v_col;
    float* decay;
    float* beta;
    uint32_t ldbeta;
    const float *a_log, *dt_bias;
    float unit_eps;
    float* out;
    float* const* states;
    const SeqSpan* spans;
    uint32_t nseq, rows, heads, groups, dim, vdim;
};
bool channel_delta_supported(uint32_t dim, uint32_t vdim);
uzu_status channel_delta_prep(hipStream_t s, const ChannelDeltaParams& p);
uzu_status channel_delta(hipStream_t s, const ChannelDeltaParams& p);

} // namespace k
} // namespace uzu
