/*
 * uzu_model_desc.h -- plain-C description of a decoder-only language model as uzu's
 * `encodable_block` layer sees it after `Engine::load_language_model`
 * (crates/backend-uzu/src/engine/language_model/mod.rs:58-116).
 *
 * It is the in-memory equivalent of `config.json` + `model.safetensors`: the same numbers the
 * reference's `config/**` structs carry, and host pointers to tensors in the reference's on-disk
 * layouts.  Both the HIP engine (include/uzu_hip_engine.h) and the CPU
 * oracle (oracle/) consume this struct, so a parity test hands the SAME bytes to both.
 *
 * All pointers are HOST pointers, owned by the caller, and only need to stay valid for the
 * duration of the `*_model_create` call that receives them.
 */
#ifndef UZU_MODEL_DESC_H
#define UZU_MODEL_DESC_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* backends/common/gpu_types/quantization_method.rs:4-9 */
typedef enum {
    UZU_QUANT_SCALE_BIAS = 0,       /* MLXSpec: deq = scale*q + bias                  */
    UZU_QUANT_SCALE_ZERO_POINT = 1, /* IntSpec asymmetric: deq = scale*q - scale*zp   */
    UZU_QUANT_SCALE_SYMMETRIC = 2,  /* IntSpec symmetric: deq = scale*q - scale*2^(b-1) */
    UZU_QUANT_NONE = 3              /* FullPrecisionSpec: bf16 weights [n,k]          */
} uzu_quant_method;

/* backends/common/gpu_types/activation_type.rs:8-14 */
typedef enum {
    UZU_ACT_SILU = 0,
    UZU_ACT_GELU_APPROX = 1,
    UZU_ACT_GELU_EXACT = 2,
    UZU_ACT_IDENTITY = 3,
    UZU_ACT_SOFTPLUS = 4,
    UZU_ACT_RELU_SQUARED = 5 /* max(z, 0)^2: the plain (ungated) dense MLP of an f32-stream design (uzu_layer_desc::mlp_plain) */
} uzu_activation_type;

/*
 * One `Linear` (encodable_block/linear/matmul.rs:39-47) = WeightMatrix in Layout::OutputInput
 * (encodable_block/weight_matrix.rs:101-162):
 *   weights      u8  [n, k/pack]            pack = 2 (4 bit, low nibble = even k) or 1 (8 bit)
 *   scales       bf16 [n, ceil(k/group)]
 *   biases       bf16 [n, ceil(k/group)]                  (ScaleBias only)
 *   zero_points  u8  [n, ceil(groups/pack)]               (ScaleZeroPoint only; 4 bit: nibble packed)
 *   out_biases   bf16 [n]                                 (Linear `biases`, optional)
 * method == UZU_QUANT_NONE: weights is bf16 [n,k], bits == 16, everything else NULL.
 * HybridSpec { incoherence_processing_mode: InputOutput, block 32, no adapter } (RHTLinearWrapper, linear/rht_wrapper.rs:140-298):
 *   input_signs  i32 [k], output_signs i32 [n] (+-1): y = OutputRht(W InputRht(x)) + out_biases; NULL = a plain linear.
 * Embedding tables (encodable_block/embedding.rs:126-341) reuse the struct with their own reading of the sign vectors:
 *   `embedding` / input table, HybridSpec { Output, block 32 }: output_signs i32 [model_dim]: lookup = OutputRht(dequantised row); a TIED
 *   table's read-out takes InputRht(row, the same signs) in front of the matmul (embedding.rs:161-188, 385-400);
 *   `output_embedding`, HybridSpec { Input, block 32 }: input_signs i32 [model_dim]: read-out = W InputRht(x) (embedding.rs:243-283).
 */
typedef struct {
    uint32_t n;          /* output_dim */
    uint32_t k;          /* input_dim */
    uint32_t bits;       /* 4, 8 or 16 */
    uint32_t group_size; /* 0 for full precision */
    uint32_t method;     /* uzu_quant_method */
    uint32_t reserved;
    const void* weights;
    const uint16_t* scales;
    const uint16_t* biases;
    const uint8_t* zero_points;
    const uint16_t* out_biases;
    const int32_t* input_signs;
    const int32_t* output_signs;
    /* HybridSpec { adapter_spec: LowRankSpec { rank } } (QLoRALinearWrapper, linear/qlora_wrapper.rs:61-252): bf16 adapters next to the
     * quantized base; y = [OutputRht]( W [InputRht](x) + (x down^T) up^T ); lora_rank == 0 = no adapter.  The sign vectors are optional
     * here (incoherence_block_size None); out_biases must be NULL (the reference asserts it). */
    uint32_t lora_rank;
    uint32_t reserved2;
    const uint16_t* adapter_down; /* bf16 [rank, k]  (weights.adapter.down_projection) */
    const uint16_t* adapter_up;   /* bf16 [n, rank]  (weights.adapter.up_projection) */
} uzu_linear_desc;

/* config/normalization.rs:10-18 + tensor `scales` f32 [dim] (encodable_block/normalization.rs:67-74) */
typedef enum {
    UZU_NORM_STATISTICS = 0,   /* RMS / mean-variance normalisation (the reference's Normalization) */
    UZU_NORM_DYNAMIC_TANH = 1, /* no statistics: y = tanh(alpha * x) * scales + biases, element by element (f32-stream designs) */
    UZU_NORM_RMS_SCALAR = 2    /* y = alpha * x / sqrt(mean(x^2) + epsilon): RMS norm with ONE gain for all coordinates (alpha; no scales tensor) (f32-stream designs) */
} uzu_norm_kind;
typedef struct {
    uint32_t present;       /* 0 => this optional norm is absent */
    uint32_t full_layer;    /* UpcastMode::FullLayer (1) vs OnlyNormalization (0) */
    uint32_t subtract_mean; /* LayerNorm-style mean subtraction */
    uint32_t kind;          /* uzu_norm_kind (the field was `reserved`: 0 = the reference's Normalization) */
    float epsilon;
    float scale_offset;     /* Option<f32>::unwrap_or(0.0) */
    const float* scales;    /* f32 [dim] or NULL (has_scale == false) */
    const float* biases;    /* f32 [dim] or NULL */
    float alpha;            /* UZU_NORM_DYNAMIC_TANH: the scalar inside the tanh; UZU_NORM_RMS_SCALAR: the gain */
    uint32_t groups;        /* f32-stream designs, UZU_NORM_STATISTICS: the row is cut into `groups` equal consecutive parts, each divided by its own root mean
                               square (dim % groups == 0); 0 or 1 = the whole row (the field was `reserved`) */
} uzu_norm_desc;

typedef enum {
    UZU_MIXER_ATTENTION = 0,
    UZU_MIXER_DELTA_NET = 1,
    /* Attention over a cached low-rank latent (f32-stream designs): per token only c = RMSNorm(W_down h) [latent_rank] is kept; a head's keys and values are
     * W_up_k c and W_up_v c, so scores and the weighted sum run in latent space (q W_up_k applied to the query, W_up_v to the result).  No rotation.  Reuses the
     * attention fields: num_heads, head_dim (query / key width per head), attention_scale, sliding_window_size, has_sinks / sinks, is_kv_sharing +
     * kv_source_layer_index (the sharing layer reads the source layer's cached latents through its OWN up projections), qkv_projection (queries only,
     * n = heads * head_dim), out_projection (k = heads * value_head_dim); and the latent_* fields at the end of uzu_layer_desc. */
    UZU_MIXER_LATENT_ATTENTION = 2,
    /* Retention (f32-stream designs): linear attention with a fixed decay per head and neither softmax nor denominator.  Per head a: S_t = decay[a] S_(t-1) +
     * k_t v_t^T (f32 [head_dim, value_head_dim], the sequence state, zero at position 0), o_t = S_t^T q_t; every head's o_t is divided by its root mean square
     * (head_norm_epsilon, no weights), the heads are concatenated, multiplied by silu(gate h) and projected.  q and k are rotated (use_rope) and k is multiplied
     * by key_scale behind its rotation.  Fields: num_heads, head_dim, value_head_dim, retention_decay, qkv_projection (rows: queries | keys | values | gate,
     * n = 2 heads head_dim + 2 heads value_head_dim), out_projection (k = heads * value_head_dim). */
    UZU_MIXER_RETENTION = 3,
    /* Gated linear recurrent unit behind a short causal convolution (f32-stream designs): two branches of lru_width channels from ONE packed projection
     * (qkv_projection rows: gate branch | recurrent branch, n = 2 lru_width, with out_biases).  The recurrent branch runs through a per-channel causal convolution
     * (dn_kernel_size taps, dn_conv_weights f32 [lru_width, taps], the last tap weighs the current position, dn_conv_biases f32 [lru_width]) giving u; the channels
     * are split into lru_blocks equal blocks with two square gate matrices each (lru_gate_weights bf16 [blocks][2 bw][bw], bw = lru_width / lru_blocks: the
     * recurrence gate's rows, then the input gate's; lru_gate_biases f32 [blocks][2 bw]): r = sigmoid(A_b u_b + a_b), i = sigmoid(B_b u_b + b_b).  With
     * a = exp(-lru_decay_rate r softplus(lru_lambda)) the state is S_t = a S_(t-1) + sqrt(1 - a^2) i u (f32 [lru_width], zero in front of position 0) and the
     * mixer's result out_projection(S_t * gelu_tanh(gate branch)) (k = lru_width).  Gates, decays and the state are f32 in both precisions; the sequence state
     * is S and the convolution's last taps - 1 inputs. */
    UZU_MIXER_GATED_LRU = 4
} uzu_mixer_kind;

/* config/rope/*.rs -- every AnyRoPEConfig variant (encodable_block/mixer/attention/rope.rs:13-114) */
typedef enum { UZU_ROPE_NONE = 0, UZU_ROPE_UNSCALED = 1, UZU_ROPE_LLAMA = 2, UZU_ROPE_LINEAR = 3, UZU_ROPE_YARN = 4,
               UZU_ROPE_LONGROPE = 5 } uzu_rope_kind;

typedef struct {
    uint32_t kind;                    /* uzu_rope_kind */
    uint32_t head_dim;                /* rope dim (may be < attention head_dim: partial rotary) */
    uint32_t max_sequence_length;
    uint32_t original_context_length; /* Llama */
    float base;
    float scaling_factor;             /* Llama / Linear */
    float low_frequency_factor;       /* Llama */
    float high_frequency_factor;      /* Llama */
    float beta_fast, beta_slow;       /* YaRN (config/rope/yarn_rope.rs) */
    uint32_t truncate;                /* YaRN */
    uint32_t reserved;
    const float* short_factor;        /* LongRoPE (config/rope/longrope.rs): f32 [head_dim / 2] */
    const float* long_factor;         /* LongRoPE: used when max_sequence_length > original_context_length */
} uzu_rope_desc;

/* MixtureOfExpertsConfig (config/mlp/mixture_of_experts.rs:9-22) + the tensors of the `mlp` subtree of a MoE layer (encodable_block/mlp/moe/mod.rs:114-160),
 * all in the model's data type (bf16), full precision:
 *   router.weights.weights [E, model_dim] (FullPrecisionSpec, Layout::OutputInput), router.biases [E]
 *   experts.up_projection.weights.weights [E, 2*d_ff, model_dim] (rows [0, d_ff) of an expert = up, [d_ff, 2 d_ff) = gate), experts.up_projection.biases [E, 2*d_ff]
 *   experts.down_projection.weights.weights [E, model_dim, d_ff], experts.down_projection.biases [E, model_dim]
 * What MoeBlock::new refuses is refused here as well: shared experts, an expert gate, a block without router / up / down biases, activations other than
 * SiLU / GELUApprox, more than 512 routed or 128 active experts, model_dim % 4 != 0 (mod.rs:84-112). */
typedef struct {
    uint32_t num_routed_experts;
    uint32_t num_active_experts; /* num_active_routed_experts */
    uint32_t expert_hidden_dim;  /* d_ff */
    uint32_t router_renorm;      /* routing_function == SoftmaxRouting: softmax over the k winners (mod.rs:110); else the raw logits */
    uint32_t gating_sel;         /* 2 = SwiGLU (expert activation SILU), 3 = GEGLU (GELUApprox)  (mod.rs:104-108) */
    float silu_alpha;            /* expert_config.activation.alpha() */
    float gate_clip_min, gate_clip_max, up_clip_min, up_clip_max; /* expert_config.{gate,up}_clipping; -inf / +inf = none */
    const uint16_t* router_weights;
    const uint16_t* router_biases;
    const uint16_t* w13;
    const uint16_t* w2;
    const uint16_t* up_biases;
    const uint16_t* down_biases;
    /* Score routing (f32-stream designs; routing == UZU_MOE_ROUTE_SCORES): scores = softmax of the router logits over ALL num_routed_experts +
     * num_identity_experts outputs; the num_active_experts largest (score + selection_bias) win; a winner's weight is its score divided by the winners'
     * score sum (+ 1e-20).  The last num_identity_experts router outputs have no tensors: such an expert returns its input.  No router / expert biases
     * (the bias pointers are NULL); router_weights is [routed + identity, model_dim]. */
    uint32_t routing;              /* uzu_moe_routing; 0 = the reference's top-k of the logits */
    uint32_t num_identity_experts;
    const float* selection_bias;   /* f32 [routed + identity]: added to the scores for the choice only */
    /* expert = down(act(gate) * (up + up_offset)) with the clipping above applied first; 0 = the plain gated product.  In an f32-stream design top-k routing
     * (routing == 0) reads router_biases (bf16 [E], optional), takes the num_active_experts largest logits (ties: the lower index) and, with router_renorm, the
     * softmax over the winners' logits as weights; the experts have no biases. */
    float up_offset;
    uint32_t reserved;
} uzu_moe_desc;
typedef enum { UZU_MOE_ROUTE_TOPK_LOGITS = 0, UZU_MOE_ROUTE_SCORES = 1 } uzu_moe_routing;

typedef enum { UZU_MLP_DENSE = 0, UZU_MLP_MOE = 1 } uzu_mlp_kind;

/* config/transformer_layer.rs:8-21 with AttentionConfig / DeltaNetConfig and a DenseMLPConfig | MixtureOfExpertsConfig */
typedef struct {
    uint32_t mixer_kind; /* uzu_mixer_kind */
    uint32_t hidden_dim; /* MLP hidden (up projection has 2*hidden rows: [up ; gate]) */
    uint32_t activation; /* uzu_activation_type of the gated MLP */
    uint32_t mlp_kind;   /* uzu_mlp_kind (the field was `reserved`: 0 = the dense MLP) */

    uzu_norm_desc pre_mixer_norm;
    uzu_norm_desc post_mixer_norm;
    uzu_norm_desc pre_mlp_norm;
    uzu_norm_desc post_mlp_norm;

    /* --- attention (config/token_mixer/attention.rs:9-29) --- */
    uint32_t num_heads;
    uint32_t num_groups; /* kv heads */
    uint32_t head_dim;
    uint32_t has_gate;   /* gate_projection_config.is_some() */
    float attention_scale; /* 0 => 1/sqrt(head_dim) */
    uint32_t use_rope;
    uzu_linear_desc qkv_projection;  /* n = (heads + 2*groups) * head_dim */
    uzu_linear_desc gate_projection; /* n = heads*head_dim */
    uzu_linear_desc out_projection;  /* k = heads*head_dim */
    uzu_norm_desc query_norm;        /* scales f32 [head_dim] */
    uzu_norm_desc key_norm;
    uint32_t sliding_window_size;    /* 0 = none; causal + window => the ring KV state of mixer/attention/state.rs:20-106 */
    uint32_t has_sinks;
    const void* sinks;               /* bf16 [heads] (mixer.sinks, mixer/attention/mod.rs:162-165) or NULL */

    /* --- gated delta net (config/token_mixer/delta_net.rs) --- */
    uint32_t dn_num_heads;      /* value heads Hv */
    uint32_t dn_num_groups;     /* key heads Hk */
    uint32_t dn_head_dim;       /* Dk (128) */
    uint32_t dn_value_head_dim; /* Dv (128) */
    uint32_t dn_kernel_size;
    float dn_norm_epsilon;
    uzu_linear_desc dn_in_proj;  /* n = 2*Hk*Dk + 2*Hv*Dv + 2*Hv */
    uzu_linear_desc dn_out_proj; /* k = Hv*Dv */
    const float* dn_conv_weights; /* f32 [conv_dim, kernel_size] */
    const float* dn_conv_biases;  /* f32 [conv_dim] or NULL */
    const float* dn_a_log;        /* f32 [Hv] */
    const float* dn_dt_bias;      /* f32 [Hv] */
    const float* dn_norm_scales;  /* f32 [Dv] */

    /* --- dense MLP (encodable_block/mlp/dense.rs) --- */
    uzu_linear_desc up_projection;   /* n = 2*hidden: rows [0,h) = up, [h,2h) = gate */
    uzu_linear_desc down_projection; /* k = hidden */

    /* --- layer options of the Gemma families (config/transformer_layer.rs:16-20, config/token_mixer/attention.rs:26-28);
     *     all zero = none of them.  NB the struct has grown in place over the rounds (it is the element type of uzu_model_desc.layers, so its size is
     *     part of the ABI): uzu_hip_desc_abi() reports the sizes the library was built with -- a caller checks them once (uzu_amd/desc.py does) --- */
    uint32_t rope_index;            /* use_rope != 0: which entry of uzu_model_desc.ropes rotates this layer (transformer.rs:101-118);
                                       ignored when num_ropes == 0 (the single `rope`) */
    uint32_t has_post_layer_scalar; /* transformer_layer.rs:61-84: pre_mlp_norm scales the residual sum, post_mlp_norm (required) its
                                       output -- unless the layer has a PLE projection, which then owns the scalar */
    float post_layer_scalar;        /* tensor `post_layer_scalar` [1] */
    uint32_t is_kv_sharing;         /* AttentionConfig::is_kv_sharing == TransformerLayerConfig::kv_source_layer_index.is_some(): the packed
                                       projection yields queries only (n = heads*head_dim), no key / value norm, no KV append; the
                                       attention reads the source layer's state (mixer/attention/mode.rs:79-84, transformer.rs:264-275) */
    uint32_t kv_source_layer_index; /* an earlier attention layer that owns its state (is_kv_sharing != 0) */
    uint32_t normalize_values;      /* AttentionConfig::value_norm_config(): scale-free RMS norm (eps 1e-6, FullLayer) of the value heads */
    uint32_t has_ple;               /* ple_config.is_some(): PerLayerEmbeddingProjection (per_layer_embedding.rs:150-271) ends the layer */
    uint32_t ple_dim;
    uint32_t ple_activation;        /* uzu_activation_type */
    uint32_t is_non_causal;         /* AttentionConfig::is_causal == false (mixer/attention/mod.rs:166-198, mask.rs:3-61): every suffix row sees every suffix row --
                                       the block attention of a DFlash draft model (encodable_block/dflash.rs).  0 = causal (the field was `reserved3`: same layout) */
    uzu_linear_desc ple_gate;       /* ple.gate: n = ple_dim, k = model_dim */
    uzu_linear_desc ple_projection; /* ple.projection: n = model_dim, k = ple_dim */
    uzu_norm_desc ple_norm;         /* ple.norm: [model_dim] */

    /* --- mixture of experts (mlp_kind == UZU_MLP_MOE: up_projection / down_projection / hidden_dim / activation above are unused) --- */
    uzu_moe_desc moe;

    /* --- layer mechanisms of the f32-stream designs (uzu_model_desc::f32_stream); all zero / NULL = none --- */
    uint32_t latent_rank;        /* UZU_MIXER_LATENT_ATTENTION: width of the cached latent */
    uint32_t value_head_dim;     /* ... value width per head (out_projection.k = num_heads * value_head_dim) */
    uzu_linear_desc latent_down;      /* n = latent_rank, k = model_dim; absent (weights NULL) on a sharing layer */
    uzu_norm_desc latent_norm;        /* RMS norm of the latent, scales [latent_rank]; absent on a sharing layer */
    uzu_linear_desc latent_up_keys;   /* n = num_heads * head_dim, k = latent_rank */
    uzu_linear_desc latent_up_values; /* n = num_heads * value_head_dim, k = latent_rank */
    /* Token shift: the mixer reads h + (h_prev - h) * token_shift, h_prev = the previous position's normalised row before this replacement (zeros at
     * position 0); the last row's h is part of the sequence state. */
    const float* token_shift;    /* f32 [model_dim] or NULL */
    /* Depth mix: with X_0 the embedding rows and X_(j+1) layer j's own result, what layer l hands on is sum_{j <= l+1} depth_weights[j] * X_j. */
    const float* depth_weights;  /* f32 [num_depth_weights] or NULL */
    uint32_t num_depth_weights;  /* l + 2 on layer l */
    uint32_t mlp_plain;          /* dense MLP without a gate: down(act(up x + b) ) + b, up_projection.n == hidden_dim */
    uint32_t no_mlp;             /* the layer ends behind its mixer */
    /* Parallel block: the mixer and the MLP both read pre_mixer_norm's rows and the layer is x <- x + (mixer(h) + mlp(h)); there is no pre_mlp_norm. */
    uint32_t parallel_block;
    /* UZU_MIXER_ATTENTION in an f32-stream design: grouped heads (num_heads queries on num_groups key / value heads, query head a reads head a / (heads / groups)),
     * key width head_dim and value width value_head_dim, qkv_projection rows = queries | keys | values (n = heads head_dim + groups (head_dim + value_head_dim);
     * a sharing layer: queries only) with out_biases, rotation of the first rope dimensions of queries and keys (use_rope, rope_index), scores
     * attention_scale <q, k>, then the soft cap, causal sliding window (sliding_window_size, 0 = all earlier positions), softmax with per-head sink logits in the
     * denominator (has_sinks + sinks, or unit_sink), out_projection.k = heads * value_head_dim.  The cache keeps rotated keys and values per position;
     * is_kv_sharing reads the source layer's cache with this layer's own queries, mask and constants. */
    float score_soft_cap;        /* s <- cap * tanh(s / cap); 0 = none */
    uint32_t unit_sink;          /* one more term exp(0) in every softmax denominator (a sink with logit 0 and no value) */
    float key_scale;             /* keys are multiplied by it behind their rotation; 0 = 1 */
    float head_norm_epsilon;     /* UZU_MIXER_RETENTION: epsilon of the per-head RMS division */
    const float* retention_decay; /* UZU_MIXER_RETENTION: f32 [num_heads] */
    /* UZU_MIXER_LATENT_ATTENTION with a rotated key part: the down projection yields latent_rank + latent_rope_dim numbers per token -- the latent (normed) and ONE
     * rotated key part shared by all heads (not normed); a query head is [head_dim | latent_rope_dim] wide and its last latent_rope_dim coordinates turn with the
     * same rotation (use_rope + rope_index, rope_interleaved); score = attention_scale (<q_plain, W_up_k c> + <q_rot, k_rot>).  The cache row is [latent | rotated part].
     * latent_packed: the down projection's rows stand behind the queries in qkv_projection (latent_down absent); has_gate then adds num_heads rows behind them:
     * head a's result is multiplied by sigmoid(gate row a . h). */
    uint32_t latent_rope_dim;
    uint32_t latent_packed;
    uint32_t rope_interleaved;   /* the rotation pairs coordinates (2i, 2i + 1) instead of (i, i + dims / 2) */
    /* UZU_MIXER_GATED_LRU (see uzu_mixer_kind) */
    uint32_t lru_width;
    uint32_t lru_blocks;
    float lru_decay_rate;
    const uint16_t* lru_gate_weights; /* bf16 [blocks][2 bw][bw] */
    const float* lru_gate_biases;     /* f32 [blocks][2 bw] */
    const float* lru_lambda;          /* f32 [lru_width] */
    /* Layer scale (f32-stream designs): the mixer's result (behind post_mixer_norm) is multiplied element by element by layer_scale_mixer before it joins the
     * stream, the MLP's (behind post_mlp_norm) by layer_scale_mlp; f32 [model_dim] or NULL.  In an f32-stream design post_mixer_norm / post_mlp_norm, query_norm /
     * key_norm (scales [head_dim], before the rotation) and UZU_NORM_STATISTICS norms (RMS, scales + scale_offset) are honoured as well. */
    const float* layer_scale_mixer;
    const float* layer_scale_mlp;
    /* A gated dense MLP in an f32-stream design (mlp_plain == 0): up_projection rows [up ; gate], hidden = clamp-gated product with the constants of
     * moe.{silu_alpha, gate_clip_*, up_clip_*, up_offset} (mlp_kind stays UZU_MLP_DENSE, no other field of `moe` is read). */
    /* Per-layer token input in an f32-stream design (has_ple, ple_dim, ple_gate, ple_projection, ple_norm with the model's ple_token_embedding): behind the MLP
     * x <- x + norm(projection(gelu_tanh(gate x) * e)), e = columns [ple_slice ple_dim, (ple_slice + 1) ple_dim) of the token's row of the side table. */
    uint32_t ple_slice;
    /* Weight sharing between layer runs (a looped stack): weights_of_layer = j + 1 makes this run use run j's tensors (its own pointers are ignored; scalars must
     * agree); every run keeps its own sequence state.  0 = its own. */
    uint32_t weights_of_layer;
    /* Re-entry of the stream: before this run x <- W [x ; x0] with x0 the embedding rows (n = model_dim, k = 2 model_dim); absent = none */
    uzu_linear_desc stream_reentry;
    /* Input convolution of the sublayers (f32-stream designs): what a sublayer reads is h + conv(h), h = its input rows (the stream itself where the pre norm is
     * absent -- with an input convolution pre_mixer_norm / pre_mlp_norm may be absent), conv = a causal convolution over positions on every channel:
     * conv(h)_t = sum_j w[:, j] h_(t - taps + 1 + j), zeros in front of the sequence; input_conv_mixer / input_conv_mlp f32 [model_dim, input_conv_taps] (either
     * may be NULL = that sublayer reads h).  The last taps - 1 inputs of each are sequence state. */
    uint32_t input_conv_taps;
    /* UZU_MIXER_ATTENTION in an f32-stream design, further options: */
    uint32_t qk_norm_whole;        /* query_norm / key_norm are ONE RMS norm over the whole projection each (scales [heads head_dim] / [groups head_dim]), not per head */
    const float* input_conv_mixer;
    const float* input_conv_mlp;
    uint32_t attention_chunk_size; /* != 0: position i sees j <= i only inside its own chunk, floor(i / size) == floor(j / size), chunks counted from position 0 */
    uint32_t values_are_keys;      /* the packed projection has no value rows: the values are the key rows as projected (before their norm and rotation);
                                      value_head_dim == head_dim */
    uint32_t rel_bias_rows;        /* != 0: a learned bias per (distance bucket, head) is added to the scaled score: rel_bias bf16 [rel_bias_rows, heads]; with
                                      E = rows / 2 the bucket of distance n is n below E, else min(rows - 1, E + floor(ln(n / E) / ln(rel_bias_max / E) (rows - E))) */
    float rel_bias_max;
    const uint16_t* rel_bias;
    const float* head_temperature; /* f32 [heads] or NULL: the scaled score of head a is multiplied by head_temperature[a] (in front of the bias) */
    /* has_gate on such a layer: num_heads more rows behind the packed projection's values; head a's result is multiplied by sigmoid(row a . h). */
    /* A second mixer beside the first (f32-stream designs): both read the same rows, the layer's mixer result is pair_scale_main * main + pair_scale_second *
     * second, each through its own out projection.  pair_mixer = 1 + uzu_mixer_kind of the second (0 = none); supported: attention with a channel-decay delta
     * rule (UZU_MIXER_DELTA_NET) as the second. */
    uint32_t pair_mixer;
    float pair_scale_main, pair_scale_second;
    /* UZU_MIXER_DELTA_NET in an f32-stream design: the gated delta rule with one decay per head and KEY CHANNEL.  dn_num_heads value heads of dn_value_head_dim on
     * dn_num_groups query / key heads of dn_head_dim (head a reads group a / (heads / groups)).  dn_in_proj rows: q | k | v | beta (heads) | decay down
     * (dn_decay_rank) | gate down (dn_gate_rank); q, k, v pass a causal convolution per channel (dn_kernel_size taps, dn_conv_weights f32 [2 groups dk + heads dv,
     * taps], no bias) and silu; q and k become unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q times dk^(-1/2); beta = sigmoid; decay[a, c] =
     * exp(-exp(dn_a_log[a]) softplus(dn_decay_up (decay down) + dn_dt_bias))[a dk + c] (dn_dt_bias f32 [heads dk]); per head S <- decay * S (rows = key
     * channels), u = beta (v - S^T k), S <- S + k u^T, o = S^T q; o / rms(o over dv, dn_norm_epsilon) * dn_norm_scales * sigmoid(dn_gate_up (gate down)); then
     * dn_out_proj.  S (f32 [heads, dk, dv], zero in front of position 0) and the convolution's last taps - 1 inputs are sequence state.  Everything behind the
     * projections and the convolution is f32 in both precisions, the two up products included. */
    uint32_t dn_channel_decay;
    uint32_t dn_decay_rank, dn_gate_rank;
    uzu_linear_desc dn_decay_up; /* n = heads dk, k = dn_decay_rank */
    uzu_linear_desc dn_gate_up;  /* n = heads dv, k = dn_gate_rank */
} uzu_layer_desc;

typedef struct {
    uint32_t vocab_size;
    uint32_t model_dim;
    uint32_t num_layers;
    uint32_t tied_embeddings;
    float input_scale;   /* embedding input_scale, default 1 */
    float logit_scale;   /* default 1 */
    float logit_soft_cap; /* 0 => none */
    uint32_t max_context_length; /* KV cache capacity = max_context_length + 1024 rows (attention/state.rs:108-122) */
    uzu_rope_desc rope;
    /* embedding table, Layout::InputOutput => stored [vocab, dim/pack]; described here with
     * n = vocab, k = model_dim exactly like the readout matmul sees it (embedding.rs:374-456). */
    uzu_linear_desc embedding;
    uzu_linear_desc output_embedding; /* untied readout; ignored when tied */
    uzu_norm_desc output_norm;
    const uzu_layer_desc* layers;

    /* --- decoder options of the Gemma families; all zero = none --- */
    uint32_t num_ropes;          /* 0: every rotating layer uses `rope` above.  Else the distinct AnyRoPEConfig values of the layers in
                                    order of first use (Transformer::new, transformer.rs:101-118): layer l rotates with ropes[rope_index] */
    uint32_t has_ple;            /* DecoderConfig::ple_model_config.is_some() (decoder.rs:85-99) */
    const uzu_rope_desc* ropes;
    uzu_norm_desc embedding_norm; /* DecoderConfig::embedding_norm_config: a Normalization of the looked-up rows (decoder.rs:68-83,149-154) */
    /* PLEModelConfig (config/per_layer_embedding.rs:5-15), PerLayerEmbedding (per_layer_embedding.rs:36-148); num_layers == the layer count */
    uint32_t ple_dim;
    uint32_t ple_vocab_size;
    float ple_embed_scale;
    float ple_model_projection_scale;
    float ple_input_scale;
    uint32_t reserved;
    uzu_linear_desc ple_token_embedding;  /* per_layer_embedding.token_embedding: n = ple_vocab_size, k = num_layers*ple_dim (an embedding table) */
    uzu_linear_desc ple_model_projection; /* per_layer_embedding.model_projection: n = num_layers*ple_dim, k = model_dim */
    uzu_norm_desc ple_projection_norm;    /* per_layer_embedding.projection_norm: [ple_dim]; epsilon as configured (the engine divides it by
                                             model_projection_scale^2, per_layer_embedding.rs:75-80) */
    /* An f32-stream design: the residual stream, norms, attention scores / weights and routers are f32 end to end (the reference's models re-round the residual
     * to bf16 at every add); weights are full-precision bf16 (UZU_QUANT_NONE); pre-norm layers x <- x + mixer(norm(x)), x <- x + mlp(norm(x)); the read-out is the
     * tied embedding table behind output_norm; logits are f32.  Such a model runs through its own forward encoder (csrc/engine_stream32.hip), batched over
     * sequences of unequal length (uzu_hip_model_step_batch). */
    uint32_t f32_stream;
    /* A second, hashed token table added to the looked-up rows (f32-stream designs): row (previous token * bigram_mul_prev + token * bigram_mul_cur) mod
     * bigram_buckets of bigram_table (bf16 [bigram_buckets + 1, model_dim], not scaled by input_scale); a sequence's first token reads the last row.  The previous
     * token is sequence state.  bigram_buckets == 0: none (the field was `reserved5`). */
    uint32_t bigram_buckets;
    uint32_t bigram_mul_prev, bigram_mul_cur;
    uzu_linear_desc bigram_table;
} uzu_model_desc;

/*
 * The DFlash draft model of the tree speculator: DFlashDraftConfig (config/dflash.rs:9-23) + the tensors of the subtree
 * `speculator.draft_model` (speculators/dflash_tfm.rs:86-107, encodable_block/dflash.rs:86-172):
 *   context_projection.*   Linear  [model_dim, model_dim * num_target_layers]   the accepted tokens' target features, side by side
 *   context_norm.scales    Normalization of the projected features (no shortcut)
 *   state_kv_projection.*  Linear  [num_layers * 2 * groups * head_dim, model_dim]   keys | values of every draft layer from one projected row
 *   layers.{i}.*           TransformerLayers with attention mixers (block attention: is_non_causal as configured) and a full KV state
 *   output_norm.scales     Normalization with the shortcut added
 * The draft model has no embedding of its own: rows are looked up in, and read out through, the TARGET model's table (dflash.rs:285,335).
 */
typedef struct {
    uint32_t model_dim;
    uint32_t hidden_dim;
    uint32_t block_size;           /* rows of one draft pass (<= ATTENTION_SUFFIX_CAPACITY = 1024) */
    uint32_t mask_token_id;
    uint32_t num_target_layers;    /* target_layer_ids.len(): the target's hidden-feature taps (stream.rs:213-214,632-633) */
    uint32_t num_layers;
    uint32_t vocab_size;
    uint32_t context_capacity;     /* DFlash::empty_state(context_capacity) (dflash.rs:174-188; language_model/state.rs:46-51: the target's max context) */
    const uint32_t* target_layer_ids;
    uzu_linear_desc context_projection;
    uzu_norm_desc context_norm;
    uzu_linear_desc state_kv_projection;
    uzu_rope_desc rope;            /* rope_config: positions context .. context + rows; max_sequence_length bounds the state */
    const uzu_layer_desc* layers;
    uzu_norm_desc output_norm;
} uzu_dflash_desc;

/*
 * The Weaver tree constructor of the speculator: WeaverConfig (config/weaver.rs:5-17) + the tensors of the subtree `speculator.weaver`
 * (encodable_block/weaver.rs:166-275, weaver_layer.rs:47-148).  All norms share norm_config (their own scales); the layers' MLP is a DenseMLP with SiLU and
 * up / down biases (weaver_layer.rs:126-131); model_dim = num_heads * rope.head_dim.
 *   embedding_norm.scales [target_embedding_dim], embedding_projection.{weights.*, biases} [model_dim, target_embedding_dim]
 *   hidden_state_norm.scales [target_model_dim], hidden_state_projection.{weights.*, biases} [model_dim, target_model_dim]
 *   blocks.{i}.{pre_attention_norm, qkv_projection [3 model_dim, model_dim], out_projection [model_dim, model_dim], pre_mlp_norm, mlp.up_projection (+ biases)
 *               [2 hidden, model_dim], mlp.down_projection (+ biases) [model_dim, hidden]}
 *   output_norm.scales [model_dim], query_projection.weights.* [target_model_dim, model_dim]
 */
typedef struct {
    uzu_norm_desc pre_attention_norm;
    uzu_norm_desc pre_mlp_norm;
    uzu_linear_desc qkv_projection;
    uzu_linear_desc out_projection;
    uzu_linear_desc up_projection;
    uzu_linear_desc down_projection;
} uzu_weaver_layer_desc;

typedef struct {
    uint32_t model_dim;
    uint32_t target_model_dim;
    uint32_t target_embedding_dim;
    uint32_t num_layers;
    uint32_t num_heads;
    uint32_t hidden_dim;
    uint32_t max_depth;
    uint32_t candidate_pool_size; /* 1..512 (CANDIDATES_MAX) */
    uzu_norm_desc embedding_norm;
    uzu_linear_desc embedding_projection;
    uzu_norm_desc hidden_state_norm;
    uzu_linear_desc hidden_state_projection;
    uzu_norm_desc output_norm;
    uzu_linear_desc query_projection;
    uzu_rope_desc rope; /* head_dim = model_dim / num_heads, max_sequence_length > max_depth */
    const uzu_weaver_layer_desc* layers;
} uzu_weaver_desc;

/* WeaverTreeShape (encodable_block/weaver.rs:33-46; dflash_tfm.rs:259-279: max_depth counts the root) */
typedef struct {
    uint32_t tree_budget;
    uint32_t max_depth;
    uint32_t dflash_depth;
    uint32_t rounds;
    uint32_t expand_per_round;
    uint32_t expand_width;
} uzu_weaver_tree_shape;

#ifdef __cplusplus
}
#endif
#endif /* UZU_MODEL_DESC_H */
