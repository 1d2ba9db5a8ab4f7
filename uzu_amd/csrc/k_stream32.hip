// k_stream32.hip -- element-wise kernels, the full-precision linear and the score-routed experts of the f32-stream designs (kernels_stream32.h).
//
// Everything here keeps f32 where such a design asks for it: the residual rows, the norm, the router and its softmax, every accumulation.  A matrix product
// reads f32 activation rows and bf16 weights; with `bf16_products` the activation operand is rounded to bf16 as it is loaded (what a bf16 activation buffer
// would have held), otherwise the product is a true f32 product.  Reductions run in a fixed order: a result does not depend on what else is in the pass.
#include "device_utils.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

namespace {

__device__ __forceinline__ float opnd(float v, uint32_t bf16_products) { return bf16_products ? round_bf16(v) : v; }

// this lane's share of <x, w> over n elements (x f32 in LDS or global, w bf16 in global): 16-byte weight loads where the row allows them (n % 8 == 0 and
// the row 16-byte aligned), element loads otherwise; the caller sums over the wave
__device__ __forceinline__ float lane_dot(const float* x, const uint16_t* w, uint32_t n, uint32_t lane, uint32_t round_x = 0) {
    float acc = 0.0f;
    if (round_x) { // operand rows that were not rounded when they were staged (read straight from global memory)
        for (uint32_t i = lane; i < n; i += 64) acc = fmaf(round_bf16(x[i]), bf16_to_f32(w[i]), acc);
        return acc;
    }
    if ((n & 7) == 0 && ((uintptr_t)w & 15) == 0) {
        for (uint32_t i0 = lane * 8; i0 < n; i0 += 512) {
            const uint4 wv = *(const uint4*)(w + i0);
            const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc = fmaf(x[i0 + 2 * j], bits_to_f32(ww[j] << 16), acc);
                acc = fmaf(x[i0 + 2 * j + 1], bits_to_f32(ww[j] & 0xFFFF0000u), acc);
            }
        }
    } else {
        for (uint32_t i = lane; i < n; i += 64) acc = fmaf(x[i], bf16_to_f32(w[i]), acc);
    }
    return acc;
}

__global__ void __launch_bounds__(256) embed_rows_f32_kernel(const uint32_t* tokens, const uint16_t* table, float* out, uint32_t vocab, uint32_t d, float scale) {
    const uint32_t r = blockIdx.x;
    uint32_t t = tokens[r];
    if (t >= vocab) t = 0;
    const uint16_t* src = table + (size_t)t * d;
    float* dst = out + (size_t)r * d;
    for (uint32_t i = threadIdx.x; i < d; i += blockDim.x) dst[i] = bf16_to_f32(src[i]) * scale; // (scale 1: the value itself)
}

// the same rows plus a hashed (previous token, token) row of a second table; the previous token of a sequence's first row of the pass is the state's
// (prev[z]), position 0 reads the table's last row
__global__ void __launch_bounds__(256) embed_pair_rows_f32_kernel(EmbedPairParams p) {
    const uint32_t r = blockIdx.x;
    const uint32_t z = p.row_seq[r];
    const SeqSpan sp = p.spans[z];
    const uint32_t i = r - sp.row0;
    uint32_t t = p.tokens[r];
    if (t >= p.vocab) t = 0;
    uint32_t row = p.buckets;
    if (sp.start + i > 0) {
        uint32_t before = i ? p.tokens[r - 1] : *p.prev[z];
        if (before >= p.vocab) before = 0;
        row = (uint32_t)(((uint64_t)before * p.mul_prev + (uint64_t)t * p.mul_cur) % p.buckets);
    }
    const uint16_t* src = p.table + (size_t)t * p.d;
    const uint16_t* add = p.pair_table + (size_t)row * p.d;
    float* dst = p.out + (size_t)r * p.d;
    for (uint32_t c = threadIdx.x; c < p.d; c += blockDim.x) dst[c] = bf16_to_f32(src[c]) * p.scale + bf16_to_f32(add[c]);
    if (sp.count == 1 && threadIdx.x == 0) *p.prev[z] = p.tokens[r]; // a sequence that brings one row: this workgroup is the only reader of the old token
}
// thread = sequence: its last token of the pass becomes the state's previous token (a launch of its own: the rows above read the old one)
__global__ void __launch_bounds__(64) embed_pair_commit_kernel(EmbedPairParams p, uint32_t nseq) {
    const uint32_t z = blockIdx.x * 64 + threadIdx.x;
    if (z >= nseq) return;
    const SeqSpan sp = p.spans[z];
    if (sp.count > 1) *p.prev[z] = p.tokens[sp.row0 + sp.count - 1];
}

constexpr int kNormUnroll = 8;
// a workgroup per row: the sum of squares as 256 strided partial sums folded in a fixed tree, then the scaled row
// (blockIdx.y = the part of a row that is normed in gridDim.y equal consecutive parts: `d` is the part's width, `ld` the row's)
__global__ void __launch_bounds__(256) rms_norm_rows_kernel(const float* x, float* out, const float* scales, float gain, float eps, const uint32_t* row_index, uint32_t d,
                                                            float offset, uint32_t ld) {
    __shared__ float s_red[256];
    const uint32_t r = blockIdx.x, part0 = blockIdx.y * d;
    const float* xr = x + (size_t)(row_index ? row_index[r] : r) * ld + part0;
    if (scales) scales += part0;
    float acc = 0.0f;
    for (uint32_t i = threadIdx.x; i < d; i += 256) acc = fmaf(xr[i], xr[i], acc);
    s_red[threadIdx.x] = acc;
    __syncthreads();
    for (uint32_t w = 128; w > 0; w >>= 1) {
        if (threadIdx.x < w) s_red[threadIdx.x] += s_red[threadIdx.x + w];
        __syncthreads();
    }
    const float inv = 1.0f / sqrtf(s_red[0] / (float)d + eps);
    float* o = out + (size_t)r * ld + part0;
    // kNormUnroll elements per thread and step, every load of a step in front of its stores (out may alias x for the compiler: a loop of load -> store pairs would
    // pay one memory round trip per element, which is what a one-row decode step's launch consists of)
    for (uint32_t i0 = threadIdx.x; i0 < d; i0 += 256 * kNormUnroll) {
        float xv[kNormUnroll], sv[kNormUnroll];
#pragma unroll
        for (int u = 0; u < kNormUnroll; ++u) {
            const uint32_t i = i0 + u * 256;
            xv[u] = i < d ? xr[i] : 0.0f;
            sv[u] = (i < d && scales) ? scales[i] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < kNormUnroll; ++u) {
            const uint32_t i = i0 + u * 256;
            if (i >= d) break;
            const float v = xv[u] * inv * gain;
            o[i] = scales ? v * (sv[u] + offset) : v;
        }
    }
}

// the same sum of squares over a sublayer's result y; the normed row joins the stream: out = residual + y * inv * (scales + offset) * layer_scale
// ... and, with `next`, the norm of the new row for the sublayer that follows (its own weights, offset and epsilon): next[r] = rms(out[r]) * (next_scales + next_offset)
__global__ void __launch_bounds__(256) rms_norm_add_rows_kernel(const float* y, const float* residual, float* out, const float* scales, float offset, const float* layer_scale,
                                                                float eps, uint32_t d, float* next, const float* next_scales, float next_offset, float next_eps, uint32_t ld) {
    __shared__ float s_red[256];
    const uint32_t r = blockIdx.x, part0 = blockIdx.y * d; // (a row normed in gridDim.y parts of width d; `next` only with one part)
    const float* yr = y + (size_t)r * ld + part0;
    scales += part0;
    if (layer_scale) layer_scale += part0;
    float acc = 0.0f;
    for (uint32_t i = threadIdx.x; i < d; i += 256) acc = fmaf(yr[i], yr[i], acc);
    s_red[threadIdx.x] = acc;
    __syncthreads();
    for (uint32_t w = 128; w > 0; w >>= 1) {
        if (threadIdx.x < w) s_red[threadIdx.x] += s_red[threadIdx.x + w];
        __syncthreads();
    }
    const float inv = 1.0f / sqrtf(s_red[0] / (float)d + eps);
    const float* res = residual + (size_t)r * ld + part0;
    float* o = out + (size_t)r * ld + part0;
    float acc2 = 0.0f;
    for (uint32_t i0 = threadIdx.x; i0 < d; i0 += 256 * kNormUnroll) { // (loads of a step in front of its stores, as in rms_norm_rows_kernel; sums in the same order)
        float yv[kNormUnroll], rv[kNormUnroll], sv[kNormUnroll], lv[kNormUnroll];
#pragma unroll
        for (int u = 0; u < kNormUnroll; ++u) {
            const uint32_t i = i0 + u * 256;
            const bool ok = i < d;
            yv[u] = ok ? yr[i] : 0.0f, rv[u] = ok ? res[i] : 0.0f, sv[u] = ok ? scales[i] : 0.0f, lv[u] = (ok && layer_scale) ? layer_scale[i] : 1.0f;
        }
#pragma unroll
        for (int u = 0; u < kNormUnroll; ++u) {
            const uint32_t i = i0 + u * 256;
            if (i >= d) break;
            float v = yv[u] * inv * (sv[u] + offset);
            if (layer_scale) v *= lv[u];
            v = rv[u] + v;
            o[i] = v;
            acc2 = fmaf(v, v, acc2);
        }
    }
    if (!next) return;
    __syncthreads(); // s_red[0] has been read by everyone
    s_red[threadIdx.x] = acc2;
    __syncthreads();
    for (uint32_t w = 128; w > 0; w >>= 1) {
        if (threadIdx.x < w) s_red[threadIdx.x] += s_red[threadIdx.x + w];
        __syncthreads();
    }
    const float inv2 = 1.0f / sqrtf(s_red[0] / (float)d + next_eps);
    float* nx = next + (size_t)r * d;
    for (uint32_t i0 = threadIdx.x; i0 < d; i0 += 256 * kNormUnroll) { // (o: the thread's own stores)
        float ov[kNormUnroll], sv[kNormUnroll];
#pragma unroll
        for (int u = 0; u < kNormUnroll; ++u) {
            const uint32_t i = i0 + u * 256;
            ov[u] = i < d ? o[i] : 0.0f, sv[u] = i < d ? next_scales[i] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < kNormUnroll; ++u) {
            const uint32_t i = i0 + u * 256;
            if (i >= d) break;
            nx[i] = ov[u] * inv2 * (sv[u] + next_offset);
        }
    }
}

__device__ __forceinline__ float gelu_tanh_f32(float z) { return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

__global__ void __launch_bounds__(256) dyn_tanh_kernel(DynTanhParams p) {
    const uint32_t r = blockIdx.x;
    const uint32_t src = p.row_index ? p.row_index[r] : r;
    const float* x = p.x + (size_t)src * p.d;
    float* out = p.out + (size_t)r * p.d;
    const uint32_t i0 = blockIdx.y * blockDim.x + threadIdx.x, step = gridDim.y * blockDim.x; // a row is spread over grid.y workgroups: one round of loads per thread
    if (!p.shift) {
        for (uint32_t i = i0; i < p.d; i += step) out[i] = fmaf(tanhf(p.alpha * x[i]), p.scales[i], p.biases ? p.biases[i] : 0.0f);
        return;
    }
    const uint32_t q = p.row_seq[r];
    const SeqSpan sp = p.spans[q];
    const bool first = r == sp.row0;
    float* prev = p.prev[q];
    const float* xl = p.x + (size_t)(sp.row0 + sp.count - 1) * p.d; // the sequence's last row of the pass
    for (uint32_t i = i0; i < p.d; i += step) {
        const float w = p.scales[i], b = p.biases ? p.biases[i] : 0.0f;
        const float h = fmaf(tanhf(p.alpha * x[i]), w, b);
        float hp;
        if (first) {
            hp = sp.start ? prev[i] : 0.0f;
            // the same thread that has read the state's element replaces it: no other block of the launch touches prev[q]
            prev[i] = sp.count == 1 ? h : fmaf(tanhf(p.alpha * xl[i]), w, b);
        } else {
            hp = fmaf(tanhf(p.alpha * x[(ptrdiff_t)i - (ptrdiff_t)p.d]), w, b);
        }
        out[i] = fmaf(hp - h, p.shift[i], h);
    }
}

__global__ void __launch_bounds__(256) depth_mix_kernel(const float* slots, size_t slot_stride, const float* w, uint32_t count, float* out, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    float acc = 0.0f;
    for (uint32_t j = 0; j < count; ++j) acc = fmaf(w[j], slots[(size_t)j * slot_stride + i], acc);
    out[i] = acc;
}

__device__ __forceinline__ float expert_act(float gate, float up, const ExpertAct& a) {
    const float g = fminf(fmaxf(gate, a.gate_min), a.gate_max), u = fminf(fmaxf(up, a.up_min), a.up_max);
    if (a.gelu) return gelu_tanh_f32(g) * (u + a.up_offset);
    return g / (1.0f + expf(-(a.alpha * g))) * (u + a.up_offset);
}

__device__ __forceinline__ float apply_act(float v, uint32_t act) {
    if (act == 1) {
        const float t = fmaxf(v, 0.0f);
        return t * t;
    }
    if (act == 2) return gelu_tanh_f32(v);
    return v;
}
// what follows the activation: the product's scale, a per-(row, product) sigmoid gate
__device__ __forceinline__ float apply_tail(float v, const LinearF32Params& p, uint32_t r, uint32_t z) {
    if (p.y_scale != 0.0f) v *= p.y_scale;
    if (p.soft_cap != 0.0f) v = p.soft_cap * tanhf(v / p.soft_cap);
    if (p.gate) v *= 1.0f / (1.0f + expf(-p.gate[(size_t)r * p.ldgate + z]));
    return v;
}
// ... and a per-(row's token, column) multiplier from a bf16 table
__device__ __forceinline__ float apply_token_mul(float v, const LinearF32Params& p, uint32_t r, uint32_t n) {
    if (!p.mul_table) return v;
    uint32_t t = p.mul_tokens[r];
    if (t >= p.mul_vocab) t = 0;
    return v * bf16_to_f32(p.mul_table[(size_t)t * p.mul_ld + p.mul_col0 + n]);
}

// thread = (row, hidden unit): a one-row decode step still spreads over ff / 256 workgroups
__global__ void __launch_bounds__(256) gated_act_rows_kernel(const float* y1, float* hidden, uint32_t ff, ExpertAct act) {
    const uint32_t f = blockIdx.x * 256 + threadIdx.x, r = blockIdx.y;
    if (f >= ff) return;
    const float* src = y1 + (size_t)r * 2 * ff;
    hidden[(size_t)r * ff + f] = expert_act(src[ff + f], src[f], act);
}

// ---- few rows: a wave per output column, RT rows per pass over the weights
template <int RT>
__global__ void __launch_bounds__(256) linear_rows_kernel(LinearF32Params p, uint32_t vec) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n = blockIdx.x * 4 + wave;
    const uint32_t r0 = blockIdx.y * RT;
    const uint32_t z = blockIdx.z;
    if (n >= p.n) return;
    const float* x = p.x + z * p.x_batch;
    const uint16_t* w = p.w + z * p.w_batch + (size_t)n * p.k;
    float acc[RT];
#pragma unroll
    for (int i = 0; i < RT; ++i) acc[i] = 0.0f;
    if (vec) {
        for (uint32_t k0 = lane * 8; k0 < p.k; k0 += 64 * 8) {
            const uint4 wv = *(const uint4*)(w + k0);
            const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
            float wf[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) wf[2 * j] = bits_to_f32(ww[j] << 16), wf[2 * j + 1] = bits_to_f32(ww[j] & 0xFFFF0000u);
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                const uint32_t r = r0 + i < p.rows ? r0 + i : p.rows - 1;
                const float4 a = *(const float4*)(x + (size_t)r * p.ldx + k0), b = *(const float4*)(x + (size_t)r * p.ldx + k0 + 4);
                const float xv[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[i] = fmaf(opnd(xv[j], p.bf16_products), wf[j], acc[i]);
            }
        }
    } else {
        for (uint32_t k0 = lane; k0 < p.k; k0 += 64) {
            const float wf = bf16_to_f32(w[k0]);
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                const uint32_t r = r0 + i < p.rows ? r0 + i : p.rows - 1;
                acc[i] = fmaf(opnd(x[(size_t)r * p.ldx + k0], p.bf16_products), wf, acc[i]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < RT; ++i) acc[i] = wave_sum(acc[i]);
    if (lane == 0) {
        const float bias = p.bias ? bf16_to_f32(p.bias[n]) : 0.0f;
        float* y = p.y + z * p.y_batch;
#pragma unroll
        for (int i = 0; i < RT; ++i) {
            const uint32_t r = r0 + i;
            if (r >= p.rows) break;
            float v = apply_token_mul(apply_tail(apply_act(acc[i] + bias, p.act), p, r, z), p, r, n);
            if (p.residual) v += p.residual[(size_t)r * p.ldr + n];
            y[(size_t)r * p.ldy + n] = v;
        }
    }
}

// ---- many rows without the matrix cores (true f32 products, and every shape the matrix-core form does not take): 64 x 64 tile, 16-deep k-steps through LDS,
// a 4 x 4 block of outputs per thread
constexpr int TM = 64, TN = 64, TK = 16;
__global__ void __launch_bounds__(256) linear_tile_kernel(LinearF32Params p) {
    __shared__ float s_a[TK][TM + 4];
    __shared__ float s_b[TK][TN + 4];
    const uint32_t z = blockIdx.z;
    const float* x = p.x + z * p.x_batch;
    const uint16_t* w = p.w + z * p.w_batch;
    const uint32_t m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    const uint32_t tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
    // loader mapping: thread -> (row / column tid >> 2 of the tile, k offsets (tid & 3) * 4 .. + 3)
    const uint32_t lr = tid >> 2, lk = (tid & 3) * 4;
    for (uint32_t k0 = 0; k0 < p.k; k0 += TK) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t kk = k0 + lk + j;
            const uint32_t r = m0 + lr, n = n0 + lr;
            s_a[lk + j][lr] = (r < p.rows && kk < p.k) ? opnd(x[(size_t)r * p.ldx + kk], p.bf16_products) : 0.0f;
            s_b[lk + j][lr] = (n < p.n && kk < p.k) ? bf16_to_f32(w[(size_t)n * p.k + kk]) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = s_a[kk][ty * 4 + i], b[i] = s_b[kk][tx * 4 + i];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
    float* y = p.y + z * p.y_batch;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t r = m0 + ty * 4 + i;
        if (r >= p.rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t n = n0 + tx * 4 + j;
            if (n >= p.n) continue;
            float v = apply_token_mul(apply_tail(apply_act(acc[i][j] + (p.bias ? bf16_to_f32(p.bias[n]) : 0.0f), p.act), p, r, z), p, r, n);
            if (p.residual) v += p.residual[(size_t)r * p.ldr + n];
            y[(size_t)r * p.ldy + n] = v;
        }
    }
}

// ---- score routing: one wave per row
constexpr uint32_t kRouteMaxOutputs = 512; // 8 per lane
// mode 0: score routing (softmax over all outputs, choice by score + selection_bias, weights = winners' scores / their sum)
// mode 1 / 2: top-k of the logits z + router_bias; weights = the winners' logits (1) or the softmax over them (2)
__global__ void __launch_bounds__(64) moe_route_scores_kernel(const float* x, const uint16_t* router, const float* selection_bias, int32_t* ids, float* weights, uint32_t d,
                                                              uint32_t outputs, uint32_t top, uint32_t mode, const uint16_t* router_bias) {
    const uint32_t r = blockIdx.x, lane = threadIdx.x;
    const float* xr = x + (size_t)r * d;
    float z[8];
    float zmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) z[j] = -INFINITY;
    for (uint32_t e = 0; e < outputs; ++e) {
        float acc = wave_sum(lane_dot(xr, router + (size_t)e * d, d, lane));
        if (router_bias) acc += bf16_to_f32(router_bias[e]);
        if ((e & 63) == lane) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if ((uint32_t)j == (e >> 6)) z[j] = acc;
        }
        zmax = fmaxf(zmax, acc);
    }
    float ex[8], sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t e = j * 64 + lane;
        ex[j] = e < outputs ? expf(z[j] - zmax) : 0.0f;
        sum += ex[j];
    }
    sum = wave_sum(sum);
    float score[8], choice[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t e = j * 64 + lane;
        score[j] = mode ? z[j] : ex[j] / sum;
        choice[j] = e < outputs ? score[j] + (selection_bias ? selection_bias[e] : 0.0f) : -INFINITY;
    }
    float first = 0.0f; // the largest winner (mode 2: the softmax's reference point)
    float wsum = 0.0f;
    float my_w = 0.0f; // lane t keeps the t-th winner's score
    int32_t my_id = 0;
    for (uint32_t t = 0; t < top; ++t) {
        float best = -INFINITY;
        uint32_t best_e = 0xFFFFFFFFu;
        float best_s = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t e = j * 64 + lane;
            if (e < outputs && (choice[j] > best || (choice[j] == best && e < best_e))) best = choice[j], best_e = e, best_s = score[j];
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, 64), os = __shfl_xor(best_s, off, 64);
            const uint32_t oe = __shfl_xor(best_e, off, 64);
            if (ob > best || (ob == best && oe < best_e)) best = ob, best_e = oe, best_s = os;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if ((uint32_t)j * 64 + lane == best_e) choice[j] = -INFINITY; // taken (a NaN row leaves best_e invalid: every lane then agrees on 0xFFFFFFFF)
        if (t == 0) first = best_s;
        if (mode == 2) best_s = expf(best_s - first);
        wsum += best_s;
        if ((t & 63) == lane && t < 64) my_w = best_s, my_id = (int32_t)best_e;
        if (t >= 64 && lane == 0) { // more winners than lanes: written as they come
            ids[(size_t)r * top + t] = (int32_t)best_e;
            weights[(size_t)r * top + t] = best_s; // (normalised below only for the first 64; top <= 64 is checked on the host)
        }
    }
    if (lane < top && lane < 64) {
        ids[(size_t)r * top + lane] = my_id;
        weights[(size_t)r * top + lane] = mode == 1 ? my_w : mode == 2 ? my_w / wsum : my_w / (wsum + 1e-20f);
    }
}

// a workgroup per (row, slot): the row once into LDS, then a wave per hidden unit (gate and up rows of the unit in the same pass)
__global__ void __launch_bounds__(256) moe_experts_gate_up_kernel(const float* x, const int32_t* ids, const uint16_t* w13, float* hidden, uint32_t d, uint32_t ff, uint32_t routed,
                                                                  uint32_t top, uint32_t bf16_products, ExpertAct act) {
    extern __shared__ float s_x[];
    const uint32_t slot = blockIdx.x, r = slot / top;
    const int32_t e = ids[slot];
    if (e < 0 || (uint32_t)e >= routed) return; // an identity expert has no hidden row
    for (uint32_t i = threadIdx.x; i < d; i += blockDim.x) s_x[i] = opnd(x[(size_t)r * d + i], bf16_products);
    __syncthreads();
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const uint16_t* base = w13 + (size_t)e * 2 * ff * d;
    for (uint32_t f = blockIdx.y * nw + wave; f < ff; f += gridDim.y * nw) {
        const uint16_t* wu = base + (size_t)f * d;
        const uint16_t* wg = base + (size_t)(ff + f) * d;
        const float au = wave_sum(lane_dot(s_x, wu, d, lane)), ag = wave_sum(lane_dot(s_x, wg, d, lane));
        if (lane == 0) hidden[(size_t)slot * ff + f] = expert_act(ag, au, act);
    }
}

// a workgroup per (row, block of outputs): the row's hidden rows into LDS, then a wave per output; the slots are added in slot order
__global__ void __launch_bounds__(256) moe_experts_down_kernel(const float* hidden, const float* x, const int32_t* ids, const float* weights, const uint16_t* w2,
                                                               const float* residual, float* y, uint32_t d, uint32_t ff, uint32_t routed, uint32_t top, uint32_t bf16_products,
                                                               uint32_t staged) {
    extern __shared__ float s_h[]; // [top][ff] (staged; hidden rows too wide for LDS are read from global memory)
    const uint32_t r = blockIdx.x;
    if (staged) {
        for (uint32_t i = threadIdx.x; i < top * ff; i += blockDim.x) {
            const int32_t e = ids[(size_t)r * top + i / ff];
            s_h[i] = (e >= 0 && (uint32_t)e < routed) ? opnd(hidden[(size_t)r * top * ff + i], bf16_products) : 0.0f;
        }
        __syncthreads();
    }
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    for (uint32_t n = blockIdx.y * nw + wave; n < d; n += gridDim.y * nw) {
        float total = residual ? residual[(size_t)r * d + n] : 0.0f;
        for (uint32_t j = 0; j < top; ++j) {
            const int32_t e = ids[(size_t)r * top + j];
            const float wt = weights[(size_t)r * top + j];
            if (e < 0) continue;
            if ((uint32_t)e >= routed) { // identity expert: the block's input itself
                total = fmaf(wt, x[(size_t)r * d + n], total);
                continue;
            }
            const float* hrow = staged ? s_h + j * ff : hidden + ((size_t)r * top + j) * ff;
            const float acc = wave_sum(lane_dot(hrow, w2 + ((size_t)e * d + n) * ff, ff, lane, staged ? 0u : bf16_products));
            total = fmaf(wt, acc, total);
        }
        if (lane == 0) y[(size_t)r * d + n] = total;
    }
}

// ---- bucketing of the (row, slot) pairs by expert for the grouped matrix-core form
__global__ void __launch_bounds__(1024) moe_bucket_kernel(const int32_t* ids, uint32_t slots, uint32_t routed, uint32_t* offsets, uint32_t* cursor) {
    extern __shared__ uint32_t s_hist[];
    for (uint32_t e = threadIdx.x; e < routed; e += blockDim.x) s_hist[e] = 0;
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < slots; i += blockDim.x) {
        const int32_t e = ids[i];
        if (e >= 0 && (uint32_t)e < routed) atomicAdd(&s_hist[e], 1u);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t run = 0;
        for (uint32_t e = 0; e < routed; ++e) {
            offsets[e] = run, cursor[e] = 0;
            run += s_hist[e];
        }
        offsets[routed] = run;
    }
}
// a pair's place inside its expert's bucket: the order of arrival (any order gives the same numbers: a row's product does not depend on its place in a tile)
__global__ void __launch_bounds__(256) moe_scatter_kernel(const int32_t* ids, uint32_t slots, uint32_t routed, uint32_t top, const uint32_t* offsets, uint32_t* cursor, uint32_t* perm,
                                                         uint32_t* slot_pos) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= slots) return;
    const int32_t e = ids[i];
    if (e < 0 || (uint32_t)e >= routed) {
        slot_pos[i] = 0xFFFFFFFFu;
        return;
    }
    const uint32_t pos = offsets[e] + atomicAdd(&cursor[e], 1u);
    perm[pos] = i / top;
    slot_pos[i] = pos;
}
__global__ void __launch_bounds__(256) moe_act_mul_kernel(const float* y1, float* hidden, const uint32_t* offsets, uint32_t routed, uint32_t ff, ExpertAct act) {
    const uint32_t pos = blockIdx.x;
    if (pos >= offsets[routed]) return;
    const float* src = y1 + (size_t)pos * 2 * ff;
    for (uint32_t f = threadIdx.x; f < ff; f += blockDim.x) {
        const float g = src[ff + f];
        hidden[(size_t)pos * ff + f] = expert_act(g, src[f], act);
    }
}
__global__ void __launch_bounds__(256) moe_combine_kernel(const float* y2, const float* x, const int32_t* ids, const float* weights, const uint32_t* slot_pos, const float* residual,
                                                         float* y, uint32_t d, uint32_t routed, uint32_t top) {
    const uint32_t r = blockIdx.x;
    for (uint32_t n = threadIdx.x; n < d; n += blockDim.x) {
        float total = residual ? residual[(size_t)r * d + n] : 0.0f;
        for (uint32_t j = 0; j < top; ++j) {
            const int32_t e = ids[(size_t)r * top + j];
            if (e < 0) continue;
            const float src = (uint32_t)e >= routed ? x[(size_t)r * d + n] : y2[(size_t)slot_pos[(size_t)r * top + j] * d + n];
            total = fmaf(weights[(size_t)r * top + j], src, total);
        }
        y[(size_t)r * d + n] = total;
    }
}

} // namespace

bool moe_experts_grouped_supported(const MoeGroupedParams& p) {
    if (!p.routed || p.rows < 64 || p.routed > 8192 || !p.y1 || !p.y2 || !p.hidden || !p.perm) return false;
    LinearF32Params q{};
    q.x = p.x, q.w = p.w13, q.y = p.y1, q.rows = p.rows * p.top, q.n = 2 * p.ff, q.k = p.d, q.ldx = p.d, q.ldy = 2 * p.ff, q.batch = p.routed, q.w_batch = (size_t)2 * p.ff * p.d;
    q.bf16_products = 1, q.row_offsets = p.offsets, q.row_map = p.perm;
    LinearF32Params r = q;
    r.x = p.hidden, r.w = p.w2, r.y = p.y2, r.n = p.d, r.k = p.ff, r.ldx = p.ff, r.ldy = p.d, r.w_batch = (size_t)p.d * p.ff, r.row_map = nullptr;
    return linear_mfma_supported(q) && linear_mfma_supported(r);
}

uzu_status moe_experts_grouped(hipStream_t s, const MoeGroupedParams& p) {
    UZU_REQUIRE(moe_experts_grouped_supported(p), "moe_experts_grouped: shape not covered");
    const uint32_t slots = p.rows * p.top;
    UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL(moe_bucket_kernel, dim3(1), dim3(1024), (size_t)p.routed * 4, s, p.ids, slots, p.routed, p.offsets, p.cursor); }, "moe_bucket"));
    UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL(moe_scatter_kernel, dim3((slots + 255) / 256), dim3(256), 0, s, p.ids, slots, p.routed, p.top, p.offsets, p.cursor, p.perm, p.slot_pos); },
                               "moe_scatter"));
    LinearF32Params q{};
    q.x = p.x, q.w = p.w13, q.y = p.y1, q.rows = slots, q.n = 2 * p.ff, q.k = p.d, q.ldx = p.d, q.ldy = 2 * p.ff, q.batch = p.routed, q.w_batch = (size_t)2 * p.ff * p.d;
    q.bf16_products = 1, q.row_offsets = p.offsets, q.row_map = p.perm;
    UZU_PROPAGATE(linear_mfma(s, q));
    UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL(moe_act_mul_kernel, dim3(slots), dim3(256), 0, s, p.y1, p.hidden, p.offsets, p.routed, p.ff, p.act); }, "moe_act_mul"));
    LinearF32Params r{};
    r.x = p.hidden, r.w = p.w2, r.y = p.y2, r.rows = slots, r.n = p.d, r.k = p.ff, r.ldx = p.ff, r.ldy = p.d, r.batch = p.routed, r.w_batch = (size_t)p.d * p.ff;
    r.bf16_products = 1, r.row_offsets = p.offsets;
    UZU_PROPAGATE(linear_mfma(s, r));
    return launch_check([&] { hipLaunchKernelGGL(moe_combine_kernel, dim3(p.rows), dim3(256), 0, s, p.y2, p.x, p.ids, p.weights, p.slot_pos, p.residual, p.y, p.d, p.routed, p.top); },
                        "moe_combine");
}

uzu_status embed_rows_f32(hipStream_t s, const uint32_t* tokens, const uint16_t* table, float* out, uint32_t rows, uint32_t vocab, uint32_t d, float scale) {
    if (!rows) return UZU_OK;
    return launch_check([&] { hipLaunchKernelGGL(embed_rows_f32_kernel, dim3(rows), dim3(256), 0, s, tokens, table, out, vocab, d, scale); }, "embed_rows_f32");
}

uzu_status embed_pair_rows_f32(hipStream_t s, const EmbedPairParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.tokens && p.table && p.pair_table && p.out && p.spans && p.row_seq && p.prev && p.buckets && p.nseq, "embed_pair_rows_f32: null argument");
    UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL(embed_pair_rows_f32_kernel, dim3(p.rows), dim3(256), 0, s, p); }, "embed_pair_rows_f32"));
    if (p.max_count == 1) return UZU_OK;
    return launch_check([&] { hipLaunchKernelGGL(embed_pair_commit_kernel, dim3((p.nseq + 63) / 64), dim3(64), 0, s, p, p.nseq); }, "embed_pair_commit");
}

uzu_status rms_norm_rows(hipStream_t s, const float* x, float* out, const float* scales, float gain, float eps, const uint32_t* row_index, uint32_t rows, uint32_t d,
                         float offset, uint32_t groups) {
    if (!rows) return UZU_OK;
    UZU_REQUIRE(x && out && d, "rms_norm_rows: null argument");
    if (!groups) groups = 1;
    UZU_REQUIRE(d % groups == 0 && groups <= 65535, "rms_norm_rows: %u coordinates in %u parts", d, groups);
    return launch_check([&] { hipLaunchKernelGGL(rms_norm_rows_kernel, dim3(rows, groups), dim3(256), 0, s, x, out, scales, gain, eps, row_index, d / groups, offset, d); },
                        "rms_norm_rows");
}

uzu_status rms_norm_add_rows(hipStream_t s, const float* y, const float* residual, float* out, const float* scales, float offset, const float* layer_scale, float eps,
                             uint32_t rows, uint32_t d, float* next, const float* next_scales, float next_offset, float next_eps, uint32_t groups) {
    if (!rows) return UZU_OK;
    UZU_REQUIRE(y && residual && out && scales && d && (!next || next_scales), "rms_norm_add_rows: null argument");
    if (!groups) groups = 1;
    UZU_REQUIRE(d % groups == 0 && groups <= 65535 && (groups == 1 || !next), "rms_norm_add_rows: %u coordinates in %u parts (the following norm only behind an undivided one)", d, groups);
    return launch_check([&] { hipLaunchKernelGGL(rms_norm_add_rows_kernel, dim3(rows, groups), dim3(256), 0, s, y, residual, out, scales, offset, layer_scale, eps, d / groups, next,
                                                 next_scales, next_offset, next_eps, d); }, "rms_norm_add_rows");
}

uzu_status gated_act_rows(hipStream_t s, const float* y1, float* hidden, uint32_t rows, uint32_t ff, const ExpertAct& act) {
    if (!rows || !ff) return UZU_OK;
    UZU_REQUIRE(y1 && hidden, "gated_act_rows: null argument");
    return launch_check([&] { hipLaunchKernelGGL(gated_act_rows_kernel, dim3((ff + 255) / 256, rows), dim3(256), 0, s, y1, hidden, ff, act); }, "gated_act_rows");
}

uzu_status dyn_tanh_norm(hipStream_t s, const DynTanhParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.x && p.out && p.scales, "dyn_tanh_norm: null argument");
    UZU_REQUIRE(!p.shift || (p.spans && p.row_seq && p.prev && !p.row_index), "dyn_tanh_norm: the token shift needs the pass's spans, row map and state rows");
    UZU_REQUIRE(!p.shift || p.x != p.out, "dyn_tanh_norm: the token shift reads neighbouring rows: not in place");
    const uint32_t gy = p.rows >= 1024 ? 1 : (p.d + 255) / 256 < 64 ? (p.d + 255) / 256 : 64;
    return launch_check([&] { hipLaunchKernelGGL(dyn_tanh_kernel, dim3(p.rows, gy), dim3(256), 0, s, p); }, "dyn_tanh_norm");
}

uzu_status depth_mix(hipStream_t s, const float* slots, size_t slot_stride, const float* w, uint32_t count, float* out, uint32_t rows, uint32_t d) {
    const size_t total = (size_t)rows * d;
    if (!total) return UZU_OK;
    return launch_check([&] { hipLaunchKernelGGL(depth_mix_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, slots, slot_stride, w, count, out, total); }, "depth_mix");
}

size_t linear_f32_bytes(const LinearF32Params& p) { return (size_t)p.batch * ((size_t)p.n * p.k * 2 + (size_t)p.rows * p.k * 4 + (size_t)p.rows * p.n * 4); }

uzu_status linear_f32(hipStream_t s, const LinearF32Params& p, const char** variant) {
    if (!p.rows || !p.n || !p.batch) return UZU_OK;
    UZU_REQUIRE(p.x && p.w && p.y && p.k, "linear_f32: null argument");
    UZU_REQUIRE(!p.residual || p.batch == 1, "linear_f32: a residual only with one product per launch");
    UZU_REQUIRE(!p.mul_table || (p.mul_tokens && p.batch == 1 && !p.row_offsets && p.mul_col0 + p.n <= p.mul_ld), "linear_f32: a token multiplier needs the rows' tokens, one product, columns inside the table");
    UZU_REQUIRE(p.ldx >= p.k && p.ldy >= p.n && p.batch <= 65535, "linear_f32: row pitch below the row length");
    if (p.row_offsets || p.row_map) { // the grouped / gathered form lives in the matrix-core kernel only
        UZU_UNSUPPORTED(!linear_mfma_supported(p), "linear_f32: grouped / gathered rows need bf16 products and 8-aligned k");
        if (variant) *variant = "linear_mfma_grouped";
        return linear_mfma(s, p);
    }
    if (p.rows <= 16) {
        const uint32_t vec = (p.k % 8 == 0 && p.ldx % 4 == 0 && p.x_batch % 4 == 0 && p.w_batch % 8 == 0 && (uintptr_t)p.x % 16 == 0 && (uintptr_t)p.w % 16 == 0) ? 1u : 0u;
        if (variant) *variant = "linear_rows";
        if (p.rows <= 2) {
            const dim3 grid((p.n + 3) / 4, (p.rows + 1) / 2, p.batch);
            return launch_check([&] { hipLaunchKernelGGL(linear_rows_kernel<2>, grid, dim3(256), 0, s, p, vec); }, "linear_rows");
        }
        const dim3 grid((p.n + 3) / 4, (p.rows + 3) / 4, p.batch);
        return launch_check([&] { hipLaunchKernelGGL(linear_rows_kernel<4>, grid, dim3(256), 0, s, p, vec); }, "linear_rows");
    }
    if (linear_mfma_supported(p)) {
        if (variant) *variant = "linear_mfma";
        return linear_mfma(s, p);
    }
    if (variant) *variant = "linear_tile";
    const dim3 grid((p.n + TN - 1) / TN, (p.rows + TM - 1) / TM, p.batch);
    UZU_REQUIRE(grid.y <= 65535, "linear_f32: too many rows for one launch");
    return launch_check([&] { hipLaunchKernelGGL(linear_tile_kernel, grid, dim3(256), 0, s, p); }, "linear_tile");
}

uzu_status moe_route_scores(hipStream_t s, const float* x, const uint16_t* router, const float* selection_bias, int32_t* ids, float* weights, uint32_t rows, uint32_t d,
                            uint32_t outputs, uint32_t top) {
    if (!rows) return UZU_OK;
    UZU_UNSUPPORTED(outputs > kRouteMaxOutputs || top > 64 || top > outputs || !top, "moe_route_scores: at most %u router outputs and 64 winners (got %u, %u)", kRouteMaxOutputs, outputs, top);
    return launch_check([&] { hipLaunchKernelGGL(moe_route_scores_kernel, dim3(rows), dim3(64), 0, s, x, router, selection_bias, ids, weights, d, outputs, top, 0u, (const uint16_t*)nullptr); }, "moe_route_scores");
}

uzu_status moe_route_topk(hipStream_t s, const float* x, const uint16_t* router, const uint16_t* router_bias, int32_t* ids, float* weights, uint32_t rows, uint32_t d,
                          uint32_t outputs, uint32_t top, uint32_t renorm) {
    if (!rows) return UZU_OK;
    UZU_UNSUPPORTED(outputs > kRouteMaxOutputs || top > 64 || top > outputs || !top, "moe_route_topk: at most %u router outputs and 64 winners (got %u, %u)", kRouteMaxOutputs, outputs, top);
    return launch_check([&] { hipLaunchKernelGGL(moe_route_scores_kernel, dim3(rows), dim3(64), 0, s, x, router, (const float*)nullptr, ids, weights, d, outputs, top, renorm ? 2u : 1u, router_bias); },
                        "moe_route_topk");
}

uzu_status moe_experts_gate_up(hipStream_t s, const float* x, const int32_t* ids, const uint16_t* w13, float* hidden, uint32_t rows, uint32_t d, uint32_t ff, uint32_t routed,
                               uint32_t top, uint32_t bf16_products, const ExpertAct& act) {
    if (!rows || !routed) return UZU_OK;
    UZU_UNSUPPORTED((size_t)d * 4 > 48 * 1024, "moe_experts_gate_up: model_dim %u does not fit the workgroup's LDS row", d);
    // few (row, slot) pairs (decode): the hidden units of a pair are spread over more workgroups, so that the expert's rows stream through many CUs
    const uint32_t want = (1024 + rows * top - 1) / (rows * top), most = (ff + 15) / 16;
    const uint32_t gy = want < 1 ? 1 : (want > most ? most : want);
    return launch_check([&] { hipLaunchKernelGGL(moe_experts_gate_up_kernel, dim3(rows * top, gy), dim3(256), (size_t)d * 4, s, x, ids, w13, hidden, d, ff, routed, top, bf16_products, act); },
                        "moe_experts_gate_up");
}

uzu_status moe_experts_down_combine(hipStream_t s, const float* hidden, const float* x, const int32_t* ids, const float* weights, const uint16_t* w2, const float* residual,
                                    float* y, uint32_t rows, uint32_t d, uint32_t ff, uint32_t routed, uint32_t top, uint32_t bf16_products) {
    if (!rows) return UZU_OK;
    const uint32_t staged = (size_t)top * ff * 4 <= 48 * 1024 ? 1u : 0u;
    const uint32_t want = (1024 + rows - 1) / rows, most = (d + 15) / 16;
    const uint32_t gy = want < 1 ? 1 : (want > most ? most : want);
    return launch_check([&] { hipLaunchKernelGGL(moe_experts_down_kernel, dim3(rows, gy), dim3(256), staged ? (size_t)top * ff * 4 : 0, s, hidden, x, ids, weights, w2, residual, y, d, ff, routed, top,
                                                  bf16_products, staged); }, "moe_experts_down_combine");
}

} // namespace k
} // namespace uzu
