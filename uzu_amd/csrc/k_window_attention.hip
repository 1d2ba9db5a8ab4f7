// k_window_attention.hip -- attention over a per-position cache of rotated keys and values for the f32-stream designs (kernels_stream32.h): rotation + key
// scaling + cache append, and the attention core with grouped heads, a soft cap on the scores, a causal sliding window and sink terms in the softmax denominator.
//
// Scores, softmax weights and the weighted sums are f32 whatever the cache holds (bf16 rows in the serving precision, f32 rows in the full-f32 mode).  A row's
// keys are walked in blocks of 64 counted from the first key the row sees, so the order of every sum depends on the row's position and the window only: not on
// how a prompt was cut into passes, and not on what else a pass carries.
#include "device_utils.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

namespace {

__device__ __forceinline__ float cache_ld(const void* p, uint32_t is_bf16, size_t i) { return is_bf16 ? bf16_to_f32(((const uint16_t*)p)[i]) : ((const float*)p)[i]; }
__device__ __forceinline__ void cache_st(void* p, uint32_t is_bf16, size_t i, float v) {
    if (is_bf16) ((uint16_t*)p)[i] = f32_to_bf16(v);
    else ((float*)p)[i] = v;
}

// a workgroup per row: query pairs in place, key pairs (+ the unrotated tail) to the cache or in place, values to the cache
__global__ void __launch_bounds__(256) rope_append_kernel(RopeAppendParams p) {
    const uint32_t r = blockIdx.x;
    const uint32_t z = p.row_seq[r];
    const SeqSpan sp = p.spans[z];
    const uint32_t t = sp.start + (r - sp.row0);
    float* row = p.qkv + (size_t)r * p.ld;
    const uint32_t half = p.rope_dim / 2;
    const float* cs = p.cosines + (size_t)t * p.rope_dim;
    const float* sn = p.sines + (size_t)t * p.rope_dim;
    // values first, as projected: with v_col == k_col the values are the keys in front of their norm and rotation
    if (p.kv_heads && p.value_caches) {
        void* vc = p.value_caches[z];
        const size_t vrow = (size_t)t * p.kv_heads * p.vdim;
        for (uint32_t idx = threadIdx.x; idx < p.kv_heads * p.vdim; idx += 256) cache_st(vc, p.cache_bf16, vrow + idx, row[p.v_col + idx]);
        __syncthreads();
    }
    if (p.norm_whole && (p.q_norm || p.k_norm)) { // one RMS norm over all query coordinates of the row, one over all key coordinates: 256 strided partial sums, a fixed tree
        __shared__ float s_red[256];
        for (int pass = 0; pass < 2; ++pass) {
            const float* w = pass ? p.k_norm : p.q_norm;
            const uint32_t n = pass ? p.kv_heads * p.dim : p.heads * p.dim;
            if (!w || !n) continue;
            float* h = pass ? row + p.k_col : row;
            float ss = 0.0f;
            for (uint32_t i = threadIdx.x; i < n; i += 256) ss = fmaf(h[i], h[i], ss);
            s_red[threadIdx.x] = ss;
            __syncthreads();
            for (uint32_t wd = 128; wd > 0; wd >>= 1) {
                if (threadIdx.x < wd) s_red[threadIdx.x] += s_red[threadIdx.x + wd];
                __syncthreads();
            }
            const float inv = 1.0f / sqrtf(s_red[0] / (float)n + p.norm_eps);
            __syncthreads();
            for (uint32_t i = threadIdx.x; i < n; i += 256) h[i] = h[i] * inv * w[i];
        }
        __syncthreads();
    } else if (p.q_norm || p.k_norm) { // a wave per head: x <- x / sqrt(mean(x^2) + eps) * w over the head's coordinates, in front of the rotation
        const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        for (uint32_t a = wave; a < p.heads + p.kv_heads; a += 4) {
            const bool is_q = a < p.heads;
            const float* w = is_q ? p.q_norm : p.k_norm;
            if (!w) continue;
            float* h = is_q ? row + (size_t)a * p.dim : row + p.k_col + (size_t)(a - p.heads) * p.dim;
            float ss = 0.0f;
            for (uint32_t i = lane; i < p.dim; i += 64) ss = fmaf(h[i], h[i], ss);
            ss = wave_sum(ss);
            const float inv = 1.0f / sqrtf(ss / (float)p.dim + p.norm_eps);
            for (uint32_t i = lane; i < p.dim; i += 64) h[i] = h[i] * inv * w[i];
        }
        __syncthreads();
    }
    for (uint32_t idx = threadIdx.x; idx < p.heads * half; idx += 256) {
        const uint32_t a = idx / half, i = idx - a * half;
        float* h = row + (size_t)a * p.dim;
        const uint32_t iu = p.interleaved ? 2 * i : i, iv = p.interleaved ? 2 * i + 1 : i + half;
        const float u = h[iu], v = h[iv], c = cs[i], s = sn[i];
        h[iu] = u * c - v * s;
        h[iv] = v * c + u * s;
    }
    if (!p.kv_heads) return;
    const float ks = p.key_scale;
    void* kc = p.key_caches ? p.key_caches[z] : nullptr;
    const size_t krow = (size_t)t * p.kv_heads * p.dim;
    for (uint32_t idx = threadIdx.x; idx < p.kv_heads * p.dim; idx += 256) {
        const uint32_t g = idx / p.dim, c = idx - g * p.dim;
        float* h = row + p.k_col + (size_t)g * p.dim;
        if (c >= p.rope_dim) {
            const float a = h[c] * ks;
            if (kc) cache_st(kc, p.cache_bf16, krow + idx, a);
            else h[c] = a;
        } else if (p.interleaved ? (c & 1) == 0 : c < half) { // the thread of a pair's first coordinate turns the pair
            const uint32_t step = p.interleaved ? 1 : half, i = p.interleaved ? c >> 1 : c;
            const float u = h[c], v = h[c + step], co = cs[i], s = sn[i];
            const float a = (u * co - v * s) * ks, b = (v * co + u * s) * ks;
            if (kc) cache_st(kc, p.cache_bf16, krow + idx, a), cache_st(kc, p.cache_bf16, krow + idx + step, b);
            else h[c] = a, h[c + step] = b;
        }
    }
}

// ---- the simple form: a wave per (row, head).  Keys in blocks of 64 from the row's first visible key: a lane scores one key of the block (the whole dot
// product, the query staged in LDS), the block's weights go through LDS, then a lane owns value coordinates lane, lane + 64, ... of the running sum.
constexpr uint32_t kMaxVecPerLane = 8; // value widths up to 512
__global__ void __launch_bounds__(64) window_attention_simple_kernel(WindowAttentionParams p) {
    extern __shared__ float s_mem[]; // [dim] query + [64] weights
    float* s_q = s_mem;
    float* s_p = s_mem + p.dim;
    const uint32_t r = blockIdx.x, a = blockIdx.y, lane = threadIdx.x;
    const uint32_t z = p.row_seq[r];
    const SeqSpan sp = p.spans[z];
    const uint32_t t = sp.start + (r - sp.row0);
    const uint32_t g = a / (p.heads / p.kv_heads);
    const void* K = p.key_caches[z];
    const void* V = p.value_caches[z];
    uint32_t lo = (p.window && t + 1 > p.window) ? t + 1 - p.window : 0u;
    if (p.chunk) lo = max(lo, t / p.chunk * p.chunk);
    const float hscale = p.head_scale ? p.scale * p.head_scale[a] : p.scale;
    const float* q = p.q + (size_t)r * p.ldq + (size_t)a * p.dim;
    for (uint32_t c = lane; c < p.dim; c += 64) s_q[c] = q[c];
    __syncthreads();
    float m = p.sinks ? p.sinks[a] : -INFINITY, l = p.sinks ? 1.0f : 0.0f;
    float acc[kMaxVecPerLane];
#pragma unroll
    for (uint32_t i = 0; i < kMaxVecPerLane; ++i) acc[i] = 0.0f;
    const size_t kpitch = (size_t)p.kv_heads * p.dim, vpitch = (size_t)p.kv_heads * p.vdim;
    for (uint32_t j0 = lo; j0 <= t; j0 += 64) {
        const uint32_t j = j0 + lane;
        float s = -INFINITY;
        if (j <= t) {
            const size_t base = (size_t)j * kpitch + (size_t)g * p.dim;
            float dot = 0.0f;
            if (p.cache_bf16) {
                const uint16_t* kr = (const uint16_t*)K + base;
                if ((p.dim & 7) == 0 && (((uintptr_t)kr) & 15) == 0) {
                    for (uint32_t c = 0; c < p.dim; c += 8) {
                        const uint4 kv = *(const uint4*)(kr + c);
                        const uint32_t w[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            dot = fmaf(s_q[c + 2 * i], bits_to_f32(w[i] << 16), dot);
                            dot = fmaf(s_q[c + 2 * i + 1], bits_to_f32(w[i] & 0xFFFF0000u), dot);
                        }
                    }
                } else {
                    for (uint32_t c = 0; c < p.dim; ++c) dot = fmaf(s_q[c], bf16_to_f32(kr[c]), dot);
                }
            } else {
                const float* kr = (const float*)K + base;
                for (uint32_t c = 0; c < p.dim; ++c) dot = fmaf(s_q[c], kr[c], dot);
            }
            s = dot * hscale;
            if (p.soft_cap != 0.0f) s = p.soft_cap * tanhf(s / p.soft_cap);
            if (p.dist_bias) s += p.dist_bias[(size_t)min(t - j, p.dist_rows - 1) * p.heads + a];
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float w = j <= t ? expf(s - m_new) : 0.0f;
        const float corr = expf(m - m_new); // (first block without a sink: exp(-inf) = 0 against l = 0 and zero sums)
        l = l * corr + wave_sum(w);
        m = m_new;
        __syncthreads();
        s_p[lane] = w;
        __syncthreads();
        const uint32_t nk = t - j0 + 1 < 64 ? t - j0 + 1 : 64;
#pragma unroll
        for (uint32_t i = 0; i < kMaxVecPerLane; ++i) {
            const uint32_t c = lane + 64 * i;
            if (c >= p.vdim) break;
            float sum = acc[i] * corr;
            const size_t vb = (size_t)j0 * vpitch + (size_t)g * p.vdim + c;
            for (uint32_t jj = 0; jj < nk; ++jj) sum = fmaf(s_p[jj], cache_ld(V, p.cache_bf16, vb + (size_t)jj * vpitch), sum);
            acc[i] = sum;
        }
    }
    float* o = p.out + ((size_t)r * p.heads + a) * p.vdim;
    const float og = p.gate ? 1.0f / (1.0f + expf(-p.gate[(size_t)r * p.ldgate + a])) : 1.0f;
#pragma unroll
    for (uint32_t i = 0; i < kMaxVecPerLane; ++i) {
        const uint32_t c = lane + 64 * i;
        if (c >= p.vdim) break;
        o[c] = p.gate ? acc[i] / l * og : acc[i] / l;
    }
}

} // namespace

uzu_status rope_append(hipStream_t s, const RopeAppendParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.qkv && p.spans && p.row_seq && p.heads && p.dim, "rope_append: null argument");
    UZU_REQUIRE(p.rope_dim % 2 == 0 && p.rope_dim <= p.dim && (!p.rope_dim || (p.cosines && p.sines)), "rope_append: rotation width %u of a head of %u (even, with its tables)", p.rope_dim, p.dim);
    UZU_REQUIRE(!p.kv_heads || ((p.key_caches != nullptr) == (p.value_caches != nullptr)), "rope_append: key and value caches come together");
    UZU_REQUIRE(p.v_col != p.k_col || !p.kv_heads || (p.vdim == p.dim && p.value_caches), "rope_append: values that are the key rows have the keys' width and go to a cache");
    return launch_check([&] { hipLaunchKernelGGL(rope_append_kernel, dim3(p.rows), dim3(256), 0, s, p); }, "rope_append");
}

uzu_status window_attention_mfma(hipStream_t s, const WindowAttentionParams& p); // k_window_attention_mfma.hip

uzu_status window_attention(hipStream_t s, const WindowAttentionParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.q && p.out && p.key_caches && p.value_caches && p.spans && p.row_seq, "window_attention: null argument");
    UZU_REQUIRE(p.heads && p.kv_heads && p.heads % p.kv_heads == 0 && p.dim && p.vdim, "window_attention: %u query heads on %u key / value heads", p.heads, p.kv_heads);
    UZU_UNSUPPORTED(p.vdim > 64 * kMaxVecPerLane || p.dim > 8192, "window_attention: value width %u (at most %u)", p.vdim, 64 * kMaxVecPerLane);
    UZU_REQUIRE(!p.dist_bias || p.dist_rows, "window_attention: a distance bias without its rows");
    if (p.form == 2 || (p.form == 0 && window_attention_mfma_supported(p))) {
        UZU_UNSUPPORTED(!window_attention_mfma_supported(p), "window_attention: the matrix-core form does not take this shape");
        return window_attention_mfma(s, p);
    }
    UZU_REQUIRE(p.heads <= 65535, "window_attention: too many heads for one launch");
    return launch_check([&] { hipLaunchKernelGGL(window_attention_simple_kernel, dim3(p.rows, p.heads), dim3(64), (size_t)(p.dim + 64) * 4, s, p); }, "window_attention");
}

} // namespace k
} // namespace uzu
