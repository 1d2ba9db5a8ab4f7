// k_latent_attention.hip -- attention over a cached low-rank latent (UZU_MIXER_LATENT_ATTENTION; kernels_stream32.h).
//
// Per token the state keeps ONE row c = RMSNorm(W_down h) of `rank` numbers for all heads.  A head's key is W_up_k c and its value W_up_v c, so
//   score(i, j) = <q_i, W_up_k c_j> = <W_up_k^T q_i, c_j>          and          sum_j p_j W_up_v c_j = W_up_v (sum_j p_j c_j):
// the engine folds W_up_k into the query (a batched product per head) and applies W_up_v to the result, and the core below is attention with one shared
// "key = value" row per token in latent space -- the cache is read once per (row, head) and never expanded.  Scores, the softmax and the weighted sum are f32
// in both precisions; a sink adds exp(sink_h) to the denominator and nothing to the sum; the window keeps keys t - window < j <= t.
//
// The summation order over the keys depends on the row's position and the window only, so a row's result is the same whatever else the pass carries.
#include "device_utils.h"
#include "gemm_convert.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

namespace {

__device__ __forceinline__ float cache_ld(const void* c, uint32_t bf16, size_t i) { return bf16 ? bf16_to_f32(((const uint16_t*)c)[i]) : ((const float*)c)[i]; }

// a wave per row
__global__ void __launch_bounds__(256) latent_norm_append_kernel(const float* x, const float* scales, float eps, void* const* caches, uint32_t cache_bf16, const SeqSpan* spans,
                                                                 const uint32_t* row_seq, uint32_t rows, uint32_t rank) {
    const uint32_t lane = threadIdx.x & 63, r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const float* xr = x + (size_t)r * rank;
    float ss = 0.0f;
    for (uint32_t i = lane; i < rank; i += 64) ss = fmaf(xr[i], xr[i], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
    const uint32_t q = row_seq[r];
    const SeqSpan sp = spans[q];
    const size_t base = (size_t)(sp.start + (r - sp.row0)) * rank;
    void* c = caches[q];
    for (uint32_t i = lane; i < rank; i += 64) {
        const float v = xr[i] * inv * scales[i];
        if (cache_bf16) ((uint16_t*)c)[base + i] = f32_to_bf16(v);
        else ((float*)c)[base + i] = v;
    }
}

// a workgroup per row: wave 0 norms the latent and writes [latent | rotated key part] to the cache, all waves turn the query heads' rotated parts into qlat
__global__ void __launch_bounds__(256) latent_rope_append_kernel(LatentRopeAppendParams p) {
    const uint32_t r = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t q = p.row_seq[r];
    const SeqSpan sp = p.spans[q];
    const uint32_t t = sp.start + (r - sp.row0);
    const float* xr = p.x + (size_t)r * p.ldx;
    const uint32_t kw = p.rank + p.rope_dim, half = p.rope_dim / 2;
    const float* cs = p.rope_dim ? p.cosines + (size_t)t * p.rope_dim : nullptr;
    const float* sn = p.rope_dim ? p.sines + (size_t)t * p.rope_dim : nullptr;
    // pair i of a rotated part: coordinates (2i, 2i + 1) or (i, i + half)
    auto lo_of = [&](uint32_t i) { return p.interleaved ? 2 * i : i; };
    auto hi_of = [&](uint32_t i) { return p.interleaved ? 2 * i + 1 : i + half; };
    if (wave == 0 && p.caches) {
        const float* c = xr + p.c_col;
        float ss = 0.0f;
        for (uint32_t i = lane; i < p.rank; i += 64) ss = fmaf(c[i], c[i], ss);
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)p.rank + p.eps);
        void* cache = p.caches[q];
        const size_t base = (size_t)t * kw;
        for (uint32_t i = lane; i < p.rank; i += 64) {
            const float v = c[i] * inv * p.scales[i];
            if (p.cache_bf16) ((uint16_t*)cache)[base + i] = f32_to_bf16(v);
            else ((float*)cache)[base + i] = v;
        }
        const float* kr = c + p.rank;
        for (uint32_t i = lane; i < half; i += 64) {
            const float u = kr[lo_of(i)], v = kr[hi_of(i)], co = cs[i], si = sn[i];
            const float a = u * co - v * si, b = v * co + u * si;
            if (p.cache_bf16) ((uint16_t*)cache)[base + p.rank + lo_of(i)] = f32_to_bf16(a), ((uint16_t*)cache)[base + p.rank + hi_of(i)] = f32_to_bf16(b);
            else ((float*)cache)[base + p.rank + lo_of(i)] = a, ((float*)cache)[base + p.rank + hi_of(i)] = b;
        }
    }
    if (!p.qlat) return;
    for (uint32_t idx = threadIdx.x; idx < p.heads * half; idx += 256) {
        const uint32_t a = idx / half, i = idx - a * half;
        const float* qr = xr + (size_t)a * p.q_width + (p.q_width - p.rope_dim);
        float* dst = p.qlat + ((size_t)r * p.heads + a) * kw + p.rank;
        const float u = qr[lo_of(i)], v = qr[hi_of(i)], co = cs[i], si = sn[i];
        dst[lo_of(i)] = u * co - v * si;
        dst[hi_of(i)] = v * co + u * si;
    }
}

// Simple form: a wave per (row, head), lane = latent elements lane, lane + 64, ...; the keys one after the other with a running maximum.
template <int NT>
__global__ void __launch_bounds__(256) latent_attention_rows_kernel(LatentAttentionParams p) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t item = blockIdx.x * 4 + (threadIdx.x >> 6); // (row, head), heads of a row next to each other: they read the same latents
    if (item >= p.rows * p.heads) return;
    const uint32_t r = item / p.heads, h = item % p.heads;
    const uint32_t q = p.row_seq[r];
    const SeqSpan sp = p.spans[q];
    const uint32_t t = sp.start + (r - sp.row0);
    const uint32_t lo = (p.window && t + 1 > p.window) ? t + 1 - p.window : 0;
    const void* cache = p.caches[q];
    const float* ql = p.qlat + ((size_t)r * p.heads + h) * p.rank;
    float qv[NT], acc[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        const uint32_t e = i * 64 + lane;
        qv[i] = e < p.rank ? ql[e] * p.scale : 0.0f;
        acc[i] = 0.0f;
    }
    // the sink takes part in the maximum and in the denominator only
    float m = p.sinks ? p.sinks[h] : -INFINITY;
    float l = p.sinks ? 1.0f : 0.0f;
    for (uint32_t j = lo; j <= t; ++j) {
        float cv[NT];
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const uint32_t e = i * 64 + lane;
            cv[i] = e < p.rank ? cache_ld(cache, p.cache_bf16, (size_t)j * p.rank + e) : 0.0f;
            s = fmaf(qv[i], cv[i], s);
        }
        s = wave_sum(s);
        const float mn = fmaxf(m, s);
        const float corr = expf(m - mn), pj = expf(s - mn); // m == -inf only before the first key of a sink-less head: corr = 0 on l = 0
        l = fmaf(l, corr, pj);
#pragma unroll
        for (int i = 0; i < NT; ++i) acc[i] = fmaf(acc[i], corr, pj * cv[i]);
        m = mn;
    }
    const float inv = 1.0f / l;
    float* out = p.out + ((size_t)r * p.heads + h) * p.rank;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        const uint32_t e = i * 64 + lane;
        if (e < p.rank) out[e] = acc[i] * inv;
    }
}

// Tiled form on the bf16 matrix cores (bf16 cache).  An ITEM is a (row, head) pair of one sequence, items numbered row-major; a wave owns 32 consecutive
// items, a workgroup four such tiles -- with 16 heads that is 8 neighbouring rows, whose windows overlap almost entirely, so a 32-key block of latents is
// staged once in LDS for 128 items.  Everything is computed transposed so that a lane owns one item:
//   S^T = C Q^T    A = the block's latent rows [key][rank] from LDS, B = the item's query fragments (registers, bf16 of the f32 latent query);
//                  the result gives a lane 16 key scores of ITS item, so the running maximum / sum are per-lane scalars (one exchange with lane ^ 32);
//   O^T += C^T P^T A = the block transposed [rank][key] from LDS, B = those 16 weights, fed as hi + lo bf16 (16 significant bits: the weights stay f32 up
//                  to the product); the accumulator columns are again "this lane's item": rescaling and the final 1 / l are per-lane multiplies.
// The k order inside an MFMA only has to agree between A and B: for O^T the lane's keys are taken in the order the S^T result already holds them.
// Scores are scaled and masked in f32 behind the MFMA; the sink enters as the initial maximum with weight 1 in the denominator.
// SPLIT (few items, many keys: decode steps): grid.y workgroups share an item tile's key blocks (block i goes to workgroup i mod grid.y) and leave unnormalised
// sums with their running maximum / denominator in p.split_ws; latent_attention_merge_kernel combines them.  The sink belongs to split 0.
template <int NB, bool SPLIT> // rank padded to RP = 32 NB
__global__ void __launch_bounds__(256) latent_attention_mfma_kernel(LatentAttentionParams p) {
    constexpr int RP = 32 * NB, CP = RP * 2 + 16, TP = 80, VEC = RP / 8;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* s_c = smem;            // [32 keys][CP bytes]
    uint8_t* s_ct = smem + 32 * CP; // [RP][TP bytes]: 32 keys + pad
    uint32_t wg = blockIdx.x, q = 0;
    SeqSpan sp{0, 0, 0};
    for (;; ++q) {
        if (q >= p.nseq) return;
        sp = p.spans[q];
        const uint32_t n = (sp.count * p.heads + 127) / 128;
        if (wg < n) break;
        wg -= n;
    }
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5;
    const uint32_t items = sp.count * p.heads;
    auto row_lo = [&](uint32_t t) { return (p.window && t + 1 > p.window) ? t + 1 - p.window : 0u; };
    // this lane's item
    const uint32_t g = wg * 128 + wave * 32 + l32;
    const bool valid = g < items;
    const uint32_t gi = valid ? g : items - 1;
    const uint32_t row = gi / p.heads, head = gi % p.heads;
    const uint32_t t = sp.start + row, lo = row_lo(t);
    // key ranges of the workgroup and of this wave
    const uint32_t g_last = (wg * 128 + 128 < items ? wg * 128 + 128 : items) - 1;
    const uint32_t kmin = row_lo(sp.start + wg * 128 / p.heads), kmax = sp.start + g_last / p.heads;
    const uint32_t w_first = wg * 128 + wave * 32;
    const bool wave_on = w_first < items;
    const uint32_t w_last = (w_first + 32 < items ? w_first + 32 : items) - 1;
    const uint32_t wave_lo = wave_on ? row_lo(sp.start + w_first / p.heads) : 0, wave_hi = wave_on ? sp.start + w_last / p.heads : 0;

    u32x4_t qf[2 * NB];
    {
        const float* qrow = p.qlat + ((size_t)(sp.row0 + row) * p.heads + head) * p.rank;
#pragma unroll
        for (int s = 0; s < 2 * NB; ++s) {
            const uint32_t k0 = s * 16 + half * 8;
            u32x4_t f{0u, 0u, 0u, 0u};
            if (valid && k0 < p.rank) { // rank % 8 == 0: a fragment is inside the row or outside it
                const f32x4_v a = *(const f32x4_v*)(qrow + k0), b = *(const f32x4_v*)(qrow + k0 + 4);
                f.x = (uint32_t)f32_to_bf16(a.x) | ((uint32_t)f32_to_bf16(a.y) << 16), f.y = (uint32_t)f32_to_bf16(a.z) | ((uint32_t)f32_to_bf16(a.w) << 16);
                f.z = (uint32_t)f32_to_bf16(b.x) | ((uint32_t)f32_to_bf16(b.y) << 16), f.w = (uint32_t)f32_to_bf16(b.z) | ((uint32_t)f32_to_bf16(b.w) << 16);
            }
            qf[s] = f;
        }
    }
    const bool with_sink = p.sinks && (!SPLIT || blockIdx.y == 0);
    float m_run = with_sink ? p.sinks[head] : -1.0e30f;
    float l_run = with_sink ? 1.0f : 0.0f;
    f32x16_t o[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[b][r] = 0.0f;
    const uint8_t* cache = (const uint8_t*)p.caches[q];
    // a cache row whose tail takes part in the scores only (value_rank < rank): the score product stops behind the row's last 16-column step, the weighted sum
    // covers the value columns' 32-column blocks only
    const uint32_t vr = p.value_rank ? p.value_rank : p.rank;
    const uint32_t nsteps = (p.rank + 15) / 16, nbv = (vr + 31) / 32;

    const uint32_t kstep = SPLIT ? 32 * gridDim.y : 32;
    for (uint32_t kb = kmin + (SPLIT ? 32 * blockIdx.y : 0); kb <= kmax; kb += kstep) {
        __syncthreads(); // the block before has been read
        for (uint32_t v = tid; v < 32 * VEC; v += 256) {
            const uint32_t key = v / VEC, e0 = (v % VEC) * 8, kk = kb + key;
            u32x4_v val{0u, 0u, 0u, 0u};
            if (kk <= kmax && e0 < p.rank) val = *(const u32x4_v*)(cache + ((size_t)kk * p.rank + e0) * 2);
            *(u32x4_v*)(s_c + key * CP + e0 * 2) = val;
            const uint32_t w[4] = {val.x, val.y, val.z, val.w};
            if (e0 >= nbv * 32) continue; // columns outside the value blocks have no transposed copy
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                *(uint16_t*)(s_ct + (e0 + 2 * e) * TP + key * 2) = (uint16_t)(w[e] & 0xFFFFu);
                *(uint16_t*)(s_ct + (e0 + 2 * e + 1) * TP + key * 2) = (uint16_t)(w[e] >> 16);
            }
        }
        __syncthreads();
        if (!wave_on || kb > wave_hi || kb + 31 < wave_lo) continue; // (wave-uniform; the barriers above are reached by every wave)
        f32x16_t st;
#pragma unroll
        for (int r = 0; r < 16; ++r) st[r] = 0.0f;
#pragma unroll
        for (int s = 0; s < 2 * NB; ++s) {
            if ((uint32_t)s < nsteps) { // (a predicate, not a break: the loop stays unrolled and qf / o statically indexed)
                const u32x4_t a = *(const u32x4_t*)(s_c + l32 * CP + (s * 16 + half * 8) * 2);
                st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, qf[s]), st, 0, 0, 0);
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t key = kb + (r & 3) + 8 * (r >> 2) + 4 * half;
            const bool ok = valid && key >= lo && key <= t;
            st[r] = ok ? st[r] * p.scale : -INFINITY;
            mx = fmaxf(mx, st[r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        const float corr = fast_exp(m_run - m_new);
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            st[r] = fast_exp(st[r] - m_new); // masked: exp(-inf) = 0
            psum += st[r];
        }
        psum += __shfl_xor(psum, 32, 64);
        l_run = fmaf(l_run, corr, psum);
        m_run = m_new;
#pragma unroll
        for (int b = 0; b < NB; ++b)
            if ((uint32_t)b < nbv)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[b][r] *= corr;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            u32x4_t hi, lw;
            uint32_t hw[4], lwv[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float p0 = st[8 * s2 + 2 * e], p1 = st[8 * s2 + 2 * e + 1];
                const uint16_t h0 = f32_to_bf16(p0), h1 = f32_to_bf16(p1);
                const uint16_t l0 = f32_to_bf16(p0 - bf16_to_f32(h0)), l1 = f32_to_bf16(p1 - bf16_to_f32(h1));
                hw[e] = (uint32_t)h0 | ((uint32_t)h1 << 16), lwv[e] = (uint32_t)l0 | ((uint32_t)l1 << 16);
            }
            hi = u32x4_t{hw[0], hw[1], hw[2], hw[3]}, lw = u32x4_t{lwv[0], lwv[1], lwv[2], lwv[3]};
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                if ((uint32_t)b < nbv) {
                    const uint8_t* cr = s_ct + (b * 32 + l32) * TP + (16 * s2 + 4 * half) * 2;
                    const u32x2_v c0 = *(const u32x2_v*)cr, c1 = *(const u32x2_v*)(cr + 16);
                    const u32x4_t cf{c0.x, c0.y, c1.x, c1.y};
                    o[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, cf), __builtin_bit_cast(bf16x8_t, hi), o[b], 0, 0, 0);
                    o[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, cf), __builtin_bit_cast(bf16x8_t, lw), o[b], 0, 0, 0);
                }
            }
        }
    }
    if (!valid) return;
    if (SPLIT) {
        float* ws = p.split_ws + (((size_t)(sp.row0 + row) * p.heads + head) * gridDim.y + blockIdx.y) * (RP + 4);
#pragma unroll
        for (int b = 0; b < NB; ++b)
            if ((uint32_t)b < nbv)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4)
                    *(f32x4_v*)(ws + b * 32 + 8 * g4 + 4 * half) = f32x4_v{o[b][4 * g4], o[b][4 * g4 + 1], o[b][4 * g4 + 2], o[b][4 * g4 + 3]};
        if (half == 0) ws[RP] = m_run, ws[RP + 1] = l_run;
        return;
    }
    const float inv = 1.0f / l_run;
    float* out = p.out + ((size_t)(sp.row0 + row) * p.heads + head) * p.rank;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            const uint32_t col = b * 32 + 8 * g4 + 4 * half;
            if (col < vr) *(f32x4_v*)(out + col) = f32x4_v{o[b][4 * g4] * inv, o[b][4 * g4 + 1] * inv, o[b][4 * g4 + 2] * inv, o[b][4 * g4 + 3] * inv};
        }
}

// a workgroup per item: out = sum_s e^(m_s - M) O_s / sum_s e^(m_s - M) l_s over the splits (a split that saw no key has l = 0 and m = -1e30: weight 0).
// The splits' weights are formed once (one thread per split, through LDS); the sums over the splits run in split order.
// (cols <= rank: the value columns; an item's row of `out` is rank wide)
__global__ void __launch_bounds__(256) latent_attention_merge_kernel(const float* ws, float* out, uint32_t items, uint32_t splits, uint32_t rank, uint32_t rp, uint32_t cols) {
    __shared__ float s_w[64];
    __shared__ float s_inv;
    const uint32_t item = blockIdx.x, tid = threadIdx.x;
    const float* base = ws + (size_t)item * splits * (rp + 4);
    if (tid < 64) {
        const float m = tid < splits ? base[(size_t)tid * (rp + 4) + rp] : -1.0e30f;
        const float M = wave_max(m);
        const float w = fast_exp(m - M);
        s_w[tid] = w;
    }
    __syncthreads();
    if (tid == 0) {
        float L = 0.0f;
        for (uint32_t s = 0; s < splits; ++s) L = fmaf(s_w[s], base[(size_t)s * (rp + 4) + rp + 1], L);
        s_inv = 1.0f / L;
    }
    __syncthreads();
    const float inv = s_inv;
    for (uint32_t e = tid; e < cols; e += blockDim.x) {
        float acc = 0.0f;
        for (uint32_t s = 0; s < splits; ++s) acc = fmaf(s_w[s], base[(size_t)s * (rp + 4) + e], acc);
        out[(size_t)item * rank + e] = acc * inv;
    }
}

} // namespace

size_t latent_attention_split_ws_bytes(uint32_t rows, uint32_t heads, uint32_t rank, uint32_t splits) {
    const uint32_t rp = rank <= 128 ? 128 : 256;
    return (size_t)rows * heads * splits * (rp + 4) * 4;
}

bool latent_attention_tiled_supported(const LatentAttentionParams& p) {
    return p.cache_bf16 && p.rank % 8 == 0 && p.rank <= 256 && p.nseq > 0 && p.tiles > 0 && (uintptr_t)p.qlat % 16 == 0 && (uintptr_t)p.out % 16 == 0;
}

uzu_status latent_norm_append(hipStream_t s, const float* x, const float* scales, float eps, void* const* caches, uint32_t cache_bf16, const SeqSpan* spans,
                              const uint32_t* row_seq, uint32_t rows, uint32_t rank) {
    if (!rows) return UZU_OK;
    UZU_REQUIRE(x && scales && caches && spans && row_seq && rank, "latent_norm_append: null argument");
    return launch_check([&] { hipLaunchKernelGGL(latent_norm_append_kernel, dim3((rows + 3) / 4), dim3(256), 0, s, x, scales, eps, caches, cache_bf16, spans, row_seq, rows, rank); },
                        "latent_norm_append");
}

uzu_status latent_rope_append(hipStream_t s, const LatentRopeAppendParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.x && p.spans && p.row_seq && p.rank && (!p.caches || p.scales), "latent_rope_append: null argument");
    UZU_REQUIRE(p.rope_dim % 2 == 0 && (!p.rope_dim || (p.cosines && p.sines && p.q_width >= p.rope_dim)), "latent_rope_append: an even rotated width with its tables");
    UZU_REQUIRE(p.c_col + p.rank + p.rope_dim <= p.ldx && (!p.qlat || p.heads * p.q_width <= p.ldx), "latent_rope_append: columns outside the row");
    return launch_check([&] { hipLaunchKernelGGL(latent_rope_append_kernel, dim3(p.rows), dim3(256), 0, s, p); }, "latent_rope_append");
}

uzu_status latent_attention(hipStream_t s, const LatentAttentionParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.qlat && p.out && p.caches && p.spans && p.row_seq && p.heads && p.rank, "latent_attention: null argument");
    UZU_UNSUPPORTED(p.rank > kLatentMaxRank, "latent_attention: latent rank %u above %u", p.rank, kLatentMaxRank);
    UZU_REQUIRE(p.value_rank <= p.rank && p.value_rank % 4 == 0, "latent_attention: value_rank is a multiple of 4 of at most rank");
    UZU_UNSUPPORTED(p.form == 2 && !latent_attention_tiled_supported(p), "latent_attention: the tiled form takes a bf16 cache, rank %% 8 == 0, rank <= 256");
    if (p.form != 1 && latent_attention_tiled_supported(p)) {
        static LdsLimit lim4, lim8, lim4s, lim8s;
        const uint32_t rp = p.rank <= 128 ? 128 : 256;
        const size_t lds = 32 * (rp * 2 + 16) + rp * 80;
        // few item tiles over many keys (decode steps): the key blocks of a tile are spread over `splits` workgroups and merged by a second launch
        const uint32_t splits = (p.split_ws && p.splits > 1 && p.splits <= 64 && latent_attention_split_ws_bytes(p.rows, p.heads, p.rank, p.splits) <= p.split_ws_bytes) ? p.splits : 1;
        if (splits > 1) {
            const dim3 grid(p.tiles, splits);
            if (rp == 128) {
                raise_lds_limit(lim4s, (const void*)latent_attention_mfma_kernel<4, true>, lds);
                UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL((latent_attention_mfma_kernel<4, true>), grid, dim3(256), lds, s, p); }, "latent_attention_mfma_split"));
            } else {
                raise_lds_limit(lim8s, (const void*)latent_attention_mfma_kernel<8, true>, lds);
                UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL((latent_attention_mfma_kernel<8, true>), grid, dim3(256), lds, s, p); }, "latent_attention_mfma_split"));
            }
            const uint32_t items = p.rows * p.heads;
            return launch_check([&] { hipLaunchKernelGGL(latent_attention_merge_kernel, dim3(items), dim3(256), 0, s, p.split_ws, p.out, items, splits, p.rank, rp, p.value_rank ? p.value_rank : p.rank); },
                                "latent_attention_merge");
        }
        if (rp == 128) {
            raise_lds_limit(lim4, (const void*)latent_attention_mfma_kernel<4, false>, lds);
            return launch_check([&] { hipLaunchKernelGGL((latent_attention_mfma_kernel<4, false>), dim3(p.tiles), dim3(256), lds, s, p); }, "latent_attention_mfma");
        }
        raise_lds_limit(lim8, (const void*)latent_attention_mfma_kernel<8, false>, lds);
        return launch_check([&] { hipLaunchKernelGGL((latent_attention_mfma_kernel<8, false>), dim3(p.tiles), dim3(256), lds, s, p); }, "latent_attention_mfma");
    }
    const uint32_t items = p.rows * p.heads;
    const dim3 grid((items + 3) / 4), block(256);
    const uint32_t nt = (p.rank + 63) / 64;
    if (nt <= 1) return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<1>, grid, block, 0, s, p); }, "latent_attention");
    if (nt <= 2) return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<2>, grid, block, 0, s, p); }, "latent_attention");
    if (nt <= 4) return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<4>, grid, block, 0, s, p); }, "latent_attention");
    if (nt <= 8) return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<8>, grid, block, 0, s, p); }, "latent_attention");
    if (nt <= 16) return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<16>, grid, block, 0, s, p); }, "latent_attention");
    return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<32>, grid, block, 0, s, p); }, "latent_attention");
}

} // namespace k
} // namespace uzu
