// k_window_attention_mfma.hip -- the matrix-core form of the attention over cached keys and values (kernels_stream32.h::window_attention): prompt-sized
// passes over bf16 caches.
//
// Items are (row, query head) pairs of ONE sequence and ONE key / value head: a wave owns 32 of them, a workgroup 128, so with heads / kv_heads = 4 a
// workgroup's 32 neighbouring rows share every staged block of 32 keys.  Both products are computed transposed with v_mfma_f32_32x32x16_bf16, so that a lane
// owns one item:
//   S^T = K Q^T     A = the key block [32][dim] from LDS, B = the item's query, rounded to bf16 as hi + lo (two products: the query keeps 16 significant bits);
//                   the result gives a lane 16 key scores of ITS item, so scale, cap, mask and the running maximum / sum are per-lane work (one exchange
//                   with lane ^ 32);
//   O^T += V^T P^T  A = the value block transposed [vdim][32] from LDS, B = those 16 weights as hi + lo bf16; rescaling and the final 1 / l are per lane.
// The k order inside an MFMA only has to agree between A and B: for O^T the lane's keys are taken in the order the S^T result already holds them.
// Scores, weights and sums are f32; the sink enters as the initial maximum with weight 1 in the denominator.
#include "device_utils.h"
#include "gemm_convert.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

namespace {

__device__ __forceinline__ void split_bf16(float a, float b, uint32_t& hi, uint32_t& lo) {
    const uint16_t h0 = f32_to_bf16(a), h1 = f32_to_bf16(b);
    const uint16_t l0 = f32_to_bf16(a - bf16_to_f32(h0)), l1 = f32_to_bf16(b - bf16_to_f32(h1));
    hi = (uint32_t)h0 | ((uint32_t)h1 << 16), lo = (uint32_t)l0 | ((uint32_t)l1 << 16);
}

// SPLIT (few items, many keys: decode steps): grid.z workgroups share an item tile's key blocks (block i goes to workgroup i mod grid.z) and leave unnormalised
// sums with their running maximum / denominator in p.split_ws; window_attention_merge_kernel combines them.  The sink belongs to split 0.
template <int NB, bool SPLIT> // dim and vdim padded to RP = 32 NB
__global__ void __launch_bounds__(256) window_attention_mfma_kernel(WindowAttentionParams p) {
    constexpr int RP = 32 * NB, KP = RP * 2 + 16, TP = 80, VEC = RP / 8;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* s_k = smem;             // [32 keys][KP bytes]
    uint8_t* s_vt = smem + 32 * KP;  // [RP][TP bytes]: 32 keys + pad
    const uint32_t hg = p.heads / p.kv_heads, g = blockIdx.y;
    uint32_t wg = blockIdx.x, z = 0;
    SeqSpan sp{0, 0, 0};
    for (;; ++z) {
        if (z >= p.nseq) return;
        sp = p.spans[z];
        const uint32_t n = (sp.count * hg + 127) / 128;
        if (wg < n) break;
        wg -= n;
    }
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5;
    const uint32_t items = sp.count * hg;
    auto row_lo = [&](uint32_t t) { // the first key the row at position t sees: the window's edge or its chunk's start, whichever is later
        uint32_t lo = (p.window && t + 1 > p.window) ? t + 1 - p.window : 0u;
        if (p.chunk) lo = max(lo, t / p.chunk * p.chunk);
        return lo;
    };
    // this lane's item
    const uint32_t it = wg * 128 + wave * 32 + l32;
    const bool valid = it < items;
    const uint32_t gi = valid ? it : items - 1;
    const uint32_t row = gi / hg, head = g * hg + gi % hg;
    const uint32_t t = sp.start + row, lo = row_lo(t);
    // key ranges of the workgroup and of this wave
    const uint32_t g_last = (wg * 128 + 128 < items ? wg * 128 + 128 : items) - 1;
    const uint32_t kmin = row_lo(sp.start + wg * 128 / hg), kmax = sp.start + g_last / hg;
    const uint32_t w_first = wg * 128 + wave * 32;
    const bool wave_on = w_first < items;
    const uint32_t w_last = (w_first + 32 < items ? w_first + 32 : items) - 1;
    const uint32_t wave_lo = wave_on ? row_lo(sp.start + w_first / hg) : 0, wave_hi = wave_on ? sp.start + w_last / hg : 0;

    u32x4_t qh[2 * NB], ql[2 * NB];
    {
        const float* qrow = p.q + (size_t)(sp.row0 + row) * p.ldq + (size_t)head * p.dim;
#pragma unroll
        for (int s = 0; s < 2 * NB; ++s) {
            const uint32_t k0 = s * 16 + half * 8;
            u32x4_t fh{0u, 0u, 0u, 0u}, fl{0u, 0u, 0u, 0u};
            if (valid && k0 < p.dim) { // dim % 8 == 0: a fragment is inside the head or outside it
                const f32x4_v a = *(const f32x4_v*)(qrow + k0), b = *(const f32x4_v*)(qrow + k0 + 4);
                uint32_t h[4], w[4];
                split_bf16(a.x, a.y, h[0], w[0]), split_bf16(a.z, a.w, h[1], w[1]), split_bf16(b.x, b.y, h[2], w[2]), split_bf16(b.z, b.w, h[3], w[3]);
                fh = u32x4_t{h[0], h[1], h[2], h[3]}, fl = u32x4_t{w[0], w[1], w[2], w[3]};
            }
            qh[s] = fh, ql[s] = fl;
        }
    }
    const bool with_sink = p.sinks && (!SPLIT || blockIdx.z == 0);
    float m_run = with_sink ? p.sinks[head] : -1.0e30f;
    float l_run = with_sink ? 1.0f : 0.0f;
    f32x16_t o[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[b][r] = 0.0f;
    const uint8_t* kc = (const uint8_t*)p.key_caches[z];
    const uint8_t* vc = (const uint8_t*)p.value_caches[z];
    const size_t kpitch = (size_t)p.kv_heads * p.dim, vpitch = (size_t)p.kv_heads * p.vdim;
    const float inv_cap = p.soft_cap != 0.0f ? 1.0f / p.soft_cap : 0.0f;
    const float hscale = p.head_scale ? p.scale * p.head_scale[head] : p.scale;

    const uint32_t kstep = SPLIT ? 32 * gridDim.z : 32;
    for (uint32_t kb = kmin + (SPLIT ? 32 * blockIdx.z : 0); kb <= kmax; kb += kstep) {
        __syncthreads(); // the block before has been read
        for (uint32_t v = tid; v < 32 * VEC; v += 256) {
            const uint32_t key = v / VEC, e0 = (v % VEC) * 8, kk = kb + key;
            u32x4_v kv{0u, 0u, 0u, 0u}, vv{0u, 0u, 0u, 0u};
            if (kk <= kmax) {
                if (e0 < p.dim) kv = *(const u32x4_v*)(kc + ((size_t)kk * kpitch + (size_t)g * p.dim + e0) * 2);
                if (e0 < p.vdim) vv = *(const u32x4_v*)(vc + ((size_t)kk * vpitch + (size_t)g * p.vdim + e0) * 2);
            }
            *(u32x4_v*)(s_k + key * KP + e0 * 2) = kv;
            const uint32_t w[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                *(uint16_t*)(s_vt + (e0 + 2 * e) * TP + key * 2) = (uint16_t)(w[e] & 0xFFFFu);
                *(uint16_t*)(s_vt + (e0 + 2 * e + 1) * TP + key * 2) = (uint16_t)(w[e] >> 16);
            }
        }
        __syncthreads();
        if (!wave_on || kb > wave_hi || kb + 31 < wave_lo) continue; // (wave-uniform; the barriers above are reached by every wave)
        f32x16_t st;
#pragma unroll
        for (int r = 0; r < 16; ++r) st[r] = 0.0f;
#pragma unroll
        for (int s = 0; s < 2 * NB; ++s) {
            const u32x4_t a = *(const u32x4_t*)(s_k + l32 * KP + (s * 16 + half * 8) * 2);
            st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, qh[s]), st, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, ql[s]), st, 0, 0, 0);
        }
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t key = kb + (r & 3) + 8 * (r >> 2) + 4 * half;
            const bool ok = valid && key >= lo && key <= t;
            float sc = st[r] * hscale;
            if (p.soft_cap != 0.0f) { // cap * tanh(s / cap), tanh(x) = 1 - 2 / (1 + e^(2x))
                const float e2 = fast_exp(2.0f * sc * inv_cap);
                sc = p.soft_cap * (1.0f - 2.0f / (1.0f + e2));
            }
            if (p.dist_bias && ok) sc += p.dist_bias[(size_t)min(t - key, p.dist_rows - 1) * p.heads + head];
            st[r] = ok ? sc : -INFINITY;
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
#pragma unroll
            for (int r = 0; r < 16; ++r) o[b][r] *= corr;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            uint32_t hw[4], lwv[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) split_bf16(st[8 * s2 + 2 * e], st[8 * s2 + 2 * e + 1], hw[e], lwv[e]);
            const u32x4_t hi{hw[0], hw[1], hw[2], hw[3]}, lw{lwv[0], lwv[1], lwv[2], lwv[3]};
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint8_t* cr = s_vt + (b * 32 + l32) * TP + (16 * s2 + 4 * half) * 2;
                const u32x2_v c0 = *(const u32x2_v*)cr, c1 = *(const u32x2_v*)(cr + 16);
                const u32x4_t cf{c0.x, c0.y, c1.x, c1.y};
                o[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, cf), __builtin_bit_cast(bf16x8_t, hi), o[b], 0, 0, 0);
                o[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, cf), __builtin_bit_cast(bf16x8_t, lw), o[b], 0, 0, 0);
            }
        }
    }
    if (!valid) return;
    if (SPLIT) {
        float* ws = p.split_ws + (((size_t)(sp.row0 + row) * p.heads + head) * gridDim.z + blockIdx.z) * (RP + 4);
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)
                *(f32x4_v*)(ws + b * 32 + 8 * g4 + 4 * half) = f32x4_v{o[b][4 * g4], o[b][4 * g4 + 1], o[b][4 * g4 + 2], o[b][4 * g4 + 3]};
        if (half == 0) ws[RP] = m_run, ws[RP + 1] = l_run;
        return;
    }
    float inv = 1.0f / l_run;
    if (p.gate) inv *= 1.0f / (1.0f + expf(-p.gate[(size_t)(sp.row0 + row) * p.ldgate + head]));
    float* out = p.out + ((size_t)(sp.row0 + row) * p.heads + head) * p.vdim;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            const uint32_t col = b * 32 + 8 * g4 + 4 * half;
            if (col < p.vdim) *(f32x4_v*)(out + col) = f32x4_v{o[b][4 * g4] * inv, o[b][4 * g4 + 1] * inv, o[b][4 * g4 + 2] * inv, o[b][4 * g4 + 3] * inv};
        }
}

// a workgroup per item: out = sum_s e^(m_s - M) O_s / sum_s e^(m_s - M) l_s over the splits, in split order (a split that saw no key has l = 0 and m = -1e30)
// (gate: the item's result times sigmoid(gate[row, head]), item = row * heads + head)
__global__ void __launch_bounds__(128) window_attention_merge_kernel(const float* ws, float* out, uint32_t splits, uint32_t vdim, uint32_t rp, const float* gate, uint32_t ldgate,
                                                                     uint32_t heads) {
    const uint32_t item = blockIdx.x, tid = threadIdx.x;
    const float* base = ws + (size_t)item * splits * (rp + 4);
    float M = -1.0e30f;
    for (uint32_t s = 0; s < splits; ++s) M = fmaxf(M, base[(size_t)s * (rp + 4) + rp]);
    float den = 0.0f;
    for (uint32_t s = 0; s < splits; ++s) den = fmaf(fast_exp(base[(size_t)s * (rp + 4) + rp] - M), base[(size_t)s * (rp + 4) + rp + 1], den);
    if (gate) den *= 1.0f + expf(-gate[(size_t)(item / heads) * ldgate + item % heads]);
    for (uint32_t c = tid; c < vdim; c += 128) {
        float acc = 0.0f;
        for (uint32_t s = 0; s < splits; ++s) acc = fmaf(fast_exp(base[(size_t)s * (rp + 4) + rp] - M), base[(size_t)s * (rp + 4) + c], acc);
        out[(size_t)item * vdim + c] = acc / den;
    }
}

uint32_t blocks_of(const WindowAttentionParams& p) {
    const uint32_t w = p.dim > p.vdim ? p.dim : p.vdim;
    return w <= 32 ? 1 : w <= 64 ? 2 : w <= 128 ? 4 : 0;
}

} // namespace

size_t window_attention_split_ws_bytes(uint32_t rows, uint32_t heads, uint32_t splits) { return (size_t)rows * heads * splits * (128 + 4) * 4; }

// bf16 caches, head widths that are multiples of 8 up to 128 (16-byte rows); prompt-sized passes, or a decode-sized pass with a workspace to split its keys
// (without one a decode step's few items would walk all their keys in one nearly empty workgroup: the simple form does that better)
static bool use_split(const WindowAttentionParams& p) {
    return p.splits > 1 && p.splits <= 64 && p.split_ws && p.split_ws_bytes >= window_attention_split_ws_bytes(p.rows, p.heads, p.splits);
}

bool window_attention_mfma_supported(const WindowAttentionParams& p) {
    const bool split = use_split(p);
    return p.cache_bf16 && blocks_of(p) && p.dim % 8 == 0 && p.vdim % 8 == 0 && p.ldq % 4 == 0 && p.kv_heads && p.heads % p.kv_heads == 0 && p.nseq && p.tiles &&
           (split || p.rows >= 16 * p.nseq) && p.kv_heads <= 65535 && ((uintptr_t)p.q & 15) == 0 && ((uintptr_t)p.out & 15) == 0;
}

uzu_status window_attention_mfma(hipStream_t s, const WindowAttentionParams& p) {
    UZU_REQUIRE(window_attention_mfma_supported(p), "window_attention: the matrix-core form does not take this shape");
    const uint32_t nb = blocks_of(p);
    const size_t lds = (size_t)32 * (32 * nb * 2 + 16) + (size_t)32 * nb * 80;
    if (use_split(p)) {
        const dim3 grid(p.tiles, p.kv_heads, p.splits);
#define UZU_WA(NB) UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL((window_attention_mfma_kernel<NB, true>), grid, dim3(256), lds, s, p); }, "window_attention_mfma_split"))
        if (nb == 1) UZU_WA(1);
        else if (nb == 2) UZU_WA(2);
        else UZU_WA(4);
#undef UZU_WA
        return launch_check([&] { hipLaunchKernelGGL(window_attention_merge_kernel, dim3(p.rows * p.heads), dim3(128), 0, s, (const float*)p.split_ws, p.out, p.splits, p.vdim, 32 * nb, p.gate, p.ldgate, p.heads); },
                            "window_attention_merge");
    }
    const dim3 grid(p.tiles, p.kv_heads);
#define UZU_WA(NB) return launch_check([&] { hipLaunchKernelGGL((window_attention_mfma_kernel<NB, false>), grid, dim3(256), lds, s, p); }, "window_attention_mfma")
    if (nb == 1) UZU_WA(1);
    if (nb == 2) UZU_WA(2);
    UZU_WA(4);
#undef UZU_WA
}

} // namespace k
} // namespace uzu
