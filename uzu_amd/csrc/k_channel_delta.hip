// k_channel_delta.hip -- the gated delta rule with one decay per head and KEY CHANNEL, for the f32-stream designs (kernels_stream32.h::channel_delta).
//
// Per value head a (reading query / key group a / (heads / groups)), with S [dk][dv] the head's state:
//     S <- diag(decay_t) S,   u = beta_t (v_t - S^T k_t),   S <- S + k_t u^T,   o_t = S^T q_t
// Everything is f32.  The value columns of S never meet: column j only needs k_t, q_t, decay_t, beta_t and v_t[j].  So a workgroup owns 16 columns of one
// (sequence, head) and sixteen threads share a column, each holding a sixteenth of its rows in registers; the two dot products of a token are sums over the
// thread's own rows in row order, then a fixed exchange between the sixteen threads.  The order of every sum is the same whatever else the pass carries and however a prompt
// was cut: prompts, portions and decode steps run this one kernel.  q, k, decay, v and beta of sixteen tokens are staged in LDS for all columns at once.
#include "device_utils.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

namespace {

__device__ __forceinline__ float softplus_f32(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// a workgroup per row: unit vectors of the query / key heads (q also times dk^(-1/2)), beta = sigmoid, decay = exp(-exp(a_log) softplus(pre + dt_bias)), in place
__global__ void __launch_bounds__(256) channel_delta_prep_kernel(ChannelDeltaParams p) {
    const uint32_t r = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float* qk = p.qkv + (size_t)r * p.ld;
    const float qs = 1.0f / sqrtf((float)p.dim);
    for (uint32_t a = wave; a < 2 * p.groups; a += 4) { // query heads, then key heads
        const bool is_q = a < p.groups;
        float* h = qk + (is_q ? p.q_col + (size_t)a * p.dim : p.k_col + (size_t)(a - p.groups) * p.dim);
        float ss = 0.0f;
        for (uint32_t i = lane; i < p.dim; i += 64) ss = fmaf(h[i], h[i], ss);
        ss = wave_sum(ss);
        const float inv = (is_q ? qs : 1.0f) / sqrtf(ss + p.unit_eps);
        for (uint32_t i = lane; i < p.dim; i += 64) h[i] *= inv;
    }
    float* dec = p.decay + (size_t)r * p.heads * p.dim;
    for (uint32_t i = threadIdx.x; i < p.heads * p.dim; i += 256) dec[i] = expf(-expf(p.a_log[i / p.dim]) * softplus_f32(dec[i] + p.dt_bias[i]));
    float* b = p.beta + (size_t)r * p.ldbeta;
    for (uint32_t i = threadIdx.x; i < p.heads; i += 256) b[i] = 1.0f / (1.0f + expf(-b[i]));
}

constexpr int kStage = 16; // tokens whose q / k / decay / v / beta are staged at once

// the sum over the 16 lanes of a row of the wave, left in every one of them: four data-parallel-primitive moves (quad swaps, then the two mirrors) -- the same
// order in every launch
__device__ __forceinline__ float row16_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));  // quad_perm [1, 0, 3, 2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));  // quad_perm [2, 3, 0, 1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true)); // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true)); // row_mirror
    return v;
}

// grid (sequence * heads, ceil(dv / 16)); thread = (column, sixteenth of the rows): a wave owns 4 columns, a workgroup 16.  RP = rows per thread (dk <= 16 RP);
// thread `part` of a column owns rows part * RP .. part * RP + RP - 1, which lie side by side in LDS (16-byte reads; a pad of four floats per part keeps the
// sixteen parts on different banks).  The next stage's rows travel from memory into registers while the current stage is worked on.
template <int RP>
__global__ void __launch_bounds__(256) channel_delta_steps_kernel(ChannelDeltaParams p) {
    constexpr int DK = 16 * RP, PW = RP >= 8 ? RP + 4 : RP, LDW = 16 * PW;
    __shared__ __attribute__((aligned(16))) float s_k[kStage][LDW], s_q[kStage][LDW], s_g[kStage][LDW];
    __shared__ float s_v[kStage][16], s_b[kStage], s_o[kStage][16];
    const uint32_t z = blockIdx.x / p.heads, a = blockIdx.x % p.heads, g = a / (p.heads / p.groups);
    const uint32_t tid = threadIdx.x, cl = tid >> 4, part = tid & 15, col = blockIdx.y * 16 + cl;
    const bool live = col < p.vdim;
    const SeqSpan sp = p.spans[z];
    float* state = p.states[z] + (size_t)a * p.dim * p.vdim;
    float S[RP];
#pragma unroll
    for (int n = 0; n < RP; ++n) {
        const uint32_t i = part * RP + n;
        S[n] = (sp.start && live && i < p.dim) ? state[(size_t)i * p.vdim + col] : 0.0f;
    }
    float pf[3 * RP], pf_v = 0.0f, pf_b = 0.0f;
    // element e * 256 + tid of a stage's [k | q | decay][token][row] block: rows beyond dk and tokens beyond the share are zeros (zero keys and queries leave the
    // padding rows of S at zero)
    auto fetch = [&](uint32_t i0) {
        const uint32_t nt = sp.count - i0 < (uint32_t)kStage ? sp.count - i0 : (uint32_t)kStage;
#pragma unroll
        for (int e = 0; e < 3 * RP; ++e) {
            const uint32_t rem = (uint32_t)(e % RP) * 256 + tid, tk = rem / DK, i = rem % DK;
            const size_t r = sp.row0 + i0 + tk;
            float v = 0.0f;
            if (tk < nt && i < p.dim) {
                if (e / RP == 0) v = p.qkv[r * p.ld + p.k_col + (size_t)g * p.dim + i];
                else if (e / RP == 1) v = p.qkv[r * p.ld + p.q_col + (size_t)g * p.dim + i];
                else v = p.decay[(r * p.heads + a) * p.dim + i];
            }
            pf[e] = v;
        }
        const uint32_t tk = tid >> 4, c = blockIdx.y * 16 + (tid & 15);
        pf_v = (tk < nt && c < p.vdim) ? p.qkv[(size_t)(sp.row0 + i0 + tk) * p.ld + p.v_col + (size_t)a * p.vdim + c] : 0.0f;
        pf_b = (tid < nt) ? p.beta[(size_t)(sp.row0 + i0 + tid) * p.ldbeta + a] : 0.0f;
    };
    auto put = [&]() {
#pragma unroll
        for (int e = 0; e < 3 * RP; ++e) {
            const uint32_t rem = (uint32_t)(e % RP) * 256 + tid, tk = rem / DK, i = rem % DK;
            float* dst = e / RP == 0 ? &s_k[0][0] : e / RP == 1 ? &s_q[0][0] : &s_g[0][0];
            dst[tk * LDW + (i / RP) * PW + i % RP] = pf[e];
        }
        s_v[tid >> 4][tid & 15] = pf_v;
        if (tid < (uint32_t)kStage) s_b[tid] = pf_b;
    };
    // a stage's results leave through LDS, one coalesced store per thread (a store per token and column from inside the chain costs 40 % of the launch)
    auto flush = [&](uint32_t i0, uint32_t nt) {
        const uint32_t tk = tid >> 4, c = blockIdx.y * 16 + (tid & 15);
        if (tk < nt && c < p.vdim) p.out[((size_t)(sp.row0 + i0 + tk) * p.heads + a) * p.vdim + c] = s_o[tk][tid & 15];
    };
    fetch(0);
    for (uint32_t i0 = 0; i0 < sp.count; i0 += kStage) {
        const uint32_t nt = sp.count - i0 < (uint32_t)kStage ? sp.count - i0 : (uint32_t)kStage;
        __syncthreads(); // the stage before has been read, its results stand in s_o
        if (i0) flush(i0 - kStage, kStage);
        put();
        __syncthreads();
        if (i0 + kStage < sp.count) fetch(i0 + kStage);
        // one token: only  S -> decayed S -> <S, k> -> u -> S  is the recurrence; the read-out <S, q> of a token overlaps the next token's chain when a full stage
        // is unrolled.  The dot products are sums of four interleaved partial sums (rows n = 0, 4, .. | 1, 5, .. | ..), then of the sixteen threads: a fixed order.
        auto step = [&](uint32_t tk) {
            const float v = s_v[tk][cl], beta = s_b[tk];
            float kk[RP], qq[RP], gg[RP];
            if constexpr (RP % 4 == 0) {
#pragma unroll
                for (int n = 0; n < RP; n += 4) {
                    const f32x4_v k4 = *(const f32x4_v*)&s_k[tk][part * PW + n], q4 = *(const f32x4_v*)&s_q[tk][part * PW + n], g4 = *(const f32x4_v*)&s_g[tk][part * PW + n];
                    kk[n] = k4.x, kk[n + 1] = k4.y, kk[n + 2] = k4.z, kk[n + 3] = k4.w;
                    qq[n] = q4.x, qq[n + 1] = q4.y, qq[n + 2] = q4.z, qq[n + 3] = q4.w;
                    gg[n] = g4.x, gg[n + 1] = g4.y, gg[n + 2] = g4.z, gg[n + 3] = g4.w;
                }
            } else {
#pragma unroll
                for (int n = 0; n < RP; ++n) kk[n] = s_k[tk][part * PW + n], qq[n] = s_q[tk][part * PW + n], gg[n] = s_g[tk][part * PW + n];
            }
            float d[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int n = 0; n < RP; ++n) {
                S[n] *= gg[n];
                d[n & 3] = fmaf(S[n], kk[n], d[n & 3]);
            }
            const float dot = row16_sum((d[0] + d[1]) + (d[2] + d[3]));
            const float u = beta * (v - dot);
            float o[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int n = 0; n < RP; ++n) {
                S[n] = fmaf(kk[n], u, S[n]);
                o[n & 3] = fmaf(S[n], qq[n], o[n & 3]);
            }
            const float out = row16_sum((o[0] + o[1]) + (o[2] + o[3]));
            if (part == 0) s_o[tk][cl] = out;
        };
        if (nt == (uint32_t)kStage) {
#pragma unroll
            for (int tk = 0; tk < kStage; ++tk) step(tk);
        } else {
            for (uint32_t tk = 0; tk < nt; ++tk) step(tk);
        }
    }
    __syncthreads();
    {
        const uint32_t last = (sp.count - 1) / kStage * kStage;
        flush(last, sp.count - last);
    }
    if (!live) return;
#pragma unroll
    for (int n = 0; n < RP; ++n) {
        const uint32_t i = part * RP + n;
        if (i < p.dim) state[(size_t)i * p.vdim + col] = S[n];
    }
}

} // namespace

bool channel_delta_supported(uint32_t dim, uint32_t vdim) { return dim >= 1 && dim <= 256 && vdim >= 1; }

uzu_status channel_delta_prep(hipStream_t s, const ChannelDeltaParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.qkv && p.decay && p.beta && p.a_log && p.dt_bias && p.heads && p.groups && p.heads % p.groups == 0 && p.dim && p.vdim, "channel_delta: null argument");
    return launch_check([&] { hipLaunchKernelGGL(channel_delta_prep_kernel, dim3(p.rows), dim3(256), 0, s, p); }, "channel_delta_prep");
}

uzu_status channel_delta(hipStream_t s, const ChannelDeltaParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.qkv && p.decay && p.beta && p.out && p.states && p.spans && p.nseq && p.heads && p.groups && p.heads % p.groups == 0, "channel_delta: null argument");
    UZU_UNSUPPORTED(!channel_delta_supported(p.dim, p.vdim), "channel_delta: heads of %u x %u (keys up to 256)", p.dim, p.vdim);
    UZU_REQUIRE((size_t)p.nseq * p.heads <= 0x7FFFFFFFu && (p.vdim + 15) / 16 <= 65535, "channel_delta: too many heads for one launch");
    const dim3 grid(p.nseq * p.heads, (p.vdim + 15) / 16);
#define UZU_CD(RP) return launch_check([&] { hipLaunchKernelGGL((channel_delta_steps_kernel<RP>), grid, dim3(256), 0, s, p); }, "channel_delta_steps")
    if (p.dim <= 16) UZU_CD(1);
    if (p.dim <= 32) UZU_CD(2);
    if (p.dim <= 64) UZU_CD(4);
    if (p.dim <= 128) UZU_CD(8);
    UZU_CD(16);
#undef UZU_CD
}

} // namespace k
} // namespace uzu
