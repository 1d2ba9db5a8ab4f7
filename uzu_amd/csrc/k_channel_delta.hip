// k_channel_delta.hip -- the gated delta rule with one decay per head and KEY CHANNEL, for the f32-stream designs (kernels_stream32.h::channel_delta).
//
// Per value head a (reading query / key group a / (heads / groups)), with S [dk][dv] the head's state:
//     S <- diag(decay_t) S,   u = beta_t (v_t - S^T k_t),   S <- S + k_t u^T,   o_t = S^T q_t
// Everything is f32.  The value columns of S never meet: column j only needs k_t, q_t, decay_t, beta_t and v_t[j].  So a workgroup owns 64 columns of one
// (sequence, head) and four threads share a column, each holding a quarter of its rows in registers; the two dot products of a token are sums over the thread's
// own rows in row order, then a fixed exchange between the four threads.  The order of every sum is the same whatever else the pass carries and however a prompt
// was cut: prompts, portions and decode steps run this one kernel.  q, k and decay of a few tokens are staged in LDS for all columns at once.
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

constexpr uint32_t kStage = 8; // tokens whose q / k / decay are staged at once

// grid (sequence * heads, ceil(dv / 64)); thread = (column, quarter of the rows); RP = rows per thread (dk <= 4 RP)
template <int RP>
__global__ void __launch_bounds__(256) channel_delta_steps_kernel(ChannelDeltaParams p) {
    __shared__ __attribute__((aligned(16))) float s_k[kStage][4 * RP], s_q[kStage][4 * RP], s_g[kStage][4 * RP];
    const uint32_t z = blockIdx.x / p.heads, a = blockIdx.x % p.heads, g = a / (p.heads / p.groups);
    const uint32_t tid = threadIdx.x, col = blockIdx.y * 64 + (tid >> 2), part = tid & 3;
    const bool live = col < p.vdim;
    const SeqSpan sp = p.spans[z];
    float* state = p.states[z] + (size_t)a * p.dim * p.vdim;
    float S[RP];
#pragma unroll
    for (int n = 0; n < RP; ++n) {
        const uint32_t i = part * RP + n;
        S[n] = (sp.start && live && i < p.dim) ? state[(size_t)i * p.vdim + col] : 0.0f;
    }
    for (uint32_t i0 = 0; i0 < sp.count; i0 += kStage) {
        const uint32_t nt = sp.count - i0 < kStage ? sp.count - i0 : kStage;
        __syncthreads(); // the stage before has been read
        for (uint32_t e = tid; e < nt * 4 * RP; e += 256) {
            const uint32_t tk = e / (4 * RP), i = e - tk * (4 * RP);
            const size_t r = sp.row0 + i0 + tk;
            const bool in = i < p.dim; // rows beyond dk: zero keys and queries leave the padding rows of S at zero
            s_k[tk][i] = in ? p.qkv[r * p.ld + p.k_col + (size_t)g * p.dim + i] : 0.0f;
            s_q[tk][i] = in ? p.qkv[r * p.ld + p.q_col + (size_t)g * p.dim + i] : 0.0f;
            s_g[tk][i] = in ? p.decay[(r * p.heads + a) * p.dim + i] : 0.0f;
        }
        __syncthreads();
        for (uint32_t tk = 0; tk < nt; ++tk) {
            const size_t r = sp.row0 + i0 + tk;
            const float v = live ? p.qkv[r * p.ld + p.v_col + (size_t)a * p.vdim + col] : 0.0f;
            const float beta = p.beta[r * p.ldbeta + a];
            const float *kk = &s_k[tk][part * RP], *qq = &s_q[tk][part * RP], *gg = &s_g[tk][part * RP];
            float dot = 0.0f;
#pragma unroll
            for (int n = 0; n < RP; ++n) {
                S[n] *= gg[n];
                dot = fmaf(S[n], kk[n], dot);
            }
            dot += __shfl_xor(dot, 1, 64);
            dot += __shfl_xor(dot, 2, 64);
            const float u = beta * (v - dot);
            float o = 0.0f;
#pragma unroll
            for (int n = 0; n < RP; ++n) {
                S[n] = fmaf(kk[n], u, S[n]);
                o = fmaf(S[n], qq[n], o);
            }
            o += __shfl_xor(o, 1, 64);
            o += __shfl_xor(o, 2, 64);
            if (live && part == 0) p.out[(r * p.heads + a) * p.vdim + col] = o;
        }
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
    UZU_REQUIRE((size_t)p.nseq * p.heads <= 0x7FFFFFFFu && (p.vdim + 63) / 64 <= 65535, "channel_delta: too many heads for one launch");
    const dim3 grid(p.nseq * p.heads, (p.vdim + 63) / 64);
#define UZU_CD(RP) return launch_check([&] { hipLaunchKernelGGL((channel_delta_steps_kernel<RP>), grid, dim3(256), 0, s, p); }, "channel_delta_steps")
    if (p.dim <= 16) UZU_CD(4);
    if (p.dim <= 32) UZU_CD(8);
    if (p.dim <= 64) UZU_CD(16);
    if (p.dim <= 128) UZU_CD(32);
    UZU_CD(64);
#undef UZU_CD
}

} // namespace k
} // namespace uzu
