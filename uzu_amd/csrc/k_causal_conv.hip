// k_causal_conv.hip -- a causal convolution over positions on every channel of a block of f32 rows, for the f32-stream designs (kernels_stream32.h): the input
// convolution of a sublayer (what the sublayer reads is h + conv(h)) and the short convolution with silu in front of a delta rule.
//
// Row r sits at position t of its sequence; tap j weighs the input of position t - (taps - 1) + j, so the last tap weighs the row itself.  Inputs in front of the
// pass come from the sequence's state (the last taps - 1 inputs, oldest first), inputs in front of position 0 are zeros whatever the state holds.  The taps are
// added in tap order whatever their source, so a row's result does not depend on how a prompt was cut into passes or on what else a pass carries.  The state is
// replaced by a launch of its own (thread = (sequence, channel)): the rows of the first launch read the old one.
#include "device_utils.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

namespace {

// the inputs of positions end - (taps - 1) .. end - 1 of sequence z, channel c: from this pass's rows, the old window, or (in front of position 0) zeros
__device__ __forceinline__ void window_update(const CausalConvParams& p, const SeqSpan& sp, uint32_t z, uint32_t c) {
    float* cs = p.states[z] + p.state_offset;
    const uint32_t keep = p.taps - 1;
    for (uint32_t s = 0; s < keep; ++s) { // ascending: an old entry is read at index s + count > s before that index is written
        float v = 0.0f;
        if (s + sp.count >= keep) v = p.x[(size_t)(sp.row0 + (s + sp.count - keep)) * p.ldx + p.x_col + c];
        else if (sp.start + sp.count + s >= keep) v = cs[(size_t)(s + sp.count) * p.channels + c];
        cs[(size_t)s * p.channels + c] = v;
    }
}

// thread = (row, channel).  A sequence that brings ONE row (a decode step) has its window replaced here: the row's own thread is the only reader of the old one.
__global__ void __launch_bounds__(256) causal_conv_rows_kernel(CausalConvParams p) {
    const uint32_t r = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= p.channels) return;
    const uint32_t z = p.row_seq[r];
    const SeqSpan sp = p.spans[z];
    const uint32_t i = r - sp.row0, t = sp.start + i;
    const float* state = p.taps > 1 ? p.states[z] + p.state_offset : nullptr;
    const float own = p.x[(size_t)r * p.ldx + p.x_col + c];
    float acc = p.bias ? p.bias[c] : 0.0f;
    for (uint32_t j = 0; j < p.taps; ++j) {
        const uint32_t back = p.taps - 1 - j;
        float xin = 0.0f;
        if (back == 0) xin = own;
        else if (back <= i) xin = p.x[(size_t)(r - back) * p.ldx + p.x_col + c];
        else if (back <= t) xin = state[(size_t)(p.taps - 1 - (back - i)) * p.channels + c]; // in front of the pass: the state's rows are positions start - (taps - 1) .. start - 1
        acc = fmaf(p.w[(size_t)c * p.taps + j], xin, acc);
    }
    if (p.act == 1) acc = acc / (1.0f + expf(-acc));
    if (p.add_input) acc = own + acc;
    p.out[(size_t)r * p.ldo + p.o_col + c] = acc;
    if (sp.count == 1 && p.taps > 1) window_update(p, sp, z, c);
}

// thread = (sequence, channel): the windows of the sequences that bring several rows (their first rows' threads read the old window in the launch before)
__global__ void __launch_bounds__(256) causal_conv_commit_kernel(CausalConvParams p) {
    const uint32_t z = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= p.channels) return;
    const SeqSpan sp = p.spans[z];
    if (sp.count == 1) return; // done by the row's own thread
    window_update(p, sp, z, c);
}

// a wave per (row, head): x / sqrt(mean(x^2) + eps) * weight * gate
__global__ void __launch_bounds__(256) head_norm_gate_kernel(HeadNormGateParams p) {
    const uint32_t lane = threadIdx.x & 63, item = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= p.rows * p.heads) return;
    const uint32_t r = item / p.heads, a = item - r * p.heads;
    float* x = p.x + (size_t)r * p.ldx + (size_t)a * p.width;
    float ss = 0.0f;
    for (uint32_t i = lane; i < p.width; i += 64) ss = fmaf(x[i], x[i], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)p.width + p.eps);
    const float* g = p.gate ? p.gate + (size_t)r * p.ldgate + (size_t)a * p.width : nullptr;
    for (uint32_t i = lane; i < p.width; i += 64) {
        float v = x[i] * inv;
        if (p.weight) v *= p.weight[i];
        if (g) v *= p.gate_sigmoid ? 1.0f / (1.0f + expf(-g[i])) : g[i] / (1.0f + expf(-g[i]));
        x[i] = v;
    }
}

} // namespace

uzu_status causal_conv_rows(hipStream_t s, const CausalConvParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.x && p.out && p.w && (p.states || p.taps == 1) && p.spans && p.row_seq && p.channels && p.taps >= 1, "causal_conv: null argument");
    UZU_REQUIRE(p.x_col + p.channels <= p.ldx && p.o_col + p.channels <= p.ldo, "causal_conv: %u channels at columns %u / %u of rows of %u / %u", p.channels, p.x_col, p.o_col, p.ldx, p.ldo);
    UZU_REQUIRE(p.out != p.x || p.taps == 1, "causal_conv: a row reads earlier rows of the pass: the result goes to another block of rows");
    return launch_check([&] { hipLaunchKernelGGL(causal_conv_rows_kernel, dim3(p.rows, (p.channels + 255) / 256), dim3(256), 0, s, p); }, "causal_conv_rows");
}

uzu_status causal_conv_commit(hipStream_t s, const CausalConvParams& p) {
    if (!p.rows || p.taps < 2 || p.max_count == 1) return UZU_OK; // (every sequence brings one row: the rows' launch has replaced the windows)
    UZU_REQUIRE(p.x && p.states && p.spans && p.nseq && p.channels, "causal_conv: null argument");
    return launch_check([&] { hipLaunchKernelGGL(causal_conv_commit_kernel, dim3(p.nseq, (p.channels + 255) / 256), dim3(256), 0, s, p); }, "causal_conv_commit");
}

uzu_status head_norm_gate_rows(hipStream_t s, const HeadNormGateParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.x && p.heads && p.width && p.heads * p.width <= p.ldx, "head_norm_gate: null argument");
    return launch_check([&] { hipLaunchKernelGGL(head_norm_gate_kernel, dim3((p.rows * p.heads + 3) / 4), dim3(256), 0, s, p); }, "head_norm_gate_rows");
}

} // namespace k
} // namespace uzu
