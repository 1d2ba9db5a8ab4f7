// k_gated_lru.hip -- the gated linear recurrent unit of the f32-stream designs (UZU_MIXER_GATED_LRU; kernels_stream32.h): the short causal convolution in front
// of it and the recurrence S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with its gates, decays and state in f32.
//
// The recurrence is element-wise per channel and linear in S, so a sequence's rows can be cut into pieces: a piece scanned from zero yields its local states L_t
// and decay products P_t = a_(first) ... a_t, and the true state is S_t = L_t + P_t * (the state in front of the piece).  The position-by-position form walks a
// sequence's rows in one thread per channel (decode steps, short portions); the pieced form cuts a prompt's rows into pieces of 32, scans every piece from zero
// in its own thread, joins the pieces' carries in order and walks the pieces again from their true carries (three launches that fill the chip).  Both leave S and
// the convolution's last taps - 1 inputs in the sequence's state.
#include "device_utils.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

namespace {

__device__ __forceinline__ float sigmoid_f32(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f32(float z) { return z > 20.0f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float gelu_tanh(float z) { return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

// thread = (row, channel)
__global__ void __launch_bounds__(256) lru_conv_kernel(GatedLruParams p) {
    const uint32_t r = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= p.width) return;
    const uint32_t z = p.row_seq[r];
    const SeqSpan sp = p.spans[z];
    const uint32_t i = r - sp.row0, t = sp.start + i;
    const float* state = p.conv_states[z];
    float acc = p.conv_b ? p.conv_b[c] : 0.0f;
    for (uint32_t j = 0; j < p.taps; ++j) {
        const uint32_t back = p.taps - 1 - j;
        float xin = 0.0f;
        if (back <= i) xin = p.branches[(size_t)(r - back) * p.ld + p.x_col + c];
        else if (back <= t) xin = state[(size_t)(p.taps - 1 - (back - i)) * p.width + c]; // a position in front of the pass: the state's rows are start - (taps - 1) .. start - 1
        acc = fmaf(p.conv_w[(size_t)c * p.taps + j], xin, acc);
    }
    p.u[(size_t)r * p.width + c] = acc;
}

struct Coef {
    float a, b;
};
// decay and input of row r, channel c (block blk, offset o inside it); sl = rate * softplus(lambda[c])
__device__ __forceinline__ Coef coef_of(const GatedLruParams& p, uint32_t r, uint32_t c, uint32_t bw, uint32_t blk, uint32_t o, float sl, float br, float bi) {
    const float* g = p.gates + (size_t)r * 2 * p.width + (size_t)blk * 2 * bw + o;
    const float rr = sigmoid_f32(g[0] + br), ii = sigmoid_f32(g[bw] + bi);
    const float la = -sl * rr;
    Coef k;
    k.a = expf(la);
    k.b = sqrtf(-expm1f(2.0f * la)) * ii * p.u[(size_t)r * p.width + c]; // 1 - a^2 without the cancellation near a = 1
    return k;
}

// the convolution's window behind the pass: positions end - (taps - 1) .. end - 1, from this pass's rows, the old window, or (in front of position 0) zeros
__device__ __forceinline__ void conv_state_update(const GatedLruParams& p, const SeqSpan& sp, uint32_t z, uint32_t c) {
    float* cs = p.conv_states[z];
    const uint32_t keep = p.taps - 1;
    for (uint32_t s = 0; s < keep; ++s) { // ascending: an old entry is read at index s + count > s before that index is written
        float v = 0.0f;
        if (s + sp.count >= keep) v = p.branches[(size_t)(sp.row0 + (s + sp.count - keep)) * p.ld + p.x_col + c];
        else if (sp.start + sp.count + s >= keep) v = cs[(size_t)(s + sp.count) * p.width + c];
        cs[(size_t)s * p.width + c] = v;
    }
}

// position by position: thread = (sequence, channel)
__global__ void __launch_bounds__(256) lru_scan_steps_kernel(GatedLruParams p) {
    const uint32_t z = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= p.width) return;
    const SeqSpan sp = p.spans[z];
    const uint32_t bw = p.width / p.blocks, blk = c / bw, o = c - blk * bw;
    const float sl = p.rate * softplus_f32(p.lambda[c]);
    const float br = p.gate_b ? p.gate_b[(size_t)blk * 2 * bw + o] : 0.0f, bi = p.gate_b ? p.gate_b[(size_t)blk * 2 * bw + bw + o] : 0.0f;
    float S = sp.start ? p.states[z][c] : 0.0f;
    for (uint32_t i = 0; i < sp.count; ++i) {
        const uint32_t r = sp.row0 + i;
        const Coef k = coef_of(p, r, c, bw, blk, o, sl, br, bi);
        S = fmaf(k.a, S, k.b);
        p.out[(size_t)r * p.width + c] = S * gelu_tanh(p.branches[(size_t)r * p.ld + c]);
    }
    p.states[z][c] = S;
    conv_state_update(p, sp, z, c);
}

// In pieces of kPieceRows rows: thread = (piece, channel), consecutive lanes on consecutive channels, so that a prompt's rows fill the chip.
//   local:  a piece scanned from zero: L (its last local state) and P (the product of its decays) per channel
//   carry:  thread = (sequence, channel) joins the pieces in order: the state in front of every piece, the sequence's state behind the pass, the convolution's window
//   out:    the piece again from its true carry; writes the rows
constexpr uint32_t kPieceRows = 32;
// piece g of the pass -> its sequence, first row (within the sequence's share) and row count; false behind the last piece
__device__ __forceinline__ bool piece_of(const GatedLruParams& p, uint32_t g, SeqSpan& sp, uint32_t& i0, uint32_t& n) {
    for (uint32_t z = 0; z < p.nseq; ++z) {
        sp = p.spans[z];
        const uint32_t np = (sp.count + kPieceRows - 1) / kPieceRows;
        if (g < np) {
            i0 = g * kPieceRows;
            n = sp.count - i0 < kPieceRows ? sp.count - i0 : kPieceRows;
            return true;
        }
        g -= np;
    }
    return false;
}

template <bool OUT>
__global__ void __launch_bounds__(256) lru_piece_kernel(GatedLruParams p) {
    const uint32_t g = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= p.width) return;
    SeqSpan sp;
    uint32_t i0, n;
    if (!piece_of(p, g, sp, i0, n)) return;
    const uint32_t bw = p.width / p.blocks, blk = c / bw, o = c - blk * bw;
    const float sl = p.rate * softplus_f32(p.lambda[c]);
    const float br = p.gate_b ? p.gate_b[(size_t)blk * 2 * bw + o] : 0.0f, bi = p.gate_b ? p.gate_b[(size_t)blk * 2 * bw + bw + o] : 0.0f;
    const size_t at = (size_t)g * p.width + c;
    if (!OUT) {
        float L = 0.0f, P = 1.0f;
        for (uint32_t i = 0; i < n; ++i) {
            const Coef k = coef_of(p, sp.row0 + i0 + i, c, bw, blk, o, sl, br, bi);
            L = fmaf(k.a, L, k.b);
            P *= k.a;
        }
        p.piece_ws[at] = L, p.piece_ws[(size_t)p.pieces * p.width + at] = P;
    } else {
        float S = p.piece_ws[(size_t)2 * p.pieces * p.width + at];
        for (uint32_t i = 0; i < n; ++i) {
            const uint32_t r = sp.row0 + i0 + i;
            const Coef k = coef_of(p, r, c, bw, blk, o, sl, br, bi);
            S = fmaf(k.a, S, k.b);
            p.out[(size_t)r * p.width + c] = S * gelu_tanh(p.branches[(size_t)r * p.ld + c]);
        }
    }
}

__global__ void __launch_bounds__(256) lru_piece_carry_kernel(GatedLruParams p) {
    const uint32_t z = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= p.width) return;
    uint32_t g = 0;
    for (uint32_t q = 0; q < z; ++q) g += (p.spans[q].count + kPieceRows - 1) / kPieceRows;
    const SeqSpan sp = p.spans[z];
    const uint32_t np = (sp.count + kPieceRows - 1) / kPieceRows;
    const size_t plane = (size_t)p.pieces * p.width;
    float S = sp.start ? p.states[z][c] : 0.0f;
    for (uint32_t q = 0; q < np; ++q) {
        const size_t at = (size_t)(g + q) * p.width + c;
        p.piece_ws[2 * plane + at] = S;
        S = fmaf(p.piece_ws[plane + at], S, p.piece_ws[at]);
    }
    p.states[z][c] = S;
    conv_state_update(p, sp, z, c);
}

uzu_status lru_check(const GatedLruParams& p) {
    UZU_REQUIRE(p.branches && p.u && p.conv_w && p.conv_states && p.spans && p.row_seq, "gated_lru: null argument");
    UZU_REQUIRE(p.width && p.blocks && p.width % p.blocks == 0 && p.taps >= 1 && p.x_col + p.width <= p.ld, "gated_lru: width %u in %u blocks, %u taps, pitch %u", p.width, p.blocks,
                p.taps, p.ld);
    return UZU_OK;
}

} // namespace

size_t lru_piece_ws_bytes(uint32_t pieces, uint32_t width) { return (size_t)3 * pieces * width * 4; }

uzu_status lru_conv(hipStream_t s, const GatedLruParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_PROPAGATE(lru_check(p));
    return launch_check([&] { hipLaunchKernelGGL(lru_conv_kernel, dim3(p.rows, (p.width + 255) / 256), dim3(256), 0, s, p); }, "lru_conv");
}

uzu_status lru_scan(hipStream_t s, const GatedLruParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_PROPAGATE(lru_check(p));
    UZU_REQUIRE(p.gates && p.out && p.lambda && p.states && p.nseq, "gated_lru: null argument");
    const bool have_ws = p.piece_ws && p.pieces && lru_piece_ws_bytes(p.pieces, p.width) <= p.piece_ws_bytes;
    UZU_REQUIRE(p.form != 2 || have_ws, "gated_lru: the pieced form needs its piece count and workspace");
    if (p.form == 2 || (p.form == 0 && have_ws && p.max_count >= 2 * kPieceRows)) {
        const dim3 grid(p.pieces, (p.width + 255) / 256);
        UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL(lru_piece_kernel<false>, grid, dim3(256), 0, s, p); }, "lru_piece_local"));
        UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL(lru_piece_carry_kernel, dim3(p.nseq, (p.width + 255) / 256), dim3(256), 0, s, p); }, "lru_piece_carry"));
        return launch_check([&] { hipLaunchKernelGGL(lru_piece_kernel<true>, grid, dim3(256), 0, s, p); }, "lru_piece_out");
    }
    return launch_check([&] { hipLaunchKernelGGL(lru_scan_steps_kernel, dim3(p.nseq, (p.width + 255) / 256), dim3(256), 0, s, p); }, "lru_scan_steps");
}

} // namespace k
} // namespace uzu
