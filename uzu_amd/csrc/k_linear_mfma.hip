// k_linear_mfma.hip -- the full-precision linear of the f32-stream designs on the bf16 matrix cores (kernels_stream32.h: linear_f32 with bf16 products).
//
//   Y[r, n] = act(sum_k bf16(X[r, k]) * W[n, k] + bias[n]) + residual[r, n]       X f32 rows, W bf16 [n, k], f32 accumulation, f32 out
//
// v_mfma_f32_32x32x16_bf16; a workgroup of four waves (2 x 2) owns a (64 MB) x (64 NB) tile, a wave MB x NB blocks of 32 x 32.  A k-step is 64 deep: the
// activation rows are rounded to bf16 on their way into LDS (what a bf16 activation buffer would have held -- the round trip through HBM is saved instead of
// the conversion), the weight rows are copied; both tiles use a 144-byte row pitch, so the 16-byte operand reads of the 64 lanes fall on distinct banks.
// The next k-step's global loads are issued before the MFMAs of the current one and stored behind them (one LDS buffer, two barriers per k-step).
// An MFMA lane holds column n = lane % 32 of a block and rows (i & 3) + 8 (i >> 2) + 4 (lane / 32): a row's 32 columns leave as one 128-byte segment.
// grid.z batches independent products of one shape (the per-head products of the latent attention).
#include "device_utils.h"
#include "gemm_convert.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

namespace {

constexpr int LK = 64;       // k-step
constexpr int PITCH = 144;   // bytes per staged row: 64 bf16 + 16 bytes of pad

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) { return (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16); }

template <int MB, int NB, bool GROUPED> // GROUPED: per-product row buckets (row_offsets) and gathered operand rows (row_map); the plain form carries neither
__global__ void __launch_bounds__(256) linear_mfma_kernel(LinearF32Params p) {
    constexpr int BM = 64 * MB, BN = 64 * NB;
    constexpr int A_PASSES = BM / 16; // 16 threads cover a row's 64 k (one float4 each), 16 rows per pass
    constexpr int B_PASSES = BN / 32; // 8 threads cover a row's 64 k (one 16-byte vector each), 32 rows per pass
    __shared__ __attribute__((aligned(16))) uint8_t s_a[BM * PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t s_b[BN * PITCH];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1, l32 = lane & 31, half = lane >> 5;
    const uint32_t z = blockIdx.z;
    const float* x = p.x + z * p.x_batch;
    const uint16_t* w = p.w + z * p.w_batch;
    uint32_t r_lo = 0, r_hi = p.rows;
    if (GROUPED) { // a grouped launch: this product's bucket of rows (workgroup-uniform: the exit comes before any barrier)
        r_lo = p.row_offsets[z], r_hi = p.row_offsets[z + 1];
        x = p.x;
    }
    const uint32_t m0 = r_lo + blockIdx.y * BM, n0 = blockIdx.x * BN;
    if (m0 >= r_hi) return;

    f32x16_t acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    f32x4_v a_reg[A_PASSES];
    u32x4_v b_reg[B_PASSES];
    const uint32_t a_row = tid >> 4, a_k = (tid & 15) * 4;
    const uint32_t b_row = tid >> 3, b_k = (tid & 7) * 8;
    auto load = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i) {
            const uint32_t r = m0 + a_row + i * 16, kk = k0 + a_k;
            const bool ok = r < r_hi && kk < p.k;
            const uint32_t sr = ok ? ((GROUPED && p.row_map) ? p.row_map[r] : r) : 0;
            const float* src = x + (size_t)sr * p.ldx + (ok ? kk : 0);
            const f32x4_v v = *(const f32x4_v*)src;
            a_reg[i] = ok ? v : f32x4_v{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int i = 0; i < B_PASSES; ++i) {
            const uint32_t n = n0 + b_row + i * 32, kk = k0 + b_k;
            const bool ok = n < p.n && kk < p.k;
            const uint16_t* src = w + (size_t)(ok ? n : 0) * p.k + (ok ? kk : 0);
            const u32x4_v v = *(const u32x4_v*)src;
            b_reg[i] = ok ? v : u32x4_v{0u, 0u, 0u, 0u};
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i) {
            const uint32_t row = a_row + i * 16;
            u32x2_v o;
            o.x = pack_bf16(a_reg[i].x, a_reg[i].y), o.y = pack_bf16(a_reg[i].z, a_reg[i].w);
            *(u32x2_v*)(s_a + row * PITCH + a_k * 2) = o;
        }
#pragma unroll
        for (int i = 0; i < B_PASSES; ++i) {
            const uint32_t row = b_row + i * 32;
            *(u32x4_v*)(s_b + row * PITCH + b_k * 2) = b_reg[i];
        }
    };

    load(0);
    for (uint32_t k0 = 0; k0 < p.k; k0 += LK) {
        __syncthreads(); // the MFMAs of the step before have read the tiles
        stage();
        __syncthreads();
        if (k0 + LK < p.k) load(k0 + LK);
#pragma unroll
        for (int s = 0; s < LK / 16; ++s) {
            u32x4_t af[MB], bfr[NB];
#pragma unroll
            for (int i = 0; i < MB; ++i) af[i] = *(const u32x4_t*)(s_a + ((wm * MB + i) * 32 + l32) * PITCH + (s * 16 + half * 8) * 2);
#pragma unroll
            for (int j = 0; j < NB; ++j) bfr[j] = *(const u32x4_t*)(s_b + ((wn * NB + j) * 32 + l32) * PITCH + (s * 16 + half * 8) * 2);
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, af[i]), __builtin_bit_cast(bf16x8_t, bfr[j]), acc[i][j], 0, 0, 0);
        }
    }

    float* y = GROUPED ? p.y : p.y + z * p.y_batch;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const uint32_t n = n0 + (wn * NB + j) * 32 + l32;
        if (n >= p.n) continue;
        const float bias = p.bias ? bf16_to_f32(p.bias[n]) : 0.0f;
#pragma unroll
        for (int i = 0; i < MB; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + (wm * MB + i) * 32 + (r & 3) + 8 * (r >> 2) + 4 * half;
                if (row >= r_hi) continue;
                float v = acc[i][j][r] + bias;
                if (p.act == 1) {
                    const float t = fmaxf(v, 0.0f);
                    v = t * t;
                } else if (p.act == 2) {
                    v = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
                }
                if (p.y_scale != 0.0f) v *= p.y_scale;
                if (p.soft_cap != 0.0f) v = p.soft_cap * tanhf(v / p.soft_cap);
                if (p.gate) v *= 1.0f / (1.0f + expf(-p.gate[(size_t)row * p.ldgate + z]));
                if (p.mul_table) {
                    uint32_t t = p.mul_tokens[row];
                    if (t >= p.mul_vocab) t = 0;
                    v *= bf16_to_f32(p.mul_table[(size_t)t * p.mul_ld + p.mul_col0 + n]);
                }
                if (p.residual) v += p.residual[(size_t)row * p.ldr + n];
                y[(size_t)row * p.ldy + n] = v;
            }
        }
    }
}

} // namespace

bool linear_mfma_supported(const LinearF32Params& p) {
    if (!p.bf16_products || (p.rows < 32 && !p.row_offsets) || p.k % 8 || p.ldx % 4 || p.x_batch % 4 || p.w_batch % 8) return false;
    if ((uintptr_t)p.x % 16 || (uintptr_t)p.w % 16) return false;
    return true;
}

uzu_status linear_mfma(hipStream_t s, const LinearF32Params& p) {
    UZU_REQUIRE(linear_mfma_supported(p), "linear_mfma: shape / alignment not covered");
    UZU_REQUIRE(p.row_offsets || !p.row_map, "linear_mfma: gathered rows only in the grouped form");
    // tile choice: the widest tile that still fills the chip; narrow outputs (the per-head products) take the narrow tiles
    if (p.row_offsets) { // grouped: every product may need the whole row range, the workgroups beyond a bucket leave at once
        const dim3 grid((p.n + 127) / 128, (p.rows + 127) / 128 + 1, p.batch);
        UZU_REQUIRE(grid.y <= 65535 && grid.z <= 65535 && !p.residual, "linear_mfma: grouped grid too large");
        return launch_check([&] { hipLaunchKernelGGL((linear_mfma_kernel<2, 2, true>), grid, dim3(256), 0, s, p); }, "linear_mfma_grouped");
    }
    const bool small_m = p.rows <= 64, small_n = p.n <= 64;
    auto tiles = [&](uint32_t bm, uint32_t bn) { return (size_t)((p.rows + bm - 1) / bm) * ((p.n + bn - 1) / bn) * p.batch; };
    if (!small_m && !small_n && tiles(128, 128) >= 256) {
        const dim3 grid((p.n + 127) / 128, (p.rows + 127) / 128, p.batch);
        UZU_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "linear_mfma: grid too large");
        return launch_check([&] { hipLaunchKernelGGL((linear_mfma_kernel<2, 2, false>), grid, dim3(256), 0, s, p); }, "linear_mfma<2,2>");
    }
    if (!small_m && (small_n || tiles(128, 64) >= 256)) {
        const dim3 grid((p.n + 63) / 64, (p.rows + 127) / 128, p.batch);
        UZU_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "linear_mfma: grid too large");
        return launch_check([&] { hipLaunchKernelGGL((linear_mfma_kernel<2, 1, false>), grid, dim3(256), 0, s, p); }, "linear_mfma<2,1>");
    }
    const dim3 grid((p.n + 63) / 64, (p.rows + 63) / 64, p.batch);
    UZU_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "linear_mfma: grid too large");
    return launch_check([&] { hipLaunchKernelGGL((linear_mfma_kernel<1, 1, false>), grid, dim3(256), 0, s, p); }, "linear_mfma<1,1>");
}

} // namespace k
} // namespace uzu
