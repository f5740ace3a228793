// One small product per head on the matrix cores: out_h[M, N] = x_h[M, K] * w_h[N, K]^T for every
// head h, where x and out are [M, width] matrices that hold the heads side by side (x_h starts at
// column h * x_stride, out_h at column h * o_stride) and w is [heads, N, K] bfloat16.  The shapes
// are those of a layer that folds a per-head expansion into its queries or applies one behind its
// attention: K and N of a few hundred, M the step's tokens.
//
// A block of four waves takes 64 rows and 128 columns of one head, a wave 64 rows x 32 columns as
// 4 x 2 tiles of mfma_f32_16x16x32_bf16 with the weights as the first operand (so that a lane ends
// with four neighbouring columns of one row, one 8-byte store).  Operands go from memory straight
// into the MFMA registers, 16 bytes a lane: with K this short every operand byte is used by all
// tiles of the wave in the same step, and the next block finds the weights in L2.  x may be 32-bit
// (rounded to bfloat16 on the way in).  GATE: out = product * sigmoid(gate) with gate 32-bit,
// [M, gate width], the heads side by side at g_stride.
#pragma once
#include "gemm_mfma.h"

constexpr int GH_BM = 64, GH_BN = 128;

template <typename TX>
__device__ __forceinline__ bf16x8_t gh_load8(const TX* p);
template <>
__device__ __forceinline__ bf16x8_t gh_load8<bf16_t>(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)p);
}
template <>
__device__ __forceinline__ bf16x8_t gh_load8<float>(const float* p) {
    float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    u32x4_t v = {f32x2_to_bf16x2(a.x, a.y), f32x2_to_bf16x2(a.z, a.w), f32x2_to_bf16x2(b.x, b.y), f32x2_to_bf16x2(b.z, b.w)};
    return __builtin_bit_cast(bf16x8_t, v);
}

template <typename TX, typename TO, bool GATE>
__global__ void __launch_bounds__(256)
gemm_heads_mfma_kernel(const TX* __restrict__ x, int ldx, int x_stride, const bf16_t* __restrict__ w,
                       TO* __restrict__ out, int ldo, int o_stride, int m, int n, int k,
                       const float* __restrict__ gate, int ldg, int g_stride) {
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int g = lane >> 4, col = lane & 15;
    int h = blockIdx.z;
    int m0 = blockIdx.y * GH_BM, n0 = blockIdx.x * GH_BN + wave * 32;
    if (n0 >= n) return;
    int m_tiles = min(4, (m - m0 + 15) / 16);                      // wave-uniform
    const bf16_t* wh = w + (size_t)h * n * k;
    const TX* xh = x + (size_t)h * x_stride;
    f32x4_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const bf16x8_t zero = __builtin_bit_cast(bf16x8_t, u32x4_t{0u, 0u, 0u, 0u});
    // Four steps of 32 along K at a time: all their operands are requested before the first product,
    // so a round of the loop is one trip to memory (K = 128 is one round).
    constexpr int STEPS = 4;
    for (int k0 = 0; k0 < k; k0 += 32 * STEPS) {
        bf16x8_t wf[STEPS][2], xf[STEPS][4];
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
            int kk = k0 + st * 32 + g * 8;
            bool k_ok = kk < k;                                     // (K is a multiple of 8)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                int gn = n0 + j * 16 + col;
                wf[st][j] = (k_ok && gn < n) ? gh_load8<bf16_t>(wh + (size_t)gn * k + kk) : zero;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int gm = m0 + i * 16 + col;
                xf[st][i] = (i < m_tiles && k_ok && gm < m) ? gh_load8<TX>(xh + (size_t)gm * ldx + kk) : zero;
            }
        }
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
            if (k0 + st * 32 >= k) break;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (i >= m_tiles) break;
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[st][j], xf[st][i], acc[i][j], 0, 0, 0);
            }
        }
    }
    // element e of acc[i][j]: column n0 + 16 j + 4 g + e, row m0 + 16 i + col
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int gm = m0 + i * 16 + col;
        if (i >= m_tiles || gm >= m) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            int gn = n0 + j * 16 + 4 * g;
            float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
            if (GATE) {
                const float* gp = gate + (size_t)gm * ldg + (size_t)h * g_stride + gn;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (gn + e < n) v[e] *= 1.0f / (1.0f + expf(-gp[e]));
            }
            TO* op = out + (size_t)gm * ldo + (size_t)h * o_stride + gn;
            if (sizeof(TO) == 2 && gn + 3 < n && ((uintptr_t)op & 7) == 0) {
                *(uint2*)op = make_uint2(f32x2_to_bf16x2(v[0], v[1]), f32x2_to_bf16x2(v[2], v[3]));       // four columns, 8 bytes
                continue;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (gn + e < n) Elem<TO>::store(op + e, v[e]);
        }
    }
}

// The same products for at most 16 rows (a decode step): a block takes 32 columns of one head and its
// four waves a quarter of K each, so that a block is one trip to memory whatever K is, and the chip
// sees heads * N / 32 blocks; the waves' sums meet in LDS in wave order, wave 0 stores.
template <typename TX, typename TO, bool GATE>
__global__ void __launch_bounds__(256)
gemm_heads_few_rows_kernel(const TX* __restrict__ x, int ldx, int x_stride, const bf16_t* __restrict__ w,
                           TO* __restrict__ out, int ldo, int o_stride, int m, int n, int k,
                           const float* __restrict__ gate, int ldg, int g_stride) {
    __shared__ float red[3][2][64][4];
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int g = lane >> 4, col = lane & 15;
    int h = blockIdx.z, n0 = blockIdx.x * 32;
    const bf16_t* wh = w + (size_t)h * n * k;
    const TX* xh = x + (size_t)h * x_stride;
    int k_quarter = ((k + 3) / 4 + 31) / 32 * 32;
    int k_lo = wave * k_quarter, k_hi = min(k, k_lo + k_quarter);
    f32x4_t acc[2] = {f32x4_t{0.f, 0.f, 0.f, 0.f}, f32x4_t{0.f, 0.f, 0.f, 0.f}};
    const bf16x8_t zero = __builtin_bit_cast(bf16x8_t, u32x4_t{0u, 0u, 0u, 0u});
    constexpr int STEPS = 4;
    for (int k0 = k_lo; k0 < k_hi; k0 += 32 * STEPS) {
        bf16x8_t wf[STEPS][2], xf[STEPS];
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
            int kk = k0 + st * 32 + g * 8;
            bool k_ok = kk < k_hi;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                int gn = n0 + j * 16 + col;
                wf[st][j] = (k_ok && gn < n) ? gh_load8<bf16_t>(wh + (size_t)gn * k + kk) : zero;
            }
            xf[st] = (k_ok && col < m) ? gh_load8<TX>(xh + (size_t)col * ldx + kk) : zero;
        }
#pragma unroll
        for (int st = 0; st < STEPS; ++st)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[st][j], xf[st], acc[j], 0, 0, 0);
    }
    if (wave > 0) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave - 1][j][lane][e] = acc[j][e];
    }
    __syncthreads();
    if (wave > 0 || col >= m) return;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        int gn = n0 + j * 16 + 4 * g;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = ((acc[j][e] + red[0][j][lane][e]) + red[1][j][lane][e]) + red[2][j][lane][e];
        if (GATE) {
            const float* gp = gate + (size_t)col * ldg + (size_t)h * g_stride + gn;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (gn + e < n) v[e] *= 1.0f / (1.0f + expf(-gp[e]));
        }
        TO* op = out + (size_t)col * ldo + (size_t)h * o_stride + gn;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (gn + e < n) Elem<TO>::store(op + e, v[e]);
    }
}
