// Kernels of mixers that carry a state of fixed size from token to token (gfx950, wave64): the
// short causal convolution in front of a recurrence, the recurrence with one scalar decay per head
// (state-space duality), and the gated norm in equal parts behind it.  Everything here is 32-bit:
// the inputs of the recurrence, step sizes, decays, the state and the norm's statistics.
//
// A step brings, per sequence b, the tokens cu_seqlens[b] .. cu_seqlens[b + 1] - 1 of the packed
// batch, in order; the sequence's state lives in row seq_slots[b] of the state tensors and is zero
// when the sequence starts.  A step of one token per sequence and a step of a whole prompt run the
// same arithmetic per token, in the same order, so the result does not depend on how a prompt
// was cut.
#include "common.h"

ROCML_LAST_ERROR_FN(recurrent)

constexpr int RC_BLOCK = 256;

__device__ __forceinline__ float rc_silu(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float rc_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// ---- causal convolution per channel ------------------------------------------------
// out[t, c] = act(bias[c] + sum_j w[c, j] * in(t - (taps - 1) + j, c)): the last column of w is
// the current token's.  Inputs before the step's first token of a sequence come from the
// sequence's state [slot, taps - 1, C] (its last taps - 1 inputs, oldest first; zeros at the
// start).  u is [T, ldu] 32-bit and the channels are its columns col0 .. col0 + C - 1.
constexpr int CONV_MAX_TAPS = 8;

__global__ void __launch_bounds__(RC_BLOCK)
causal_conv_kernel(const float* __restrict__ u, int ldu, int col0, int n_channels, int taps,
                   const float* __restrict__ w, const float* __restrict__ bias, const float* __restrict__ state,
                   const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                   const int* __restrict__ seq_slots, float* __restrict__ out, long long total, int silu) {
    long long idx = (long long)blockIdx.x * RC_BLOCK + threadIdx.x;
    if (idx >= total) return;
    int t = (int)(idx / n_channels), c = (int)(idx - (long long)t * n_channels);
    int b = token_seq[t];
    int local = t - cu_seqlens[b];
    const float* st = state + (size_t)seq_slots[b] * (taps - 1) * n_channels;
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        int src = local - (taps - 1) + j;
        float v = src >= 0 ? u[(size_t)(t - (taps - 1) + j) * ldu + col0 + c] : st[(size_t)(taps - 1 + src) * n_channels + c];
        acc = fmaf(w[(size_t)c * taps + j], v, acc);
    }
    out[idx] = silu ? rc_silu(acc) : acc;
}

// The state after the step: the last taps - 1 inputs of each sequence, taken from the step's
// tokens and, where the step brought fewer, from the old state.  Runs after the outputs.
__global__ void __launch_bounds__(RC_BLOCK)
causal_conv_state_kernel(const float* __restrict__ u, int ldu, int col0, int n_channels, int taps,
                         float* __restrict__ state, const int* __restrict__ cu_seqlens,
                         const int* __restrict__ seq_slots, long long total) {
    long long idx = (long long)blockIdx.x * RC_BLOCK + threadIdx.x;
    if (idx >= total) return;
    int b = (int)(idx / n_channels), c = (int)(idx - (long long)b * n_channels);
    int first = cu_seqlens[b], n = cu_seqlens[b + 1] - first;
    float* st = state + (size_t)seq_slots[b] * (taps - 1) * n_channels;
    float keep[CONV_MAX_TAPS];
#pragma unroll
    for (int k = 0; k < CONV_MAX_TAPS; ++k) {
        if (k >= taps - 1) break;
        int src = n - (taps - 1) + k;
        keep[k] = src >= 0 ? u[(size_t)(first + src) * ldu + col0 + c] : st[(size_t)(taps - 1 + src) * n_channels + c];
    }
#pragma unroll
    for (int k = 0; k < CONV_MAX_TAPS; ++k) {
        if (k >= taps - 1) break;
        st[(size_t)k * n_channels + c] = keep[k];
    }
}

ROCML_EXPORT int rocml_causal_conv(const float* u, int ldu, int col0, int n_tokens, int n_channels, int taps,
                                   const float* w, const float* bias, float* state, int n_slots,
                                   const int* token_seq, const int* cu_seqlens, const int* seq_slots, int n_seqs,
                                   float* out, int silu, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && n_channels > 0 && n_seqs >= 0 && n_slots > 0, "causal_conv: bad sizes T=%d C=%d B=%d", n_tokens,
                  n_channels, n_seqs);
    ROCML_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "causal_conv: %d taps (1 to %d)", taps, CONV_MAX_TAPS);
    ROCML_REQUIRE(col0 >= 0 && ldu >= col0 + n_channels, "causal_conv: row stride %d too small for columns %d..%d", ldu, col0,
                  col0 + n_channels);
    ROCML_REQUIRE(u && w && out && token_seq && cu_seqlens && seq_slots && (taps == 1 || state), "causal_conv: missing arguments");
    if (n_tokens == 0 || n_seqs == 0) return 0;
    long long total = (long long)n_tokens * n_channels;
    causal_conv_kernel<<<ceil_div(total, RC_BLOCK), RC_BLOCK, 0, stream>>>(u, ldu, col0, n_channels, taps, w, bias, state, token_seq,
                                                                           cu_seqlens, seq_slots, out, total, silu);
    ROCML_CHECK_LAUNCH("causal_conv");
    if (taps > 1) {
        long long st_total = (long long)n_seqs * n_channels;
        causal_conv_state_kernel<<<ceil_div(st_total, RC_BLOCK), RC_BLOCK, 0, stream>>>(u, ldu, col0, n_channels, taps, state,
                                                                                       cu_seqlens, seq_slots, st_total);
        ROCML_CHECK_LAUNCH("causal_conv state");
    }
    return 0;
}

// ---- the recurrence ----------------------------------------------------------------
// Per head a (group g = a / (H / G)) and token t, with x_t [P], B_t and C_t [N] from xbc (rows of
// [x: H * P | B: G * N | C: G * N]) and the raw step size from column dt_col0 + a of dtsrc:
//     dt = softplus(raw + dt_bias[a]),  S <- exp(-exp(A_log[a]) dt) S + dt B_t x_t^T,
//     y_t = S^T C_t + D[a] x_t.
// The columns of S (one per value p) do not depend on each other: a block takes one sequence, one
// head and SC_PT values and walks the sequence's tokens in order; thread (p, r) keeps the state
// entries n = r, r + SC_R, ... of column p in registers and the SC_R threads of a column add up
// their parts of S^T C by butterfly.  Tokens come through LDS tc at a time (at most SC_MAX_TC).  State layout:
// [slot, H, P, N].
constexpr int SC_R = 16, SC_PT = RC_BLOCK / SC_R, SC_MAX_TC = 32;

template <int NI>
__global__ void __launch_bounds__(RC_BLOCK)
ssd_scan_kernel(const float* __restrict__ xbc, int ldx, const float* __restrict__ dtsrc, int lddt, int dt_col0,
                const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
                float* __restrict__ state, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots,
                float* __restrict__ y, int n_heads, int head_dim, int n_state, int n_groups, int tc) {
    extern __shared__ float sc_smem[];
    float* bs = sc_smem;                       // [tc][N]
    float* cs = bs + tc * n_state;             // [tc][N]
    float* xs = cs + tc * n_state;             // [tc][SC_PT]
    float* ys = xs + tc * SC_PT;               // [tc][SC_PT]
    float* dts = ys + tc * SC_PT;              // [tc]
    float* decs = dts + tc;                    // [tc]
    int p0 = blockIdx.x * SC_PT, head = blockIdx.y, b = blockIdx.z;
    int tid = threadIdx.x, r = tid % SC_R, pl = tid / SC_R;
    int p = p0 + pl;
    bool p_ok = p < head_dim;
    int group = head / (n_heads / n_groups);
    int inner = n_heads * head_dim;
    int first = cu_seqlens[b], n_tok = cu_seqlens[b + 1] - first;
    float* st = state + (((size_t)seq_slots[b] * n_heads + head) * head_dim + (p_ok ? p : 0)) * n_state;
    float s[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        int n = r + i * SC_R;
        s[i] = (p_ok && n < n_state) ? st[n] : 0.f;
    }
    float a_rate = expf(a_log[head]), bias = dt_bias[head], skip = d_skip[head];
    for (int c0 = 0; c0 < n_tok; c0 += tc) {
        int nt = min(tc, n_tok - c0);
        __syncthreads();                          // the previous chunk's outputs have been written out
        for (int i = tid; i < nt * n_state; i += RC_BLOCK) {
            int tt = i / n_state, n = i - tt * n_state;
            const float* row = xbc + (size_t)(first + c0 + tt) * ldx + inner + (size_t)group * n_state + n;
            bs[i] = row[0];
            cs[i] = row[(size_t)n_groups * n_state];
        }
        for (int i = tid; i < nt * SC_PT; i += RC_BLOCK) {
            int tt = i / SC_PT, pp = i - tt * SC_PT;
            xs[i] = p0 + pp < head_dim ? xbc[(size_t)(first + c0 + tt) * ldx + (size_t)head * head_dim + p0 + pp] : 0.f;
        }
        if (tid < nt) {
            float dt = rc_softplus(dtsrc[(size_t)(first + c0 + tid) * lddt + dt_col0 + head] + bias);
            dts[tid] = dt;
            decs[tid] = expf(-a_rate * dt);
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            float dec = decs[tt], xv = xs[tt * SC_PT + pl];
            float dtx = dts[tt] * xv;
            const float* bt = bs + tt * n_state;
            const float* ct = cs + tt * n_state;
            float part = 0.f;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                int n = r + i * SC_R;
                if (n < n_state) {
                    s[i] = fmaf(dec, s[i], dtx * bt[n]);
                    part = fmaf(s[i], ct[n], part);
                }
            }
#pragma unroll
            for (int off = SC_R / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, 64);
            if (r == 0) ys[tt * SC_PT + pl] = fmaf(skip, xv, part);
        }
        __syncthreads();
        for (int i = tid; i < nt * SC_PT; i += RC_BLOCK) {
            int tt = i / SC_PT, pp = i - tt * SC_PT;
            if (p0 + pp < head_dim) y[(size_t)(first + c0 + tt) * inner + (size_t)head * head_dim + p0 + pp] = ys[i];
        }
    }
    if (p_ok) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int n = r + i * SC_R;
            if (n < n_state) st[n] = s[i];
        }
    }
}

ROCML_EXPORT int rocml_ssd_scan(const float* xbc, int ldx, const float* dtsrc, int lddt, int dt_col0,
                                const float* dt_bias, const float* a_log, const float* d_skip, float* state, int n_slots,
                                const int* cu_seqlens, const int* seq_slots, int n_seqs, int n_tokens, float* y,
                                int n_heads, int head_dim, int n_state, int n_groups, hipStream_t stream) {
    ROCML_REQUIRE(n_heads > 0 && head_dim > 0 && n_state > 0 && n_groups > 0 && n_heads % n_groups == 0,
                  "ssd_scan: bad sizes heads=%d head=%d state=%d groups=%d", n_heads, head_dim, n_state, n_groups);
    ROCML_REQUIRE(n_state <= 16 * SC_R, "ssd_scan: a state of %d exceeds %d", n_state, 16 * SC_R);
    ROCML_REQUIRE(ldx >= n_heads * head_dim + 2 * n_groups * n_state, "ssd_scan: input rows of %d are too short", ldx);
    ROCML_REQUIRE(dt_col0 >= 0 && lddt >= dt_col0 + n_heads, "ssd_scan: step-size rows of %d are too short", lddt);
    ROCML_REQUIRE(xbc && dtsrc && dt_bias && a_log && d_skip && state && cu_seqlens && seq_slots && y && n_slots > 0,
                  "ssd_scan: missing arguments");
    ROCML_REQUIRE(n_seqs >= 0 && n_seqs < 65536 && n_heads < 65536, "ssd_scan: too many sequences or heads for one launch");
    if (n_seqs == 0 || n_tokens == 0) return 0;
    dim3 grid(ceil_div(head_dim, SC_PT), n_heads, n_seqs);
    int tc = n_state <= 128 ? SC_MAX_TC : SC_MAX_TC / 2;          // 64 KB of LDS at most
    size_t lds = (size_t)(2 * tc * n_state + 2 * tc * SC_PT + 2 * tc) * sizeof(float);
    int ni = ceil_div(n_state, SC_R);
#define SCAN(NI_)                                                                                              \
    ssd_scan_kernel<NI_><<<grid, RC_BLOCK, lds, stream>>>(xbc, ldx, dtsrc, lddt, dt_col0, dt_bias, a_log, d_skip, \
                                                          state, cu_seqlens, seq_slots, y, n_heads, head_dim,  \
                                                          n_state, n_groups, tc)
    if (ni <= 1) SCAN(1);
    else if (ni <= 2) SCAN(2);
    else if (ni <= 3) SCAN(3);
    else if (ni <= 4) SCAN(4);
    else if (ni <= 6) SCAN(6);
    else if (ni <= 8) SCAN(8);
    else if (ni <= 12) SCAN(12);
    else SCAN(16);
#undef SCAN
    ROCML_CHECK_LAUNCH("ssd_scan");
    return 0;
}

// ---- gated norm in equal parts ------------------------------------------------------
// out[t, i] = v / sqrt(mean over i's part of v^2 + eps) * gain[i],  v = y[t, i] * silu(z[t, i]):
// the gate comes before the norm, and each of the `parts` equal parts of a row has a root mean
// square of its own.  z is 32-bit in rows of ldz numbers starting at column z_col0.
__device__ __forceinline__ float rc_block_sum(float v, float* scratch) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) scratch[threadIdx.x / WAVE] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < RC_BLOCK / WAVE; ++w) total += scratch[w];
    return total;
}

template <typename TO>
__global__ void __launch_bounds__(RC_BLOCK)
gated_part_norm_kernel(const float* __restrict__ y, const float* __restrict__ z, int ldz, int z_col0,
                       const float* __restrict__ gain, TO* __restrict__ out, int n, int parts, float eps) {
    __shared__ float scratch[RC_BLOCK / WAVE];
    int t = blockIdx.x, part = blockIdx.y;
    int width = n / parts, i0 = part * width;
    const float* yr = y + (size_t)t * n + i0;
    const float* zr = z + (size_t)t * ldz + z_col0 + i0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += RC_BLOCK) {
        float v = yr[i] * rc_silu(zr[i]);
        ss = fmaf(v, v, ss);
    }
    float inv = 1.0f / sqrtf(rc_block_sum(ss, scratch) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += RC_BLOCK) {
        float v = yr[i] * rc_silu(zr[i]);
        Elem<TO>::store(out + (size_t)t * n + i0 + i, v * inv * gain[i0 + i]);
    }
}

ROCML_EXPORT int rocml_gated_part_norm(const float* y, const float* z, int ldz, int z_col0, const float* gain, void* out,
                                       int out_dtype, int n_rows, int n, int parts, float eps, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && n > 0 && parts > 0 && n % parts == 0, "gated_part_norm: %d values do not fall into %d equal parts", n,
                  parts);
    ROCML_REQUIRE(z_col0 >= 0 && ldz >= z_col0 + n, "gated_part_norm: gate rows of %d are too short", ldz);
    ROCML_REQUIRE(parts < 65536, "gated_part_norm: too many parts");
    if (n_rows == 0) return 0;
    dim3 grid(n_rows, parts);
    if (out_dtype == ROCML_F32)
        gated_part_norm_kernel<float><<<grid, RC_BLOCK, 0, stream>>>(y, z, ldz, z_col0, gain, (float*)out, n, parts, eps);
    else if (out_dtype == ROCML_BF16)
        gated_part_norm_kernel<bf16_t><<<grid, RC_BLOCK, 0, stream>>>(y, z, ldz, z_col0, gain, (bf16_t*)out, n, parts, eps);
    else return rocml_fail("gated_part_norm: unknown dtype code %d", out_dtype);
    ROCML_CHECK_LAUNCH("gated_part_norm");
    return 0;
}
