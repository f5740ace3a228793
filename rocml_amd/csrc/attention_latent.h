// bfloat16 attention over a cache of latent rows on the gfx950 matrix cores.
//
// The cache holds one row of DK numbers per position, [page, 64, DK]; all query heads share it (one
// key/value "head"), a key is the whole row and its value is the row's first DV numbers.  A layer
// whose keys and values are expanded from a latent vector reaches this form by folding the key
// expansion into its queries and the value expansion into a product behind the attention.
//
// Rows of work are the (token, head) pairs of a step: the queries [T, H, DK] and the outputs
// [T, H, DV] are plain matrices of T * H rows, and row r of a sequence's new tokens stands at
// position pos0 + r / H.  A block takes 64 RT consecutive rows of one sequence (RT tiles of 16 per
// wave: the 16 columns of an MFMA; RT = 2 for prompts, where every key operand read from LDS then
// feeds two products and a loaded key serves 128 rows, RT = 1 for the few rows of a decode step and
// for the widest sizes, whose two tiles of outputs and queries would not fit a lane's 512 registers)
// and one split of their keys; keys come 32 at a time through LDS, once as
// rows (the first product, S^T = K Q^T, reads 8 numbers of a key per lane) and once transposed
// (the second, O^T = V^T P^T, reads 8 keys of a number per lane): the transposition happens on
// the way into LDS, the cache keeps the rows only.  With many rows per sequence (a prompt) the
// 64 rows share every key they load; with few (a decode step: H rows per sequence) the key range
// is cut into splits whose partial results a second kernel merges by log-sum-exp, in split order.
//
// Online softmax per column as in attention_mfma.h; scores scaled after the dot product, base-2
// exponentials.  A window limits the keys of a row to (pos - window, pos].
// KD: 32-number steps of the first product (DK <= 32 KD), DT: 16-number tiles of the output
// (DV <= 16 DT); numbers beyond DK or DV are zeros in LDS and in the query operand.
#pragma once
#include "attention_mfma.h"

constexpr int AL_ROWS = 64;           // rows of a block
constexpr int AL_KEYS = 32;           // keys of a piece
constexpr int AL_VROW = AL_KEYS + 8;  // bf16 per row of the transposed piece (16 bytes of padding)
constexpr float AL_LAZY_MAX = 8.0f;   // how far a row's maximum may run ahead of its exponents' reference (powers of two)

// Where the transposed piece keeps number d of the keys (bf16 units): rows of AL_VROW and 32 more
// after every eight rows, so that rows eight apart, which neighbouring groups of lanes write at
// the same time, lie 16 banks apart.
__device__ __forceinline__ int al_vrow_at(int d) { return d * AL_VROW + (d >> 3) * 32; }

// Keys as rows: the first product's tile u reads key 8 (c / 4) + 4 u + c % 4 in lane column c; that key
// is stored at row 16 u + c, so the 16 lanes of a tile read 16 consecutive rows.  A thread that
// stages the piece takes the two keys of one column c (they are 4 apart) and writes rows c and
// 16 + c: 16 neighbouring lanes write 16 consecutive rows.  In the transposed copy the two keys
// stand side by side (key 8 G + 4 u + i at place 8 G + 2 i + u of its row), one 4-byte store; the
// probabilities are packed in the same order.

template <int KD, int DT>
struct LatentLds {
    static constexpr int K_ROW = KD * 32 + 8;                               // bf16 per key row
    static constexpr int BYTES = (AL_KEYS * K_ROW + DT * 16 * AL_VROW + DT * 2 * 32) * 2;
};

template <int KD, int DT, int RT>
__global__ void __launch_bounds__(256)
attn_latent_mfma_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ cache,
                        const int* __restrict__ block_table, int bt_width, const int* __restrict__ cu_seqlens,
                        int n_seqs, const int* __restrict__ token_pos, int n_heads, int dk, int dv,
                        float scale_log2e, int window, int n_splits, float* __restrict__ part_o,
                        float* __restrict__ part_ml) {
    using L = LatentLds<KD, DT>;
    extern __shared__ uint4 al_smem[];
    bf16_t* sk = (bf16_t*)al_smem;                    // [AL_KEYS][K_ROW]
    bf16_t* sv = sk + AL_KEYS * L::K_ROW;             // [DT * 16] rows at al_vrow_at
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int g = lane >> 4, col = lane & 15;
    int split = blockIdx.y;
    // which sequence and which of its row tiles
    int tile = blockIdx.x, b = 0, tok0 = 0, n_rows = 0;
    for (; b < n_seqs; ++b) {
        tok0 = cu_seqlens[b];
        n_rows = (cu_seqlens[b + 1] - tok0) * n_heads;
        int tiles = (n_rows + AL_ROWS * RT - 1) / (AL_ROWS * RT);
        if (tile < tiles) break;
        tile -= tiles;
    }
    if (b >= n_seqs) return;
    const int* pages = block_table + (size_t)b * bt_width;
    int pos0 = token_pos[tok0];
    int row0 = tile * AL_ROWS * RT, row1 = min(n_rows, row0 + AL_ROWS * RT) - 1;        // the block's rows
    int w_first = row0 + wave * 16 * RT, w_last = min(row1, w_first + 16 * RT - 1);    // the wave's rows
    bool wave_active = w_first <= row1;
    int wave_lo = window > 0 ? max(0, pos0 + w_first / n_heads - window + 1) : 0;     // first key any of the wave's rows sees
    int wave_hi = pos0 + w_last / n_heads;                                            // last key
    int blk_lo = window > 0 ? max(0, pos0 + row0 / n_heads - window + 1) : 0;
    int blk_hi = pos0 + row1 / n_heads;
    int first_piece = blk_lo / AL_KEYS, last_piece = blk_hi / AL_KEYS;

    // zeros where the sizes stop short of the tiles: they are never written again
    for (int i = tid; i < L::BYTES / 16; i += 256) al_smem[i] = make_uint4(0u, 0u, 0u, 0u);

    // Per tile of 16 rows: the lane's column is one row of work.  Q^T operand: 8 numbers per lane and step.
    bool row_ok[RT];
    int my_pos[RT], my_lo[RT];
    size_t grow[RT];
    bf16x8_t qf[RT][KD];
    float m[RT], l[RT];
    f32x4_t o[RT][DT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        int my_row = w_first + rt * 16 + col;
        row_ok[rt] = my_row <= row1;
        my_pos[rt] = pos0 + (row_ok[rt] ? my_row : row1) / n_heads;
        my_lo[rt] = window > 0 ? max(0, my_pos[rt] - window + 1) : 0;
        grow[rt] = (size_t)tok0 * n_heads + (row_ok[rt] ? my_row : row1);
        const bf16_t* qrow = q + grow[rt] * dk + g * 8;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            bool ok = row_ok[rt] && kd * 32 + g * 8 < dk;
            uint4 v = ok ? *(const uint4*)(qrow + kd * 32) : make_uint4(0u, 0u, 0u, 0u);
            qf[rt][kd] = __builtin_bit_cast(bf16x8_t, v);
        }
        m[rt] = -INFINITY;
        l[rt] = 0.f;
#pragma unroll
        for (int i = 0; i < DT; ++i) o[rt][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    // A piece on its way: a thread takes the two keys of a column (see above) and 8 numbers of both.
    int dk8 = dk / 8, dv8 = dv / 8;
    int items = (AL_KEYS / 2) * dk8;
    constexpr int MAX_ITEMS = (AL_KEYS / 2) * (KD * 4) / 256 + 1;
    uint4 ra[MAX_ITEMS], rb[MAX_ITEMS];
    auto request_piece = [&](int piece) {
        int key0 = piece * AL_KEYS;
        int phys = max(pages[key0 / AM_PAGE], 0);       // (a page that is not there holds no visible key)
        const bf16_t* base = cache + ((size_t)phys * AM_PAGE + key0 % AM_PAGE) * dk;
#pragma unroll
        for (int i = 0; i < MAX_ITEMS; ++i) {
            int w = tid + i * 256;
            if (w < items) {
                int c = w & 15, dc = w >> 4;            // 16 neighbouring lanes: the 16 columns, the same 8 numbers
                int ka = 8 * (c >> 2) + (c & 3);
                ra[i] = *(const uint4*)(base + (size_t)ka * dk + dc * 8);
                rb[i] = *(const uint4*)(base + (size_t)(ka + 4) * dk + dc * 8);
            }
        }
    };
    auto store_piece = [&]() {
#pragma unroll
        for (int i = 0; i < MAX_ITEMS; ++i) {
            int w = tid + i * 256;
            if (w < items) {
                int c = w & 15, dc = w >> 4;
                *(uint4*)(sk + c * L::K_ROW + dc * 8) = ra[i];
                *(uint4*)(sk + (16 + c) * L::K_ROW + dc * 8) = rb[i];
                if (dc < dv8) {
                    const uint32_t a[4] = {ra[i].x, ra[i].y, ra[i].z, ra[i].w};
                    const uint32_t bw[4] = {rb[i].x, rb[i].y, rb[i].z, rb[i].w};
                    uint32_t* dst = (uint32_t*)(sv + al_vrow_at(dc * 8) + 2 * c);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        // numbers 2j and 2j + 1 of both keys, the two keys side by side
                        dst[(2 * j) * (AL_VROW / 2)] = (a[j] & 0xffffu) | (bw[j] << 16);
                        dst[(2 * j + 1) * (AL_VROW / 2)] = (a[j] >> 16) | (bw[j] & 0xffff0000u);
                    }
                }
            }
        }
    };

    int piece = first_piece + split;
    if (piece <= last_piece) request_piece(piece);
    for (; piece <= last_piece; piece += n_splits) {
        __syncthreads();                 // the piece before has been multiplied (first round: the zeros are written)
        store_piece();
        __syncthreads();
        if (piece + n_splits <= last_piece) request_piece(piece + n_splits);
        int key0 = piece * AL_KEYS;
        if (!wave_active || key0 > wave_hi || key0 + AL_KEYS - 1 < wave_lo) continue;      // wave-uniform
        // scores of 2 x 16 keys: row r of tile u is key 8 (r / 4) + 4 u + r % 4, so that element i of
        // s[rt][u] in lane (g, col) is key 8 g + 4 u + i of the column's row of work
        f32x4_t s[RT][2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) s[rt][u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            const bf16_t* krow = sk + (16 * u + col) * L::K_ROW + g * 8;       // key 8 (col / 4) + 4 u + col % 4
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) {
                bf16x8_t kf = __builtin_bit_cast(bf16x8_t, *(const uint4*)(krow + kd * 32));
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    s[rt][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[rt][kd], s[rt][u], 0, 0, 0);
            }
        }
        bf16x8_t pf[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            float mx = -INFINITY;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    int key = key0 + g * 8 + u * 4 + i;
                    float v = (row_ok[rt] && key >= my_lo[rt] && key <= my_pos[rt]) ? s[rt][u][i] * scale_log2e : -INFINITY;
                    s[rt][u][i] = v;
                    mx = fmaxf(mx, v);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            // The exponents' reference m follows a row's maximum only when that has grown by more than
            // AL_LAZY_MAX: any reference gives the same quotient at the end, the probabilities stay below
            // 2^AL_LAZY_MAX, and the sums and outputs so far are rescaled only for a row's first pieces
            // instead of with every piece (the outputs are the bulk of a lane's registers).
            if (__builtin_amdgcn_ballot_w64(mx > m[rt] + AL_LAZY_MAX)) {
                float m_new = fmaxf(m[rt], mx);
                float corr = fast_exp2(m[rt] - (m_new == -INFINITY ? 0.f : m_new));
                l[rt] *= corr;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) o[rt][dt] = o[rt][dt] * corr;
                m[rt] = m_new;
            }
            float m_use = m[rt] == -INFINITY ? 0.f : m[rt];
            float sum = 0.f;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s[rt][u][i] = fast_exp2(s[rt][u][i] - m_use);
                    sum += s[rt][u][i];
                }
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            l[rt] += sum;
            // P^T operand: slot 2 i + u = key 8 g + 4 u + i, the order of the transposed copy
            pf[rt] = __builtin_bit_cast(bf16x8_t, make_uint4(pack_bf16x2(s[rt][0][0], s[rt][1][0]), pack_bf16x2(s[rt][0][1], s[rt][1][1]),
                                                             pack_bf16x2(s[rt][0][2], s[rt][1][2]), pack_bf16x2(s[rt][0][3], s[rt][1][3])));
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            bf16x8_t vf = __builtin_bit_cast(bf16x8_t, *(const uint4*)(sv + al_vrow_at(dt * 16 + col) + g * 8));
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[rt], o[rt][dt], 0, 0, 0);
        }
    }
    // element i of o[rt][dt] is number 16 dt + 4 g + i of the column's row
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (!row_ok[rt]) continue;
        if (n_splits == 1) {
            float inv = 1.0f / l[rt];
            bf16_t* orow = out + grow[rt] * dv;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                int d = dt * 16 + 4 * g;
                if (d < dv)       // (dv is a multiple of 8: four numbers are inside or outside together)
                    *(uint2*)(orow + d) = make_uint2(pack_bf16x2(o[rt][dt][0] * inv, o[rt][dt][1] * inv),
                                                     pack_bf16x2(o[rt][dt][2] * inv, o[rt][dt][3] * inv));
            }
        } else {
            size_t slot = grow[rt] * n_splits + split;
            float* po = part_o + slot * dv;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                int d = dt * 16 + 4 * g;
                if (d < dv) *(float4*)(po + d) = make_float4(o[rt][dt][0], o[rt][dt][1], o[rt][dt][2], o[rt][dt][3]);
            }
            if (g == 0) {
                part_ml[slot * 2] = m[rt];
                part_ml[slot * 2 + 1] = l[rt];
            }
        }
    }
}

// Log-sum-exp merge of the splits of a row, in split order: one block per row.  At most 64 splits:
// lane s of every wave fetches split s's reference and sum, so these loads go out together; the
// weights then sit in LDS and every thread sums its numbers over the splits, eight loads at a time.
__global__ void attn_latent_reduce_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                          bf16_t* __restrict__ out, int n_splits, int dv) {
    __shared__ float wgt[64];
    size_t row = blockIdx.x;
    const float* ml = part_ml + row * n_splits * 2;
    const float* po = part_o + row * n_splits * dv;
    int lane = threadIdx.x & 63;
    bool has = lane < n_splits;
    float ms = has ? ml[lane * 2] : -INFINITY;
    float ls = has ? ml[lane * 2 + 1] : 0.f;
    float mm = wave_max(ms);
    float w = ms == -INFINITY ? 0.f : fast_exp2(ms - mm);
    if (threadIdx.x < 64) wgt[lane] = w;
    float inv_l = 1.0f / wave_sum(ls * w);          // every wave computes the same sum
    __syncthreads();
    for (int d = threadIdx.x; d < dv; d += blockDim.x) {
        float acc = 0.f;
        for (int s0 = 0; s0 < n_splits; s0 += 8) {
            float v[8];
#pragma unroll
            for (int s = 0; s < 8; ++s) v[s] = po[(size_t)min(s0 + s, n_splits - 1) * dv + d];
#pragma unroll
            for (int s = 0; s < 8; ++s) acc += s0 + s < n_splits ? v[s] * wgt[s0 + s] : 0.f;
        }
        out[row * dv + d] = f32_to_bf16(acc * inv_l);
    }
}
