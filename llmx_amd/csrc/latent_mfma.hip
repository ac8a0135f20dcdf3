// Latent attention on the matrix cores (bfloat16): the attention of latent.hip for steps whose sizes the 16x16x32
// instruction takes (latent C a multiple of 16 up to 512, C + R a multiple of 32, pages of a multiple of 8 tokens).
//
// Decoded rows (one row of a request in the step) share out their context: blocks of 128 keys each go to an item of their
// own, which stores partial sums, and a second kernel joins them (so a decoded row's bits depend on its own context
// only, never on the batch; against the same row inside a prompt portion they differ by rounding).
// An item is one wave and up to 16 columns; a column is a (row, head) pair: the heads head0 .. head0 + heads - 1 of the rows
// row0 .. row0 + rows - 1 of one request (rows * heads <= 16).  All heads read the same cached rows, so one key tile serves
// all 16 columns.  The item walks the request's keys in segments of 64 absolute positions up to its last row's position:
//   scores  S[keys x cols] = K[keys x (C+R)] . Q^T, 4 tiles of 16 keys a segment, Q^T read from LDS, K straight from the cache;
//   online softmax a column (keys beyond the column's own position weigh 0; a segment that lies wholly beyond it changes
//   none of the column's bits: max unchanged, correction exp(0) = 1, weights 0);
//   values  O[C x cols] = O * correction + V^T[C x keys] . P, V^T straight from the transposed copy of the latents
//   (cache_t [pages, C, page_tokens]: 8 consecutive keys of one dim are one 16-byte load).
// Key -> tile row follows the accumulator layout: row r of score tile u of a 32-key chunk holds key 8 (r / 4) + 4 u + r % 4, so
// that a lane's eight weights of a chunk belong to eight consecutive keys, the k-slots it feeds the value product.
// A column's arithmetic depends on its own position and its request's cache only, and on segments of absolute
// positions: the same bits in any step, beside any other rows.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

struct LatentMfmaArgs {
    const bf16_t* q_lat;    // [H, T, C]
    const bf16_t* q_rot;    // [H, T, R]
    const bf16_t* cache;    // [pages, page_tokens, C + R]
    const bf16_t* cache_t;  // [pages, C, page_tokens]
    const int* pos;
    const int* row_entry;
    const int* tables;
    const int* items;       // [n_items, 8]: row0, rows, head0, heads, key_begin, key_end, slot, -
    bf16_t* out;            // [H, T, C]
    float* part_o;          // [slots, 16, C]: a split item's sums, not yet divided
    float* part_ml;         // [slots, 16, 2]: its maximum and its sum of weights
    float scale;
    int T, H, C, R, page_tokens, max_blocks;
};

#define LM_SEG 64
#define LM_ITEM_INTS 8
#define LM_KSTEPS 6     // k-steps of 32 dims whose key loads are in flight together
#define LM_VTILES 16    // dim tiles of 16 whose value loads are in flight together

// An item with slot < 0 walks all keys up to its last row's position and stores the finished rows.  A split item (one
// decoded row, the keys key_begin .. key_end - 1, a multiple of 64 apart) stores its unnormalized sums, maximum and sum
// of weights in its slot; the merge kernel joins a column's slots in key order.
template <int CT>
__global__ void __launch_bounds__(64) latent_attention_mfma_kernel(LatentMfmaArgs a) {
    extern __shared__ __align__(16) bf16_t qs[];   // [16][C + R + 8]
    const int lane = threadIdx.x, col = lane & 15, g = lane >> 4;
    const int* item = a.items + LM_ITEM_INTS * (size_t)blockIdx.x;
    const int row0 = item[0], rows = item[1], head0 = item[2], heads = item[3], slot = item[6];
    const int C = a.C, R = a.R, CR = C + R, ldq = CR + 8, pt = a.page_tokens;
    const int n_cols = rows * heads;

    // the columns' queries into LDS, 16 bytes a lane and turn, eight turns' loads in flight together; columns without a
    // (row, head) hold zeros
    {
        const int per_col = CR / 8, chunks = 16 * per_col;
        for (int i0 = lane; i0 < chunks; i0 += 64 * 8) {
            uint4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i = i0 + 64 * u;
                const int c = i / per_col, d = 8 * (i % per_col);
                v[u] = uint4{0, 0, 0, 0};
                if (i < chunks && c < n_cols) {
                    const int r = row0 + c / heads, h = head0 + c % heads;
                    v[u] = d < C ? *reinterpret_cast<const uint4*>(a.q_lat + ((size_t)h * a.T + r) * C + d)
                                 : *reinterpret_cast<const uint4*>(a.q_rot + ((size_t)h * a.T + r) * R + (d - C));
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i = i0 + 64 * u;
                if (i < chunks) *reinterpret_cast<uint4*>(qs + (i / per_col) * ldq + 8 * (i % per_col)) = v[u];
            }
        }
    }
    __syncthreads();

    const bool live = col < n_cols;
    const int c_row = row0 + (live ? col / heads : 0), c_head = head0 + (live ? col % heads : 0);
    const int p_col = a.pos[c_row];
    const int p_max = a.pos[row0 + rows - 1];
    const int* table = a.tables + (size_t)a.row_entry[row0] * a.max_blocks;
    const int steps = CR / 32;
    const int last_group = (p_max / 8) * 8;
    const int key_begin = slot < 0 ? 0 : item[4];
    const int key_last = slot < 0 ? p_max : min(item[5] - 1, p_max);

    f32x4_t o[CT];
#pragma unroll
    for (int dt = 0; dt < CT; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float m = -INFINITY, l = 0.0f;

    for (int seg0 = key_begin; seg0 <= key_last; seg0 += LM_SEG) {
        // this lane's key row of each of the segment's four score tiles (tile v = 2 * chunk + u)
        const bf16_t* kp[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            int key = seg0 + 32 * (v >> 1) + 8 * (col >> 2) + 4 * (v & 1) + (col & 3);
            key = key < p_max ? key : p_max;     // keys beyond the last row's position weigh nothing; read a key that exists
            kp[v] = a.cache + ((size_t)table[key / pt] * pt + key % pt) * CR + 8 * g;
        }
        f32x4_t s[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) s[v] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        for (int st0 = 0; st0 < steps; st0 += LM_KSTEPS) {
            // every load of the group is asked for before the first product; a step past the end reads the last step's keys
            // again and multiplies them by zeros
            bf16x8_t kf[LM_KSTEPS][4], qf[LM_KSTEPS];
#pragma unroll
            for (int j = 0; j < LM_KSTEPS; ++j) {
                const int st = st0 + j < steps ? st0 + j : steps - 1;
#pragma unroll
                for (int v = 0; v < 4; ++v) kf[j][v] = *reinterpret_cast<const bf16x8_t*>(kp[v] + 32 * st);
            }
#pragma unroll
            for (int j = 0; j < LM_KSTEPS; ++j) {
                const int st = st0 + j < steps ? st0 + j : steps - 1;
                const uint4 q = *reinterpret_cast<const uint4*>(qs + col * ldq + 32 * st + 8 * g);
                const uint4 used = st0 + j < steps ? q : uint4{0, 0, 0, 0};
                qf[j] = __builtin_bit_cast(bf16x8_t, used);
            }
#pragma unroll
            for (int j = 0; j < LM_KSTEPS; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v) s[v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[j][v], qf[j], s[v], 0, 0, 0);
        }
        // s[v][i]: key seg0 + 32 (v / 2) + 8 g + 4 (v % 2) + i against column `col`
        float top = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = seg0 + 32 * (v >> 1) + 8 * g + 4 * (v & 1) + i;
                s[v][i] = key <= p_col ? s[v][i] * a.scale : -INFINITY;
                top = fmaxf(top, s[v][i]);
            }
        top = rows_max4(top);
        const float m_new = fmaxf(m, top);           // finite from the first segment on: its first key counts for every column
        const float correction = __expf(m - m_new);  // 0 in the first segment, 1 where the segment holds no key of the column
        float sum = 0.0f;
        bf16x8_t pf[2];
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float w = s[v][i] == -INFINITY ? 0.0f : __expf(s[v][i] - m_new);
                sum += w;
                pf[v >> 1][4 * (v & 1) + i] = (__bf16)w;
            }
        l = l * correction + rows_sum4(sum);
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < CT; ++dt) o[dt] = f32x4_t{o[dt][0] * correction, o[dt][1] * correction, o[dt][2] * correction, o[dt][3] * correction};
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            int key0 = seg0 + 32 * c + 8 * g;
            key0 = key0 < last_group ? key0 : last_group;   // a group wholly beyond the last key weighs nothing; read one that exists
            const bf16_t* vp = a.cache_t + ((size_t)table[key0 / pt] * C + col) * pt + key0 % pt;
#pragma unroll
            for (int d0 = 0; d0 < CT; d0 += LM_VTILES) {
                bf16x8_t vf[LM_VTILES < CT ? LM_VTILES : CT];
#pragma unroll
                for (int j = 0; j < (LM_VTILES < CT ? LM_VTILES : CT); ++j) {
                    const int dt = 16 * (d0 + j) < C ? d0 + j : 0;     // a tile past the latent reads the first one again; its product is dropped
                    vf[j] = *reinterpret_cast<const bf16x8_t*>(vp + (size_t)16 * dt * pt);
                }
#pragma unroll
                for (int j = 0; j < (LM_VTILES < CT ? LM_VTILES : CT); ++j)
                    if (16 * (d0 + j) < C) o[d0 + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[j], pf[c], o[d0 + j], 0, 0, 0);
            }
        }
    }
    if (slot >= 0) {
        float* po = a.part_o + ((size_t)slot * 16 + col) * C;
#pragma unroll
        for (int dt = 0; dt < CT; ++dt)
            if (16 * dt < C) *reinterpret_cast<f32x4_t*>(po + 16 * dt + 4 * g) = o[dt];
        if (g == 0) {
            a.part_ml[((size_t)slot * 16 + col) * 2] = m;
            a.part_ml[((size_t)slot * 16 + col) * 2 + 1] = l;
        }
        return;
    }
    if (!live) return;
    bf16_t* out = a.out + ((size_t)c_head * a.T + c_row) * C;
    const float inv = 1.0f / l;
#pragma unroll
    for (int dt = 0; dt < CT; ++dt) {
        if (16 * dt < C) {
#pragma unroll
            for (int i = 0; i < 4; ++i) out[16 * dt + 4 * g + i] = f32_to_bf16(o[dt][i] * inv);
        }
    }
}

// Joins the slots of a decoded row's split items, in key order: with M the largest of the slots' maxima,
// out = sum_i O_i e^(m_i - M) / sum_i l_i e^(m_i - M).  merges [n, 8]: row, head0, heads, first slot, slots.
// One workgroup a column (blockIdx.y): the slots' weights are formed once into LDS, then every thread adds its dims over
// the slots in order, eight slots' loads in flight.
#define LM_MERGE_MAX 1024    // slots of one column whose weights fit the workgroup's LDS; longer columns take rounds
__global__ void __launch_bounds__(256) latent_attention_merge_kernel(const int* __restrict__ merges, const float* __restrict__ part_o,
                                                                   const float* __restrict__ part_ml, bf16_t* __restrict__ out, int T, int C) {
    __shared__ float weight[LM_MERGE_MAX];
    __shared__ float scratch[4];
    const int* mg = merges + LM_ITEM_INTS * (size_t)blockIdx.x;
    const int row = mg[0], head0 = mg[1], heads = mg[2], slot0 = mg[3], n = mg[4];
    const int c = blockIdx.y;
    if (c >= heads) return;
    // M: every thread takes slots tid, tid + 256, ...; the workgroup's maximum does not depend on the order
    float M = -INFINITY;
    for (int i = threadIdx.x; i < n; i += 256) M = fmaxf(M, part_ml[((size_t)(slot0 + i) * 16 + c) * 2]);
    M = wave_max(M);
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = M;
    __syncthreads();
    M = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
    float acc[2] = {0.0f, 0.0f};    // dims tid and tid + 256 (C <= 512)
    float L = 0.0f;
    for (int i0 = 0; i0 < n; i0 += LM_MERGE_MAX) {
        const int round = min(LM_MERGE_MAX, n - i0);
        __syncthreads();
        for (int i = threadIdx.x; i < round; i += 256) weight[i] = __expf(part_ml[((size_t)(slot0 + i0 + i) * 16 + c) * 2] - M);
        __syncthreads();
        for (int i = 0; i < round; ++i) L += part_ml[((size_t)(slot0 + i0 + i) * 16 + c) * 2 + 1] * weight[i];   // in slot order, by every thread alike
        for (int i = 0; i < round; i += 8) {
            float v[8][2];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int at = i + u < round ? i + u : round - 1;
                const float* po = part_o + ((size_t)(slot0 + i0 + at) * 16 + c) * C;
#pragma unroll
                for (int e = 0; e < 2; ++e) v[u][e] = threadIdx.x + 256 * e < C ? po[threadIdx.x + 256 * e] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (i + u < round) {
                    acc[0] += v[u][0] * weight[i + u];
                    acc[1] += v[u][1] * weight[i + u];
                }
        }
    }
    const float inv = 1.0f / L;
#pragma unroll
    for (int e = 0; e < 2; ++e)
        if (threadIdx.x + 256 * e < C) out[((size_t)(head0 + c) * T + row) * C + threadIdx.x + 256 * e] = f32_to_bf16(acc[e] * inv);
}

// ---------------------------------------------------------------------------
// Rows of a prompt portion: a workgroup of four waves takes four column tiles (64 columns: consecutive rows of one request
// with the same heads) and walks the keys once for all of them.  Of a segment's 64 keys wave w scores keys 16w .. 16w + 15
// against all four tiles (one key load serves four products); the weights go through LDS (float32, [column][key]); of the
// value product wave w owns the latent dims [w C/4, (w + 1) C/4) of all four tiles (one value load serves four products).
// Maxima are exact in any order; a column's sum of weights is added from LDS by the lanes and in the order of the
// one-wave kernel, and the value product sees the same weights in the same k-slots: a column gets that kernel's bits.
// With one column tile (LW_TILES 1) the same workgroup serves decoded rows: the item is a block of a row's context (see the
// one-wave kernel's split items), all of a segment's key loads and the wave's value loads are asked for together before
// the first product, and the item stores its sums, maximum and sum of weights for the join.
#define LW_LDW 68     // floats a column's 64 weights take in LDS (padded)

template <int DPW, int LW_TILES, int KS>    // dim tiles of 16 a wave owns; column tiles; k-steps whose key loads are in flight together
__global__ void __launch_bounds__(256) latent_attention_tiles_kernel(LatentMfmaArgs a) {
    constexpr int COLS = 16 * LW_TILES;
    constexpr bool EARLY_VALUES = LW_TILES == 1;
    extern __shared__ __align__(16) bf16_t qs[];   // [64][C + R + 8], then the weights and the waves' maxima
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 15, g = lane >> 4;
    const int* item = a.items + LM_ITEM_INTS * (size_t)blockIdx.x;
    const int row0 = item[0], rows = item[1], head0 = item[2], heads = item[3], slot = item[6];
    const int C = a.C, R = a.R, CR = C + R, ldq = CR + 8, pt = a.page_tokens;
    const int per = heads >= 16 ? 1 : 16 / heads;      // rows a column tile holds
    float* ws = reinterpret_cast<float*>(qs + COLS * ldq);        // [2][COLS][LW_LDW]
    float* pmax = ws + 2 * COLS * LW_LDW;                           // [2][4][COLS]

    {
        const int per_col = CR / 8, chunks = COLS * per_col;
        for (int i0 = tid; i0 < chunks; i0 += 256 * 8) {
            uint4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i = i0 + 256 * u;
                const int cc = i / per_col, d = 8 * (i % per_col);
                const int c = cc & 15, r = (cc >> 4) * per + c / heads;
                v[u] = uint4{0, 0, 0, 0};
                if (i < chunks && c < per * heads && r < rows) {
                    const int h = head0 + c % heads;
                    v[u] = d < C ? *reinterpret_cast<const uint4*>(a.q_lat + ((size_t)h * a.T + row0 + r) * C + d)
                                 : *reinterpret_cast<const uint4*>(a.q_rot + ((size_t)h * a.T + row0 + r) * R + (d - C));
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i = i0 + 256 * u;
                if (i < chunks) *reinterpret_cast<uint4*>(qs + (i / per_col) * ldq + 8 * (i % per_col)) = v[u];
            }
        }
    }
    __syncthreads();

    bool live[LW_TILES];
    int p_col[LW_TILES], c_row[LW_TILES];
#pragma unroll
    for (int ct = 0; ct < LW_TILES; ++ct) {
        const int r = ct * per + col / heads;
        live[ct] = col < per * heads && r < rows;
        c_row[ct] = row0 + (live[ct] ? r : 0);
        p_col[ct] = a.pos[c_row[ct]];
    }
    const int c_head = head0 + col % heads;
    const int p_max = a.pos[row0 + rows - 1];
    const int* table = a.tables + (size_t)a.row_entry[row0] * a.max_blocks;
    const int steps = CR / 32;
    const int last_group = (p_max / 8) * 8;
    const int key_begin = slot < 0 ? 0 : item[4];
    const int key_last = slot < 0 ? p_max : min(item[5] - 1, p_max);

    f32x4_t o[LW_TILES][DPW];
    float m[LW_TILES], l[LW_TILES];
#pragma unroll
    for (int ct = 0; ct < LW_TILES; ++ct) {
        m[ct] = -INFINITY;
        l[ct] = 0.0f;
#pragma unroll
        for (int dt = 0; dt < DPW; ++dt) o[ct][dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }

    for (int seg0 = key_begin; seg0 <= key_last; seg0 += LM_SEG) {
        const int buf = (seg0 / LM_SEG) & 1;
        float* wbuf = ws + buf * COLS * LW_LDW;
        float* mbuf = pmax + buf * 4 * COLS;
        // scores of this wave's 16 keys (key 16 wave + lane % 16 in the tile's row lane % 16) against the four tiles
        int key = seg0 + 16 * wave + col;
        key = key < p_max ? key : p_max;
        const bf16_t* kp = a.cache + ((size_t)table[key / pt] * pt + key % pt) * CR + 8 * g;
        f32x4_t s[LW_TILES];
#pragma unroll
        for (int ct = 0; ct < LW_TILES; ++ct) s[ct] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        // the wave's value loads of the segment (its dim tiles, both chunks): with one column tile they are asked for now,
        // with the keys, and wait for nothing but the page ids
        bf16x8_t vf[2][DPW];
        auto value_loads = [&](int c) {
            int key0 = seg0 + 32 * c + 8 * g;
            key0 = key0 < last_group ? key0 : last_group;
            const bf16_t* vp = a.cache_t + ((size_t)table[key0 / pt] * C + col) * pt + key0 % pt;
#pragma unroll
            for (int dt = 0; dt < DPW; ++dt) {
                const int tile = 16 * (wave * DPW + dt) < C ? wave * DPW + dt : 0;
                vf[c][dt] = *reinterpret_cast<const bf16x8_t*>(vp + (size_t)16 * tile * pt);
            }
        };
        if (EARLY_VALUES) {
            value_loads(0);
            value_loads(1);
        }
        for (int st0 = 0; st0 < steps; st0 += KS) {
            bf16x8_t kf[KS];
#pragma unroll
            for (int j = 0; j < KS; ++j) kf[j] = *reinterpret_cast<const bf16x8_t*>(kp + 32 * (st0 + j < steps ? st0 + j : steps - 1));
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                const int st = st0 + j < steps ? st0 + j : steps - 1;
#pragma unroll
                for (int ct = 0; ct < LW_TILES; ++ct) {
                    const uint4 q = *reinterpret_cast<const uint4*>(qs + (16 * ct + col) * ldq + 32 * st + 8 * g);
                    const uint4 used = st0 + j < steps ? q : uint4{0, 0, 0, 0};
                    s[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[j], __builtin_bit_cast(bf16x8_t, used), s[ct], 0, 0, 0);
                }
            }
        }
        // s[ct][i]: key seg0 + 16 wave + 4 g + i against column `col` of tile ct
#pragma unroll
        for (int ct = 0; ct < LW_TILES; ++ct) {
            float top = -INFINITY;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s[ct][i] = seg0 + 16 * wave + 4 * g + i <= p_col[ct] ? s[ct][i] * a.scale : -INFINITY;
                top = fmaxf(top, s[ct][i]);
            }
            top = rows_max4(top);
            if (g == 0) mbuf[wave * COLS + 16 * ct + col] = top;
        }
        __syncthreads();
        float correction[LW_TILES];
#pragma unroll
        for (int ct = 0; ct < LW_TILES; ++ct) {
            const int cc = 16 * ct + col;
            const float top = fmaxf(fmaxf(mbuf[cc], mbuf[COLS + cc]), fmaxf(mbuf[2 * COLS + cc], mbuf[3 * COLS + cc]));
            const float m_new = fmaxf(m[ct], top);
            correction[ct] = __expf(m[ct] - m_new);
            m[ct] = m_new;
            f32x4_t w;
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = s[ct][i] == -INFINITY ? 0.0f : __expf(s[ct][i] - m_new);
            *reinterpret_cast<f32x4_t*>(wbuf + cc * LW_LDW + 16 * wave + 4 * g) = w;
        }
        __syncthreads();
        bf16x8_t pf[LW_TILES][2];
#pragma unroll
        for (int ct = 0; ct < LW_TILES; ++ct) {
            // the lane's 16 weights of the segment in the one-wave kernel's order: keys 32 c + 8 g + 4 u + i over c, u, i
            const float* wc = wbuf + (16 * ct + col) * LW_LDW + 8 * g;
            float sum = 0.0f;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const f32x4_t w = *reinterpret_cast<const f32x4_t*>(wc + 32 * (v >> 1) + 4 * (v & 1));
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    sum += w[i];
                    pf[ct][v >> 1][4 * (v & 1) + i] = (__bf16)w[i];
                }
            }
            l[ct] = l[ct] * correction[ct] + rows_sum4(sum);
#pragma unroll
            for (int dt = 0; dt < DPW; ++dt)
                o[ct][dt] = f32x4_t{o[ct][dt][0] * correction[ct], o[ct][dt][1] * correction[ct], o[ct][dt][2] * correction[ct], o[ct][dt][3] * correction[ct]};
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            if (!EARLY_VALUES) value_loads(c);
#pragma unroll
            for (int dt = 0; dt < DPW; ++dt)
                if (16 * (wave * DPW + dt) < C) {
#pragma unroll
                    for (int ct = 0; ct < LW_TILES; ++ct) o[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[c][dt], pf[ct][c], o[ct][dt], 0, 0, 0);
                }
        }
    }
    if (slot >= 0) {       // a block of a decoded row's context (one column tile): sums, maximum and sum of weights for the join
        float* po = a.part_o + ((size_t)slot * 16 + col) * C;
#pragma unroll
        for (int dt = 0; dt < DPW; ++dt) {
            const int d0 = 16 * (wave * DPW + dt);
            if (d0 < C) *reinterpret_cast<f32x4_t*>(po + d0 + 4 * g) = o[0][dt];
        }
        if (wave == 0 && g == 0) {
            a.part_ml[((size_t)slot * 16 + col) * 2] = m[0];
            a.part_ml[((size_t)slot * 16 + col) * 2 + 1] = l[0];
        }
        return;
    }
#pragma unroll
    for (int ct = 0; ct < LW_TILES; ++ct) {
        if (!live[ct]) continue;
        bf16_t* out = a.out + ((size_t)c_head * a.T + c_row[ct]) * C;
        const float inv = 1.0f / l[ct];
#pragma unroll
        for (int dt = 0; dt < DPW; ++dt) {
            const int d0 = 16 * (wave * DPW + dt);
            if (d0 < C) {
#pragma unroll
                for (int i = 0; i < 4; ++i) out[d0 + 4 * g + i] = f32_to_bf16(o[ct][dt][i] * inv);
            }
        }
    }
}

extern "C" int llmx_latent_attention_mfma_ok(int C, int R, int page_tokens) {
    return C >= 16 && C <= 512 && C % 16 == 0 && R >= 0 && R % 8 == 0 && (C + R) % 32 == 0 && page_tokens > 0 && page_tokens % 8 == 0 ? 1 : 0;
}

extern "C" int llmx_latent_attention_mfma(const void* q_lat, const void* q_rot, const void* cache, const void* cache_t, const int* pos,
                                          const int* row_entry, const int* tables, const int* items, int n_items, int n_tile_items, int n_row_items,
                                          const int* merges, int n_merges,
                                          void* out, float* part_o, float* part_ml, float scale, int T, int H, int C, int R, int page_tokens,
                                          int max_blocks, hipStream_t stream) {
    if (n_items <= 0 && n_tile_items <= 0 && n_row_items <= 0) return 0;
    if (!llmx_latent_attention_mfma_ok(C, R, page_tokens)) return -2;
    if (n_merges > 0 && (!merges || !part_o || !part_ml)) return -2;
    LatentMfmaArgs a{(const bf16_t*)q_lat, (const bf16_t*)q_rot, (const bf16_t*)cache, (const bf16_t*)cache_t, pos, row_entry, tables, items,
                     (bf16_t*)out, part_o, part_ml, scale, T, H, C, R, page_tokens, max_blocks};
#define LLMX_LT(DPW, TILES, KS, count, first)                                                                                        \
    {                                                                                                                                 \
        static bool raised = false;                                                                                                   \
        if (!raised) {                                                                                                                \
            if (hipFuncSetAttribute((const void*)latent_attention_tiles_kernel<DPW, TILES, KS>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) return -1; \
            raised = true;                                                                                                            \
        }                                                                                                                             \
        a.items = items + LM_ITEM_INTS * (size_t)(first);                                                                             \
        const size_t lds = sizeof(bf16_t) * 16 * TILES * (size_t)(C + R + 8) + sizeof(float) * (2 * 16 * TILES * LW_LDW + 2 * 4 * 16 * TILES); \
        hipLaunchKernelGGL((latent_attention_tiles_kernel<DPW, TILES, KS>), dim3(count), dim3(256), lds, stream, a);                 \
    }
    if (n_tile_items > 0) {      // the list's first items: four column tiles each, a workgroup of four waves
        llmx_note_launch(LK_LATENT_ATTENTION_TILES);
        if (C <= 64) LLMX_LT(1, 4, 6, n_tile_items, 0)
        else if (C <= 128) LLMX_LT(2, 4, 6, n_tile_items, 0)
        else if (C <= 256) LLMX_LT(4, 4, 6, n_tile_items, 0)
        else LLMX_LT(8, 4, 6, n_tile_items, 0)
    }
    if (n_row_items > 0) {       // then the decoded rows' items: one column tile, a workgroup of four waves
        llmx_note_launch(LK_LATENT_ATTENTION_ROWS);
        if (C <= 64) LLMX_LT(1, 1, 18, n_row_items, n_tile_items)
        else if (C <= 128) LLMX_LT(2, 1, 18, n_row_items, n_tile_items)
        else if (C <= 256) LLMX_LT(4, 1, 18, n_row_items, n_tile_items)
        else LLMX_LT(8, 1, 18, n_row_items, n_tile_items)
    }
#undef LLMX_LT
    if (n_items > 0) {
        llmx_note_launch(LK_LATENT_ATTENTION_MFMA);
        a.items = items + LM_ITEM_INTS * (size_t)(n_tile_items + n_row_items);
        const size_t lds = sizeof(bf16_t) * 16 * (size_t)(C + R + 8);
        const dim3 grid(n_items), block(64);
        if (C <= 64) hipLaunchKernelGGL(latent_attention_mfma_kernel<4>, grid, block, lds, stream, a);
        else if (C <= 128) hipLaunchKernelGGL(latent_attention_mfma_kernel<8>, grid, block, lds, stream, a);
        else if (C <= 256) hipLaunchKernelGGL(latent_attention_mfma_kernel<16>, grid, block, lds, stream, a);
        else hipLaunchKernelGGL(latent_attention_mfma_kernel<32>, grid, block, lds, stream, a);
    }
    if (n_merges > 0) {
        llmx_note_launch(LK_LATENT_ATTENTION_MERGE);
        hipLaunchKernelGGL(latent_attention_merge_kernel, dim3(n_merges, 16), dim3(256), 0, stream, merges, part_o, part_ml, (bf16_t*)out, T, C);
    }
    return LLMX_CHECK_LAUNCH();
}
