// Latent attention on the matrix cores (bfloat16): the attention of latent.hip for steps whose sizes the 16x16x32
// instruction takes (latent C a multiple of 16 up to 512, C + R a multiple of 32, pages of a multiple of 8 tokens).
//
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
    const int* items;       // [n_items, 4]: row0, rows, head0, heads
    bf16_t* out;            // [H, T, C]
    float scale;
    int T, H, C, R, page_tokens, max_blocks;
};

#define LM_SEG 64

template <int CT>
__global__ void __launch_bounds__(64) latent_attention_mfma_kernel(LatentMfmaArgs a) {
    extern __shared__ __align__(16) bf16_t qs[];   // [16][C + R + 8]
    const int lane = threadIdx.x, col = lane & 15, g = lane >> 4;
    const int* item = a.items + 4 * (size_t)blockIdx.x;
    const int row0 = item[0], rows = item[1], head0 = item[2], heads = item[3];
    const int C = a.C, R = a.R, CR = C + R, ldq = CR + 8, pt = a.page_tokens;
    const int n_cols = rows * heads;

    // the columns' queries into LDS, 16 bytes a lane and turn; columns without a (row, head) hold zeros
    for (int c = 0; c < 16; ++c) {
        const bool in = c < n_cols;
        const int r = row0 + (in ? c / heads : 0), h = head0 + (in ? c % heads : 0);
        const bf16_t* ql = a.q_lat + ((size_t)h * a.T + r) * C;
        const bf16_t* qr = a.q_rot + ((size_t)h * a.T + r) * R;
        for (int d = 8 * lane; d < CR; d += 8 * 64) {
            uint4 v = uint4{0, 0, 0, 0};
            if (in) v = d < C ? *reinterpret_cast<const uint4*>(ql + d) : *reinterpret_cast<const uint4*>(qr + (d - C));
            *reinterpret_cast<uint4*>(qs + c * ldq + d) = v;
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

    f32x4_t o[CT];
#pragma unroll
    for (int dt = 0; dt < CT; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float m = -INFINITY, l = 0.0f;

    for (int seg0 = 0; seg0 <= p_max; seg0 += LM_SEG) {
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
        for (int st = 0; st < steps; ++st) {
            const bf16x8_t qf = *reinterpret_cast<const bf16x8_t*>(qs + col * ldq + 32 * st + 8 * g);
            bf16x8_t kf[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) kf[v] = *reinterpret_cast<const bf16x8_t*>(kp[v] + 32 * st);
#pragma unroll
            for (int v = 0; v < 4; ++v) s[v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[v], qf, s[v], 0, 0, 0);
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
        const float m_new = fmaxf(m, top);           // finite from the first segment on: key 0 counts for every column
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
            for (int dt = 0; dt < CT; ++dt) {
                if (16 * dt < C) {
                    const bf16x8_t vf = *reinterpret_cast<const bf16x8_t*>(vp + (size_t)16 * dt * pt);
                    o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[c], o[dt], 0, 0, 0);
                }
            }
        }
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

extern "C" int llmx_latent_attention_mfma_ok(int C, int R, int page_tokens) {
    return C >= 16 && C <= 512 && C % 16 == 0 && R >= 0 && R % 8 == 0 && (C + R) % 32 == 0 && page_tokens > 0 && page_tokens % 8 == 0 ? 1 : 0;
}

extern "C" int llmx_latent_attention_mfma(const void* q_lat, const void* q_rot, const void* cache, const void* cache_t, const int* pos,
                                          const int* row_entry, const int* tables, const int* items, int n_items, void* out, float scale, int T,
                                          int H, int C, int R, int page_tokens, int max_blocks, hipStream_t stream) {
    if (n_items <= 0) return 0;
    if (!llmx_latent_attention_mfma_ok(C, R, page_tokens)) return -2;
    llmx_note_launch(LK_LATENT_ATTENTION_MFMA);
    LatentMfmaArgs a{(const bf16_t*)q_lat, (const bf16_t*)q_rot, (const bf16_t*)cache, (const bf16_t*)cache_t, pos, row_entry, tables, items,
                     (bf16_t*)out, scale, T, H, C, R, page_tokens, max_blocks};
    const size_t lds = sizeof(bf16_t) * 16 * (size_t)(C + R + 8);
    const dim3 grid(n_items), block(64);
    if (C <= 64) hipLaunchKernelGGL(latent_attention_mfma_kernel<4>, grid, block, lds, stream, a);
    else if (C <= 128) hipLaunchKernelGGL(latent_attention_mfma_kernel<8>, grid, block, lds, stream, a);
    else if (C <= 256) hipLaunchKernelGGL(latent_attention_mfma_kernel<16>, grid, block, lds, stream, a);
    else hipLaunchKernelGGL(latent_attention_mfma_kernel<32>, grid, block, lds, stream, a);
    return LLMX_CHECK_LAUNCH();
}
