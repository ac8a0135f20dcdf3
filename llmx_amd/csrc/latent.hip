// Latent attention: the cache keeps, for every token, one latent vector of C values (shared by all heads, RMS-normed)
// followed by one rotated key part of R values.  A head's key for a token is [W_uk_h c | k_rot] and its value W_uv_h c;
// neither is ever formed: the query's unrotated part is taken through W_uk_h^T first (q_lat = W_uk_h^T q_plain, C values),
// so that score = (q_lat . c + q_rot . k_rot) * scale, and the weighted sum of latents goes through W_uv_h afterwards.
// Both products with W_uk / W_uv are grouped products (one group a head) outside this file; here are the step before
// them (norm, rotation, cache write, queries laid out head by head), the attention over the paged latents, and the
// per-head output gate.
//
// Layouts: proj [T, ldp] float32 holds q (H heads of [D unrotated | R rotated]) at column 0 and [C latent | R key part]
// at column q_width; cache [pages, page_tokens, C + R]; q_plain [H, T, D], q_rot [H, T, R], q_lat and the attention's
// result [H, T, C] (head-major, so that a head's rows are one group of the grouped products).
#include "common.h"

struct LatentPrepArgs {
    const float* proj;
    const float* norm_w;    // [C]
    const float* cos_sin;   // [positions, dims]: cos of the dims/2 pairs, then sin (any magnitude factor already inside)
    const int* pos;
    const int* row_entry;
    const int* tables;
    void* q_plain;
    void* q_rot;
    void* cache;
    void* cache_t;          // null, or a second copy of the latents [pages, C, page_tokens] (transposed within the page)
    float eps;
    int T, ldp, H, D, R, C, dims, page_tokens, max_blocks, write_cache;
};

// Element r of a rotated part `part` (R values, the first `dims` of them rotated as interleaved pairs (2i, 2i+1) by the
// angle of frequency i): (u, v) -> (u cos - v sin, v cos + u sin).
__device__ __forceinline__ float rotated_interleaved(const float* __restrict__ part, const float* __restrict__ cs, int r, int dims) {
    const float x = part[r];
    if (r >= dims) return x;
    const bool first = (r & 1) == 0;
    const float y = part[first ? r + 1 : r - 1];
    const float c = cs[r >> 1], s = cs[dims / 2 + (r >> 1)];
    return first ? fmaf(-y, s, x * c) : fmaf(y, s, x * c);
}

template <typename TQ, typename TC>
__global__ void __launch_bounds__(256) latent_prep_kernel(LatentPrepArgs a) {
    __shared__ float scratch[4];
    const int t = blockIdx.x;
    const float* row = a.proj + (size_t)t * a.ldp;
    const int p = a.pos[t];
    const float* cs = a.cos_sin + (size_t)p * a.dims;
    const int DR = a.D + a.R;
    if (blockIdx.y == 0) {
        TQ* qp = (TQ*)a.q_plain;
        TQ* qr = (TQ*)a.q_rot;
        int h = threadIdx.x / DR, d = threadIdx.x % DR;
        const int step_h = 256 / DR, step_d = 256 % DR;
        for (int i = threadIdx.x; i < a.H * DR; i += 256) {
            if (d < a.D) st(qp + ((size_t)h * a.T + t) * a.D + d, row[i]);
            else st(qr + ((size_t)h * a.T + t) * a.R + (d - a.D), rotated_interleaved(row + h * DR + a.D, cs, d - a.D, a.dims));
            h += step_h;
            d += step_d;
            if (d >= DR) {
                d -= DR;
                ++h;
            }
        }
        return;
    }
    if (!a.write_cache) return;
    const float* lat = row + a.H * DR;
    const float s = block_sum<4>(strided_squares<256>(lat, a.C), scratch);
    const float r = 1.0f / sqrtf(s / (float)a.C + a.eps);
    const int page = a.tables[(size_t)a.row_entry[t] * a.max_blocks + p / a.page_tokens];
    TC* out = (TC*)a.cache + ((size_t)page * a.page_tokens + p % a.page_tokens) * (a.C + a.R);
    TC* out_t = a.cache_t ? (TC*)a.cache_t + (size_t)page * a.C * a.page_tokens + p % a.page_tokens : nullptr;
    for (int i = threadIdx.x; i < a.C; i += 256) {
        const float c = lat[i] * (r * a.norm_w[i]);
        st(out + i, c);
        if (out_t) st(out_t + (size_t)i * a.page_tokens, c);
    }
    for (int i = threadIdx.x; i < a.R; i += 256) st(out + a.C + i, rotated_interleaved(lat + a.C, cs, i, a.dims));
}

extern "C" int llmx_latent_prep(const float* proj, const float* norm_w, const float* cos_sin, const int* pos, const int* row_entry,
                                const int* tables, void* q_plain, void* q_rot, void* cache, void* cache_t, int dtype, float eps, int T, int ldp, int H, int D,
                                int R, int C, int dims, int page_tokens, int max_blocks, int write_cache, hipStream_t stream) {
    if (T <= 0) return 0;
    if (dims % 2 || dims > R || D + R <= 0 || C <= 0 || H * (D + R) + C + R > ldp) return -2;
    llmx_note_launch(LK_LATENT_PREP);
    LatentPrepArgs a{proj, norm_w, cos_sin, pos, row_entry, tables, q_plain, q_rot, cache, cache_t, eps, T, ldp, H, D, R, C, dims, page_tokens, max_blocks, write_cache};
    if (dtype == LLMX_F32) hipLaunchKernelGGL((latent_prep_kernel<float, float>), dim3(T, 2), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((latent_prep_kernel<bf16_t, bf16_t>), dim3(T, 2), dim3(256), 0, stream, a);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// The universal kernel: one wave per (row, head).  Keys lo..p of the row's request are walked in tiles of 64 absolute
// positions with an online softmax; lane j of a tile forms the score of key 64*tile + j, for the weighted sum lane d
// owns latent dims d, d + 64, ... and walks the tile's keys in order.  A row's arithmetic depends on its own position
// and request only.  Any sizes with C <= 2048 and C + R <= 4096, float32 or bfloat16.
struct LatentAttnArgs {
    const void* q_lat;   // [H, T, C]
    const void* q_rot;   // [H, T, R]
    const void* cache;   // [pages, page_tokens, C + R]
    const int* pos;
    const int* row_entry;
    const int* tables;
    void* out;           // [H, T, C]
    float scale;
    int T, H, C, R, page_tokens, max_blocks, window;
};

#define LAT_MAX_C 2048
#define LAT_MAX_CR 4096

template <typename T>
__global__ void __launch_bounds__(64) latent_attention_generic_kernel(LatentAttnArgs a) {
    __shared__ float qs[LAT_MAX_CR];
    __shared__ float ps[64];
    __shared__ int row_at[64];   // page * page_tokens + slot of each key of the tile
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int C = a.C, R = a.R, CR = C + R;
    const int p = a.pos[t];
    const int* table = a.tables + (size_t)a.row_entry[t] * a.max_blocks;
    const T* ql = (const T*)a.q_lat + ((size_t)h * a.T + t) * C;
    const T* qr = (const T*)a.q_rot + ((size_t)h * a.T + t) * R;
    const T* cache = (const T*)a.cache;
    for (int d = lane; d < C; d += 64) qs[d] = ld(ql + d);
    for (int d = lane; d < R; d += 64) qs[C + d] = ld(qr + d);
    __syncthreads();

    int lo = (a.window > 0 && p - a.window + 1 > 0) ? p - a.window + 1 : 0;
    float m = -INFINITY, l = 0.0f;
    float acc[LAT_MAX_C / 64];
#pragma unroll
    for (int i = 0; i < LAT_MAX_C / 64; ++i) acc[i] = 0.0f;

    for (int j0 = (lo / 64) * 64; j0 <= p; j0 += 64) {
        const int j = j0 + lane;
        const bool seen = j >= lo && j <= p;
        float s = -INFINITY;
        int at = 0;
        if (seen) {
            at = table[j / a.page_tokens] * a.page_tokens + j % a.page_tokens;
            const T* key = cache + (size_t)at * CR;
            float dot = 0.0f;
            for (int d = 0; d < CR; ++d) dot = fmaf(qs[d], ld(key + d), dot);
            s = dot * a.scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float w = seen ? expf(s - m_new) : 0.0f;
        const float correction = expf(m - m_new);   // 0 on the first tile (m = -inf)
        ps[lane] = w;
        row_at[lane] = at;
        __syncthreads();
        const int n = min(64, p - j0 + 1);
        float tile_sum = 0.0f;
        for (int i = 0; i < n; ++i) tile_sum += ps[i];   // keys before lo hold 0
        l = l * correction + tile_sum;
#pragma unroll
        for (int i = 0; i < LAT_MAX_C / 64; ++i) {
            const int d = lane + 64 * i;
            if (d < C) {
                float v = acc[i] * correction;
                for (int jj = 0; jj < n; ++jj) v = fmaf(ps[jj], ld(cache + (size_t)row_at[jj] * CR + d), v);
                acc[i] = v;
            }
        }
        m = m_new;
        __syncthreads();
    }
    T* out = (T*)a.out + ((size_t)h * a.T + t) * C;
#pragma unroll
    for (int i = 0; i < LAT_MAX_C / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < C) st(out + d, acc[i] / l);
    }
}

extern "C" int llmx_latent_attention_generic(const void* q_lat, const void* q_rot, const void* cache, const int* pos, const int* row_entry,
                                             const int* tables, void* out, int dtype, float scale, int T, int H, int C, int R, int page_tokens,
                                             int max_blocks, int window, hipStream_t stream) {
    if (T <= 0 || H <= 0) return 0;
    if (C <= 0 || C > LAT_MAX_C || R < 0 || C + R > LAT_MAX_CR) return -2;
    llmx_note_launch(LK_LATENT_ATTENTION_GENERIC);
    LatentAttnArgs a{q_lat, q_rot, cache, pos, row_entry, tables, out, scale, T, H, C, R, page_tokens, max_blocks, window};
    if (dtype == LLMX_F32) hipLaunchKernelGGL(latent_attention_generic_kernel<float>, dim3(T, H), dim3(64), 0, stream, a);
    else hipLaunchKernelGGL(latent_attention_generic_kernel<bf16_t>, dim3(T, H), dim3(64), 0, stream, a);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// Per-head output gate and the change of layout before the output projection:
// out[t, h*V + d] = sigmoid(gate[t*ldg + h]) * values[h, t, d], values float32 [H, T, V], out in the activation type.
template <typename TO>
__global__ void __launch_bounds__(256) head_gate_kernel(const float* __restrict__ values, const float* __restrict__ gate, int ldg,
                                                      TO* __restrict__ out, int T, int H, int V) {
    const int t = blockIdx.x;
    int h = threadIdx.x / V, d = threadIdx.x % V;
    const int step_h = 256 / V, step_d = 256 % V;
    for (int i = threadIdx.x; i < H * V; i += 256) {
        const float g = gate ? 1.0f / (1.0f + expf(-gate[(size_t)t * ldg + h])) : 1.0f;
        st(out + (size_t)t * H * V + i, g * values[((size_t)h * T + t) * V + d]);
        h += step_h;
        d += step_d;
        if (d >= V) {
            d -= V;
            ++h;
        }
    }
}

extern "C" int llmx_head_gate(const float* values, const float* gate, int ldg, void* out, int out_dtype, int T, int H, int V, hipStream_t stream) {
    if (T <= 0 || H <= 0 || V <= 0) return 0;
    llmx_note_launch(LK_HEAD_GATE);
    if (out_dtype == LLMX_F32) hipLaunchKernelGGL(head_gate_kernel<float>, dim3(T), dim3(256), 0, stream, values, gate, ldg, (float*)out, T, H, V);
    else hipLaunchKernelGGL(head_gate_kernel<bf16_t>, dim3(T), dim3(256), 0, stream, values, gate, ldg, (bf16_t*)out, T, H, V);
    return LLMX_CHECK_LAUNCH();
}
