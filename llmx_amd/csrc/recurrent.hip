// Gated element-wise recurrences over the rows of a step, with a float32 state a request in state slots.
//
// minGRU form: for channel c of a request's rows t = 0 .. n-1 (in position order)
//     z = sigmoid(a[t,c] + bz[c]),  u = b[t,c] + bx[c],  cand = u >= 0 ? u + 1/2 : sigmoid(u),
//     S = (1 - z) * S + z * cand,   out[t,c] = S * silu(g[t,c]),
// where a | b | g are the three thirds of a row of `zxg` (the pre-activations of the gate, the candidate and the output
// gate, float32).  S starts from the request's state slot `slot_read` and ends in `slot_write` (they may be the same):
// a step that computes into a second slot needs no copy of the state first.  One thread owns a channel of a request and
// walks its rows in order, so the state after a row is the same bits however the rows were cut into steps.
#include "common.h"

struct ScanArgs {
    const float* zxg;        // [T, 3W]
    const float* bz;         // [W] or null
    const float* bx;         // [W] or null
    float* state;            // [slots, W]
    const int* slot_read;    // [n_entries]
    const int* slot_write;   // [n_entries]
    const int* entry_rows;   // [n_entries, 2]: first row, rows
    void* out;               // [T, W] in the activation type
    int W;
};

__device__ __forceinline__ float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }

#define SCAN_AHEAD 8
template <typename TO>
__global__ void __launch_bounds__(64) mingru_scan_kernel(ScanArgs a) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    const int e = blockIdx.y;
    if (c >= a.W) return;
    const int row0 = a.entry_rows[2 * e], n = a.entry_rows[2 * e + 1];
    const float bz = a.bz ? a.bz[c] : 0.0f, bx = a.bx ? a.bx[c] : 0.0f;
    float S = a.state[(size_t)a.slot_read[e] * a.W + c];
    const size_t ld = 3 * (size_t)a.W;
    TO* out = (TO*)a.out;
    for (int t0 = 0; t0 < n; t0 += SCAN_AHEAD) {
        float za[SCAN_AHEAD], ua[SCAN_AHEAD], ga[SCAN_AHEAD];
        // a round's loads are asked for together; the chain below then runs without waiting for memory
#pragma unroll
        for (int k = 0; k < SCAN_AHEAD; ++k) {
            const int t = t0 + k < n ? t0 + k : n - 1;
            const float* row = a.zxg + (size_t)(row0 + t) * ld;
            za[k] = row[c];
            ua[k] = row[a.W + c];
            ga[k] = row[2 * a.W + c];
        }
#pragma unroll
        for (int k = 0; k < SCAN_AHEAD; ++k) {
            if (t0 + k < n) {
                const float z = sigmoid_f(za[k] + bz);
                const float u = ua[k] + bx;
                const float cand = u >= 0.0f ? u + 0.5f : sigmoid_f(u);
                S = (1.0f - z) * S + z * cand;
                const float g = ga[k];
                st(out + (size_t)(row0 + t0 + k) * a.W + c, S * (g * sigmoid_f(g)));
            }
        }
    }
    a.state[(size_t)a.slot_write[e] * a.W + c] = S;
}

extern "C" int llmx_mingru_scan(const float* zxg, const float* bz, const float* bx, float* state, const int* slot_read, const int* slot_write,
                                const int* entry_rows, void* out, int out_dtype, int n_entries, int W, hipStream_t stream) {
    if (n_entries <= 0 || W <= 0) return 0;
    llmx_note_launch(LK_GATED_SCAN);
    ScanArgs a{zxg, bz, bx, state, slot_read, slot_write, entry_rows, out, W};
    const dim3 grid((W + 63) / 64, n_entries);
    if (out_dtype == LLMX_F32) hipLaunchKernelGGL(mingru_scan_kernel<float>, grid, dim3(64), 0, stream, a);
    else hipLaunchKernelGGL(mingru_scan_kernel<bf16_t>, grid, dim3(64), 0, stream, a);
    return LLMX_CHECK_LAUNCH();
}
