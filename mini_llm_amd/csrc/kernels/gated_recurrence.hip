// A gated linear recurrence whose forget gate also decides what is written (HGRN2), for gfx950. Per head
// with d key channels and dv value channels, token by token:
//   f_i = l_i + (1 - l_i) sigmoid(fraw_i + b_i)      (a lower bound l per channel)
//   S[i, e] <- f_i S[i, e] + (1 - f_i) v_e;   o_e = sum_i S[i, e] silu(qraw_i)
// The state S ([head][d][dv], dv contiguous, fp32) lives in a per-request slot and is carried from step to
// step. Gates, state and sums are fp32; the inputs are the fp32 rows of the input projection.
//
// One wavefront per (sequence, head, 64 value columns, slice of GR_ROWS key channels): a lane owns one value
// column and keeps its slice of the state in registers; the gate and the query of a slice's channel are the
// same for all lanes, so lane i works them out for channel i and they go round through LDS. The sum over the
// key channels is split over the slices: slice s leaves its share in y + s * part_stride, and the reader (the
// norm that follows) adds the shares in the order of s.
#include "common.h"

#define GR_ROWS 32

namespace {

__device__ __forceinline__ float gr_sigmoid(float v) { return 1.f / (1.f + expf(-v)); }

// MODE 0: every portion of the step is one chunk: from the slot's state, results to y, the state back to the slot.
// Portions longer than GR_CHUNK tokens are cut into chunks that run side by side, in three launches:
// MODE 1: every chunk from a zero state; it leaves its last state and the product of its gates in the workspace;
//         then hgrn2_chunk_states_kernel walks a sequence's chunks in order, S <- F_c S + L_c, leaves in the
//         workspace the state each chunk starts from, and writes the last state to the slot;
// MODE 2: every chunk again, from the state it starts from, results to y.
// The sums are those of the token-by-token recurrence in another order.
// Workspace per chunk and head: [d * dv] the chunk's state, then [d] the product of its gates.
#define GR_CHUNK 32

template <int MODE>
__global__ void __launch_bounds__(64)
hgrn2_scan_kernel(const float* __restrict__ proj, int ld, int q_col, int f_col, int v_col, const float* __restrict__ f_bias,
                  const float* __restrict__ lower, const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                  float* __restrict__ state, size_t slot_floats, float* __restrict__ y, int ldy, size_t part_stride, int H, int d,
                  int dv, int n_tiles, int n_slices, int write, int n_seqs, float* __restrict__ ws) {
    __shared__ float fq[2][2 * GR_ROWS];        // per token in turn: [f | q] of the slice's channels
    const int lane = threadIdx.x;
    int w = blockIdx.x;
    const int slice = w % n_slices; w /= n_slices;
    const int tile = w % n_tiles; w /= n_tiles;
    const int h = w % H;
    w /= H;
    int b, first, n, chunk_id = 0;
    if (MODE == 0) {
        b = w;
        first = cu_q[b];
        n = cu_q[b + 1] - first;
    } else {
        // which sequence and which of its chunks
        chunk_id = w;
        int c = w;
        for (b = 0; b < n_seqs; ++b) {
            first = cu_q[b];
            n = cu_q[b + 1] - first;
            const int nc = (n + GR_CHUNK - 1) / GR_CHUNK;
            if (c < nc) break;
            c -= nc;
        }
        if (b >= n_seqs) return;                // a surplus workgroup
        first += c * GR_CHUNK;
        n = min(GR_CHUNK, n - c * GR_CHUNK);
    }
    const int slot = state_slots[b];
    if (slot < 0) return;
    const int e = tile * 64 + lane, i0 = slice * GR_ROWS;
    const int rows = min(GR_ROWS, d - i0);
    const bool col_ok = e < dv;
    float* S = state + static_cast<size_t>(slot) * slot_floats + (static_cast<size_t>(h) * d + i0) * dv + (col_ok ? e : 0);
    float* W = ws ? ws + (static_cast<size_t>(chunk_id) * H + h) * (static_cast<size_t>(d) * dv + d) : nullptr;
    float* WS = W ? W + static_cast<size_t>(i0) * dv + (col_ok ? e : 0) : nullptr;
    float s[GR_ROWS];
#pragma unroll
    for (int i = 0; i < GR_ROWS; ++i) {
        // (the start: the slot's state, zero, or what the pass over the chunks left for this chunk)
        const float* from = MODE == 2 ? WS : S;
        s[i] = (MODE != 1 && i < rows && col_ok) ? from[static_cast<size_t>(i) * dv] : 0.f;
    }
    // the channel this lane prepares: lanes 0..31 the gate of channel lane, lanes 32..63 the query of channel lane - 32
    const int ch = lane % GR_ROWS;
    const bool ch_ok = ch < rows;
    const int c = h * d + i0 + (ch_ok ? ch : 0);
    const float lo = lower[c], fb = f_bias ? f_bias[c] : 0.f;
    float cum = 1.f;                            // (lanes 0..31) the product of the channel's gates over the chunk
    // A token's inputs are asked for one token ahead (from a clamped, always valid row), so that the round trip to
    // memory runs beside the arithmetic of the token before.
    const int col = lane < GR_ROWS ? f_col + c : q_col + c;
    const int vcol = v_col + h * dv + (col_ok ? e : 0);
    float raw = 0.f, v_next = 0.f;
    if (n > 0) {
        raw = proj[static_cast<size_t>(first) * ld + col];
        v_next = proj[static_cast<size_t>(first) * ld + vcol];
    }
    for (int k = 0; k < n; ++k) {
        const float z = raw, v = col_ok ? v_next : 0.f;
        const float* ahead = proj + static_cast<size_t>(first + min(k + 1, n - 1)) * ld;
        raw = ahead[col];
        v_next = ahead[vcol];
        float val;
        if (lane < GR_ROWS) { val = lo + (1.f - lo) * gr_sigmoid(z + fb); cum *= val; }
        else val = z * gr_sigmoid(z);
        float* cur = fq[k & 1];
        cur[lane] = ch_ok ? val : 0.f;
        wave_lds_sync();
        float o = 0.f;
#pragma unroll
        for (int i = 0; i < GR_ROWS; ++i) {
            const float f = cur[i], qi = cur[GR_ROWS + i];
            s[i] = f * s[i] + (1.f - f) * v;
            o = fmaf(s[i], qi, o);
        }
        if (MODE != 1 && col_ok) y[slice * part_stride + static_cast<size_t>(first + k) * ldy + h * dv + e] = o;
    }
    if (MODE == 0 && write && col_ok) {
#pragma unroll
        for (int i = 0; i < GR_ROWS; ++i)
            if (i < rows) S[static_cast<size_t>(i) * dv] = s[i];
    }
    if (MODE == 1) {
        if (col_ok) {
#pragma unroll
            for (int i = 0; i < GR_ROWS; ++i)
                if (i < rows) WS[static_cast<size_t>(i) * dv] = s[i];
        }
        if (tile == 0 && lane < GR_ROWS && ch_ok) W[static_cast<size_t>(d) * dv + i0 + ch] = cum;
    }
}

// One thread per (sequence, head, key channel, value column): the sequence's chunks in order. In the workspace a
// chunk's own last state is replaced by the state it starts from.
__global__ void hgrn2_chunk_states_kernel(const int* __restrict__ cu_q, const int* __restrict__ state_slots, float* __restrict__ state,
                                          size_t slot_floats, float* __restrict__ ws, int H, int d, int dv, int n_seqs, int write) {
    const long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    const long long per_seq = static_cast<long long>(H) * d * dv;
    if (idx >= per_seq * n_seqs) return;
    const int b = static_cast<int>(idx / per_seq);
    const long long r = idx % per_seq;
    const int h = static_cast<int>(r / (static_cast<long long>(d) * dv)), i = static_cast<int>(r / dv % d);
    const int slot = state_slots[b];
    if (slot < 0) return;
    int chunk0 = 0;
    for (int bb = 0; bb < b; ++bb) chunk0 += (cu_q[bb + 1] - cu_q[bb] + GR_CHUNK - 1) / GR_CHUNK;
    const int nc = (cu_q[b + 1] - cu_q[b] + GR_CHUNK - 1) / GR_CHUNK;
    float* sp = state + static_cast<size_t>(slot) * slot_floats + r;
    float S = *sp;
    const size_t per_chunk = static_cast<size_t>(d) * dv + d;
    for (int c = 0; c < nc; ++c) {
        float* W = ws + (static_cast<size_t>(chunk0 + c) * H + h) * per_chunk;
        const float L = W[r % (static_cast<long long>(d) * dv)], F = W[static_cast<size_t>(d) * dv + i];
        W[r % (static_cast<long long>(d) * dv)] = S;
        S = F * S + L;
    }
    if (write) *sp = S;
}

// out[t, :] = [a[t, :] | b[t, :]] in the output's dtype (two fp32 streams side by side, as one product's input)
template <typename T>
__global__ void concat_cast_kernel(const float* __restrict__ a, const float* __restrict__ b, int D, T* __restrict__ out, long long total) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / (2 * D);
    const int c = static_cast<int>(i % (2 * D));
    out[i] = from_float<T>(c < D ? a[t * D + c] : b[t * D + c - D]);
}

// out[t, j] = act(gu[t, j]) * gu[t, F + j]: the two halves of a joined gate/up product
template <typename T>
__global__ void glu_act_kernel(const T* __restrict__ gu, int ld, int F, T* __restrict__ out, int ldo, long long total) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / F;
    const int j = static_cast<int>(i % F);
    const float g = to_float(gu[t * ld + j]), u = to_float(gu[t * ld + F + j]);
    out[t * ldo + j] = from_float<T>((sizeof(T) == 4 ? gelu_tanh_precise(g) : gelu_tanh(g)) * u);
}

}  // namespace

extern "C" {

int mllm_hgrn2_parts(int d) { return (d + GR_ROWS - 1) / GR_ROWS; }

// proj [T, ld] fp32 holds, per token, the raw queries (H * d from q_col), raw gates (H * d from f_col) and values
// (H * dv from v_col). y: mllm_hgrn2_parts(d) shares of [T, ldy], part_stride floats apart. The state of a
// request lies state_offset floats into its slot.
int mllm_hgrn2_scan(const float* proj, int ld, int q_col, int f_col, int v_col, const float* f_bias, const float* lower,
                    const int* cu_q, const int* state_slots, float* state, size_t slot_floats, size_t state_offset, float* y, int ldy,
                    size_t part_stride, int T, int B, int max_q_len, int H, int d, int dv, int write, float* workspace,
                    hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    if (H < 1 || d < 1 || dv < 1 || lower == nullptr) return -1;
    const int n_tiles = (dv + 63) / 64, n_slices = (d + GR_ROWS - 1) / GR_ROWS;
    const long long per = static_cast<long long>(H) * n_tiles * n_slices;
    if (max_q_len <= GR_CHUNK || workspace == nullptr) {
        if (per * B >= (1ll << 31)) return -1;
        hgrn2_scan_kernel<0><<<static_cast<int>(per * B), 64, 0, stream>>>(proj, ld, q_col, f_col, v_col, f_bias, lower, cu_q, state_slots,
                                                                          state + state_offset, slot_floats, y, ldy, part_stride, H, d, dv,
                                                                          n_tiles, n_slices, write, B, nullptr);
        MLLM_LAUNCH_CHECK();
        return 0;
    }
    const long long chunks = T / GR_CHUNK + B;          // an upper bound; surplus workgroups leave at once
    if (per * chunks >= (1ll << 31)) return -1;
    hgrn2_scan_kernel<1><<<static_cast<int>(per * chunks), 64, 0, stream>>>(proj, ld, q_col, f_col, v_col, f_bias, lower, cu_q, state_slots,
                                                                           state + state_offset, slot_floats, y, ldy, part_stride, H, d, dv,
                                                                           n_tiles, n_slices, write, B, workspace);
    MLLM_LAUNCH_CHECK();
    const long long cells = static_cast<long long>(B) * H * d * dv;
    hgrn2_chunk_states_kernel<<<static_cast<int>((cells + 255) / 256), 256, 0, stream>>>(cu_q, state_slots, state + state_offset, slot_floats,
                                                                                        workspace, H, d, dv, B, write);
    MLLM_LAUNCH_CHECK();
    hgrn2_scan_kernel<2><<<static_cast<int>(per * chunks), 64, 0, stream>>>(proj, ld, q_col, f_col, v_col, f_bias, lower, cu_q, state_slots,
                                                                           state + state_offset, slot_floats, y, ldy, part_stride, H, d, dv,
                                                                           n_tiles, n_slices, write, B, workspace);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// Floats of workspace that a step of T tokens in B sequences needs when its longest portion exceeds a chunk.
size_t mllm_hgrn2_workspace_floats(int T, int B, int H, int d, int dv) {
    return static_cast<size_t>(T / GR_CHUNK + B) * H * (static_cast<size_t>(d) * dv + d);
}
int mllm_hgrn2_chunk() { return GR_CHUNK; }

int mllm_concat_cast(const float* a, const float* b, int T, int D, void* out, int dtype, hipStream_t stream) {
    if (T <= 0 || D <= 0) return 0;
    const long long total = static_cast<long long>(T) * 2 * D;
    const int blocks = static_cast<int>((total + 255) / 256);
    if (dtype == MLLM_F32) concat_cast_kernel<float><<<blocks, 256, 0, stream>>>(a, b, D, static_cast<float*>(out), total);
    else concat_cast_kernel<bf16_t><<<blocks, 256, 0, stream>>>(a, b, D, static_cast<bf16_t*>(out), total);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// -1: an activation other than the tanh form of GELU (code 1)
int mllm_glu_act(const void* gu, int ld, int T, int F, int act, void* out, int ldo, int dtype, hipStream_t stream) {
    if (T <= 0 || F <= 0) return 0;
    if (act != EPI_GELU_TANH) return -1;
    const long long total = static_cast<long long>(T) * F;
    const int blocks = static_cast<int>((total + 255) / 256);
    if (dtype == MLLM_F32) glu_act_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<const float*>(gu), ld, F, static_cast<float*>(out), ldo, total);
    else glu_act_kernel<bf16_t><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(gu), ld, F, static_cast<bf16_t*>(out), ldo, total);
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
