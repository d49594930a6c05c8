// State-space mixer kernels for gfx950: the short causal convolution with its carried inputs, and the
// selective scan (Mamba-2 form: one decay per head and token) over a step's portions, the state carried
// in a per-request slot. Everything here is fp32.
//
// A request's slot holds [taps - 1][channels] convolution inputs (oldest first), then the scan's state
// laid out [head][p][n] (n contiguous).
#include <algorithm>

#include "common.h"

namespace {

__device__ __forceinline__ float silu_precise(float v) { return v / (1.f + expf(-v)); }
// log(1 + exp(v)) without overflow, no clamp
__device__ __forceinline__ float softplus_precise(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// out[t, ch] = silu(bias[ch] + sum_j w[ch, j] * in(t - (taps - 1 - j), ch)): inputs before the portion come
// from the slot's carried rows (zeros for a fresh request: the slot was cleared). One thread per (t, ch).
__global__ void conv_silu_kernel(const float* __restrict__ proj, int ld, int col0, int C, const float* __restrict__ w,
                                 const float* __restrict__ bias, int taps, const int* __restrict__ token_seq,
                                 const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                                 const float* __restrict__ state, size_t slot_floats, float* __restrict__ out, int ldo,
                                 long long total) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = static_cast<int>(i / C), ch = static_cast<int>(i % C);
    const int b = token_seq[t], slot = state_slots[b];
    if (slot < 0) return;
    const int first = cu_q[b], k = t - first;
    const float* carried = state + static_cast<size_t>(slot) * slot_floats;
    float acc = bias[ch];
    for (int j = 0; j < taps; ++j) {
        const int idx = k - (taps - 1 - j);
        const float v = idx >= 0 ? proj[static_cast<size_t>(first + idx) * ld + col0 + ch]
                                 : carried[static_cast<size_t>(taps - 1 + idx) * C + ch];
        acc += w[static_cast<size_t>(ch) * taps + j] * v;
    }
    out[static_cast<size_t>(t) * ldo + ch] = silu_precise(acc);
}

// The slot's carried rows after the portion: its last taps - 1 inputs, older ones shifted out; a portion
// shorter than that keeps the newest of the old rows. One thread per (sequence, channel); taps - 1 <= 15.
__global__ void conv_carry_kernel(const float* __restrict__ proj, int ld, int col0, int C, int taps,
                                  const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                                  float* __restrict__ state, size_t slot_floats, int B) {
    const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= static_cast<long long>(B) * C) return;
    const int b = static_cast<int>(i / C), ch = static_cast<int>(i % C);
    const int slot = state_slots[b];
    if (slot < 0) return;
    const int first = cu_q[b], n = cu_q[b + 1] - first, keep = taps - 1;
    float* carried = state + static_cast<size_t>(slot) * slot_floats;
    float fresh[15];
#pragma unroll
    for (int r = 0; r < 15; ++r) {
        if (r < keep) {
            const int idx = n - keep + r;
            fresh[r] = idx >= 0 ? proj[static_cast<size_t>(first + idx) * ld + col0 + ch]
                                : carried[static_cast<size_t>(r + n) * C + ch];
        }
    }
#pragma unroll
    for (int r = 0; r < 15; ++r)
        if (r < keep) carried[static_cast<size_t>(r) * C + ch] = fresh[r];
}

// The scan. For head h (group g = h / (H / G)) and token t, in order:
//   dt = softplus(raw_dt[t, h] + dt_bias[h]);  a = exp(-exp(A_log[h]) dt)
//   S[n, p] = a S[n, p] + dt B[t, g, n] x[t, h, p];   y[t, h, p] = sum_n S[n, p] C[t, g, n] + D[h] x[t, h, p]
// One wavefront per (chunk of a sequence's portion, head, 64 / LANES_N values of p): LANES_N consecutive
// lanes share a p and split n (lane l of the group holds n = l, l + LANES_N, ...: up to NPT of them in
// registers), so the sum over n is a sum inside the lane group and no wavefront waits for another. The next
// token's operands are requested before this token's are used. xbc rows: [x: H*P | B: G*N | C: G*N].
//
// A portion longer than `chunk` tokens is cut into chunks that are scanned side by side: the first starts
// from the slot's state, the others from zero, and each leaves its last state in `chunk_state`
// ([chunk][H][P][N]) and, per token, the logarithm of the decay accumulated since its chunk began in `cumlog`
// ([T, H]). ssm_chunk_join_kernel then adds what the earlier chunks contribute. A portion of one chunk
// (decoding) is finished here and its state goes straight back to the slot.
struct ChunkOf {
    int b, k, n_chunks, first_chunk;      // sequence, chunk within it, chunks of the sequence, where its chunks' states start
                                          // (only portions of several chunks keep states: at most 2 T / chunk of them)
};
__device__ __forceinline__ ChunkOf chunk_of(int index, const int* cu_q, int n_seqs, int chunk) {
    ChunkOf c{0, index, 0, 0};
    for (; c.b < n_seqs; ++c.b) {
        c.n_chunks = max(1, (cu_q[c.b + 1] - cu_q[c.b] + chunk - 1) / chunk);
        if (c.k < c.n_chunks) return c;
        c.k -= c.n_chunks;
        if (c.n_chunks > 1) c.first_chunk += c.n_chunks;
    }
    c.b = -1;
    return c;
}

template <int NPT, int LANES_N>
__global__ void __launch_bounds__(64)
ssm_scan_kernel(const float* __restrict__ xbc, int ldx, const float* __restrict__ raw_dt, int ldd,
                const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dskip,
                const int* __restrict__ cu_q, const int* __restrict__ state_slots, int n_seqs, float* __restrict__ state,
                size_t slot_floats, size_t scan_offset, float* __restrict__ y, int ldy, int H, int P, int N, int G,
                int write, int chunk, float* __restrict__ chunk_state, float* __restrict__ cumlog) {
    const int lane = threadIdx.x, ln = lane % LANES_N, pl = lane / LANES_N;
    const int h = blockIdx.y;
    const ChunkOf co = chunk_of(blockIdx.z, cu_q, n_seqs, chunk);
    if (co.b < 0) return;                                      // surplus workgroup
    const int slot = state_slots[co.b];
    if (slot < 0) return;
    const int p = blockIdx.x * (64 / LANES_N) + pl;
    const bool p_ok = p < P;
    const int pc = p_ok ? p : P - 1;
    const int g = h / (H / G), inner = H * P;
    const int t0 = cu_q[co.b] + co.k * chunk, t1 = min(t0 + chunk, cu_q[co.b + 1]);
    float* sp = state + static_cast<size_t>(slot) * slot_floats + scan_offset + (static_cast<size_t>(h) * P + pc) * N;
    float S[NPT];
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
        const int n = j * LANES_N + ln;
        S[j] = (co.k == 0 && n < N) ? sp[n] : 0.f;
    }
    const float bias = dt_bias[h], neg_rate = -expf(A_log[h]), skip = Dskip[h];
    const int b_col = inner + g * N, c_col = inner + G * N + g * N;
    // operands of the token at hand, and of the next one (loaded one token ahead)
    float xv = 0.f, dtr = 0.f, Bv[NPT], Cv[NPT];
    auto load = [&](int t, float& x_, float& d_, float (&B_)[NPT], float (&C_)[NPT]) {
        const float* row = xbc + static_cast<size_t>(t) * ldx;
        x_ = row[h * P + pc];
        d_ = raw_dt[static_cast<size_t>(t) * ldd + h];
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const int n = min(j * LANES_N + ln, N - 1);
            B_[j] = row[b_col + n];
            C_[j] = row[c_col + n];
        }
    };
    if (t0 < t1) load(t0, xv, dtr, Bv, Cv);
    float cum = 0.f;
    for (int t = t0; t < t1; ++t) {
        float xn = 0.f, dn = 0.f, Bn[NPT], Cn[NPT];
        const int tn = min(t + 1, t1 - 1);
        load(tn, xn, dn, Bn, Cn);
        const float dt = softplus_precise(dtr + bias);
        const float a = expf(neg_rate * dt), dx = dt * xv;
        cum += neg_rate * dt;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            if (j * LANES_N + ln < N) {
                S[j] = a * S[j] + dx * Bv[j];
                acc += S[j] * Cv[j];
            }
        }
        acc = group_sum<LANES_N>(acc);
        if (ln == 0 && p_ok) y[static_cast<size_t>(t) * ldy + h * P + p] = acc + skip * xv;
        if (co.n_chunks > 1 && blockIdx.x == 0 && lane == 0) cumlog[static_cast<size_t>(t) * H + h] = cum;
        xv = xn; dtr = dn;
#pragma unroll
        for (int j = 0; j < NPT; ++j) { Bv[j] = Bn[j]; Cv[j] = Cn[j]; }
    }
    if (!p_ok) return;
    if (co.n_chunks > 1) sp = chunk_state + ((static_cast<size_t>(co.first_chunk + co.k) * H + h) * P + p) * N;
    if (write || co.n_chunks > 1) {
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const int n = j * LANES_N + ln;
            if (n < N) sp[n] = S[j];
        }
    }
}

// What the chunks before chunk k of a portion contribute to it (see ssm_scan_kernel): with A_j the whole
// decay of chunk j and L_j its last local state, the state at the start of chunk k is
//   S = L_0 for k = 1;  S <- A_j S + L_j for j = 1 .. k - 1,
// every token t of chunk k gets  y[t] += exp(cumlog[t]) sum_n C[t, n] S[n, p], and the portion's last chunk
// writes A_k S + L_k back to the slot. Same grid and lane layout as the scan.
template <int NPT, int LANES_N>
__global__ void __launch_bounds__(64)
ssm_chunk_join_kernel(const float* __restrict__ xbc, int ldx, const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                      int n_seqs, float* __restrict__ state, size_t slot_floats, size_t scan_offset, float* __restrict__ y,
                      int ldy, int H, int P, int N, int G, int write, int chunk, const float* __restrict__ chunk_state,
                      const float* __restrict__ cumlog) {
    const int lane = threadIdx.x, ln = lane % LANES_N, pl = lane / LANES_N;
    const int h = blockIdx.y;
    const ChunkOf co = chunk_of(blockIdx.z, cu_q, n_seqs, chunk);
    if (co.b < 0 || co.k == 0) return;                         // surplus, or a first chunk: nothing comes before it
    const int slot = state_slots[co.b];
    if (slot < 0) return;
    const int p = blockIdx.x * (64 / LANES_N) + pl;
    const bool p_ok = p < P;
    const int pc = p_ok ? p : P - 1;
    const int g = h / (H / G), inner = H * P;
    const int q0 = cu_q[co.b], q1 = cu_q[co.b + 1];
    auto local_state = [&](int j) { return chunk_state + ((static_cast<size_t>(co.first_chunk + j) * H + h) * P + pc) * N; };
    auto chunk_decay = [&](int j) { return expf(cumlog[static_cast<size_t>(min(q0 + (j + 1) * chunk, q1) - 1) * H + h]); };
    float S[NPT];
    {
        const float* l0 = local_state(0);
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const int n = j * LANES_N + ln;
            S[j] = n < N ? l0[n] : 0.f;
        }
    }
    for (int c = 1; c < co.k; ++c) {
        const float a = chunk_decay(c);
        const float* lc = local_state(c);
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const int n = j * LANES_N + ln;
            if (n < N) S[j] = a * S[j] + lc[n];
        }
    }
    const int t0 = q0 + co.k * chunk, t1 = min(t0 + chunk, q1);
    const int c_col = inner + G * N + g * N;
    for (int t = t0; t < t1; ++t) {
        const float* row = xbc + static_cast<size_t>(t) * ldx;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const int n = j * LANES_N + ln;
            if (n < N) acc += S[j] * row[c_col + n];
        }
        acc = group_sum<LANES_N>(acc);
        if (ln == 0 && p_ok) y[static_cast<size_t>(t) * ldy + h * P + p] += expf(cumlog[static_cast<size_t>(t) * H + h]) * acc;
    }
    if (write && p_ok && co.k == co.n_chunks - 1) {
        const float a = chunk_decay(co.k);
        const float* lk = local_state(co.k);
        float* sp = state + static_cast<size_t>(slot) * slot_floats + scan_offset + (static_cast<size_t>(h) * P + p) * N;
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const int n = j * LANES_N + ln;
            if (n < N) sp[n] = a * S[j] + lk[n];
        }
    }
}

}  // namespace

extern "C" {

// Convolution + silu of columns [col0, col0 + C) of proj's rows into out [T, C]; then, with `write`, the
// slots' carried rows are brought up to date (a second kernel: it overwrites what the first one reads).
// -1: taps outside 1..16.
int mllm_conv_silu(const float* proj, int ld, int col0, int C, const float* w, const float* bias, int taps,
                   const int* token_seq, const int* cu_q, const int* state_slots, float* state, size_t slot_floats,
                   float* out, int ldo, int T, int B, int write, hipStream_t stream) {
    if (T <= 0 || C <= 0) return 0;
    if (taps < 1 || taps > 16) return -1;
    const long long total = static_cast<long long>(T) * C;
    conv_silu_kernel<<<static_cast<int>((total + 255) / 256), 256, 0, stream>>>(proj, ld, col0, C, w, bias, taps, token_seq, cu_q,
                                                                                state_slots, state, slot_floats, out, ldo, total);
    MLLM_LAUNCH_CHECK();
    if (write && taps > 1) {
        const long long pairs = static_cast<long long>(B) * C;
        conv_carry_kernel<<<static_cast<int>((pairs + 255) / 256), 256, 0, stream>>>(proj, ld, col0, C, taps, cu_q, state_slots, state,
                                                                                    slot_floats, B);
        MLLM_LAUNCH_CHECK();
    }
    return 0;
}

// Tokens of a chunk, and what the chunks' workspace must hold for a step of T tokens in B sequences.
#define SSM_CHUNK 64
static size_t chunk_states(int T) { return 2 * static_cast<size_t>(T) / SSM_CHUNK + 1; }
size_t mllm_ssm_scan_workspace_floats(int T, int B, int H, int P, int N) {
    (void)B;
    return chunk_states(T) * H * P * N + static_cast<size_t>(T) * H;
}

// The scan over every sequence's portion (see the kernels). `workspace` (mllm_ssm_scan_workspace_floats floats)
// is needed when a portion is longer than one chunk (max_q_len > 64). -1: H is no multiple of G, N > 1024, or
// the workspace is missing.
int mllm_ssm_scan(const float* xbc, int ldx, const float* raw_dt, int ldd, const float* dt_bias, const float* A_log,
                  const float* Dskip, const int* cu_q, const int* state_slots, float* state, size_t slot_floats,
                  size_t scan_offset, float* y, int ldy, int T, int B, int max_q_len, int H, int P, int N, int G, int write,
                  float* workspace, hipStream_t stream) {
    if (B <= 0 || T <= 0) return 0;
    if (H < 1 || G < 1 || H % G != 0 || N < 1 || N > 1024 || P < 1) return -1;
    const bool chunked = max_q_len > SSM_CHUNK;
    if (chunked && workspace == nullptr) return -1;
    const int n_chunks = chunked ? T / SSM_CHUNK + B : B;
    float* chunk_state = workspace;
    float* cumlog = workspace ? workspace + chunk_states(T) * H * P * N : nullptr;
    int lanes = 1;
    while (lanes < 64 && lanes * 16 < N) lanes *= 2;       // sixteen n a lane
#define SCAN(L)                                                                                                       \
    do {                                                                                                              \
        const dim3 grid((P + 64 / L - 1) / (64 / L), H, n_chunks);                                                    \
        ssm_scan_kernel<16, L><<<grid, 64, 0, stream>>>(xbc, ldx, raw_dt, ldd, dt_bias, A_log, Dskip, cu_q, state_slots, B, \
                                                        state, slot_floats, scan_offset, y, ldy, H, P, N, G, write,   \
                                                        SSM_CHUNK, chunk_state, cumlog);                              \
        if (chunked)                                                                                                  \
            ssm_chunk_join_kernel<16, L><<<grid, 64, 0, stream>>>(xbc, ldx, cu_q, state_slots, B, state, slot_floats, \
                                                                  scan_offset, y, ldy, H, P, N, G, write, SSM_CHUNK,  \
                                                                  chunk_state, cumlog);                               \
    } while (0)
    switch (lanes) {
        case 1: SCAN(1); break;
        case 2: SCAN(2); break;
        case 4: SCAN(4); break;
        case 8: SCAN(8); break;
        case 16: SCAN(16); break;
        case 32: SCAN(32); break;
        default: SCAN(64); break;
    }
#undef SCAN
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
