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
// One wavefront per (sequence, head, 64 / LANES_N values of p): LANES_N consecutive lanes share a p and
// split n (lane l of the group holds n = l, l + LANES_N, ...: up to NPT of them in registers), so the sum over
// n is a sum inside the lane group and no wavefront waits for another. The next token's operands are
// requested before this token's are used. xbc rows: [x: H*P | B: G*N | C: G*N].
template <int NPT, int LANES_N>
__global__ void __launch_bounds__(64)
ssm_scan_kernel(const float* __restrict__ xbc, int ldx, const float* __restrict__ raw_dt, int ldd,
                const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dskip,
                const int* __restrict__ cu_q, const int* __restrict__ state_slots, float* __restrict__ state,
                size_t slot_floats, size_t scan_offset, float* __restrict__ y, int ldy, int H, int P, int N, int G,
                int write) {
    const int lane = threadIdx.x, ln = lane % LANES_N, pl = lane / LANES_N;
    const int h = blockIdx.y, b = blockIdx.z;
    const int slot = state_slots[b];
    if (slot < 0) return;
    const int p = blockIdx.x * (64 / LANES_N) + pl;
    const bool p_ok = p < P;
    const int pc = p_ok ? p : P - 1;
    const int g = h / (H / G), inner = H * P;
    const int t0 = cu_q[b], t1 = cu_q[b + 1];
    float* sp = state + static_cast<size_t>(slot) * slot_floats + scan_offset + (static_cast<size_t>(h) * P + pc) * N;
    float S[NPT];
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
        const int n = j * LANES_N + ln;
        S[j] = n < N ? sp[n] : 0.f;
    }
    const float bias = dt_bias[h], neg_rate = -expf(A_log[h]), skip = Dskip[h];
    const int b_col = inner + g * N, c_col = inner + G * N + g * N;
    // operands of the token at hand, and of the next one (loaded one token ahead)
    float xv, dtr, Bv[NPT], Cv[NPT];
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
    for (int t = t0; t < t1; ++t) {
        float xn = 0.f, dn = 0.f, Bn[NPT], Cn[NPT];
        const int tn = min(t + 1, t1 - 1);
        load(tn, xn, dn, Bn, Cn);
        const float dt = softplus_precise(dtr + bias);
        const float a = expf(neg_rate * dt), dx = dt * xv;
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
        xv = xn; dtr = dn;
#pragma unroll
        for (int j = 0; j < NPT; ++j) { Bv[j] = Bn[j]; Cv[j] = Cn[j]; }
    }
    if (write && p_ok) {
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const int n = j * LANES_N + ln;
            if (n < N) sp[n] = S[j];
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

// The scan over every sequence's portion (see the kernel). -1: H is no multiple of G, or N > 1024.
int mllm_ssm_scan(const float* xbc, int ldx, const float* raw_dt, int ldd, const float* dt_bias, const float* A_log,
                  const float* Dskip, const int* cu_q, const int* state_slots, float* state, size_t slot_floats,
                  size_t scan_offset, float* y, int ldy, int B, int H, int P, int N, int G, int write,
                  hipStream_t stream) {
    if (B <= 0) return 0;
    if (H < 1 || G < 1 || H % G != 0 || N < 1 || N > 1024 || P < 1) return -1;
    int lanes = 1;
    while (lanes < 64 && lanes * 8 < N) lanes *= 2;        // eight n a lane where 64 lanes suffice, else sixteen
#define SCAN(NPT, L)                                                                                              \
    ssm_scan_kernel<NPT, L><<<dim3((P + 64 / L - 1) / (64 / L), H, B), 64, 0, stream>>>(                          \
        xbc, ldx, raw_dt, ldd, dt_bias, A_log, Dskip, cu_q, state_slots, state, slot_floats, scan_offset, y, ldy, \
        H, P, N, G, write)
    switch (lanes) {
        case 1: SCAN(8, 1); break;
        case 2: SCAN(8, 2); break;
        case 4: SCAN(8, 4); break;
        case 8: SCAN(8, 8); break;
        case 16: SCAN(8, 16); break;
        case 32: SCAN(8, 32); break;
        default:
            if (N <= 512) SCAN(8, 64); else SCAN(16, 64);
            break;
    }
#undef SCAN
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
