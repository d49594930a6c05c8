// Latent attention for gfx950: keys and values of all heads are expanded from one cached latent row per
// token, c [R], beside one rotated key part [Dr] that the heads share. The pages hold rows [c | k_rot]
// (E = R + Dr columns) and nothing per head. Attention runs in the latent's space:
//   score(t, h, j) = scale * ( (W_uk_h^T q_plain[t,h]) . c_j + q_rot[t,h] . k_rot_j )
//   out[t, h]      = W_uv_h ( sum_j softmax_j(score) c_j )
// so a query is first carried into the latent space ("absorbed": qa [T, H, E]), attention is a
// one-key-head attention over the page rows whose values are the rows' first R columns, and the result
// (o_lat [T, H, R]) is expanded per head afterwards. Scores, softmax, norms and angles are fp32.
#include <algorithm>

#include "common.h"

namespace {

// Turn of the interleaved pair (u, v) at position p by the angle p * base^(-2i/dims); the angle in double.
__device__ __forceinline__ void turn_pair(float u, float v, int pos, int i, double log2_base, int dims, float& a, float& b) {
    const double f = exp2(-2.0 * static_cast<double>(i) / static_cast<double>(dims) * log2_base);
    const double angle = static_cast<double>(pos) * f;
    const float c = static_cast<float>(cos(angle)), s = static_cast<float>(sin(angle));
    a = u * c - v * s;
    b = v * c + u * s;
}

// One wavefront per token:
//   cq[t]  = rmsnorm(dq[t]) * wq                                      (the query latent, activation dtype)
//   page row slots[t] = [ c = rmsnorm(dkv[t, :R]) * wkv | turned dkv[t, R:R+Dr] ]   (if dkv is given and slot >= 0)
// The first rot_dims of the Dr columns are turned in interleaved pairs, the rest pass unchanged.
template <typename T>
__global__ void __launch_bounds__(64)
latent_prepare_kernel(const float* __restrict__ dq, int ld_dq, int Rq, const float* __restrict__ wq, T* __restrict__ cq,
                      int ld_cq, const float* __restrict__ dkv, int ld_dkv, int R, int Dr, const float* __restrict__ wkv,
                      T* __restrict__ pages, T* __restrict__ vt_pages, int page_size, const int* __restrict__ slots,
                      const int* __restrict__ positions, float eps, double log2_base, int rot_dims) {
    const int t = blockIdx.x, lane = threadIdx.x;
    // Up to 8 values a lane of each latent are requested up front, without conditions (a loop of unknown length
    // would wait for every load before it asks for the next); longer latents read the rest in a loop.
    const float* qrow = dq + static_cast<size_t>(t) * ld_dq;
    const int slot = dkv ? slots[t] : -1;
    const bool fill = dkv != nullptr && slot >= 0;
    const float* row = fill ? dkv + static_cast<size_t>(t) * ld_dkv : qrow;
    const int Rk = fill ? R : Rq;                              // (no latent to fill: the loads below repeat the query's)
    float qv[8], kv[8], qw[8], kw[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int iq = min(lane + 64 * u, Rq - 1), ik = min(lane + 64 * u, Rk - 1);
        qv[u] = qrow[iq];
        qw[u] = wq[iq];
        kv[u] = row[ik];
        kw[u] = fill ? wkv[ik] : 0.f;
    }
    {
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) if (lane + 64 * u < Rq) ss += qv[u] * qv[u];
        for (int i = lane + 512; i < Rq; i += 64) ss += qrow[i] * qrow[i];
        const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Rq) + eps);
        T* o = cq + static_cast<size_t>(t) * ld_cq;
#pragma unroll
        for (int u = 0; u < 8; ++u) if (lane + 64 * u < Rq) o[lane + 64 * u] = from_float<T>(qv[u] * inv * qw[u]);
        for (int i = lane + 512; i < Rq; i += 64) o[i] = from_float<T>(qrow[i] * inv * wq[i]);
    }
    if (!fill) return;
    T* o = pages + static_cast<size_t>(slot) * (R + Dr);
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) if (lane + 64 * u < R) ss += kv[u] * kv[u];
    for (int i = lane + 512; i < R; i += 64) ss += row[i] * row[i];
    const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(R) + eps);
    // (vt_pages, optional: the latent once more, transposed page by page, [page][R][page_size], which is the
    // operand shape of the matrix-core kernel's second product)
    T* vt = vt_pages ? vt_pages + static_cast<size_t>(slot / page_size) * page_size * R + slot % page_size : nullptr;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int i = lane + 64 * u;
        if (i < R) {
            const T c = from_float<T>(kv[u] * inv * kw[u]);
            o[i] = c;
            if (vt) vt[static_cast<size_t>(i) * page_size] = c;
        }
    }
    for (int i = lane + 512; i < R; i += 64) {
        const T c = from_float<T>(row[i] * inv * wkv[i]);
        o[i] = c;
        if (vt) vt[static_cast<size_t>(i) * page_size] = c;
    }
    const int pos = positions[t];
    for (int i = lane; i < rot_dims / 2; i += 64) {
        float a, b;
        turn_pair(row[R + 2 * i], row[R + 2 * i + 1], pos, i, log2_base, rot_dims, a, b);
        o[R + 2 * i] = from_float<T>(a);
        o[R + 2 * i + 1] = from_float<T>(b);
    }
    for (int i = rot_dims + lane; i < Dr; i += 64) o[R + i] = from_float<T>(row[R + i]);
}

// Queries into the latent space. q rows: per head [Dn plain | Dr to be turned]; w_ukt [R, H * Dn] is the key
// expansion transposed (column h*Dn + d of row r expands latent column r into the head's plain key dimension d).
// For 8 tokens and one head a workgroup:
//   qa[t, h, r] = sum_d q[t, h, d] * w_ukt[r, h*Dn + d]      (thread per r)
//   qa[t, h, R + i] = the turned rotary part of q[t, h]
// (Any dtype and sizes; bfloat16 at sizes in steps of 32 goes to head_linear_mfma_kernel.)
template <typename T>
__global__ void __launch_bounds__(256)
latent_absorb_kernel(const T* __restrict__ q, int ldq, const T* __restrict__ w_uk, int ldw, T* __restrict__ qa, int ldqa,
                     const int* __restrict__ positions, int n_tokens, int H, int Dn, int Dr, int R, double log2_base,
                     int rot_dims) {
    extern __shared__ float q_s[];                   // [8][Dn]
    const int h = blockIdx.y, t0 = blockIdx.z * 8, E = R + Dr;
    const int nt = min(8, n_tokens - t0);
    for (int i = threadIdx.x; i < 8 * Dn; i += 256) {
        const int tt = i / Dn, d = i % Dn;
        q_s[i] = tt < nt ? to_float(q[static_cast<size_t>(t0 + tt) * ldq + h * (Dn + Dr) + d]) : 0.f;
    }
    __syncthreads();
    for (int r = blockIdx.x * 256 + threadIdx.x; r < R; r += gridDim.x * 256) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const T* wrow = w_uk + static_cast<size_t>(r) * ldw + static_cast<size_t>(h) * Dn;
        for (int d = 0; d < Dn; ++d) {
            const float wv = to_float(wrow[d]);
#pragma unroll
            for (int tt = 0; tt < 8; ++tt) acc[tt] += q_s[tt * Dn + d] * wv;
        }
#pragma unroll
        for (int tt = 0; tt < 8; ++tt)
            if (tt < nt) qa[static_cast<size_t>(t0 + tt) * ldqa + h * E + r] = from_float<T>(acc[tt]);
    }
    if (blockIdx.x == 0) {
        for (int i = threadIdx.x; i < nt * (Dr / 2 + Dr); i += 256) {
            // the first nt * rot_dims/2 indices turn pairs, the rest copy what is not turned
            const int tt = i / (Dr / 2 + Dr), k = i % (Dr / 2 + Dr);
            const T* src = q + static_cast<size_t>(t0 + tt) * ldq + h * (Dn + Dr) + Dn;
            T* dst = qa + static_cast<size_t>(t0 + tt) * ldqa + h * E + R;
            if (k < Dr / 2) {
                if (k < rot_dims / 2) {
                    float a, b;
                    turn_pair(to_float(src[2 * k]), to_float(src[2 * k + 1]), positions[t0 + tt], k, log2_base, rot_dims, a, b);
                    dst[2 * k] = from_float<T>(a);
                    dst[2 * k + 1] = from_float<T>(b);
                }
            } else {
                const int c = k - Dr / 2;
                if (c >= rot_dims) dst[c] = src[c];
            }
        }
    }
}

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
union Frag8 {
    bf16x8 v;
    u32x4 q;
    uint32_t w[4];
};

// One small product per head on the matrix cores (bfloat16, fp32 sums), operands straight from memory:
//   out[t, h*out_hs + n] = sum_k a[t, h*a_hs + k] * w[(h*w_head_rows + n) * ldw + h*w_head_cols + k],  n < N, k < K
// (w_head_rows = N, w_head_cols = 0: every head has its own rows of w; w_head_rows = 0, w_head_cols = K: its own
// columns). A workgroup takes 64 tokens, one head and 64 values of n; a wavefront 16 tokens: the weights are the
// MFMA's A operand, so a lane ends up with four neighbouring n of one token. K is a multiple of 32; rows and head
// offsets are 16-byte aligned. With `positions`, the workgroups of the first n tile also carry the `tail` columns
// behind a head's K inputs over to behind its N outputs, the first rot_dims of them turned in interleaved pairs.
__global__ void __launch_bounds__(256)
head_linear_mfma_kernel(const bf16_t* __restrict__ a, int lda, int a_hs, const bf16_t* __restrict__ w, int ldw, int w_head_rows,
                        int w_head_cols, bf16_t* __restrict__ out, int ldo, int out_hs, int n_tokens, int N, int K,
                        const int* __restrict__ positions, int tail, int rot_dims, double log2_base) {
    const int lane = threadIdx.x % 64, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int G = lane / 16, c16 = lane % 16;
    const int h = blockIdx.y, t0 = blockIdx.x * 64, n_base = blockIdx.z * 64;
    const int tok = min(t0 + 16 * wave + c16, n_tokens - 1);
    const bf16_t* arow = a + static_cast<size_t>(tok) * lda + static_cast<size_t>(h) * a_hs + 8 * G;
    const bf16_t* wbase = w + static_cast<size_t>(h) * w_head_rows * ldw + static_cast<size_t>(h) * w_head_cols + 8 * G;
    const bf16_t* wrow[4];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) wrow[ct] = wbase + static_cast<size_t>(min(n_base + 16 * ct + c16, N - 1)) * ldw;
    f32x4 acc[4];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) acc[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < K; k += 32) {
        Frag8 af, wf[4];
        af.q = *reinterpret_cast<const u32x4*>(arow + k);
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) wf[ct].q = *reinterpret_cast<const u32x4*>(wrow[ct] + k);
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[ct].v, af.v, acc[ct], 0, 0, 0);
    }
    if (t0 + 16 * wave + c16 < n_tokens) {
        bf16_t* orow = out + static_cast<size_t>(tok) * ldo + static_cast<size_t>(h) * out_hs;
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            const int n = n_base + 16 * ct + 4 * G;            // acc[ct][r] is output n + r of this lane's token
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < N) orow[n + r] = float_to_bf16(acc[ct][r]);
        }
    }
    if (positions != nullptr && blockIdx.z == 0) {
        const int nt = min(64, n_tokens - t0), per = tail / 2 + tail;
        for (int i = threadIdx.x; i < nt * per; i += 256) {
            const int tt = i / per, k = i % per;
            const bf16_t* src = a + static_cast<size_t>(t0 + tt) * lda + static_cast<size_t>(h) * a_hs + K;
            bf16_t* dst = out + static_cast<size_t>(t0 + tt) * ldo + static_cast<size_t>(h) * out_hs + N;
            if (k < tail / 2) {
                if (k < rot_dims / 2) {
                    float u, v;
                    turn_pair(to_float(src[2 * k]), to_float(src[2 * k + 1]), positions[t0 + tt], k, log2_base, rot_dims, u, v);
                    dst[2 * k] = float_to_bf16(u);
                    dst[2 * k + 1] = float_to_bf16(v);
                }
            } else {
                const int c = k - tail / 2;
                if (c >= rot_dims) dst[c] = src[c];
            }
        }
    }
}

// Attention of one token's heads over its sequence's page rows. One workgroup per (token, group of up to HG
// heads), four wavefronts; a wavefront owns the heads wave, wave + 4, ... of the group. Keys are staged in
// LDS 64 at a time (rows padded to an odd number of 32-bit words so that the lanes, one key each, read
// without bank conflicts); a head's running maximum, sum and output (R columns, fp32) live in LDS.
// Position i sees j with 0 <= i - j < window (window 0: every earlier key).
//   LDS: q_s [HG][E] f32 | o_s [HG][R] f32 | p_s [4][64] f32 | k_s [64][KS] T
template <typename T>
__global__ void __launch_bounds__(256)
latent_attention_kernel(const T* __restrict__ qa, int ldqa, const T* __restrict__ pages, const int* __restrict__ block_tables,
                        int max_blocks, const int* __restrict__ token_seq, const int* __restrict__ positions, int H, int HG,
                        int R, int Dr, int page_size, float scale_log2, int window, T* __restrict__ o_lat, int ldo, int KS) {
    extern __shared__ float lds[];
    const int E = R + Dr;
    // (bfloat16 rows are read two columns a word: an odd row gets one more column, zero in the queries and in LDS)
    const int Eq = sizeof(T) == 2 ? E + (E & 1) : E;
    float* q_s = lds;
    float* o_s = q_s + HG * Eq;
    float* p_s = o_s + HG * R;
    T* k_s = reinterpret_cast<T*>(p_s + 4 * 64);
    const int t = blockIdx.x, h0 = blockIdx.y * HG, nh = min(HG, H - h0);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const int pos = positions[t];
    const int* table = block_tables + static_cast<size_t>(token_seq[t]) * max_blocks;
    for (int i = threadIdx.x; i < nh * Eq; i += 256) {
        const int hh = i / Eq, c = i % Eq;
        q_s[i] = c < E ? to_float(qa[static_cast<size_t>(t) * ldqa + (h0 + hh) * E + c]) * scale_log2 : 0.f;
    }
    for (int i = threadIdx.x; i < nh * R; i += 256) o_s[i] = 0.f;
    // per head of this wavefront: running maximum and sum (up to 8 heads a wavefront: HG <= 32)
    float m_run[8], l_run[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) { m_run[u] = -INFINITY; l_run[u] = 0.f; }
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int words = sizeof(T) == 2 ? Eq / 2 : E;          // 32-bit words of a key row in LDS
    const bool by_words = sizeof(T) == 4 || (E & 1) == 0;   // (an odd bfloat16 row does not start on a word)
    for (int k0 = lo; k0 <= pos; k0 += 64) {
        const int nk = min(64, pos + 1 - k0);
        __syncthreads();                                   // the tile before is used up
        if (by_words) {
            for (int i = threadIdx.x; i < nk * words; i += 256) {
                const int j = i / words, c = i % words, kp = k0 + j;
                const size_t row = static_cast<size_t>(table[kp / page_size]) * page_size + kp % page_size;
                reinterpret_cast<uint32_t*>(k_s)[j * KS + c] = reinterpret_cast<const uint32_t*>(pages + row * E)[c];
            }
        } else {
            for (int i = threadIdx.x; i < nk * Eq; i += 256) {
                const int j = i / Eq, c = i % Eq, kp = k0 + j;
                const size_t row = static_cast<size_t>(table[kp / page_size]) * page_size + kp % page_size;
                k_s[static_cast<size_t>(j) * 2 * KS + c] = c < E ? pages[row * E + c] : from_float<T>(0.f);
            }
        }
        __syncthreads();
        const uint32_t* kw = reinterpret_cast<const uint32_t*>(k_s) + min(lane, nk - 1) * KS;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int hh = wave + 4 * u;
            if (hh < nh) {
                const float* qh = q_s + hh * Eq;
                float s = 0.f;
                if (sizeof(T) == 2) {
                    for (int c = 0; c < words; ++c) {
                        const uint32_t w2 = kw[c];
                        s += qh[2 * c] * __uint_as_float(w2 << 16) + qh[2 * c + 1] * __uint_as_float(w2 & 0xffff0000u);
                    }
                } else {
                    for (int c = 0; c < words; ++c) s += qh[c] * __uint_as_float(kw[c]);
                }
                if (lane >= nk) s = -INFINITY;
                const float m_new = fmaxf(m_run[u], wave_max(s));
                const float pj = lane < nk ? exp2_for<T>(s - m_new) : 0.f;
                const float corr = exp2_for<T>(m_run[u] - m_new);          // (first tile: 2^-inf = 0)
                l_run[u] = l_run[u] * corr + wave_sum(pj);
                m_run[u] = m_new;
                p_s[wave * 64 + lane] = pj;
                wave_lds_sync();
                float* oh = o_s + hh * R;
                for (int c = lane; c < R; c += 64) {
                    float acc = oh[c] * corr;
                    for (int j = 0; j < nk; ++j) acc += p_s[wave * 64 + j] * to_float(k_s[static_cast<size_t>(j) * (sizeof(T) == 2 ? 2 * KS : KS) + c]);
                    oh[c] = acc;
                }
                wave_lds_sync();
            }
        }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int hh = wave + 4 * u;
        if (hh < nh) {
            const float inv = 1.f / l_run[u];
            for (int c = lane; c < R; c += 64)
                o_lat[static_cast<size_t>(t) * ldo + (h0 + hh) * R + c] = from_float<T>(o_s[hh * R + c] * inv);
        }
    }
}

// Per-head expansion of the attention result: out[t, h*Dv + e] = sum_r w_uv[h*Dv + e, r] * o_lat[t, h, r].
// One wavefront per output column (lanes over r, coalesced weight reads), 8 tokens a pass.
template <typename T>
__global__ void __launch_bounds__(256)
latent_expand_kernel(const T* __restrict__ o_lat, int ldo, const T* __restrict__ w_uv, int ldw, T* __restrict__ out, int ldout,
                     int n_tokens, int H, int Dv, int R) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const int col = blockIdx.x * 4 + wave;
    if (col >= H * Dv) return;
    const int h = col / Dv;
    const T* wr = w_uv + static_cast<size_t>(col) * ldw;
    for (int t0 = blockIdx.y * 8; t0 < n_tokens; t0 += gridDim.y * 8) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int r = lane; r < R; r += 64) {
            const float wv = to_float(wr[r]);
#pragma unroll
            for (int tt = 0; tt < 8; ++tt) {
                const int t = min(t0 + tt, n_tokens - 1);
                acc[tt] += wv * to_float(o_lat[static_cast<size_t>(t) * ldo + h * R + r]);
            }
        }
#pragma unroll
        for (int tt = 0; tt < 8; ++tt) {
            const float v = wave_sum(acc[tt]);
            if (lane == 0 && t0 + tt < n_tokens) out[static_cast<size_t>(t0 + tt) * ldout + col] = from_float<T>(v);
        }
    }
}

// Prompt portions on the matrix cores (bfloat16, fp32 softmax). A query row is a (token, head) pair; a
// sequence's rows are numbered token by token, head by head, and a workgroup takes 64 consecutive rows (its
// four wavefronts 16 each), which lie on few neighbouring tokens, so they share their keys: one staging of a
// 64-key tile serves all of them. Everything is computed transposed, one query row per lane, as in the
// framework's other prompt-attention kernel (attention_prefill.hip):
//   S^T = K Q^T    A = 16 page rows x 32 columns from LDS, B = the lane's absorbed query, in registers
//   O^T = C^T P^T  A = 16 latent columns x 32 keys, B = P^T straight from the S^T accumulators
// The second product's A operand needs 8 keys of one latent column side by side, which the page-transposed
// copy of the latent holds ([page][R][page_size]): its 16-byte pieces go to LDS as they are, keys outside
// the tile's range set to zero (a page's tail may hold anything). E = 32 * KS, R = 16 * DT.
// (The widest sizes keep 128 accumulators, 70 query registers and a tile's staging registers a lane: they get the
// whole register file, one wavefront per SIMD, which is also all their LDS allows.)
template <int KS, int DT>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, (KS + DT > 30) ? 1 : 2)))
latent_prefill_kernel(const bf16_t* __restrict__ qa, const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ vt_pages,
                      const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ cu_q,
                      const int* __restrict__ ctx_len, int n_seqs, int H, int page_size, float scale_log2e, int window,
                      bf16_t* __restrict__ o_lat, int nsplit, float* __restrict__ partials, int single_tokens) {
    constexpr int E = 32 * KS, R = 16 * DT, BN = 64, KSTRIDE = E + 8, VSTRIDE = BN + 8, CH = E / 8;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    bf16_t* Ks = reinterpret_cast<bf16_t*>(smem);                    // [BN][KSTRIDE]
    bf16_t* Vt = Ks + BN * KSTRIDE;                                  // [R][VSTRIDE]
    int* sm_table = reinterpret_cast<int*>(Vt + R * VSTRIDE);        // the sequence's block table

    int tile = gridDim.x - 1 - blockIdx.x, b = 0, q_begin = 0, q_len = 0;
    if (single_tokens) {
        // every sequence brings one token: its tiles follow from the tile's index, without the walk over the
        // sequences below, whose every step waits for a load
        const int per = (H + 63) / 64;
        b = tile / per;
        tile -= b * per;
        if (b < n_seqs) { q_begin = b; q_len = 1; }
    } else {
        for (; b < n_seqs; ++b) {
            q_begin = cu_q[b];
            q_len = cu_q[b + 1] - q_begin;
            const int nt = (q_len * H + 63) / 64;
            if (tile < nt) break;
            tile -= nt;
        }
    }
    if (b >= n_seqs) return;                       // surplus workgroup; the whole workgroup leaves
    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int G = lane / 16, c16 = lane % 16;
    const int rows = q_len * H, start = ctx_len[b] - q_len;
    const int rho0 = tile * 64, rho = rho0 + wave * 16 + c16;
    const bool q_ok = rho < rows;
    const int rho_c = min(rho, rows - 1);
    const int p = start + rho_c / H;                              // this lane's position
    const int p_first = start + rho0 / H, p_last = start + min(rho0 + 63, rows - 1) / H;
    const int k_lo = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int shift = __ffs(page_size) - 1;
    const int* gtable = block_tables + static_cast<size_t>(b) * max_blocks;
    for (int i = tid; i <= (p_last >> shift); i += 256) sm_table[i] = gtable[i];
    __syncthreads();

    Frag8 qf[KS];
    const bf16_t* qrow = qa + (static_cast<size_t>(q_begin) * H + rho_c) * E;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks].q = *reinterpret_cast<const u32x4*>(qrow + 32 * ks + 8 * G);

    float m = -INFINITY, l = 0.f;
    f32x4 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int pg_lo = k_lo >> shift, pg_hi = p_last >> shift;

    // With nsplit > 1 (few rows in the step: decoding) the workgroups blockIdx.y = 0 .. nsplit - 1 share the
    // key tiles of these rows and leave their states unmerged in `partials`.
    int kt_begin = k_lo / BN, kt_end = p_last / BN + 1;
    if (nsplit > 1) {
        const int per = (kt_end - kt_begin + nsplit - 1) / nsplit;
        kt_begin += static_cast<int>(blockIdx.y) * per;
        kt_end = min(kt_end, kt_begin + per);
    }
    static_assert(DT % 2 == 0, "the transposed latent is staged in whole rounds of the workgroup");
    for (int kt = kt_begin; kt < kt_end; ++kt) {
        const int j_base = kt * BN;
        // Staging. All loads of a tile are issued first (a fixed number per thread: 64 * E / 8 pieces of page rows
        // over 256 threads are KS each, R * 8 pieces of the transposed latent DT / 2 each), then written to LDS: a
        // load inside a loop of unknown length would be waited for before the next one is asked for.
        // Page rows, row-major; a key outside [k_lo, p_last] is replaced by one inside (always a held page; its
        // scores are masked below). The latent transposed: 8 keys of one column a piece, keys outside the range
        // set to zero.
        u32x4 kreg[KS], vreg[DT / 2];
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            const int idx = tid + 256 * u, j = idx / CH, c = idx % CH;
            const int key = min(max(j_base + j, k_lo), p_last);
            const size_t row = (static_cast<size_t>(sm_table[key >> shift]) << shift) + (key & (page_size - 1));
            kreg[u] = *reinterpret_cast<const u32x4*>(k_pages + row * E + 8 * c);
        }
#pragma unroll
        for (int u = 0; u < DT / 2; ++u) {
            const int idx = tid + 256 * u, col = idx / (BN / 8), part = idx % (BN / 8);
            const int key0 = j_base + 8 * part;
            const int pg = min(max(key0 >> shift, pg_lo), pg_hi);
            vreg[u] = *reinterpret_cast<const u32x4*>(vt_pages + (static_cast<size_t>(sm_table[pg]) << shift) * R +
                                                      static_cast<size_t>(col) * page_size + (key0 & (page_size - 1)));
        }
        __syncthreads();                           // the tile before is used up
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            const int idx = tid + 256 * u, j = idx / CH, c = idx % CH;
            *reinterpret_cast<u32x4*>(Ks + j * KSTRIDE + 8 * c) = kreg[u];
        }
#pragma unroll
        for (int u = 0; u < DT / 2; ++u) {
            const int idx = tid + 256 * u, col = idx / (BN / 8), part = idx % (BN / 8);
            const int key0 = j_base + 8 * part;
            u32x4 v = vreg[u];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int ka = key0 + 2 * e, kb = ka + 1;
                const uint32_t keep = ((ka >= k_lo && ka <= p_last) ? 0x0000ffffu : 0u) | ((kb >= k_lo && kb <= p_last) ? 0xffff0000u : 0u);
                v[e] &= keep;
            }
            *reinterpret_cast<u32x4*>(Vt + col * VSTRIDE + 8 * part) = v;
        }
        __syncthreads();
        // S^T: s[nt][r] is the score of key j_base + 16 nt + 4 G + r with this lane's query row
        float s[4][4];
        float tile_max = -INFINITY;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8 a = *reinterpret_cast<const bf16x8*>(Ks + (16 * nt + c16) * KSTRIDE + 32 * ks + 8 * G);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[ks].v, acc, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int j = j_base + 16 * nt + 4 * G + r;
                const bool seen = q_ok && j <= p && (window <= 0 || j > p - window);
                s[nt][r] = seen ? acc[r] : -INFINITY;
                tile_max = fmaxf(tile_max, s[nt][r]);
            }
        }
        tile_max = rows_max(tile_max);             // the four lane groups of a query row agree on the maximum
        const float m_new = fmaxf(m, tile_max * scale_log2e);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2(m - m_use);
        m = m_new;
        float psum = 0.f;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                s[nt][r] = fast_exp2(fmaf(s[nt][r], scale_log2e, -m_use));
                psum += s[nt][r];
            }
        l = l * alpha + psum;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[dt][r] *= alpha;
        // O^T += C^T P^T over slabs of 32 keys: k slot i of lane group G stands for key 32 slab + 4 G + i
        // (i < 4) or 32 slab + 16 + 4 G + i - 4 (i >= 4) in both operands
#pragma unroll
        for (int slab = 0; slab < 2; ++slab) {
            Frag8 pf;
            pf.w[0] = pack_bf16x2(s[2 * slab][0], s[2 * slab][1]);
            pf.w[1] = pack_bf16x2(s[2 * slab][2], s[2 * slab][3]);
            pf.w[2] = pack_bf16x2(s[2 * slab + 1][0], s[2 * slab + 1][1]);
            pf.w[3] = pack_bf16x2(s[2 * slab + 1][2], s[2 * slab + 1][3]);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const uint32_t* vrow = reinterpret_cast<const uint32_t*>(Vt + (16 * dt + c16) * VSTRIDE);
                Frag8 vf;
                vf.w[0] = vrow[16 * slab + 2 * G];
                vf.w[1] = vrow[16 * slab + 2 * G + 1];
                vf.w[2] = vrow[16 * slab + 8 + 2 * G];
                vf.w[3] = vrow[16 * slab + 8 + 2 * G + 1];
                o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, o[dt], 0, 0, 0);
            }
        }
    }
    l = rows_sum(l);
    if (!q_ok) return;
    if (nsplit > 1) {
        // this split's state of the row: [maximum (base 2, scaled), sum, unnormalised output]; a split that saw
        // no key leaves maximum -inf, sum 0, zeros
        float* st = partials + ((static_cast<size_t>(q_begin) * H + rho) * nsplit + blockIdx.y) * (R + 2);
        if (G == 0) { st[0] = m; st[1] = l; }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) st[2 + 16 * dt + 4 * G + r] = o[dt][r];
        return;
    }
    const float inv = 1.0f / l;
    // o[dt][r] is latent column 16 dt + 4 G + r of this lane's query row
    bf16_t* orow = o_lat + (static_cast<size_t>(q_begin) * H + rho) * R;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        uint2 pk;
        pk.x = pack_bf16x2(o[dt][0] * inv, o[dt][1] * inv);
        pk.y = pack_bf16x2(o[dt][2] * inv, o[dt][3] * inv);
        *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * G) = pk;
    }
}

// The splits' states of a row merged: o = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s. One wavefront per row
// (up to 64 splits: lane s weighs split s; the weights pass through LDS; the outputs are added in the order of
// the splits, four columns a lane at a time, every load issued before the first use).
__global__ void __launch_bounds__(256)
latent_merge_kernel(const float* __restrict__ partials, int n_rows, int nsplit, int R, bf16_t* __restrict__ o_lat) {
    __shared__ float weights[4][64];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const int row = blockIdx.x * 4 + wave;
    if (row >= n_rows) return;
    const float* st = partials + static_cast<size_t>(row) * nsplit * (R + 2);
    const float* mine = st + static_cast<size_t>(min(lane, nsplit - 1)) * (R + 2);
    const float m = lane < nsplit ? mine[0] : -INFINITY, l = lane < nsplit ? mine[1] : 0.f;
    const float M = wave_max(m);
    const float wgt = fast_exp2(m - M);
    const float inv = 1.0f / wave_sum(wgt * l);
    weights[wave][lane] = wgt * inv;
    wave_lds_sync();
    for (int c = 4 * lane; c < R; c += 256) {
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int sp = 0; sp < nsplit; ++sp) {
            // (R + 2 is even and c a multiple of 4: the columns of a state are 8-byte aligned)
            const float2 a = *reinterpret_cast<const float2*>(st + static_cast<size_t>(sp) * (R + 2) + 2 + c);
            const float2 b = *reinterpret_cast<const float2*>(st + static_cast<size_t>(sp) * (R + 2) + 4 + c);
            const float ws = weights[wave][sp];
            acc.x += ws * a.x; acc.y += ws * a.y; acc.z += ws * b.x; acc.w += ws * b.y;
        }
        uint2 pk;
        pk.x = pack_bf16x2(acc.x, acc.y);
        pk.y = pack_bf16x2(acc.z, acc.w);
        *reinterpret_cast<uint2*>(o_lat + static_cast<size_t>(row) * R + c) = pk;
    }
}

constexpr int MAX_LDS = 160 * 1024;

}  // namespace

extern "C" {

// See latent_prepare_kernel. dkv may be null (a layer that reads another layer's pages). -1: an odd rot_dims
// or one beyond Dr.
int mllm_latent_prepare(const float* dq, int ld_dq, int Rq, const float* wq, void* cq, int ld_cq, const float* dkv, int ld_dkv,
                        int R, int Dr, const float* wkv, void* pages, void* vt_pages, int page_size, const int* slots,
                        const int* positions, int T, float eps, double base, int rot_dims, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (rot_dims < 0 || rot_dims % 2 != 0 || rot_dims > Dr || !(base > 0) || (vt_pages != nullptr && page_size < 1)) return -1;
    const double l2 = log2(base);
    if (dtype == MLLM_F32)
        latent_prepare_kernel<float><<<T, 64, 0, stream>>>(dq, ld_dq, Rq, wq, static_cast<float*>(cq), ld_cq, dkv, ld_dkv, R, Dr, wkv,
                                                           static_cast<float*>(pages), static_cast<float*>(vt_pages), page_size, slots, positions,
                                                           eps, l2, rot_dims);
    else
        latent_prepare_kernel<bf16_t><<<T, 64, 0, stream>>>(dq, ld_dq, Rq, wq, static_cast<bf16_t*>(cq), ld_cq, dkv, ld_dkv, R, Dr, wkv,
                                                            static_cast<bf16_t*>(pages), static_cast<bf16_t*>(vt_pages), page_size, slots, positions,
                                                            eps, l2, rot_dims);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// See latent_absorb_kernel; w_uk is the key expansion transposed, [R, H * Dn]. -1: rot_dims odd or beyond Dr, Dr
// odd; -2: Dn too large for the LDS.
int mllm_latent_absorb(const void* q, int ldq, const void* w_uk, int ldw, void* qa, int ldqa, const int* positions, int T, int H,
                       int Dn, int Dr, int R, double base, int rot_dims, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (rot_dims < 0 || rot_dims % 2 != 0 || rot_dims > Dr || Dr % 2 != 0 || !(base > 0)) return -1;
    const double l2 = log2(base);
    const auto aligned16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    if (dtype == MLLM_BF16 && Dn % 32 == 0 && ldq % 8 == 0 && (Dn + Dr) % 8 == 0 && ldw % 8 == 0 && aligned16(q) && aligned16(w_uk)) {
        head_linear_mfma_kernel<<<dim3((T + 63) / 64, H, (R + 63) / 64), 256, 0, stream>>>(
            static_cast<const bf16_t*>(q), ldq, Dn + Dr, static_cast<const bf16_t*>(w_uk), ldw, 0, Dn, static_cast<bf16_t*>(qa), ldqa, R + Dr,
            T, R, Dn, positions, Dr, rot_dims, l2);
        MLLM_LAUNCH_CHECK();
        return 0;
    }
    const size_t lds = static_cast<size_t>(8) * Dn * sizeof(float);
    if (lds > 64 * 1024) return -2;
    const dim3 grid((R + 255) / 256, H, (T + 7) / 8);
    if (dtype == MLLM_F32)
        latent_absorb_kernel<float><<<grid, 256, lds, stream>>>(static_cast<const float*>(q), ldq, static_cast<const float*>(w_uk), ldw,
                                                                static_cast<float*>(qa), ldqa, positions, T, H, Dn, Dr, R, l2, rot_dims);
    else
        latent_absorb_kernel<bf16_t><<<grid, 256, lds, stream>>>(static_cast<const bf16_t*>(q), ldq, static_cast<const bf16_t*>(w_uk), ldw,
                                                                 static_cast<bf16_t*>(qa), ldqa, positions, T, H, Dn, Dr, R, l2, rot_dims);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// See latent_attention_kernel. -1: sizes the kernel's accesses do not allow; -2: a head's rows do not fit the LDS.
int mllm_latent_attention(const void* qa, int ldqa, const void* pages, const int* block_tables, int max_blocks,
                          const int* token_seq, const int* positions, int T, int H, int R, int Dr, int page_size, float scale,
                          int window, void* o_lat, int ldo, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    const int E = R + Dr, esz = dtype == MLLM_F32 ? 4 : 2;
    if (H < 1 || R < 1 || Dr < 0 || page_size < 1) return -1;
    if ((reinterpret_cast<uintptr_t>(pages) & 3) != 0) return -1;
    const int Eq = dtype == MLLM_F32 ? E : E + (E & 1);
    int words = dtype == MLLM_F32 ? E : Eq / 2;
    const int KS = words | 1;                                    // an odd row stride, in 32-bit words
    auto lds_for = [&](int hg) {
        return static_cast<size_t>(hg) * (Eq + R) * 4 + 4 * 64 * 4 + static_cast<size_t>(64) * KS * 4;
    };
    int HG = std::min(H, 32);
    while (HG > 1 && lds_for(HG) > static_cast<size_t>(MAX_LDS)) HG = (HG + 1) / 2;
    if (lds_for(HG) > static_cast<size_t>(MAX_LDS)) return -2;
    const size_t lds = lds_for(HG);
    const dim3 grid(T, (H + HG - 1) / HG);
    const float scale_log2 = scale * 1.4426950408889634f;
    (void)esz;
#define LATENT_ATTN(TYPE)                                                                                              \
    do {                                                                                                               \
        static size_t allowed = 64 * 1024;                                                                             \
        if (lds > allowed) {                                                                                           \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(latent_attention_kernel<TYPE>),           \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, MAX_LDS);                   \
            if (e != hipSuccess) return static_cast<int>(e);                                                           \
            allowed = MAX_LDS;                                                                                         \
        }                                                                                                              \
        latent_attention_kernel<TYPE><<<grid, 256, lds, stream>>>(                                                     \
            static_cast<const TYPE*>(qa), ldqa, static_cast<const TYPE*>(pages), block_tables, max_blocks, token_seq, \
            positions, H, HG, R, Dr, page_size, scale_log2, window, static_cast<TYPE*>(o_lat), ldo, KS);               \
    } while (0)
    if (dtype == MLLM_F32) LATENT_ATTN(float); else LATENT_ATTN(bf16_t);
#undef LATENT_ATTN
    MLLM_LAUNCH_CHECK();
    return 0;
}

// The matrix-core kernel (see latent_prefill_kernel): qa [T*H, E] and o_lat [T*H, R] contiguous bfloat16.
// nsplit > 1: every row's key tiles are shared by nsplit workgroups whose states meet in `partials`
// (n_rows * nsplit * (R + 2) floats, n_rows = T*H) and are merged by a second kernel. single_tokens != 0: every
// sequence brings exactly one token (n_tiles_upper is then n_seqs * ceil(H / 64)). n_tiles_upper: an upper bound of sum over sequences of ceil(q_len * H / 64). Returns -2 when the
// sizes are not ones it is built for (E and R among (128, 96), (96, 64), (160, 128), (288, 256), (544, 512), (576, 512);
// page sizes 8 to 64, powers of two; a block table that fits the LDS beside the tiles): the caller then runs
// mllm_latent_attention.
int mllm_latent_attention_tiles(const void* qa, const void* k_pages, const void* vt_pages, const int* block_tables,
                                int max_blocks, const int* cu_q, const int* ctx_len, int n_seqs, int n_tiles_upper, int H,
                                int R, int Dr, int page_size, float scale, int window, void* o_lat, int n_rows, int nsplit,
                                float* partials, int single_tokens, hipStream_t stream) {
    if (n_seqs <= 0 || n_tiles_upper <= 0) return 0;
    const int E = R + Dr;
    if (nsplit < 1 || nsplit > 64 || (nsplit > 1 && (partials == nullptr || n_rows < 1))) return -1;
    if (E % 32 != 0 || R % 16 != 0 || page_size < 8 || page_size > 64 || (page_size & (page_size - 1)) != 0) return -2;
    if (((reinterpret_cast<uintptr_t>(qa) | reinterpret_cast<uintptr_t>(k_pages) | reinterpret_cast<uintptr_t>(vt_pages) |
          reinterpret_cast<uintptr_t>(o_lat)) & 15) != 0)
        return -2;
    const size_t lds = static_cast<size_t>(64) * (E + 8) * 2 + static_cast<size_t>(R) * 72 * 2 + static_cast<size_t>(max_blocks) * 4;
    if (lds > static_cast<size_t>(MAX_LDS)) return -2;
    const float sl2 = scale * 1.44269504088896340736f;
#define LP_CASE(KS, DT)                                                                                              \
    if (E == 32 * KS && R == 16 * DT) {                                                                              \
        static bool allowed = false;                                                                                 \
        if (!allowed) {                                                                                              \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(latent_prefill_kernel<KS, DT>),         \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, MAX_LDS);                 \
            if (e != hipSuccess) return static_cast<int>(e);                                                         \
            allowed = true;                                                                                          \
        }                                                                                                            \
        latent_prefill_kernel<KS, DT><<<dim3(n_tiles_upper, nsplit), 256, lds, stream>>>(                            \
            static_cast<const bf16_t*>(qa), static_cast<const bf16_t*>(k_pages), static_cast<const bf16_t*>(vt_pages), \
            block_tables, max_blocks, cu_q, ctx_len, n_seqs, H, page_size, sl2, window, static_cast<bf16_t*>(o_lat), \
            nsplit, partials, single_tokens);                                                                        \
        MLLM_LAUNCH_CHECK();                                                                                         \
        if (nsplit > 1) {                                                                                            \
            latent_merge_kernel<<<(n_rows + 3) / 4, 256, 0, stream>>>(partials, n_rows, nsplit, R,                   \
                                                                     static_cast<bf16_t*>(o_lat));                  \
            MLLM_LAUNCH_CHECK();                                                                                     \
        }                                                                                                            \
        return 0;                                                                                                    \
    }
    LP_CASE(4, 6) LP_CASE(3, 4) LP_CASE(5, 8) LP_CASE(9, 16) LP_CASE(17, 32) LP_CASE(18, 32)
#undef LP_CASE
    return -2;
}

int mllm_latent_expand(const void* o_lat, int ldo, const void* w_uv, int ldw, void* out, int ldout, int T, int H, int Dv, int R,
                       int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (dtype == MLLM_BF16 && R % 32 == 0 && ldo % 8 == 0 && ldw % 8 == 0 && (reinterpret_cast<uintptr_t>(o_lat) & 15) == 0 &&
        (reinterpret_cast<uintptr_t>(w_uv) & 15) == 0) {
        head_linear_mfma_kernel<<<dim3((T + 63) / 64, H, (Dv + 63) / 64), 256, 0, stream>>>(
            static_cast<const bf16_t*>(o_lat), ldo, R, static_cast<const bf16_t*>(w_uv), ldw, Dv, 0, static_cast<bf16_t*>(out), ldout, Dv, T, Dv,
            R, nullptr, 0, 0, 0.0);
        MLLM_LAUNCH_CHECK();
        return 0;
    }
    const dim3 grid((H * Dv + 3) / 4, std::min((T + 7) / 8, 64));
    if (dtype == MLLM_F32)
        latent_expand_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(o_lat), ldo, static_cast<const float*>(w_uv), ldw,
                                                              static_cast<float*>(out), ldout, T, H, Dv, R);
    else
        latent_expand_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<const bf16_t*>(o_lat), ldo, static_cast<const bf16_t*>(w_uv), ldw,
                                                               static_cast<bf16_t*>(out), ldout, T, H, Dv, R);
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
