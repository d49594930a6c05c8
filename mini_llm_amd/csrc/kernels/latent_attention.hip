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
//   page row slots[t] = [ rmsnorm(dkv[t, :R]) * wkv | turned dkv[t, R:R+Dr] ]   (if dkv is given and slot >= 0)
// The first rot_dims of the Dr columns are turned in interleaved pairs, the rest pass unchanged.
template <typename T>
__global__ void __launch_bounds__(64)
latent_prepare_kernel(const float* __restrict__ dq, int ld_dq, int Rq, const float* __restrict__ wq, T* __restrict__ cq,
                      int ld_cq, const float* __restrict__ dkv, int ld_dkv, int R, int Dr, const float* __restrict__ wkv,
                      T* __restrict__ pages, const int* __restrict__ slots, const int* __restrict__ positions, float eps,
                      double log2_base, int rot_dims) {
    const int t = blockIdx.x, lane = threadIdx.x;
    {
        const float* row = dq + static_cast<size_t>(t) * ld_dq;
        float ss = 0.f;
        for (int i = lane; i < Rq; i += 64) ss += row[i] * row[i];
        const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Rq) + eps);
        T* o = cq + static_cast<size_t>(t) * ld_cq;
        for (int i = lane; i < Rq; i += 64) o[i] = from_float<T>(row[i] * inv * wq[i]);
    }
    if (dkv == nullptr) return;
    const int slot = slots[t];
    if (slot < 0) return;
    const float* row = dkv + static_cast<size_t>(t) * ld_dkv;
    T* o = pages + static_cast<size_t>(slot) * (R + Dr);
    float ss = 0.f;
    for (int i = lane; i < R; i += 64) ss += row[i] * row[i];
    const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(R) + eps);
    for (int i = lane; i < R; i += 64) o[i] = from_float<T>(row[i] * inv * wkv[i]);
    const int pos = positions[t];
    for (int i = lane; i < rot_dims / 2; i += 64) {
        float a, b;
        turn_pair(row[R + 2 * i], row[R + 2 * i + 1], pos, i, log2_base, rot_dims, a, b);
        o[R + 2 * i] = from_float<T>(a);
        o[R + 2 * i + 1] = from_float<T>(b);
    }
    for (int i = rot_dims + lane; i < Dr; i += 64) o[R + i] = from_float<T>(row[R + i]);
}

// Queries into the latent space. q rows: per head [Dn plain | Dr to be turned]; w_uk [H * Dn, R] (row h*Dn + d
// expands latent column r into the head's plain key dimension d). For 8 tokens and one head a workgroup:
//   qa[t, h, r] = sum_d q[t, h, d] * w_uk[h*Dn + d, r]      (thread per r: the weight reads are coalesced)
//   qa[t, h, R + i] = the turned rotary part of q[t, h]
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
        const T* wcol = w_uk + static_cast<size_t>(h) * Dn * ldw + r;
        for (int d = 0; d < Dn; ++d) {
            const float wv = to_float(wcol[static_cast<size_t>(d) * ldw]);
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
    float* q_s = lds;
    float* o_s = q_s + HG * E;
    float* p_s = o_s + HG * R;
    T* k_s = reinterpret_cast<T*>(p_s + 4 * 64);
    const int t = blockIdx.x, h0 = blockIdx.y * HG, nh = min(HG, H - h0);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const int pos = positions[t];
    const int* table = block_tables + static_cast<size_t>(token_seq[t]) * max_blocks;
    for (int i = threadIdx.x; i < nh * E; i += 256)
        q_s[i] = to_float(qa[static_cast<size_t>(t) * ldqa + h0 * E + i]) * scale_log2;
    for (int i = threadIdx.x; i < nh * R; i += 256) o_s[i] = 0.f;
    // per head of this wavefront: running maximum and sum (up to 8 heads a wavefront: HG <= 32)
    float m_run[8], l_run[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) { m_run[u] = -INFINITY; l_run[u] = 0.f; }
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int words = sizeof(T) == 2 ? E / 2 : E;           // 32-bit words of a key row (E even for bfloat16)
    for (int k0 = lo; k0 <= pos; k0 += 64) {
        const int nk = min(64, pos + 1 - k0);
        __syncthreads();                                   // the tile before is used up
        for (int i = threadIdx.x; i < nk * words; i += 256) {
            const int j = i / words, c = i % words, kp = k0 + j;
            const size_t row = static_cast<size_t>(table[kp / page_size]) * page_size + kp % page_size;
            reinterpret_cast<uint32_t*>(k_s)[j * KS + c] = reinterpret_cast<const uint32_t*>(pages + row * E)[c];
        }
        __syncthreads();
        const uint32_t* kw = reinterpret_cast<const uint32_t*>(k_s) + min(lane, nk - 1) * KS;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int hh = wave + 4 * u;
            if (hh < nh) {
                const float* qh = q_s + hh * E;
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

constexpr int MAX_LDS = 160 * 1024;

}  // namespace

extern "C" {

// See latent_prepare_kernel. dkv may be null (a layer that reads another layer's pages). -1: an odd rot_dims
// or one beyond Dr.
int mllm_latent_prepare(const float* dq, int ld_dq, int Rq, const float* wq, void* cq, int ld_cq, const float* dkv, int ld_dkv,
                        int R, int Dr, const float* wkv, void* pages, const int* slots, const int* positions, int T, float eps,
                        double base, int rot_dims, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (rot_dims < 0 || rot_dims % 2 != 0 || rot_dims > Dr || !(base > 0)) return -1;
    const double l2 = log2(base);
    if (dtype == MLLM_F32)
        latent_prepare_kernel<float><<<T, 64, 0, stream>>>(dq, ld_dq, Rq, wq, static_cast<float*>(cq), ld_cq, dkv, ld_dkv, R, Dr, wkv,
                                                           static_cast<float*>(pages), slots, positions, eps, l2, rot_dims);
    else
        latent_prepare_kernel<bf16_t><<<T, 64, 0, stream>>>(dq, ld_dq, Rq, wq, static_cast<bf16_t*>(cq), ld_cq, dkv, ld_dkv, R, Dr, wkv,
                                                            static_cast<bf16_t*>(pages), slots, positions, eps, l2, rot_dims);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// See latent_absorb_kernel. -1: rot_dims odd or beyond Dr, Dr odd; -2: Dn too large for the LDS.
int mllm_latent_absorb(const void* q, int ldq, const void* w_uk, int ldw, void* qa, int ldqa, const int* positions, int T, int H,
                       int Dn, int Dr, int R, double base, int rot_dims, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (rot_dims < 0 || rot_dims % 2 != 0 || rot_dims > Dr || Dr % 2 != 0 || !(base > 0)) return -1;
    const size_t lds = static_cast<size_t>(8) * Dn * sizeof(float);
    if (lds > 64 * 1024) return -2;
    const dim3 grid((R + 255) / 256, H, (T + 7) / 8);
    const double l2 = log2(base);
    if (dtype == MLLM_F32)
        latent_absorb_kernel<float><<<grid, 256, lds, stream>>>(static_cast<const float*>(q), ldq, static_cast<const float*>(w_uk), ldw,
                                                                static_cast<float*>(qa), ldqa, positions, T, H, Dn, Dr, R, l2, rot_dims);
    else
        latent_absorb_kernel<bf16_t><<<grid, 256, lds, stream>>>(static_cast<const bf16_t*>(q), ldq, static_cast<const bf16_t*>(w_uk), ldw,
                                                                 static_cast<bf16_t*>(qa), ldqa, positions, T, H, Dn, Dr, R, l2, rot_dims);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// See latent_attention_kernel. -1: sizes the kernel's accesses do not allow (E odd in bfloat16); -2: a head's
// rows do not fit the LDS.
int mllm_latent_attention(const void* qa, int ldqa, const void* pages, const int* block_tables, int max_blocks,
                          const int* token_seq, const int* positions, int T, int H, int R, int Dr, int page_size, float scale,
                          int window, void* o_lat, int ldo, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    const int E = R + Dr, esz = dtype == MLLM_F32 ? 4 : 2;
    if (H < 1 || R < 1 || Dr < 0 || page_size < 1 || (dtype != MLLM_F32 && E % 2 != 0)) return -1;
    if ((reinterpret_cast<uintptr_t>(pages) & 3) != 0) return -1;
    int words = dtype == MLLM_F32 ? E : E / 2;
    const int KS = words | 1;                                    // an odd row stride, in 32-bit words
    auto lds_for = [&](int hg) {
        return static_cast<size_t>(hg) * (E + R) * 4 + 4 * 64 * 4 + static_cast<size_t>(64) * KS * 4;
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

int mllm_latent_expand(const void* o_lat, int ldo, const void* w_uv, int ldw, void* out, int ldout, int T, int H, int Dv, int R,
                       int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
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
