// Hybrid-mixer LM engine: a decoder whose layers mix tokens either with a linear recurrence (HGRN2, mLSTM, a real-gated diagonal
// unit behind a short convolution, a matrix state with token shift and per-channel decay, retention, the gated delta rule behind
// short convolutions) or with attention over a paged cache (a sliding window that also keeps one mean key / value per block of
// older tokens, plain causal attention with normed q / k / v -- optionally behind a short convolution, rotated, with a softmax
// sink --, or attention over a cached low-rank latent).  Two mixers may run side by side on one input; a layer is sequential or
// parallel, with an optional layer scale; its feed-forward is dense or a routed mixture of experts.  A contiguous range of layers
// may run several times with the same weights; every run owns its cache or recurrent state.
//
// Numeric rule of this engine: the residual stream, norms, rotary angles, attention scores / softmax, gates, decays and every
// recurrent state are fp32.  The engine's dtype (bf16 or fp32) is the storage of the large matrices, of the K / V cache and of
// the GEMM operands (fp32 accumulation either way); fp32 mode multiplies in plain fp32 FMA.
// One step = a ragged set of rows: each request contributes its next tokens (a prompt portion or one decoded token); rows of
// one request are contiguous and in position order.  Nothing a row computes depends on which other rows share the step:
// every reduction runs in an order fixed by the row's own sizes.
#include <math.h>

#include <vector>

#include "vox_internal.h"

namespace {

typedef __bf16 hb_bf16x8 __attribute__((ext_vector_type(8)));
typedef float hb_f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float hb_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float hb_wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
// sum of v over a block of 256 threads in a fixed order: butterfly per wave, the four wave sums added in wave order
__device__ __forceinline__ float hb_block_sum256(float v, float* red) {
    v = hb_wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return ((red[0] + red[1]) + red[2]) + red[3];
}
__device__ __forceinline__ float hb_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float hb_logsigmoid(float x) { return fminf(x, 0.0f) - log1pf(expf(-fabsf(x))); }

__device__ __forceinline__ float hb_ld(const float* p) { return *p; }
__device__ __forceinline__ float hb_ld(const bf16_t* p) { return bf2f(*p); }
__device__ __forceinline__ void hb_st(float* p, float v) { *p = v; }
__device__ __forceinline__ void hb_st(bf16_t* p, float v) { *p = f2bf(v); }
// what a GEMM operand of the engine's dtype sees of an fp32 activation
template <typename T> __device__ __forceinline__ float hb_operand(float v);
template <> __device__ __forceinline__ float hb_operand<float>(float v) { return v; }
template <> __device__ __forceinline__ float hb_operand<bf16_t>(float v) { return bfround(v); }

// A lane-chunked dot product in k_hb_gemv's order: chunks of CH at lane*CH + 64*CH*i, then a butterfly.  xs multiplies x before it
// becomes an operand.
template <typename T>
__device__ __forceinline__ float hb_dot_wave(const T* w, const float* x, int K, bool vec, int lane, float xs = 1.0f) {
    constexpr int CH = sizeof(T) == 2 ? 8 : 4;
    float a = 0.f;
    if (vec) {
        for (int k = lane * CH; k < K; k += 64 * CH) {
            float wv[CH];
            if (sizeof(T) == 2) {
                const uint4 u = *(const uint4*)(w + k);
                wv[0] = bflo(u.x); wv[1] = bfhi(u.x); wv[2] = bflo(u.y); wv[3] = bfhi(u.y);
                if (CH == 8) { wv[4] = bflo(u.z); wv[5] = bfhi(u.z); wv[6] = bflo(u.w); wv[7] = bfhi(u.w); }
            } else {
                const float4 u = *(const float4*)(w + k);
                wv[0] = u.x; wv[1] = u.y; wv[2] = u.z; wv[3] = u.w;
            }
#pragma unroll
            for (int i = 0; i < CH; ++i) a = fmaf(wv[i], hb_operand<T>(x[k + i] * xs), a);
        }
    } else {
        for (int k = lane; k < K; k += 64) a = fmaf(hb_ld(w + k), hb_operand<T>(x[k] * xs), a);
    }
    return hb_wave_sum(a);
}
// HB_EPI_SOFTCAP: v <- arg * tanh(v / arg) (arg = the product's hb_rowmap::epi_arg)
// HB_EPI_RESID_SCALED: c += v * col_scale[column] (a layer scale; arg = that column's entry); HB_EPI_SCALE: v <- v * arg
enum { HB_EPI_STORE = 0, HB_EPI_GELU = 1, HB_EPI_RESID = 2, HB_EPI_TANH = 3, HB_EPI_SOFTCAP = 4, HB_EPI_RESID_SCALED = 5, HB_EPI_SCALE = 6 };
template <int EPI> __device__ __forceinline__ void hb_epilogue(float* c, float acc, float bias, float arg = 0.f) {
    float v = acc + bias;
    if (EPI == HB_EPI_GELU) v = 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
    if (EPI == HB_EPI_TANH) v = tanhf(v);
    if (EPI == HB_EPI_SOFTCAP) v = arg * tanhf(v / arg);
    if (EPI == HB_EPI_SCALE) v = v * arg;
    if (EPI == HB_EPI_RESID) v = *c + v;
    if (EPI == HB_EPI_RESID_SCALED) v = *c + v * arg;
    *c = v;
}
__device__ __forceinline__ float hb_gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.79788456080286535588f * (z + 0.044715f * z * z * z)));
}
// Several products in one launch: product z uses the matrix Wt + z*w_stride, the activations A + z*a_stride, the outputs
// C + z*c_stride and the bias + z*b_stride (a strided batch: block-diagonal matrices, projections that each read their own input).
// count != NULL (routed experts): product z takes the gathered rows list[z*cap + 0 .. count[z]); the A row of list entry v is
// v / a_div, its C row is v; a_scale != NULL: the A row of entry v is multiplied by a_scale[v] before it becomes an operand.
struct hb_rowmap {
    const int* count;
    const int* list;
    int cap, a_div;
    long w_stride, a_stride, c_stride, b_stride;
    const float* a_scale;
    float epi_arg;
    const float* col_scale;     // HB_EPI_RESID_SCALED: [N] fp32
};
static inline hb_rowmap hb_plain() { return hb_rowmap{nullptr, nullptr, 0, 1, 0, 0, 0, 0, nullptr, 0.f, nullptr}; }
template <int EPI> __device__ __forceinline__ float hb_epi_arg(const hb_rowmap& rm, int col) {
    return EPI == HB_EPI_RESID_SCALED ? rm.col_scale[col] : rm.epi_arg;
}

// ---- embedding gather: x[row] = table[id]; the second half of both residual buffers keeps the embedding output ----------
// A bigram table (bg.table != NULL) adds row (prev * mul_prev + id * mul_cur) mod buckets, prev being the token before this one in its
// sequence: the previous row of the request, or what the request's state slot remembers, or nothing at position 0 (row `buckets`).
// Steps with one row per request (bg.store) also leave the row's id in the slot; other steps do that in k_hb_store_prev, after every
// block of this launch has read its predecessor.
struct hb_bigram {
    const void* table;
    int* prev;              // [slots]
    int buckets, mul_prev, mul_cur, store;
};
__device__ __forceinline__ int hb_clamp_id(int id, int vocab) { return id < 0 ? 0 : (id >= vocab ? vocab - 1 : id); }
template <typename T>
__global__ __launch_bounds__(256) void k_hb_embed(const T* table, const int* ids, int id_stride, float* xa, float* xb, int W, int vocab,
                                                  float scale, hb_bigram bg, const int* pos, const int* row_req, const int* req_rows,
                                                  const int* req_state) {
    const int row = blockIdx.x;
    const int id = hb_clamp_id(ids[(size_t)row * id_stride], vocab);
    const T* extra = nullptr;
    if (bg.table) {
        const int r = row_req[row];
        long b = bg.buckets;
        if (pos[row] > 0) {
            const int before = row > req_rows[r] ? hb_clamp_id(ids[(size_t)(row - 1) * id_stride], vocab) : bg.prev[req_state[r]];
            b = ((long)before * bg.mul_prev + (long)id * bg.mul_cur) % bg.buckets;
        }
        extra = (const T*)bg.table + (size_t)b * W;
        __syncthreads();        // (one row per request: the slot is read above by every thread before thread 0 replaces it)
        if (bg.store && threadIdx.x == 0) bg.prev[req_state[r]] = id;
    }
    for (int i = threadIdx.x; i < W; i += 256) {
        float v = hb_ld(table + (size_t)id * W + i) * scale;
        if (extra) v += hb_ld(extra + i);
        xa[(size_t)row * 2 * W + i] = v;
        xa[(size_t)row * 2 * W + W + i] = v;
        xb[(size_t)row * 2 * W + W + i] = v;
    }
}
__global__ void k_hb_store_prev(const int* ids, int id_stride, int vocab, const int* req_rows, const int* req_state, int* prev, int n_req) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r < n_req && req_rows[r + 1] > req_rows[r]) prev[req_state[r]] = hb_clamp_id(ids[(size_t)(req_rows[r + 1] - 1) * id_stride], vocab);
}

// ---- layer norm with a weight and no bias, fp32; optional row gather ----------------------------------------------------
// mean, then the mean of the squared deviations (two passes over the row).  NV > 0: the row (width <= 256 * NV) is read once
// into registers; NV = 0: any width, three reads.  Same sums in the same order either way.
template <int NV>
__global__ __launch_bounds__(256) void k_hb_layernorm(const float* x, long ldx, const int* rows, const float* w, float* y, long ldy, int W,
                                                      float eps) {
    __shared__ float red[2][4];
    const int r = blockIdx.x, src = rows ? rows[r] : r;
    const float* xr = x + (size_t)src * ldx;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    float xv[NV > 0 ? NV : 1];
    float s = 0.f;
    if (NV > 0) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int k = threadIdx.x + i * 256;
            xv[i] = k < W ? xr[k] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) s += xv[i];
    } else {
        for (int i = threadIdx.x; i < W; i += 256) s += xr[i];
    }
    s = hb_wave_sum(s);
    if (lane == 0) red[0][wv] = s;
    __syncthreads();
    const float mean = (((red[0][0] + red[0][1]) + red[0][2]) + red[0][3]) / (float)W;
    float q = 0.f;
    if (NV > 0) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const float d = threadIdx.x + i * 256 < W ? xv[i] - mean : 0.f;
            q += d * d;
        }
    } else {
        for (int i = threadIdx.x; i < W; i += 256) {
            const float d = xr[i] - mean;
            q += d * d;
        }
    }
    q = hb_wave_sum(q);
    if (lane == 0) red[1][wv] = q;
    __syncthreads();
    const float var = (((red[1][0] + red[1][1]) + red[1][2]) + red[1][3]) / (float)W;
    const float inv = 1.0f / sqrtf(var + eps);
    if (NV > 0) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int k = threadIdx.x + i * 256;
            if (k < W) y[(size_t)r * ldy + k] = (xv[i] - mean) * inv * w[k];
        }
    } else {
        for (int i = threadIdx.x; i < W; i += 256) y[(size_t)r * ldy + i] = (xr[i] - mean) * inv * w[i];
    }
}
static void hb_layernorm(hipStream_t st, int n, const float* x, long ldx, const int* rows, const float* w, float* y, long ldy, int W, float eps) {
    if (W <= 1024) hipLaunchKernelGGL(k_hb_layernorm<4>, dim3(n), dim3(256), 0, st, x, ldx, rows, w, y, ldy, W, eps);
    else if (W <= 4096) hipLaunchKernelGGL(k_hb_layernorm<16>, dim3(n), dim3(256), 0, st, x, ldx, rows, w, y, ldy, W, eps);
    else hipLaunchKernelGGL(k_hb_layernorm<0>, dim3(n), dim3(256), 0, st, x, ldx, rows, w, y, ldy, W, eps);
}

// ---- RMS norm over `groups` equal consecutive slices of the row, fp32; optional row gather; one or two weights --------------
// Every slice is divided by its own sqrt(mean square + eps); y1 = that * w1 and (w2 != NULL) y2 = that * w2: the two norms of a
// parallel layer share their statistics.  One wave per slice (waves take slices w, w + 4, ...): lane-strided sum of squares, then
// a butterfly — an order fixed by the slice length.
__global__ __launch_bounds__(256) void k_hb_rms_groups(const float* x, long ldx, const int* rows, const float* w1, float* y1, const float* w2,
                                                       float* y2, long ldy, int W, int groups, float eps) {
    const int r = blockIdx.x, src = rows ? rows[r] : r, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int Wg = W / groups;
    // 16-byte requests when every slice and row starts on one (a property of the sizes, not of the step); the lane-strided order of
    // the scalar form otherwise
    const bool vec = (Wg % 4 == 0) && (ldx % 4 == 0) && (ldy % 4 == 0) && (((size_t)x | (size_t)y1 | (size_t)w1 | (size_t)y2 | (size_t)w2) & 15) == 0;
    for (int g = wv + 4 * blockIdx.y; g < groups; g += 4 * gridDim.y) {
        const float* xr = x + (size_t)src * ldx + (size_t)g * Wg;
        float ss = 0.f;
        if (vec) {
            for (int i = lane * 4; i < Wg; i += 256) {
                const float4 v = *(const float4*)(xr + i);
                ss = fmaf(v.x, v.x, ss); ss = fmaf(v.y, v.y, ss); ss = fmaf(v.z, v.z, ss); ss = fmaf(v.w, v.w, ss);
            }
        } else {
            for (int i = lane; i < Wg; i += 64) ss = fmaf(xr[i], xr[i], ss);
        }
        ss = hb_wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)Wg + eps);
        if (vec) {
            for (int i = lane * 4; i < Wg; i += 256) {
                const float4 v = *(const float4*)(xr + i), a = *(const float4*)(w1 + g * Wg + i);
                *(float4*)(y1 + (size_t)r * ldy + g * Wg + i) = make_float4(v.x * inv * a.x, v.y * inv * a.y, v.z * inv * a.z, v.w * inv * a.w);
                if (w2) {
                    const float4 b2 = *(const float4*)(w2 + g * Wg + i);
                    *(float4*)(y2 + (size_t)r * ldy + g * Wg + i) = make_float4(v.x * inv * b2.x, v.y * inv * b2.y, v.z * inv * b2.z, v.w * inv * b2.w);
                }
            }
        } else {
            for (int i = lane; i < Wg; i += 64) {
                const float v = xr[i] * inv;
                y1[(size_t)r * ldy + g * Wg + i] = v * w1[g * Wg + i];
                if (w2) y2[(size_t)r * ldy + g * Wg + i] = v * w2[g * Wg + i];
            }
        }
    }
}

// The same norm over ONE slice (the whole row), all four waves on it: thread-strided sum of squares, butterfly per wave, the four wave
// sums added in wave order -- an order fixed by the width.
__global__ __launch_bounds__(256) void k_hb_rms_row(const float* x, long ldx, const int* rows, const float* w1, float* y1, const float* w2, float* y2,
                                                    long ldy, int W, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x, src = rows ? rows[r] : r, tid = threadIdx.x;
    const float* xr = x + (size_t)src * ldx;
    const bool vec = (W % 4 == 0) && (ldx % 4 == 0) && (ldy % 4 == 0) && (((size_t)x | (size_t)y1 | (size_t)w1 | (size_t)y2 | (size_t)w2) & 15) == 0;
    float ss = 0.f;
    if (vec) {
        for (int i = tid * 4; i < W; i += 1024) {
            const float4 v = *(const float4*)(xr + i);
            ss = fmaf(v.x, v.x, ss); ss = fmaf(v.y, v.y, ss); ss = fmaf(v.z, v.z, ss); ss = fmaf(v.w, v.w, ss);
        }
    } else {
        for (int i = tid; i < W; i += 256) ss = fmaf(xr[i], xr[i], ss);
    }
    const float inv = 1.0f / sqrtf(hb_block_sum256(ss, red) / (float)W + eps);
    if (vec) {
        for (int i = tid * 4; i < W; i += 1024) {
            const float4 v = *(const float4*)(xr + i), a = *(const float4*)(w1 + i);
            *(float4*)(y1 + (size_t)r * ldy + i) = make_float4(v.x * inv * a.x, v.y * inv * a.y, v.z * inv * a.z, v.w * inv * a.w);
            if (w2) {
                const float4 b2 = *(const float4*)(w2 + i);
                *(float4*)(y2 + (size_t)r * ldy + i) = make_float4(v.x * inv * b2.x, v.y * inv * b2.y, v.z * inv * b2.z, v.w * inv * b2.w);
            }
        }
    } else {
        for (int i = tid; i < W; i += 256) {
            const float v = xr[i] * inv;
            y1[(size_t)r * ldy + i] = v * w1[i];
            if (w2) y2[(size_t)r * ldy + i] = v * w2[i];
        }
    }
}

// ---- GEMM  C[M,N] (+)= A[M,K] . W[N,K]^T + bias ---------------------------------------------------------------------------
// bf16: both operands staged in LDS as bf16 (activations rounded once), v_mfma_f32_16x16x32_bf16; four waves, 64 output columns
// per block, BM = 64 (2 x 2 tiles per wave) or BM = 16 (one tile per wave).  Every edge (M, N, K) is guarded at the LDS fill.
template <int BM, int EPI>
__global__ __launch_bounds__(256) void k_hb_gemm_bf16(const float* A, long lda, const bf16_t* Wt, const float* bias, float* C, long ldc, int M,
                                                      int N, int K, hb_rowmap rm) {
    constexpr int BK = 64, LD = BK + 8;
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * LD];
    __shared__ __attribute__((aligned(16))) bf16_t Ws[64 * LD];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * 64;
    const int* lst = nullptr;
    Wt += (size_t)blockIdx.z * rm.w_stride;
    A += (size_t)blockIdx.z * rm.a_stride;
    C += (size_t)blockIdx.z * rm.c_stride;
    if (bias) bias += (size_t)blockIdx.z * rm.b_stride;
    if (rm.count) {
        M = rm.count[blockIdx.z];
        if (m0 >= M) return;
        lst = rm.list + (size_t)blockIdx.z * rm.cap;
    }
    constexpr int MT = BM == 64 ? 2 : 1, NT = BM == 64 ? 2 : 1;
    const int mt0 = BM == 64 ? (wv >> 1) * 2 : 0, nt0 = BM == 64 ? (wv & 1) * 2 : wv;
    hb_f32x4 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = hb_f32x4{0.f, 0.f, 0.f, 0.f};
    const bool a_vec = (K % 4 == 0) && (lda % 4 == 0) && ((((size_t)A) & 15) == 0);
    const bool w_vec = (K % 8 == 0) && ((((size_t)Wt) & 15) == 0);
    // the next k-tile's global requests are issued before the current tile's products and land in registers meanwhile
    constexpr int NA = BM * 16 / 256;
    float4 ra[NA];
    uint4 rw[2];
    const float* arow[NA];
    float asc[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        const int gm = m0 + ((tid + i * 256) >> 4);
        arow[i] = gm < M ? A + (size_t)(lst ? lst[gm] / rm.a_div : gm) * lda : nullptr;
        asc[i] = gm < M && lst && rm.a_scale ? rm.a_scale[lst[gm]] : 1.0f;
    }
    auto fetch = [&](int k0) {
        // A tile: BM x 64 fp32
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const int gk = k0 + ((tid + i * 256) & 15) * 4;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (arow[i]) {
                const float* p = arow[i] + gk;
                if (a_vec && gk + 3 < K) v = *(const float4*)p;
                else {
                    if (gk < K) v.x = p[0];
                    if (gk + 1 < K) v.y = p[1];
                    if (gk + 2 < K) v.z = p[2];
                    if (gk + 3 < K) v.w = p[3];
                }
            }
            ra[i] = v;
        }
        // W tile: 64 x 64 bf16
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = tid + i * 256;
            const int gn = n0 + (idx >> 3), gk = k0 + (idx & 7) * 8;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (gn < N) {
                const bf16_t* p = Wt + (size_t)gn * K + gk;
                if (w_vec && gk + 7 < K) v = *(const uint4*)p;
                else {
                    bf16_t t[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) t[e] = gk + e < K ? p[e] : (bf16_t)0;
                    v.x = t[0] | ((u32)t[1] << 16); v.y = t[2] | ((u32)t[3] << 16);
                    v.z = t[4] | ((u32)t[5] << 16); v.w = t[6] | ((u32)t[7] << 16);
                }
            }
            rw[i] = v;
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const int idx = tid + i * 256;
            uint2 o;
            o.x = pack_bf2(ra[i].x * asc[i], ra[i].y * asc[i]);
            o.y = pack_bf2(ra[i].z * asc[i], ra[i].w * asc[i]);
            *(uint2*)(As + (idx >> 4) * LD + (idx & 15) * 4) = o;
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = tid + i * 256;
            *(uint4*)(Ws + (idx >> 3) * LD + (idx & 7) * 8) = rw[i];
        }
        __syncthreads();
        if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
        for (int ks = 0; ks < BK; ks += 32) {
            hb_bf16x8 af[MT], bfr[NT];
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                union { uint4 u; hb_bf16x8 b; } cv;
                cv.u = *(const uint4*)(As + ((mt0 + i) * 16 + (lane & 15)) * LD + ks + (lane >> 4) * 8);
                af[i] = cv.b;
            }
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                union { uint4 u; hb_bf16x8 b; } cv;
                cv.u = *(const uint4*)(Ws + ((nt0 + j) * 16 + (lane & 15)) * LD + ks + (lane >> 4) * 8);
                bfr[j] = cv.b;
            }
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int gn = n0 + (nt0 + j) * 16 + (lane & 15);
            if (gn >= N) continue;
            const float b = bias ? bias[gn] : 0.f;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int gm = m0 + (mt0 + i) * 16 + (lane >> 4) * 4 + r;
                if (gm < M) hb_epilogue<EPI>(C + (size_t)(lst ? lst[gm] : gm) * ldc + gn, acc[i][j][r], b, hb_epi_arg<EPI>(rm, gn));
            }
        }
}

// fp32: LDS-tiled FMA, 64 output columns per block, BM = 64 (4 x 4 per thread) or 16 (1 x 4 per thread); k ascending per element.
template <int BM, int EPI>
__global__ __launch_bounds__(256) void k_hb_gemm_f32(const float* A, long lda, const float* Wt, const float* bias, float* C, long ldc, int M,
                                                     int N, int K, hb_rowmap rm) {
    constexpr int BK = 16, RM = BM / 16;
    __shared__ float As[BK][BM + 4];
    __shared__ float Ws[BK][64 + 4];
    __shared__ int arow[BM];
    __shared__ float asc[BM];
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * 64;
    const int* lst = nullptr;
    Wt += (size_t)blockIdx.z * rm.w_stride;
    A += (size_t)blockIdx.z * rm.a_stride;
    C += (size_t)blockIdx.z * rm.c_stride;
    if (bias) bias += (size_t)blockIdx.z * rm.b_stride;
    if (rm.count) {
        M = rm.count[blockIdx.z];
        if (m0 >= M) return;
        lst = rm.list + (size_t)blockIdx.z * rm.cap;
    }
    for (int r = tid; r < BM; r += 256) {
        arow[r] = m0 + r < M ? (lst ? lst[m0 + r] : m0 + r) : -1;
        asc[r] = m0 + r < M && lst && rm.a_scale ? rm.a_scale[lst[m0 + r]] : 1.0f;
    }
    __syncthreads();
    float acc[RM][4];
#pragma unroll
    for (int i = 0; i < RM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += BK) {
        for (int idx = tid; idx < BM * BK; idx += 256) {
            const int r = idx / BK, c = idx % BK;
            const int gm = m0 + r, gk = k0 + c;
            As[c][r] = (gm < M && gk < K) ? A[(size_t)(lst ? arow[r] / rm.a_div : gm) * lda + gk] * asc[r] : 0.f;
        }
        for (int idx = tid; idx < 64 * BK; idx += 256) {
            const int r = idx / BK, c = idx % BK;
            const int gn = n0 + r, gk = k0 + c;
            Ws[c][r] = (gn < N && gk < K) ? Wt[(size_t)gn * K + gk] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float a[RM], b[4];
#pragma unroll
            for (int i = 0; i < RM; ++i) a[i] = As[k][ty * RM + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < RM; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < RM; ++i) {
        const int gm = m0 + ty * RM + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tx * 4 + j;
            if (gn < N) hb_epilogue<EPI>(C + (size_t)arow[ty * RM + i] * ldc + gn, acc[i][j], bias ? bias[gn] : 0.f, hb_epi_arg<EPI>(rm, gn));
        }
    }
}

// 1..8 rows (decode): a wave streams CPW weight rows (output columns) at once, 16 bytes per lane and request, against one read of
// the activations; lanes own k-chunks c, c + 64, ...; butterfly at the end.  The order of each output's sum depends on K only.
template <typename T, int MR, int EPI, int HB_GEMV_CPW>
__global__ __launch_bounds__(256) void k_hb_gemv(const float* A, long lda, const T* Wt, const float* bias, float* C, long ldc, int M, int N,
                                                 int K, hb_rowmap rm) {
    const int lane = threadIdx.x & 63, n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * HB_GEMV_CPW;
    if (n0 >= N) return;
    Wt += (size_t)blockIdx.y * rm.w_stride;
    A += (size_t)blockIdx.y * rm.a_stride;
    C += (size_t)blockIdx.y * rm.c_stride;
    if (bias) bias += (size_t)blockIdx.y * rm.b_stride;
    constexpr int CH = sizeof(T) == 2 ? 8 : 4;
    float acc[MR][HB_GEMV_CPW];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int j = 0; j < HB_GEMV_CPW; ++j) acc[m][j] = 0.f;
    const T* wr[HB_GEMV_CPW];
#pragma unroll
    for (int j = 0; j < HB_GEMV_CPW; ++j) wr[j] = Wt + (size_t)(n0 + j < N ? n0 + j : N - 1) * K;
    const bool vec = (K % CH == 0) && ((((size_t)Wt) & 15) == 0) && (lda % 4 == 0) && ((((size_t)A) & 15) == 0);
    if (vec) {
        for (int k = lane * CH; k < K; k += 64 * CH) {
            float w[HB_GEMV_CPW][CH];
#pragma unroll
            for (int j = 0; j < HB_GEMV_CPW; ++j) {
                if (sizeof(T) == 2) {
                    const uint4 u = *(const uint4*)(wr[j] + k);
                    w[j][0] = bflo(u.x); w[j][1] = bfhi(u.x); w[j][2] = bflo(u.y); w[j][3] = bfhi(u.y);
                    if (CH == 8) { w[j][4] = bflo(u.z); w[j][5] = bfhi(u.z); w[j][6] = bflo(u.w); w[j][7] = bfhi(u.w); }
                } else {
                    const float4 u = *(const float4*)(wr[j] + k);
                    w[j][0] = u.x; w[j][1] = u.y; w[j][2] = u.z; w[j][3] = u.w;
                }
            }
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                if (m >= M) break;
                const float* xr = A + (size_t)m * lda + k;
#pragma unroll
                for (int e = 0; e < CH; e += 4) {
                    const float4 x4 = *(const float4*)(xr + e);
                    const float x[4] = {hb_operand<T>(x4.x), hb_operand<T>(x4.y), hb_operand<T>(x4.z), hb_operand<T>(x4.w)};
#pragma unroll
                    for (int j = 0; j < HB_GEMV_CPW; ++j) {
                        acc[m][j] = fmaf(w[j][e], x[0], acc[m][j]);
                        acc[m][j] = fmaf(w[j][e + 1], x[1], acc[m][j]);
                        acc[m][j] = fmaf(w[j][e + 2], x[2], acc[m][j]);
                        acc[m][j] = fmaf(w[j][e + 3], x[3], acc[m][j]);
                    }
                }
            }
        }
    } else {
        for (int k = lane; k < K; k += 64) {
#pragma unroll
            for (int j = 0; j < HB_GEMV_CPW; ++j) {
                const float w = hb_ld(wr[j] + k);
#pragma unroll
                for (int m = 0; m < MR; ++m)
                    if (m < M) acc[m][j] = fmaf(w, hb_operand<T>(A[(size_t)m * lda + k]), acc[m][j]);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int j = 0; j < HB_GEMV_CPW; ++j) {
            const float sum = hb_wave_sum(acc[m][j]);
            if (m < M && n0 + j < N && lane == 0) hb_epilogue<EPI>(C + (size_t)m * ldc + n0 + j, sum, bias ? bias[n0 + j] : 0.f, hb_epi_arg<EPI>(rm, n0 + j));
        }
}

// One-row steps: the weight-only LayerNorm of the row fused in front of the GEMV.  Every wave takes the row's statistics itself
// (mean, then the mean of the squared deviations; lane-chunked sums and a butterfly, an order fixed by K), so the row is read three
// times from cache instead of once from a normalised copy, and a dependent launch is saved.  Needs K % 8 == 0 (4 for fp32).
template <typename T, int EPI, int CPW>
__global__ __launch_bounds__(256) void k_hb_ln_gemv(const float* X, long ldx, const int* rows, const float* lnw, float eps, const T* Wt,
                                                    const float* bias, float* C, int N, int K, int rms, float epi_arg) {
    const int lane = threadIdx.x & 63, n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * CPW;
    if (n0 >= N) return;
    constexpr int CH = sizeof(T) == 2 ? 8 : 4;
    const float* xr = X + (size_t)(rows ? rows[0] : 0) * ldx;
    // rms != 0: the RMS norm over the whole row (no mean is taken off)
    float mean = 0.f;
    if (!rms) {
        float s = 0.f;
        for (int k = lane * CH; k < K; k += 64 * CH)
#pragma unroll
            for (int e = 0; e < CH; e += 4) {
                const float4 x4 = *(const float4*)(xr + k + e);
                s += x4.x; s += x4.y; s += x4.z; s += x4.w;
            }
        mean = hb_wave_sum(s) / (float)K;
    }
    float q = 0.f;
    for (int k = lane * CH; k < K; k += 64 * CH)
#pragma unroll
        for (int e = 0; e < CH; e += 4) {
            const float4 x4 = *(const float4*)(xr + k + e);
            const float d0 = x4.x - mean, d1 = x4.y - mean, d2 = x4.z - mean, d3 = x4.w - mean;
            q += d0 * d0; q += d1 * d1; q += d2 * d2; q += d3 * d3;
        }
    const float inv = 1.0f / sqrtf(hb_wave_sum(q) / (float)K + eps);
    float acc[CPW];
#pragma unroll
    for (int j = 0; j < CPW; ++j) acc[j] = 0.f;
    const T* wr[CPW];
#pragma unroll
    for (int j = 0; j < CPW; ++j) wr[j] = Wt + (size_t)(n0 + j < N ? n0 + j : N - 1) * K;
    for (int k = lane * CH; k < K; k += 64 * CH) {
        float w[CPW][CH];
#pragma unroll
        for (int j = 0; j < CPW; ++j) {
            if (sizeof(T) == 2) {
                const uint4 u = *(const uint4*)(wr[j] + k);
                w[j][0] = bflo(u.x); w[j][1] = bfhi(u.x); w[j][2] = bflo(u.y); w[j][3] = bfhi(u.y);
                if (CH == 8) { w[j][4] = bflo(u.z); w[j][5] = bfhi(u.z); w[j][6] = bflo(u.w); w[j][7] = bfhi(u.w); }
            } else {
                const float4 u = *(const float4*)(wr[j] + k);
                w[j][0] = u.x; w[j][1] = u.y; w[j][2] = u.z; w[j][3] = u.w;
            }
        }
#pragma unroll
        for (int e = 0; e < CH; e += 4) {
            const float4 x4 = *(const float4*)(xr + k + e), g4 = *(const float4*)(lnw + k + e);
            const float x[4] = {hb_operand<T>((x4.x - mean) * inv * g4.x), hb_operand<T>((x4.y - mean) * inv * g4.y),
                                hb_operand<T>((x4.z - mean) * inv * g4.z), hb_operand<T>((x4.w - mean) * inv * g4.w)};
#pragma unroll
            for (int j = 0; j < CPW; ++j) {
                acc[j] = fmaf(w[j][e], x[0], acc[j]);
                acc[j] = fmaf(w[j][e + 1], x[1], acc[j]);
                acc[j] = fmaf(w[j][e + 2], x[2], acc[j]);
                acc[j] = fmaf(w[j][e + 3], x[3], acc[j]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < CPW; ++j) {
        const float sum = hb_wave_sum(acc[j]);
        if (n0 + j < N && lane == 0) hb_epilogue<EPI>(C + n0 + j, sum, bias ? bias[n0 + j] : 0.f, epi_arg);
    }
}
// true: the fused form was launched (one row, aligned operands); false: the caller normalises and multiplies in two launches
template <typename T>
bool hb_try_ln_gemv(hipStream_t st, int epi, const float* X, long ldx, const int* rows, const float* lnw, float eps, const T* W, const float* bias,
                    float* C, int N, int K, int rms = 0, float epi_arg = 0.f) {
    constexpr int CH = sizeof(T) == 2 ? 8 : 4;
    if (K % CH || (ldx & 3) || ((size_t)X & 15) || ((size_t)W & 15) || ((size_t)lnw & 15)) return false;
    const bool wide = N >= 16 * 1024;
    const dim3 g(wide ? (N + 15) / 16 : (N + 3) / 4), b(256);
#define HB_LN(EPI_) \
    do { \
        if (wide) hipLaunchKernelGGL((k_hb_ln_gemv<T, EPI_, 4>), g, b, 0, st, X, ldx, rows, lnw, eps, W, bias, C, N, K, rms, epi_arg); \
        else hipLaunchKernelGGL((k_hb_ln_gemv<T, EPI_, 1>), g, b, 0, st, X, ldx, rows, lnw, eps, W, bias, C, N, K, rms, epi_arg); \
    } while (0)
    if (epi == HB_EPI_GELU) HB_LN(HB_EPI_GELU);
    else if (epi == HB_EPI_SCALE) HB_LN(HB_EPI_SCALE);
    else if (epi != HB_EPI_STORE) return false;
    else HB_LN(HB_EPI_STORE);
#undef HB_LN
    return true;
}

// 2..16 rows, bf16: one MFMA row tile; a block owns 16 output columns and its eight waves take the 32-wide k-steps w, w + 8, ...
// with both fragments straight from memory (the weight fragment is one 16-byte request per lane, the activation fragment two,
// converted to bf16 in registers); the eight partial tiles are added in wave order.  Needs K % 32 == 0.
template <int EPI>
__global__ __launch_bounds__(512) void k_hb_gemm_rows16(const float* A, long lda, const bf16_t* Wt, const float* bias, float* C, long ldc, int M,
                                                        int N, int K, hb_rowmap rm) {
    __shared__ float red[8][16][17];
    Wt += (size_t)blockIdx.y * rm.w_stride;
    A += (size_t)blockIdx.y * rm.a_stride;
    C += (size_t)blockIdx.y * rm.c_stride;
    if (bias) bias += (size_t)blockIdx.y * rm.b_stride;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int n0 = blockIdx.x * 16, col = lane & 15, kb = lane >> 4;
    const int nsteps = K >> 5;
    hb_f32x4 acc = hb_f32x4{0.f, 0.f, 0.f, 0.f};
    const bf16_t* wrow = Wt + (size_t)(n0 + col < N ? n0 + col : N - 1) * K + kb * 8;
    const float* arow = A + (size_t)(col < M ? col : M - 1) * lda + kb * 8;
    const bool rowok = col < M;
    constexpr int U = 8;
    for (int s0 = wv; s0 < nsteps; s0 += 8 * U) {
        uint4 wf[U];
        float4 a0[U], a1[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int sidx = s0 + 8 * u;
            const bool valid = sidx < nsteps;
            const int k = (valid ? sidx : s0) << 5;
            wf[u] = *(const uint4*)(wrow + k);
            a0[u] = *(const float4*)(arow + k);
            a1[u] = *(const float4*)(arow + k + 4);
            if (!valid || !rowok) { a0[u] = make_float4(0.f, 0.f, 0.f, 0.f); a1[u] = a0[u]; }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            union { uint4 q; hb_bf16x8 b; } af, bfv;
            af.q.x = pack_bf2(a0[u].x, a0[u].y); af.q.y = pack_bf2(a0[u].z, a0[u].w);
            af.q.z = pack_bf2(a1[u].x, a1[u].y); af.q.w = pack_bf2(a1[u].z, a1[u].w);
            bfv.q = wf[u];
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af.b, bfv.b, acc, 0, 0, 0);
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wv][kb * 4 + r][col] = acc[r];
    __syncthreads();
    if (wv == 0 && n0 + col < N) {
        const float bz = bias ? bias[n0 + col] : 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = kb * 4 + r;
            if (row < M) hb_epilogue<EPI>(C + (size_t)row * ldc + n0 + col, ((((((red[0][row][col] + red[1][row][col]) + red[2][row][col]) + red[3][row][col]) + red[4][row][col]) + red[5][row][col]) + red[6][row][col]) + red[7][row][col], bz, hb_epi_arg<EPI>(rm, n0 + col));
        }
    }
}
// every operand of every product of a strided batch is 16-byte aligned
static inline bool hb_batch_aligned(const hb_rowmap& rm, int nz, size_t wsize) {
    return nz == 1 || ((rm.w_stride * wsize) % 16 == 0 && (rm.a_stride * 4) % 16 == 0);
}
template <int EPI>
bool hb_try_rows16(hipStream_t st, const float* A, long lda, const bf16_t* W, const float* bias, float* C, long ldc, int M, int N, int K,
                   const hb_rowmap& rm, int nz) {
    if (M < 2 || M > 16 || (K & 31) || (lda & 3) || ((size_t)A & 15) || ((size_t)W & 15) || !hb_batch_aligned(rm, nz, 2)) return false;
    hipLaunchKernelGGL((k_hb_gemm_rows16<EPI>), dim3((N + 15) / 16, nz), dim3(512), 0, st, A, lda, W, bias, C, ldc, M, N, K, rm);
    return true;
}
template <int EPI>
bool hb_try_rows16(hipStream_t, const float*, long, const float*, const float*, float*, long, int, int, int, const hb_rowmap&, int) { return false; }

// rm.count != NULL: `groups` gathered GEMMs of at most M rows each in one launch (see hb_rowmap)
template <int EPI>
int hb_gemm_tiles(hipStream_t st, const float* A, long lda, const bf16_t* W, const float* bias, float* C, long ldc, int M, int N, int K,
                  hb_rowmap rm = hb_plain(), int groups = 1) {
    if (M <= 16) hipLaunchKernelGGL((k_hb_gemm_bf16<16, EPI>), dim3((N + 63) / 64, 1, groups), dim3(256), 0, st, A, lda, W, bias, C, ldc, M, N, K, rm);
    else hipLaunchKernelGGL((k_hb_gemm_bf16<64, EPI>), dim3((N + 63) / 64, (M + 63) / 64, groups), dim3(256), 0, st, A, lda, W, bias, C, ldc, M, N, K, rm);
    return VOX_OK;
}
template <int EPI>
int hb_gemm_tiles(hipStream_t st, const float* A, long lda, const float* W, const float* bias, float* C, long ldc, int M, int N, int K,
                  hb_rowmap rm = hb_plain(), int groups = 1) {
    if (M <= 16) hipLaunchKernelGGL((k_hb_gemm_f32<16, EPI>), dim3((N + 63) / 64, 1, groups), dim3(256), 0, st, A, lda, W, bias, C, ldc, M, N, K, rm);
    else hipLaunchKernelGGL((k_hb_gemm_f32<64, EPI>), dim3((N + 63) / 64, (M + 63) / 64, groups), dim3(256), 0, st, A, lda, W, bias, C, ldc, M, N, K, rm);
    return VOX_OK;
}
// nz > 1: a strided batch of nz products (rm gives the strides) in one launch
template <typename T, int EPI>
int hb_gemm_epi(hipStream_t st, const float* A, long lda, const T* W, const float* bias, float* C, long ldc, int M, int N, int K,
                const hb_rowmap& rm, int nz) {
    if (M <= 0 || N <= 0) return VOX_OK;
    // four columns per wave once that still leaves a block for every compute unit several times over
    const bool wide = N >= 16 * 1024;
    const dim3 g(wide ? (N + 15) / 16 : (N + 3) / 4, nz), b(256);
#define HB_GEMV(MR_) \
    do { \
        if (wide) hipLaunchKernelGGL((k_hb_gemv<T, MR_, EPI, 4>), g, b, 0, st, A, lda, W, bias, C, ldc, M, N, K, rm); \
        else hipLaunchKernelGGL((k_hb_gemv<T, MR_, EPI, 1>), g, b, 0, st, A, lda, W, bias, C, ldc, M, N, K, rm); \
    } while (0)
    if (hb_try_rows16<EPI>(st, A, lda, W, bias, C, ldc, M, N, K, rm, nz)) {}
    else if (M == 1) HB_GEMV(1);
    else if (M == 2) HB_GEMV(2);
    else if (M <= 4) HB_GEMV(4);
    else if (M <= 8) HB_GEMV(8);
#undef HB_GEMV
    else return hb_gemm_tiles<EPI>(st, A, lda, W, bias, C, ldc, M, N, K, rm, nz);
    return VOX_OK;
}
template <typename T>
int hb_gemm(hipStream_t st, int epi, const float* A, long lda, const T* W, const float* bias, float* C, long ldc, int M, int N, int K,
            const hb_rowmap& rm = hb_plain(), int nz = 1) {
    if (epi == HB_EPI_GELU) return hb_gemm_epi<T, HB_EPI_GELU>(st, A, lda, W, bias, C, ldc, M, N, K, rm, nz);
    if (epi == HB_EPI_RESID) return hb_gemm_epi<T, HB_EPI_RESID>(st, A, lda, W, bias, C, ldc, M, N, K, rm, nz);
    if (epi == HB_EPI_TANH) return hb_gemm_epi<T, HB_EPI_TANH>(st, A, lda, W, bias, C, ldc, M, N, K, rm, nz);
    if (epi == HB_EPI_SOFTCAP) return hb_gemm_epi<T, HB_EPI_SOFTCAP>(st, A, lda, W, bias, C, ldc, M, N, K, rm, nz);
    if (epi == HB_EPI_RESID_SCALED) return hb_gemm_epi<T, HB_EPI_RESID_SCALED>(st, A, lda, W, bias, C, ldc, M, N, K, rm, nz);
    if (epi == HB_EPI_SCALE) return hb_gemm_epi<T, HB_EPI_SCALE>(st, A, lda, W, bias, C, ldc, M, N, K, rm, nz);
    return hb_gemm_epi<T, HB_EPI_STORE>(st, A, lda, W, bias, C, ldc, M, N, K, rm, nz);
}

// ---- linear recurrences ------------------------------------------------------------------------------------------------------
// One block per (request, head, 64 value columns); wave w owns DPW consecutive key dims of those columns and keeps its part of
// the state in registers for the whole portion (loaded from the request's slot unless the portion starts the sequence, written
// back at the end).  Per token: the block stages the token's per-dim factors in LDS, every thread updates its DPW state values
// and accumulates its partial output, the partials of the waves are added in wave order.  The order of every sum depends on
// (dim, DPW) only, never on how the tokens are cut into steps.
#define HB_SCAN_MAX_WAVES 16

// The inputs of TT tokens at a time are staged in LDS by the whole block (activations applied there, one memory round trip per
// tile instead of one per token); TT only groups requests, it does not enter any sum.
// HGRN2: S_t = diag(f_t) S_{t-1} + (1 - f_t) v_t^T,  o_t = S_t^T q_t.
// proj row = [q (H*dim) | f (H*dim) | v (H*vdim)] pre-activation (bias already added).
template <int DPW>
__global__ __launch_bounds__(64 * HB_SCAN_MAX_WAVES) void k_hb_hgrn2_scan(const float* proj, long ldp, float* out, long ldo, const float* lower,
                                                                          float* state, const int* req_rows, const int* req_state,
                                                                          const int* pos, int H, int dim, int vdim, int TT) {
    extern __shared__ float sm[];
    const int nw = blockDim.x >> 6, dpad = nw * DPW;
    float* fs = sm;                       // [TT][dpad]
    float* qs = fs + TT * dpad;           // [TT][dpad]
    float* vs = qs + TT * dpad;           // [TT][64]
    float* part = vs + TT * 64;           // [2][nw][64]
    const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, w = threadIdx.x >> 6, c = blockIdx.z * 64 + lane;
    const int d0 = w * DPW;
    const int rs = req_rows[r], re = req_rows[r + 1];
    if (rs >= re) return;
    const bool ok = c < vdim, fresh = pos[rs] == 0;
    float* St = state + ((size_t)req_state[r] * H + h) * dim * vdim;
    float S[DPW];
#pragma unroll
    for (int i = 0; i < DPW; ++i) S[i] = (ok && !fresh && d0 + i < dim) ? St[(size_t)(d0 + i) * vdim + c] : 0.f;
    int flip = 0;
    for (int t0 = rs; t0 < re; t0 += TT) {
        const int nt = re - t0 < TT ? re - t0 : TT;
        __syncthreads();
        for (int idx = threadIdx.x; idx < nt * dpad; idx += blockDim.x) {
            const int tt = idx / dpad, d = idx - tt * dpad;
            float q = 0.f, f = 0.f;
            if (d < dim) {
                const float* p = proj + (size_t)(t0 + tt) * ldp;
                const float qv = p[h * dim + d], lo = lower[h * dim + d];
                q = qv * hb_sigmoid(qv);
                f = lo + (1.0f - lo) * hb_sigmoid(p[H * dim + h * dim + d]);
            }
            qs[idx] = q;
            fs[idx] = f;
        }
        for (int idx = threadIdx.x; idx < nt * 64; idx += blockDim.x) {
            const int tt = idx >> 6, cc = blockIdx.z * 64 + (idx & 63);
            vs[idx] = cc < vdim ? proj[(size_t)(t0 + tt) * ldp + 2 * H * dim + h * vdim + cc] : 0.f;
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float v = vs[tt * 64 + lane];
            const float* ft = fs + tt * dpad + d0;
            const float* qt = qs + tt * dpad + d0;
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < DPW; ++i) {
                const float f = ft[i];
                const float sv = f * S[i] + (1.0f - f) * v;
                S[i] = sv;
                o = fmaf(sv, qt[i], o);
            }
            float* pt = part + flip * nw * 64;
            pt[w * 64 + lane] = o;
            __syncthreads();
            if (w == 0 && ok) {
                float sum = pt[lane];
                for (int k = 1; k < nw; ++k) sum += pt[k * 64 + lane];
                out[(size_t)(t0 + tt) * ldo + h * vdim + c] = sum;
            }
            flip ^= 1;
        }
    }
    if (ok)
#pragma unroll
        for (int i = 0; i < DPW; ++i)
            if (d0 + i < dim) St[(size_t)(d0 + i) * vdim + c] = S[i];
}

// mLSTM with the running-maximum stabiliser.
// proj row = [q (H*dim) | k (H*dim) | v (H*vdim) | g (H*vdim) | i (H) | f (H)].  State per (slot, head): S [dim][vdim], n [dim], m.
// Every thread of wave w carries the same copy of its wave's n values and of m; value tile 0 writes them back.
template <int DPW>
__global__ __launch_bounds__(64 * HB_SCAN_MAX_WAVES) void k_hb_mlstm_scan(const float* proj, long ldp, float* out, long ldo, float* state,
                                                                          const int* req_rows, const int* req_state, const int* pos, int H,
                                                                          int dim, int vdim, float cap, int TT) {
    extern __shared__ float sm[];
    const int nw = blockDim.x >> 6, dpad = nw * DPW;
    float* ks = sm;                       // [TT][dpad]
    float* qs = ks + TT * dpad;           // [TT][dpad]
    float* vs = qs + TT * dpad;           // [TT][64]
    float* gs = vs + TT * 64;             // [TT][2]: log input gate, log forget gate
    float* part = gs + TT * 2;            // [2][nw][65]: partial outputs and (column 64) partial n.q
    const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, w = threadIdx.x >> 6, c = blockIdx.z * 64 + lane;
    const int d0 = w * DPW;
    const int rs = req_rows[r], re = req_rows[r + 1];
    if (rs >= re) return;
    const bool ok = c < vdim, fresh = pos[rs] == 0;
    const size_t per = (size_t)dim * vdim + dim + 1;
    float* St = state + ((size_t)req_state[r] * H + h) * per;
    float* nt_ = St + (size_t)dim * vdim;
    float S[DPW], nn[DPW];
#pragma unroll
    for (int i = 0; i < DPW; ++i) {
        S[i] = (ok && !fresh && d0 + i < dim) ? St[(size_t)(d0 + i) * vdim + c] : 0.f;
        nn[i] = (!fresh && d0 + i < dim) ? nt_[d0 + i] : 0.f;
    }
    float m = fresh ? 0.f : nt_[dim];
    const float qscale = 1.0f / sqrtf((float)dim);
    const int off_k = H * dim, off_v = 2 * H * dim, off_i = 2 * H * dim + 2 * H * vdim, off_f = off_i + H;
    int flip = 0;
    for (int t0 = rs; t0 < re; t0 += TT) {
        const int nt = re - t0 < TT ? re - t0 : TT;
        __syncthreads();
        for (int idx = threadIdx.x; idx < nt * dpad; idx += blockDim.x) {
            const int tt = idx / dpad, d = idx - tt * dpad;
            const float* p = proj + (size_t)(t0 + tt) * ldp;
            ks[idx] = d < dim ? p[off_k + h * dim + d] : 0.f;
            qs[idx] = d < dim ? p[h * dim + d] * qscale : 0.f;
        }
        for (int idx = threadIdx.x; idx < nt * 64; idx += blockDim.x) {
            const int tt = idx >> 6, cc = blockIdx.z * 64 + (idx & 63);
            vs[idx] = cc < vdim ? proj[(size_t)(t0 + tt) * ldp + off_v + h * vdim + cc] : 0.f;
        }
        for (int tt = threadIdx.x; tt < nt; tt += blockDim.x) {
            const float* p = proj + (size_t)(t0 + tt) * ldp;
            gs[2 * tt] = cap * tanhf(p[off_i + h] / cap);
            gs[2 * tt + 1] = hb_logsigmoid(cap * tanhf(p[off_f + h] / cap));
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float ig = gs[2 * tt], fg = gs[2 * tt + 1];
            const float mn = fmaxf(fg + m, ig);
            const float a = expf(fg + m - mn), b = expf(ig - mn);
            const float bv = b * vs[tt * 64 + lane];
            const float* kt = ks + tt * dpad + d0;
            const float* qt = qs + tt * dpad + d0;
            float o = 0.f, nq = 0.f;
#pragma unroll
            for (int i = 0; i < DPW; ++i) {
                const float kv = kt[i], qv = qt[i];
                nn[i] = a * nn[i] + b * kv;
                nq = fmaf(nn[i], qv, nq);
                const float sv = a * S[i] + kv * bv;
                S[i] = sv;
                o = fmaf(sv, qv, o);
            }
            float* pt = part + flip * nw * 65;
            pt[w * 65 + lane] = o;
            if (lane == 0) pt[w * 65 + 64] = nq;
            m = mn;
            __syncthreads();
            if (w == 0 && ok) {
                float sum = pt[lane], nsum = pt[64];
                for (int k = 1; k < nw; ++k) { sum += pt[k * 65 + lane]; nsum += pt[k * 65 + 64]; }
                out[(size_t)(t0 + tt) * ldo + h * vdim + c] = sum / (fmaxf(fabsf(nsum), expf(-m)) + 1e-6f);
            }
            flip ^= 1;
        }
    }
#pragma unroll
    for (int i = 0; i < DPW; ++i)
        if (d0 + i < dim) {
            if (ok) St[(size_t)(d0 + i) * vdim + c] = S[i];
            if (blockIdx.z == 0 && lane == 0) nt_[d0 + i] = nn[i];
        }
    if (blockIdx.z == 0 && threadIdx.x == 0) nt_[dim] = m;
}

// Rotation of the newer mixers: dims i and i + rot/2 (i < rot/2) of a vector form a pair (u, v) that position p turns by the angle
// p * inv_freq[i] into (u cos - v sin, v cos + u sin); dims at or beyond rot pass unchanged.  x: the vector, d: the dim asked for.
__device__ __forceinline__ float hb_rot_half(const float* x, int d, int rot, float p, const float* inv_freq) {
    const float v = x[d];
    if (d >= rot) return v;
    const int half = rot >> 1, i = d < half ? d : d - half;
    float sn, cs;
    sincosf(p * inv_freq[i], &sn, &cs);
    return d < half ? v * cs - x[d + half] * sn : v * cs + x[d - half] * sn;
}

// Retention: S_t = decay_h S_{t-1} + k_t v_t^T, o_t = S_t^T q_t, one fixed decay per head, no softmax and no denominator.
// proj row = [q (H*dim) | k (H*dim) | v (H*vdim) | gate (H*vdim)].  q and k are rotated while they are staged (hb_rot_half on their
// first `rot` dims), k is then multiplied by kscale.  Block, waves and the order of every sum as in the scans above.
// Long portions run the request's rows in chunks of `chunk_len` side by side (modes as for the shift-decay scan below):
//   mode 0  the whole portion from the slot's state, outputs and state stored
//   mode 1  chunk z from a zero state, no outputs: its final state goes to the workspace
//   mode 2  chunk z replayed from its carry (left in the workspace by k_hb_retention_carry), outputs written
// Workspace entry of chunk k of request r: index rs / chunk_len + r + k, [H][dim*vdim] floats each.
template <int DPW>
__global__ __launch_bounds__(64 * HB_SCAN_MAX_WAVES) void k_hb_retention_scan(const float* proj, long ldp, float* out, long ldo, const float* decay,
                                                                              const float* inv_freq, float* state, const int* req_rows,
                                                                              const int* req_state, const int* pos, int H, int dim, int vdim,
                                                                              int rot, float kscale, int TT, int mode, int chunk_len, float* ws) {
    extern __shared__ float sm[];
    const int nw = blockDim.x >> 6, dpad = nw * DPW;
    float* ks = sm;                       // [TT][dpad]
    float* qs = ks + TT * dpad;           // [TT][dpad]
    float* vs = qs + TT * dpad;           // [TT][64]
    float* part = vs + TT * 64;           // [2][nw][64]
    const int vt = (vdim + 63) >> 6, chunk = mode == 0 ? 0 : blockIdx.z / vt, tile = mode == 0 ? blockIdx.z : blockIdx.z % vt;
    const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, w = threadIdx.x >> 6, c = tile * 64 + lane;
    const int d0 = w * DPW;
    const int rs0 = req_rows[r], re0 = req_rows[r + 1];
    const int rs = mode == 0 ? rs0 : rs0 + chunk * chunk_len;
    if (rs >= re0) return;
    const int re = mode == 0 || rs + chunk_len > re0 ? re0 : rs + chunk_len;
    const bool ok = c < vdim, fresh = pos[rs0] == 0;
    float* St = state + ((size_t)req_state[r] * H + h) * dim * vdim;
    if (mode != 0) St = ws + ((size_t)(rs0 / chunk_len + r + chunk) * H + h) * ((size_t)dim * vdim);
    const bool load = mode == 2 || (mode == 0 && !fresh);
    const float dec = decay[h];
    float S[DPW];
#pragma unroll
    for (int i = 0; i < DPW; ++i) S[i] = (ok && load && d0 + i < dim) ? St[(size_t)(d0 + i) * vdim + c] : 0.f;
    int flip = 0;
    for (int t0 = rs; t0 < re; t0 += TT) {
        const int nt = re - t0 < TT ? re - t0 : TT;
        __syncthreads();
        for (int idx = threadIdx.x; idx < nt * dpad; idx += blockDim.x) {
            const int tt = idx / dpad, d = idx - tt * dpad;
            float q = 0.f, k = 0.f;
            if (d < dim) {
                const float* p = proj + (size_t)(t0 + tt) * ldp + h * dim;
                const float pf = (float)pos[t0 + tt];
                k = hb_rot_half(p + H * dim, d, rot, pf, inv_freq) * kscale;
                if (mode != 1) q = hb_rot_half(p, d, rot, pf, inv_freq);
            }
            qs[idx] = q;
            ks[idx] = k;
        }
        for (int idx = threadIdx.x; idx < nt * 64; idx += blockDim.x) {
            const int tt = idx >> 6, cc = tile * 64 + (idx & 63);
            vs[idx] = cc < vdim ? proj[(size_t)(t0 + tt) * ldp + 2 * H * dim + h * vdim + cc] : 0.f;
        }
        __syncthreads();
        if (mode == 1) {
            for (int tt = 0; tt < nt; ++tt) {
                const float v = vs[tt * 64 + lane];
                const float* kt = ks + tt * dpad + d0;
#pragma unroll
                for (int i = 0; i < DPW; ++i) S[i] = dec * S[i] + kt[i] * v;
            }
            continue;
        }
        for (int tt = 0; tt < nt; ++tt) {
            const float v = vs[tt * 64 + lane];
            const float* kt = ks + tt * dpad + d0;
            const float* qt = qs + tt * dpad + d0;
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < DPW; ++i) {
                const float sv = dec * S[i] + kt[i] * v;
                S[i] = sv;
                o = fmaf(sv, qt[i], o);
            }
            float* pt = part + flip * nw * 64;
            pt[w * 64 + lane] = o;
            __syncthreads();
            if (w == 0 && ok) {
                float sum = pt[lane];
                for (int k2 = 1; k2 < nw; ++k2) sum += pt[k2 * 64 + lane];
                out[(size_t)(t0 + tt) * ldo + h * vdim + c] = sum;
            }
            flip ^= 1;
        }
    }
    if (mode == 2) return;
    if (ok)
#pragma unroll
        for (int i = 0; i < DPW; ++i)
            if (d0 + i < dim) St[(size_t)(d0 + i) * vdim + c] = S[i];
}
// Between the two chunked passes: the slot's state is pushed through the request's chunks in order, S <- decay^rows S + B_k; every
// chunk's workspace entry receives its carry-in in place of B_k, the slot the final state.  decay^rows is formed by repeated
// multiplication (at most chunk_len factors).
__global__ __launch_bounds__(256) void k_hb_retention_carry(float* ws, float* state, const float* decay, const int* req_rows, const int* req_state,
                                                            const int* pos, int H, int dim, int vdim, int chunk_len) {
    const int r = blockIdx.x, h = blockIdx.y;
    const int rs = req_rows[r], re = req_rows[r + 1];
    if (rs >= re) return;
    const int nc = (re - rs + chunk_len - 1) / chunk_len;
    const bool fresh = pos[rs] == 0;
    const size_t per = (size_t)dim * vdim;
    float* St = state + ((size_t)req_state[r] * H + h) * per;
    float* w0 = ws + ((size_t)(rs / chunk_len + r) * H + h) * per;
    const float dec = decay[h];
    float full = 1.f, last = 1.f;
    for (int i = 0; i < chunk_len; ++i) full *= dec;
    for (int i = 0; i < (re - rs) - (nc - 1) * chunk_len; ++i) last *= dec;
    for (size_t e = (size_t)blockIdx.z * 256 + threadIdx.x; e < per; e += (size_t)256 * gridDim.z) {
        float S = fresh ? 0.f : St[e];
        for (int k = 0; k < nc; ++k) {
            float* wk = w0 + (size_t)k * H * per;
            const float B = wk[e];
            wk[e] = S;
            S = (k == nc - 1 ? last : full) * S + B;
        }
        St[e] = S;
    }
}

// ---- latent attention: what a row leaves in the cache, and its query ----------------------------------------------------------
// proj row = [query latent (q_rank) | key / value latent (R) | rotated key part (r) | gate (H) | ...].  Block (row, 0): the query latent
// is RMS-normed with its weight in place.  Block (row, 1): the key / value latent is RMS-normed with its weight into the row's cache
// entry [R + r] (engine dtype), followed by the rotated key part (hb_rot_half on its first `rot` dims).
template <typename T>
__global__ __launch_bounds__(256) void k_hb_latent_prep(float* proj, long ldp, T* cache, const float* qn, const float* kn, const float* inv_freq,
                                                        const int* pos, const int* page, const int* slot, int q_rank, int R, int r, int rot,
                                                        int ps, float eps) {
    __shared__ float red[4];
    const int row = blockIdx.x;
    float* p = proj + (size_t)row * ldp;
    if (blockIdx.y == 0) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < q_rank; i += 256) ss = fmaf(p[i], p[i], ss);
        const float inv = 1.0f / sqrtf(hb_block_sum256(ss, red) / (float)q_rank + eps);
        for (int i = threadIdx.x; i < q_rank; i += 256) p[i] = p[i] * inv * qn[i];
        return;
    }
    const float* x = p + q_rank;
    float ss = 0.f;
    for (int i = threadIdx.x; i < R; i += 256) ss = fmaf(x[i], x[i], ss);
    const float inv = 1.0f / sqrtf(hb_block_sum256(ss, red) / (float)R + eps);
    T* dst = cache + ((size_t)page[row] * ps + slot[row]) * (size_t)(R + r);
    for (int i = threadIdx.x; i < R; i += 256) hb_st(dst + i, x[i] * inv * kn[i]);
    const float pf = (float)pos[row];
    for (int d = threadIdx.x; d < r; d += 256) hb_st(dst + R + d, hb_rot_half(x + R, d, rot, pf, inv_freq));
}
// q row = per head [plain (dim) | rotated (r)]; qa row = per head [query against the latent (R) | rotated part (r)].  The first part
// of qa is a product of its own (the plain part times the head's key expansion); this fills the second.
__global__ __launch_bounds__(64) void k_hb_latent_qrot(const float* q, long ldq, float* qa, long ldqa, const float* inv_freq, const int* pos, int dim,
                                                       int R, int r, int rot) {
    const int row = blockIdx.x, h = blockIdx.y;
    const float* src = q + (size_t)row * ldq + (size_t)h * (dim + r) + dim;
    float* dst = qa + (size_t)row * ldqa + (size_t)h * (R + r) + R;
    const float pf = (float)pos[row];
    for (int d = threadIdx.x; d < r; d += 64) dst[d] = hb_rot_half(src, d, rot, pf, inv_freq);
}

// per (row, head): o / rms(o) over vdim, times a weight (per_head_w: indexed over all heads, else shared [vdim]; NULL: none), times
// a gate (gate_mode 1: sigmoid(g), 2: g * sigmoid(g); g = proj[row][gate_off + h*vdim + j]), times out_scale.  In place.
enum { HB_GATE_NONE = 0, HB_GATE_SIGMOID = 1, HB_GATE_SILU = 2 };
__global__ __launch_bounds__(64) void k_hb_head_norm(float* o, long ldo, const float* w, int per_head_w, const float* proj, long ldp, int gate_off,
                                                     int gate_mode, int vdim, float eps, float out_scale) {
    const int row = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    float* p = o + (size_t)row * ldo + (size_t)h * vdim;
    float ss = 0.f;
    for (int j = lane; j < vdim; j += 64) ss = fmaf(p[j], p[j], ss);
    ss = hb_wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
    for (int j = lane; j < vdim; j += 64) {
        float v = p[j] * inv;
        if (w) v *= w[per_head_w ? h * vdim + j : j];
        if (gate_mode != HB_GATE_NONE) {
            const float g = proj[(size_t)row * ldp + gate_off + h * vdim + j];
            v *= gate_mode == HB_GATE_SIGMOID ? hb_sigmoid(g) : g * hb_sigmoid(g);
        }
        p[j] = v * out_scale;
    }
}

// ---- real-gated linear recurrent unit behind a short causal convolution ------------------------------------------------------
// proj row = [gated branch y (C) | recurrent branch x (C) | u = conv(x) (C) | gate pre-activations, per block r (bs) then i (bs)].
// State of a slot: [taps][C]: row 0 the recurrent state, rows 1 .. taps-1 the last taps-1 inputs of the convolution, oldest first.
// u[row][c] = conv_b[c] + sum_j conv_w[c][j] * x[position - (taps-1-j)][c]; inputs before the step's first row come from the slot,
// inputs before the sequence are zero (so a portion that starts at position 0 never reads the slot).
__global__ __launch_bounds__(256) void k_hb_conv_causal(float* proj, long ldp, const float* cw, const float* cb, const float* state,
                                                        const int* pos, const int* row_req, const int* req_rows, const int* req_state, int C,
                                                        int taps) {
    const int row = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int r = row_req[row], rs = req_rows[r], p = pos[row], p0 = pos[rs];
    const float* hist = state + (size_t)req_state[r] * taps * C + C;
    float acc = cb ? cb[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j, q = p - back;
        if (q < 0) continue;
        const float v = row - back >= rs ? proj[(size_t)(row - back) * ldp + C + c] : hist[(size_t)(q - (p0 - (taps - 1))) * C + c];
        acc = fmaf(cw[(size_t)c * taps + j], v, acc);
    }
    proj[(size_t)row * ldp + 2 * C + c] = acc;
}
// One thread per (request, channel): walks the portion's tokens in order.  Per token: r, i = sigmoid(gate pre-activations),
// a = exp(-rec_scale * r * softplus(lam)), S <- a S + sqrt(1 - a^2) (i u), out = S * gelu_tanh(y) * out_scale.  The inputs of 8 tokens
// are fetched and their gates evaluated before the 8 dependent updates.  At the end the slot's convolution history is shifted:
// entry i <- the input at position (end - (taps-1) + i), from this step's rows or from the old history (ascending i, in place).
__global__ __launch_bounds__(64) void k_hb_rglru_scan(const float* proj, long ldp, float* out, long ldo, const float* lam, float* state,
                                                      const int* req_rows, const int* req_state, const int* pos, int C, int bs, int taps,
                                                      float rec_scale, float out_scale) {
    const int r = blockIdx.x, c = blockIdx.y * 64 + threadIdx.x;
    if (c >= C) return;
    const int rs = req_rows[r], re = req_rows[r + 1];
    if (rs >= re) return;
    float* st = state + (size_t)req_state[r] * taps * C;
    const int p0 = pos[rs];
    float S = p0 == 0 ? 0.f : st[c];
    const float lv = lam[c];
    const float sp = lv > 20.f ? lv : log1pf(expf(lv));
    const int blk = c / bs, j = c - blk * bs;
    const size_t off_r = (size_t)3 * C + (size_t)blk * 2 * bs + j, off_i = off_r + bs;
    for (int t0 = rs; t0 < re; t0 += 8) {
        float a[8], b[8], y[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int t = t0 + k < re ? t0 + k : re - 1;
            const float* pr = proj + (size_t)t * ldp;
            const float rg = hb_sigmoid(pr[off_r]), ig = hb_sigmoid(pr[off_i]);
            const float la = -rec_scale * rg * sp;
            a[k] = expf(la);
            b[k] = sqrtf(-expm1f(2.0f * la)) * (ig * pr[2 * C + c]);      // 1 - a^2 without the cancellation near a = 1
            y[k] = hb_gelu_tanh(pr[c]);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (t0 + k < re) {
                S = a[k] * S + b[k];
                out[(size_t)(t0 + k) * ldo + c] = S * y[k] * out_scale;
            }
    }
    st[c] = S;
    const int n = re - rs;
    for (int i = 0; i < taps - 1; ++i) {
        const int q = p0 + n - (taps - 1) + i;
        float v = 0.f;
        if (q >= p0) v = proj[(size_t)(rs + q - p0) * ldp + C + c];
        else if (q >= 0) v = st[(size_t)(1 + i + n) * C + c];
        st[(size_t)(1 + i) * C + c] = v;
    }
}

// Long portions: the same recurrence with the request's rows cut into 32 chunks that run side by side.  Block = 32 channels x 32
// chunks.  Pass 1: every thread evaluates the gates of its chunk (a and b = sqrt(1 - a^2) i u replace the gate pre-activations in
// proj) and reduces the chunk to S_out = A S_in + B.  Pass 2: the carry into chunk k is the slot's state pushed through chunks
// 0 .. k-1 in order.  Pass 3: the chunk is replayed from its carry with the recurrence itself and the outputs are written.
#define HB_LRU_CHUNKS 32
__global__ __launch_bounds__(1024) void k_hb_rglru_scan_chunked(float* proj, long ldp, float* out, long ldo, const float* lam, float* state,
                                                                const int* req_rows, const int* req_state, const int* pos, int C, int bs,
                                                                int taps, float rec_scale, float out_scale) {
    __shared__ float sA[HB_LRU_CHUNKS][32], sB[HB_LRU_CHUNKS][32];
    const int r = blockIdx.x, cl = threadIdx.x & 31, k = threadIdx.x >> 5, c = blockIdx.y * 32 + cl;
    const int rs = req_rows[r], re = req_rows[r + 1];
    if (rs >= re) return;
    const bool ok = c < C;
    const int cc = ok ? c : C - 1;
    const int n = re - rs, len = (n + HB_LRU_CHUNKS - 1) / HB_LRU_CHUNKS;
    const int tb = rs + k * len < re ? rs + k * len : re, te = tb + len < re ? tb + len : re;
    float* st = state + (size_t)req_state[r] * taps * C;
    const int p0 = pos[rs];
    const float lv = lam[cc];
    const float sp = lv > 20.f ? lv : log1pf(expf(lv));
    const int blk = cc / bs, j = cc - blk * bs;
    const size_t off_r = (size_t)3 * C + (size_t)blk * 2 * bs + j, off_i = off_r + bs;
    float A = 1.f, B = 0.f;
    for (int t0 = tb; t0 < te; t0 += 4) {
        float a[4], b[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int t = t0 + q < te ? t0 + q : te - 1;
            const float* pr = proj + (size_t)t * ldp;
            const float rg = hb_sigmoid(pr[off_r]), ig = hb_sigmoid(pr[off_i]);
            const float la = -rec_scale * rg * sp;
            a[q] = expf(la);
            b[q] = sqrtf(-expm1f(2.0f * la)) * (ig * pr[2 * C + cc]);      // 1 - a^2 without the cancellation near a = 1
        }
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (t0 + q < te) {
                float* pr = proj + (size_t)(t0 + q) * ldp;
                if (ok) { pr[off_r] = a[q]; pr[off_i] = b[q]; }
                B = a[q] * B + b[q];
                A *= a[q];
            }
    }
    sA[k][cl] = A;
    sB[k][cl] = B;
    __syncthreads();
    float S = p0 == 0 ? 0.f : st[cc];
    for (int q = 0; q < k; ++q) S = sA[q][cl] * S + sB[q][cl];
    for (int t = tb; t < te; ++t) {
        const float* pr = proj + (size_t)t * ldp;
        S = pr[off_r] * S + pr[off_i];
        if (ok) out[(size_t)t * ldo + c] = S * hb_gelu_tanh(pr[cc]) * out_scale;
    }
    if (!ok) return;
    // chunks behind the portion's end are empty (A = 1, B = 0): the last thread of a channel holds the final state
    if (k == HB_LRU_CHUNKS - 1) st[c] = S;
    if (k == 0)
        for (int i = 0; i < taps - 1; ++i) {
            const int q = p0 + n - (taps - 1) + i;
            float v = 0.f;
            if (q >= p0) v = proj[(size_t)(rs + q - p0) * ldp + C + c];
            else if (q >= 0) v = st[(size_t)(1 + i + n) * C + c];
            st[(size_t)(1 + i) * C + c] = v;
        }
}

// ---- short causal convolution over the channels of a fused projection ----------------------------------------------------------
// y[p][c] = sum_j w[c][j] * u[p - (taps-1-j)][c], j ascending (oldest input first), no bias; inputs before the step's first row come
// from the slot's history ([taps-1][C], oldest first: the rows at positions p0-(taps-1) .. p0-1 of a portion that starts at p0),
// inputs before the sequence are zero (a portion that starts at position 0 never reads the slot).  u = columns [0, C) of proj.
__device__ __forceinline__ float hb_conv_taps(const float* proj, long ldp, const float* cw, const float* hist, int row, int rs, int p, int p0,
                                              int c, int C, int taps) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j, q = p - back;
        if (q < 0) continue;
        const float v = row - back >= rs ? proj[(size_t)(row - back) * ldp + c] : hist[(size_t)(q - (p0 - (taps - 1))) * C + c];
        acc = fmaf(cw[(size_t)c * taps + j], v, acc);
    }
    return acc;
}
// After every row of the step has read its inputs: history entry i <- the input at position (end - (taps-1) + i), from this step's rows
// or from the old history (ascending i, in place: entry i reads old entry i + rows).  One thread per channel of one request.
__device__ __forceinline__ void hb_conv_hist_update(const float* proj, long ldp, float* hist, int rs, int re, int p0, int c, int C, int taps) {
    const int n = re - rs;
    for (int i = 0; i < taps - 1; ++i) {
        const int q = p0 + n - (taps - 1) + i;
        float v = 0.f;
        if (q >= p0) v = proj[(size_t)(rs + q - p0) * ldp + c];
        else if (q >= 0) v = hist[(size_t)(i + n) * C + c];
        hist[(size_t)i * C + c] = v;
    }
}

// ---- gated delta rule ----------------------------------------------------------------------------------------------------------------
// Columns of a projection row (see hb_delta): the fused projection [q | k | v | beta | decay input | gate input], then what the mixer
// derives from it: decay and gate pre-activations of the bottleneck forms, the convolved q | k | v, the decays, q . k per key head.
struct hb_delta_layout {
    int nq, nqkv, off_b, off_din, off_gin, n_in, ndec, off_dec, off_gate, off_c, off_g, off_kq, n_proj;
};
__device__ __forceinline__ float hb_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }
// First launch, one thread per (row, element): q | k | v through the convolution and silu; decay g = exp(-exp(a_log[h]) *
// softplus(d + dt_bias)); beta = sigmoid in place.
__global__ __launch_bounds__(256) void k_hb_delta_conv(float* proj, long ldp, const float* cw, const float* state, long per_slot, long hist_off,
                                                       const float* a_log, const float* dt_bias, const int* pos, const int* row_req,
                                                       const int* req_rows, const int* req_state, hb_delta_layout y, int H, int dim, int taps,
                                                       int decay_channels) {
    const int row = blockIdx.x, idx = blockIdx.y * 256 + threadIdx.x;
    float* pr = proj + (size_t)row * ldp;
    if (idx < y.nqkv) {
        const int r = row_req[row], rs = req_rows[r];
        const float* hist = state + (size_t)req_state[r] * per_slot + hist_off;
        const float a = hb_conv_taps(proj, ldp, cw, hist, row, rs, pos[row], pos[rs], idx, y.nqkv, taps);
        pr[y.off_c + idx] = a * hb_sigmoid(a);
    } else if (idx < y.nqkv + y.ndec) {
        const int i = idx - y.nqkv, hh = decay_channels ? i / dim : i;
        pr[y.off_g + i] = expf(-expf(a_log[hh]) * hb_softplus(pr[y.off_dec + i] + dt_bias[i]));
    } else if (idx < y.nqkv + y.ndec + H) {
        const int h = idx - y.nqkv - y.ndec;
        pr[y.off_b + h] = hb_sigmoid(pr[y.off_b + h]);
    }
}
// Second launch.  Blocks (row, g < G), two waves: q head g and k head g of the convolved row to unit vectors (x / sqrt(sum x^2 + 1e-6)),
// q times dim^-1/2, then q . k.  Blocks (row, G + j) of a request's last row: the convolution's history of 128 channels moves on (every
// row has read it in the first launch).
__global__ __launch_bounds__(128) void k_hb_delta_unit(float* proj, long ldp, float* state, long per_slot, long hist_off, const int* pos,
                                                       const int* row_req, const int* req_rows, const int* req_state, hb_delta_layout y, int G,
                                                       int dim, int taps) {
    __shared__ float xs[2][HB_SCAN_MAX_WAVES * 64];
    const int row = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    if ((int)blockIdx.y >= G) {
        const int r = row_req[row], rs = req_rows[r], re = req_rows[r + 1], c = ((int)blockIdx.y - G) * 128 + threadIdx.x;
        if (row != re - 1 || c >= y.nqkv) return;
        hb_conv_hist_update(proj, ldp, state + (size_t)req_state[r] * per_slot + hist_off, rs, re, pos[rs], c, y.nqkv, taps);
        return;
    }
    const int g = blockIdx.y;
    float* pr = proj + (size_t)row * ldp;
    float* x = pr + y.off_c + (wv ? y.nq : 0) + (size_t)g * dim;
    float ss = 0.f;
    for (int d = lane; d < dim; d += 64) ss = fmaf(x[d], x[d], ss);
    ss = hb_wave_sum(ss);
    const float inv = (1.0f / sqrtf(ss + 1e-6f)) * (wv ? 1.0f : 1.0f / sqrtf((float)dim));
    for (int d = lane; d < dim; d += 64) {
        const float v = x[d] * inv;
        x[d] = v;
        xs[wv][d] = v;
    }
    __syncthreads();
    if (wv == 0) {
        float dot = 0.f;
        for (int d = lane; d < dim; d += 64) dot = fmaf(xs[0][d], xs[1][d], dot);
        dot = hb_wave_sum(dot);
        if (lane == 0) pr[y.off_kq + g] = dot;
    }
}
// Per head: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  Block = (request, head, 64 value columns); wave w keeps DPW
// key dims of the state in registers for the whole portion.  Per token every thread decays its part of the state and forms its share of
// (g S)^T k and (g S)^T q; the waves' shares are added in wave order; then u is known to every thread, the state takes k u^T, and the
// output is (g S)^T q + u (k . q), which is S^T q after the write.  The order of every sum depends on (dim, DPW) only.
// Long portions run the request's rows in chunks of `chunk_len` side by side (the recurrence is linear in S, column by column):
//   HB_SCAN_WHOLE   the whole portion from the slot's state, outputs and state stored
//   HB_SCAN_REDUCE  chunk z from a zero state without outputs -> B; and with the identity as state and zero values -> the chunk's
//                   transition A [dim][dim], stored transposed (value tiles beyond vdim carry the identity's columns)
//   HB_SCAN_REPLAY  chunk z replayed from its carry (left in the workspace by k_hb_delta_carry), outputs written
// Workspace entry of chunk k of request r: index rs / chunk_len + r + k, [H][dim * (vdim + dim)] floats: B [dim][vdim], then A^T.
enum { HB_SCAN_WHOLE = 0, HB_SCAN_REDUCE = 1, HB_SCAN_REPLAY = 2 };
template <int DPW>
__global__ __launch_bounds__(64 * HB_SCAN_MAX_WAVES) void k_hb_delta_scan(const float* proj, long ldp, float* out, long ldo, float* state,
                                                                          long per_slot, const int* req_rows, const int* req_state,
                                                                          const int* pos, int H, int G, int dim, int vdim, hb_delta_layout y,
                                                                          int decay_channels, int TT, int mode, int chunk_len, float* ws,
                                                                          const float* head_w, int gate_mode, float eps, float out_scale) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    const int nw = blockDim.x >> 6, dpad = nw * DPW;
    float* qs = sm;                       // [TT][dpad]
    float* ks = qs + TT * dpad;           // [TT][dpad]
    float* gs = ks + TT * dpad;           // [TT][dpad]
    float* vs = gs + TT * dpad;           // [TT][64]
    float* sc = vs + TT * 64;             // [TT][2]: beta, q . k
    float* part = sc + TT * 2;            // [2][nw][2][64]
    const int vt = (vdim + 63) >> 6, at = (dim + 63) >> 6, tiles = mode == HB_SCAN_REDUCE ? vt + at : vt;
    const int chunk = mode == HB_SCAN_WHOLE ? 0 : blockIdx.z / tiles, tile = mode == HB_SCAN_WHOLE ? blockIdx.z : blockIdx.z % tiles;
    const bool ident = tile >= vt;        // this block carries columns of the chunk's transition
    const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int c = (ident ? tile - vt : tile) * 64 + lane, ncol = ident ? dim : vdim;
    const int d0 = w * DPW, gq = h / (H / G);
    const int rs0 = req_rows[r], re0 = req_rows[r + 1];
    const int rs = mode == HB_SCAN_WHOLE ? rs0 : rs0 + chunk * chunk_len;
    if (rs >= re0) return;
    const int re = mode == HB_SCAN_WHOLE || rs + chunk_len > re0 ? re0 : rs + chunk_len;
    const bool ok = c < ncol, fresh = pos[rs0] == 0;
    const size_t per_ws = (size_t)dim * (vdim + dim);
    float* St = state + (size_t)req_state[r] * per_slot + (size_t)h * dim * vdim;
    if (mode != HB_SCAN_WHOLE) St = ws + ((size_t)(rs0 / chunk_len + r + chunk) * H + h) * per_ws + (ident ? (size_t)dim * vdim : 0);
    const bool load = mode == HB_SCAN_REPLAY || (mode == HB_SCAN_WHOLE && !fresh);
    float S[DPW];
#pragma unroll
    for (int i = 0; i < DPW; ++i) {
        S[i] = (ok && load && d0 + i < dim) ? St[(size_t)(d0 + i) * ncol + c] : 0.f;
        if (ident && d0 + i == c && ok) S[i] = 1.f;
    }
    int flip = 0;
    for (int t0 = rs; t0 < re; t0 += TT) {
        const int nt = re - t0 < TT ? re - t0 : TT;
        __syncthreads();
        for (int idx = threadIdx.x; idx < nt * dpad; idx += blockDim.x) {
            const int tt = idx / dpad, d = idx - tt * dpad;
            float q = 0.f, k = 0.f, g = 0.f;
            if (d < dim) {
                const float* p = proj + (size_t)(t0 + tt) * ldp;
                q = p[y.off_c + gq * dim + d];
                k = p[y.off_c + y.nq + gq * dim + d];
                g = p[y.off_g + (decay_channels ? h * dim + d : h)];
            }
            qs[idx] = q; ks[idx] = k; gs[idx] = g;
        }
        for (int idx = threadIdx.x; idx < nt * 64; idx += blockDim.x) {
            const int tt = idx >> 6, cc = tile * 64 + (idx & 63);
            vs[idx] = !ident && cc < vdim ? proj[(size_t)(t0 + tt) * ldp + y.off_c + 2 * y.nq + h * vdim + cc] : 0.f;
        }
        for (int tt = threadIdx.x; tt < nt; tt += blockDim.x) {
            const float* p = proj + (size_t)(t0 + tt) * ldp;
            sc[2 * tt] = p[y.off_b + h];
            sc[2 * tt + 1] = p[y.off_kq + gq];
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float v = vs[tt * 64 + lane], beta = sc[2 * tt], kq = sc[2 * tt + 1];
            // the token's factors of this wave's dims, four at a time (every staged array starts on a 16-byte boundary)
            const float4* qt = (const float4*)(qs + tt * dpad + d0);
            const float4* kt = (const float4*)(ks + tt * dpad + d0);
            const float4* gt = (const float4*)(gs + tt * dpad + d0);
            float kr[DPW];
            float pk = 0.f, pq = 0.f;
#pragma unroll
            for (int i = 0; i < DPW; i += 4) {
                const float4 g4 = gt[i >> 2], k4 = kt[i >> 2], q4 = qt[i >> 2];
                kr[i] = k4.x; kr[i + 1] = k4.y; kr[i + 2] = k4.z; kr[i + 3] = k4.w;
                float sv = g4.x * S[i];
                S[i] = sv; pk = fmaf(sv, k4.x, pk); pq = fmaf(sv, q4.x, pq);
                sv = g4.y * S[i + 1];
                S[i + 1] = sv; pk = fmaf(sv, k4.y, pk); pq = fmaf(sv, q4.y, pq);
                sv = g4.z * S[i + 2];
                S[i + 2] = sv; pk = fmaf(sv, k4.z, pk); pq = fmaf(sv, q4.z, pq);
                sv = g4.w * S[i + 3];
                S[i + 3] = sv; pk = fmaf(sv, k4.w, pk); pq = fmaf(sv, q4.w, pq);
            }
            float* pt = part + flip * nw * 128;
            pt[w * 128 + lane] = pk;
            pt[w * 128 + 64 + lane] = pq;
            __syncthreads();
            float pred = pt[lane];
            for (int k2 = 1; k2 < nw; ++k2) pred += pt[k2 * 128 + lane];
            const float u = beta * (v - pred);
#pragma unroll
            for (int i = 0; i < DPW; ++i) S[i] = fmaf(kr[i], u, S[i]);
            if (w == 0 && mode != HB_SCAN_REDUCE) {
                float o = 0.f;
                if (ok) {
                    float oq = pt[64 + lane];
                    for (int k2 = 1; k2 < nw; ++k2) oq += pt[k2 * 128 + 64 + lane];
                    o = fmaf(u, kq, oq);
                }
                if (head_w) {
                    // the block holds the whole head (vdim <= 64): unit RMS, the shared weight, the gate and the mixer's scale here
                    const float inv = 1.0f / sqrtf(hb_wave_sum(o * o) / (float)vdim + eps);
                    float gm = 1.0f;
                    if (ok && gate_mode != HB_GATE_NONE) {
                        const float gv = proj[(size_t)(t0 + tt) * ldp + y.off_gate + h * vdim + c];
                        gm = gate_mode == HB_GATE_SIGMOID ? hb_sigmoid(gv) : gv * hb_sigmoid(gv);
                    }
                    o = o * inv * (ok ? head_w[c] : 0.f) * gm * out_scale;
                }
                if (ok) out[(size_t)(t0 + tt) * ldo + h * vdim + c] = o;
            }
            flip ^= 1;
        }
    }
    if (mode == HB_SCAN_REPLAY) return;
    if (ok)
#pragma unroll
        for (int i = 0; i < DPW; ++i)
            if (d0 + i < dim) St[ident ? (size_t)c * dim + d0 + i : (size_t)(d0 + i) * ncol + c] = S[i];
}
// Between the two chunked passes: the slot's state is pushed through the request's chunks in order, S <- A_k S + B_k (A_k [dim][dim]
// times S [dim][vdim], sums over the key dim in ascending order); every chunk's workspace entry receives its carry-in in place of B_k,
// the slot the final state.  The columns of S are independent: one block per (request, head, 16 value columns), dim <= 128.  Thread =
// (key row d, a share of the 16 columns); the block's columns of S live in LDS between the chunks.  A_k is stored transposed, so row e of
// A_k^T is one coalesced request of the block's threads; the values of the next 32 rows (or of the first rows of A_k+1, which does not
// depend on the carry) are on their way from memory while the current 32 are multiplied.
// ROWS = 64 (dim <= 64) or 128: key rows with a thread each; the 256 / ROWS thread groups share the 16 columns.
#define HB_DC_COLS 16
template <int ROWS>
__global__ __launch_bounds__(256) void k_hb_delta_carry(float* ws, float* state, long per_slot, const int* req_rows, const int* req_state,
                                                        const int* pos, int H, int dim, int vdim, int chunk_len) {
    constexpr int CPT = HB_DC_COLS / (256 / ROWS), EG = 32;      // columns per thread (4 | 8); rows of A^T per group
    __shared__ __attribute__((aligned(16))) float cur[2][ROWS * HB_DC_COLS];
    const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int rs = req_rows[r], re = req_rows[r + 1];
    if (rs >= re) return;
    const int d = tid % ROWS, c0 = (tid / ROWS) * CPT, cb = blockIdx.z * HB_DC_COLS;
    const int nc = (re - rs + chunk_len - 1) / chunk_len, ng = (dim + EG - 1) / EG;
    const bool fresh = pos[rs] == 0, dok = d < dim;
    const size_t per_ws = (size_t)dim * (vdim + dim);
    float* St = state + (size_t)req_state[r] * per_slot + (size_t)h * dim * vdim;
    float* w0 = ws + ((size_t)(rs / chunk_len + r) * H + h) * per_ws;
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
        const int c = cb + c0 + j;
        cur[0][d * HB_DC_COLS + c0 + j] = (dok && c < vdim && !fresh) ? St[(size_t)d * vdim + c] : 0.f;
    }
    float ar[EG];
    auto fetch = [&](int k, int g) {      // A_k[d][g*EG .. g*EG + EG) from the transposed store (zeros beyond dim)
        const float* AT = w0 + (size_t)k * H * per_ws + (size_t)dim * vdim;
#pragma unroll
        for (int i = 0; i < EG; ++i) {
            const int e = g * EG + i;
            ar[i] = (dok && e < dim) ? AT[(size_t)e * dim + d] : 0.f;
        }
    };
    fetch(0, 0);
    int flip = 0;
    for (int k = 0; k < nc; ++k) {
        float* wk = w0 + (size_t)k * H * per_ws;
        float acc[CPT], bk[CPT];
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
            const int c = cb + c0 + j;
            bk[j] = (dok && c < vdim) ? wk[(size_t)d * vdim + c] : 0.f;
            acc[j] = 0.f;
        }
        __syncthreads();                // the carry-in is complete
        const float* cv0 = cur[flip] + c0;
        for (int g = 0; g < ng; ++g) {
            float a[EG];
#pragma unroll
            for (int i = 0; i < EG; ++i) a[i] = ar[i];
            if (g + 1 < ng) fetch(k, g + 1);
            else if (k + 1 < nc) fetch(k + 1, 0);
#pragma unroll
            for (int i = 0; i < EG; ++i) {
                const int e = g * EG + i < ROWS ? g * EG + i : ROWS - 1;      // (rows beyond dim meet a = 0)
                const float4 v0 = *(const float4*)(cv0 + e * HB_DC_COLS);
                acc[0] = fmaf(a[i], v0.x, acc[0]); acc[1] = fmaf(a[i], v0.y, acc[1]); acc[2] = fmaf(a[i], v0.z, acc[2]); acc[3] = fmaf(a[i], v0.w, acc[3]);
                if (CPT == 8) {
                    const float4 v1 = *(const float4*)(cv0 + e * HB_DC_COLS + 4);
                    acc[CPT - 4] = fmaf(a[i], v1.x, acc[CPT - 4]); acc[CPT - 3] = fmaf(a[i], v1.y, acc[CPT - 3]);
                    acc[CPT - 2] = fmaf(a[i], v1.z, acc[CPT - 2]); acc[CPT - 1] = fmaf(a[i], v1.w, acc[CPT - 1]);
                }
            }
        }
        // S <- A S + B into the other buffer; the chunk's entry receives its carry-in
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
            const int c = cb + c0 + j;
            if (dok && c < vdim) wk[(size_t)d * vdim + c] = cur[flip][d * HB_DC_COLS + c0 + j];
            cur[flip ^ 1][d * HB_DC_COLS + c0 + j] = acc[j] + bk[j];
        }
        flip ^= 1;
    }
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
        const int c = cb + c0 + j;
        if (dok && c < vdim) St[(size_t)d * vdim + c] = cur[flip][d * HB_DC_COLS + c0 + j];
    }
}

// ---- matrix-state recurrence with token shift and a data-dependent decay per key channel ------------------------------------
// mixes[s][row] = h[row] + (h_prev - h[row]) * mu[s], s < 5; h_prev is the previous row of the request, or what the slot keeps
// behind its matrix state (the previous step's last normed input), or zero at position 0.
__global__ __launch_bounds__(256) void k_hb_shift_mix(const float* h, long ldh, const float* mu, float* mixes, long rows_stride, const float* state,
                                                      long per_slot, long prev_off, const int* pos, const int* row_req, const int* req_rows,
                                                      const int* req_state, int W) {
    const int row = blockIdx.x;
    const int r = row_req[row], rs = req_rows[r];
    const float* prev = row > rs ? h + (size_t)(row - 1) * ldh : (pos[row] == 0 ? nullptr : state + (size_t)req_state[r] * per_slot + prev_off);
    for (int i = blockIdx.y * 256 + threadIdx.x; i < W; i += 256 * gridDim.y) {
        const float x = h[(size_t)row * ldh + i], d = (prev ? prev[i] : 0.f) - x;
#pragma unroll
        for (int s2 = 0; s2 < 5; ++s2) mixes[(size_t)s2 * rows_stride + (size_t)row * W + i] = x + d * mu[(size_t)s2 * W + i];
    }
}
// Few-row steps: the five mixes and their projections in one launch.  A wave per output column n of [r | k | v | g | bottleneck]:
// its mix index is min(n / HD, 4); the operand x = h + (h_prev - h) * mu is formed in registers (the values k_hb_shift_mix stores),
// summed in k_hb_gemv's order; the bottleneck's columns take tanh.
template <typename T, int MR>
__global__ __launch_bounds__(256) void k_hb_shift_gemv(const float* h, long ldh, const float* mu, const T* Wt, const float* bias, float* C, long ldc,
                                                       const float* state, long per_slot, long prev_off, const int* pos, const int* row_req,
                                                       const int* req_rows, const int* req_state, int M, int N, int HD, int W) {
    const int lane = threadIdx.x & 63, n = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    const int seg = n / HD < 4 ? n / HD : 4;
    const float* mus = mu + (size_t)seg * W;
    const T* wr = Wt + (size_t)n * W;
    constexpr int CH = sizeof(T) == 2 ? 8 : 4;
    const float* prev[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        prev[m] = nullptr;
        if (m < M) {
            const int r = row_req[m], rs = req_rows[r];
            prev[m] = m > rs ? h + (size_t)(m - 1) * ldh : (pos[m] == 0 ? nullptr : state + (size_t)req_state[r] * per_slot + prev_off);
        }
    }
    float acc[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m] = 0.f;
    const bool vec = (W % CH == 0) && (ldh % 4 == 0) && ((per_slot | prev_off) % 4 == 0) &&
                     ((((size_t)Wt) | ((size_t)h) | ((size_t)mu) | ((size_t)state)) & 15) == 0;
    if (vec) {
        for (int k = lane * CH; k < W; k += 64 * CH) {
            float w[CH];
            if (sizeof(T) == 2) {
                const uint4 u = *(const uint4*)(wr + k);
                w[0] = bflo(u.x); w[1] = bfhi(u.x); w[2] = bflo(u.y); w[3] = bfhi(u.y);
                if (CH == 8) { w[4] = bflo(u.z); w[5] = bfhi(u.z); w[6] = bflo(u.w); w[7] = bfhi(u.w); }
            } else {
                const float4 u = *(const float4*)(wr + k);
                w[0] = u.x; w[1] = u.y; w[2] = u.z; w[3] = u.w;
            }
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                if (m >= M) break;
#pragma unroll
                for (int e = 0; e < CH; e += 4) {
                    const float4 x4 = *(const float4*)(h + (size_t)m * ldh + k + e), m4 = *(const float4*)(mus + k + e);
                    const float4 p4 = prev[m] ? *(const float4*)(prev[m] + k + e) : make_float4(0.f, 0.f, 0.f, 0.f);
                    acc[m] = fmaf(w[e], hb_operand<T>(x4.x + (p4.x - x4.x) * m4.x), acc[m]);
                    acc[m] = fmaf(w[e + 1], hb_operand<T>(x4.y + (p4.y - x4.y) * m4.y), acc[m]);
                    acc[m] = fmaf(w[e + 2], hb_operand<T>(x4.z + (p4.z - x4.z) * m4.z), acc[m]);
                    acc[m] = fmaf(w[e + 3], hb_operand<T>(x4.w + (p4.w - x4.w) * m4.w), acc[m]);
                }
            }
        }
    } else {
        for (int k = lane; k < W; k += 64) {
            const float w = hb_ld(wr + k);
#pragma unroll
            for (int m = 0; m < MR; ++m)
                if (m < M) {
                    const float x = h[(size_t)m * ldh + k], d = (prev[m] ? prev[m][k] : 0.f) - x;
                    acc[m] = fmaf(w, hb_operand<T>(x + d * mus[k]), acc[m]);
                }
        }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        const float sum = hb_wave_sum(acc[m]);
        if (m < M && lane == 0) {
            const float v = sum + (bias && seg < 4 ? bias[n] : 0.f);
            C[(size_t)m * ldc + n] = seg == 4 ? tanhf(v) : v;
        }
    }
}
// proj row = [r | k | v | g (H*dim each) | decay bottleneck (lora) | decay pre-activation d (H*dim)]; decay = exp(-exp(d)).
// Block = (request, head, 64 value columns); wave w keeps DPW key dims of the state in registers for the whole portion.  Per
// token: o = sum_i (S_i + bonus_i k_i v) r_i, then S_i <- decay_i S_i + k_i v; the waves' partial outputs are added in wave order.
// Block (r, 0, 0) finally stores the request's last normed input behind the matrix state (the next step's h_prev).
// Long portions run the request's rows in chunks of `chunk_len` side by side (mode 1, 2 with k_hb_shift_decay_carry between them):
//   mode 0  the whole portion from the slot's state, outputs, state and previous input stored (few-row steps)
//   mode 1  chunk z from a zero state, no outputs: its final state B and the product A of its decays go to the workspace
//   mode 2  chunk z replayed from its carry (left in the workspace by the carry kernel), outputs written
// Workspace entry of chunk k of request r: index rs / chunk_len + r + k (unique: the chunks of the requests before r number at most
// rs / chunk_len + r), [H][dim*dim + dim] floats each.
template <int DPW>
__global__ __launch_bounds__(64 * HB_SCAN_MAX_WAVES) void k_hb_shift_decay_scan(const float* proj, long ldp, float* out, long ldo, const float* bonus,
                                                                                float* state, long per_slot, const float* h, long ldh, int W,
                                                                                const int* req_rows, const int* req_state, const int* pos,
                                                                                int H, int dim, int lora, int TT, const float* head_w, float eps,
                                                                                float out_scale, int mode, int chunk_len, float* ws) {
    extern __shared__ float sm[];
    const int nw = blockDim.x >> 6, dpad = nw * DPW;
    float* rsm = sm;                       // [TT][dpad]
    float* ksm = rsm + TT * dpad;          // [TT][dpad]
    float* wsm = ksm + TT * dpad;          // [TT][dpad]
    float* vsm = wsm + TT * dpad;          // [TT][64]
    float* part = vsm + TT * 64;           // [2][nw][64]
    const int vt = (dim + 63) >> 6, chunk = mode == HB_SCAN_WHOLE ? 0 : blockIdx.z / vt, tile = mode == HB_SCAN_WHOLE ? blockIdx.z : blockIdx.z % vt;
    const int r = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x & 63, w = threadIdx.x >> 6, c = tile * 64 + lane;
    const int d0 = w * DPW;
    const int rs0 = req_rows[r], re0 = req_rows[r + 1];
    const int rs = mode == HB_SCAN_WHOLE ? rs0 : rs0 + chunk * chunk_len;
    if (rs >= re0) return;
    const int re = mode == HB_SCAN_WHOLE || rs + chunk_len > re0 ? re0 : rs + chunk_len;
    const bool ok = c < dim, fresh = pos[rs0] == 0;
    float* slot = state + (size_t)req_state[r] * per_slot;
    float* St = slot + (size_t)hd * dim * dim;
    if (mode != HB_SCAN_WHOLE) St = ws + ((size_t)(rs0 / chunk_len + r + chunk) * H + hd) * ((size_t)dim * dim + dim);
    const bool load = mode == HB_SCAN_REPLAY || (mode == HB_SCAN_WHOLE && !fresh);
    float S[DPW], u[DPW], A[DPW];
#pragma unroll
    for (int i = 0; i < DPW; ++i) {
        S[i] = (ok && load && d0 + i < dim) ? St[(size_t)(d0 + i) * dim + c] : 0.f;
        u[i] = d0 + i < dim ? bonus[hd * dim + d0 + i] : 0.f;
        A[i] = 1.f;
    }
    const int HD = H * dim, off_d = 4 * HD + lora;
    int flip = 0;
    for (int t0 = rs; t0 < re; t0 += TT) {
        const int nt = re - t0 < TT ? re - t0 : TT;
        __syncthreads();
        for (int idx = threadIdx.x; idx < nt * dpad; idx += blockDim.x) {
            const int tt = idx / dpad, d = idx - tt * dpad;
            float rv = 0.f, kv = 0.f, wv = 0.f;
            if (d < dim) {
                const float* p = proj + (size_t)(t0 + tt) * ldp + hd * dim + d;
                rv = p[0];
                kv = p[HD];
                wv = expf(-expf(p[off_d]));
            }
            rsm[idx] = rv; ksm[idx] = kv; wsm[idx] = wv;
        }
        for (int idx = threadIdx.x; idx < nt * 64; idx += blockDim.x) {
            const int tt = idx >> 6, cc = tile * 64 + (idx & 63);
            vsm[idx] = cc < dim ? proj[(size_t)(t0 + tt) * ldp + 2 * HD + hd * dim + cc] : 0.f;
        }
        __syncthreads();
        if (mode == HB_SCAN_REDUCE) {
            for (int tt = 0; tt < nt; ++tt) {
                const float v = vsm[tt * 64 + lane];
                const float* kt = ksm + tt * dpad + d0;
                const float* wt = wsm + tt * dpad + d0;
#pragma unroll
                for (int i = 0; i < DPW; ++i) {
                    S[i] = wt[i] * S[i] + kt[i] * v;
                    A[i] *= wt[i];
                }
            }
            continue;
        }
        for (int tt = 0; tt < nt; ++tt) {
            const float v = vsm[tt * 64 + lane];
            const float* rt = rsm + tt * dpad + d0;
            const float* kt = ksm + tt * dpad + d0;
            const float* wt = wsm + tt * dpad + d0;
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < DPW; ++i) {
                const float kv = kt[i] * v;
                o = fmaf(S[i] + u[i] * kv, rt[i], o);
                S[i] = wt[i] * S[i] + kv;
            }
            float* pt = part + flip * nw * 64;
            pt[w * 64 + lane] = o;
            __syncthreads();
            if (w == 0) {
                float sum = 0.f;
                if (ok) {
                    sum = pt[lane];
                    for (int k = 1; k < nw; ++k) sum += pt[k * 64 + lane];
                }
                if (head_w) {
                    // the block holds the whole head (dim <= 64): unit RMS, weight, silu gate and the mixer's scale here
                    const float inv = 1.0f / sqrtf(hb_wave_sum(sum * sum) / (float)dim + eps);
                    const float g = ok ? proj[(size_t)(t0 + tt) * ldp + 3 * HD + hd * dim + c] : 0.f;
                    sum = sum * inv * (ok ? head_w[hd * dim + c] : 0.f) * (g * hb_sigmoid(g)) * out_scale;
                }
                if (ok) out[(size_t)(t0 + tt) * ldo + hd * dim + c] = sum;
            }
            flip ^= 1;
        }
    }
    if (mode == HB_SCAN_REPLAY) return;
#pragma unroll
    for (int i = 0; i < DPW; ++i)
        if (d0 + i < dim) {
            if (ok) St[(size_t)(d0 + i) * dim + c] = S[i];
            if (mode == HB_SCAN_REDUCE && tile == 0 && lane == 0) St[(size_t)dim * dim + d0 + i] = A[i];
        }
    if (mode == HB_SCAN_WHOLE && hd == 0 && blockIdx.z == 0) {
        float* prev = slot + (size_t)H * dim * dim;
        for (int i = threadIdx.x; i < W; i += blockDim.x) prev[i] = h[(size_t)(re - 1) * ldh + i];
    }
}
// Between the two chunked passes: the slot's state is pushed through the request's chunks in order, S <- A_k S + B_k; every chunk's
// workspace entry receives its carry-in in place of B_k, the slot the final state and the request's last normed input.
__global__ __launch_bounds__(256) void k_hb_shift_decay_carry(float* ws, float* state, long per_slot, const float* h, long ldh, int W,
                                                              const int* req_rows, const int* req_state, const int* pos, int H, int dim,
                                                              int chunk_len) {
    const int r = blockIdx.x, hd = blockIdx.y;
    const int rs = req_rows[r], re = req_rows[r + 1];
    if (rs >= re) return;
    const int nc = (re - rs + chunk_len - 1) / chunk_len;
    const bool fresh = pos[rs] == 0;
    float* slot = state + (size_t)req_state[r] * per_slot;
    float* St = slot + (size_t)hd * dim * dim;
    const size_t per = (size_t)dim * dim + dim;
    float* w0 = ws + ((size_t)(rs / chunk_len + r) * H + hd) * per;
    for (int e = blockIdx.z * 256 + threadIdx.x; e < dim * dim; e += 256 * gridDim.z) {
        const int kd = e / dim;
        float S = fresh ? 0.f : St[e];
        for (int k = 0; k < nc; ++k) {
            float* wk = w0 + (size_t)k * H * per;
            const float B = wk[e], A = wk[(size_t)dim * dim + kd];
            wk[e] = S;
            S = A * S + B;
        }
        St[e] = S;
    }
    if (hd == 0 && blockIdx.z == 0) {
        float* prev = slot + (size_t)H * dim * dim;
        for (int i = threadIdx.x; i < W; i += 256) prev[i] = h[(size_t)(re - 1) * ldh + i];
    }
}

// ---- attention: rotary (interleaved pairs, first `rot` dims) + unit RMS on q and k, K / V into the paged cache -----------
// proj row = [q (H*dim) | k (G*dim) | v (G*vdim) | gate (H)].  Cache of one run: K [pages*ps][G*dim] then V [pages*ps][G*vdim].
// Options of the plain causal form: a weight on the normed q / k (shared by heads), a query temperature
// 1 + coef * ln(floor((p + 1) / every) + 1) at position p (coef 0: none), values divided by their RMS over vdim before they are cached.
#define HB_MAX_DPL 8   // dims per lane: dim <= 512
struct hb_qkv_opts {
    const float *q_norm, *k_norm;
    float temp_coef;
    int temp_every, v_unit;
};
template <typename T>
__global__ __launch_bounds__(64) void k_hb_attn_prep(float* proj, long ldp, T* cache, const float* inv_freq, const int* pos, const int* page,
                                                     const int* slot, int H, int G, int dim, int vdim, int rot, int ps, long v_base, float eps,
                                                     float* pool, const int* row_req, const int* ptab, int pts, int P, int ppp, hb_qkv_opts op) {
    const int row = blockIdx.x, hb = blockIdx.y, lane = threadIdx.x;
    const bool is_q = hb < H;
    const int g = hb - H;
    float* src = proj + (size_t)row * ldp + (is_q ? hb * dim : H * dim + g * dim);
    const float p = (float)pos[row];
    float y[HB_MAX_DPL];
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < HB_MAX_DPL; ++e) {
        const int d = lane + e * 64;
        y[e] = 0.f;
        if (d < dim) {
            float v = src[d];
            if (d < rot) {
                const float ang = p * inv_freq[d >> 1];
                float sn, cs;
                sincosf(ang, &sn, &cs);
                const float other = src[d ^ 1];
                v = (d & 1) ? (v * cs + other * sn) : (v * cs - other * sn);
            }
            y[e] = v;
            ss = fmaf(v, v, ss);
        }
    }
    ss = hb_wave_sum(ss);
    float inv = 1.0f / sqrtf(ss / (float)dim + eps);
    const float* nw = is_q ? op.q_norm : op.k_norm;
    const float temp = is_q && op.temp_coef != 0.f ? 1.0f + op.temp_coef * logf((float)((pos[row] + 1) / op.temp_every) + 1.0f) : 1.0f;
    const size_t tok = (size_t)page[row] * ps + slot[row];
    // every lane has read its inputs (both pair members) before anyone overwrites: one wave, the reduction above is the fence
#pragma unroll
    for (int e = 0; e < HB_MAX_DPL; ++e) {
        const int d = lane + e * 64;
        if (d < dim) {
            float o = y[e] * inv;
            if (nw) o *= nw[d];
            if (is_q) src[d] = o * temp;
            else hb_st(cache + tok * (size_t)(G * dim) + g * dim + d, o);
        }
    }
    if (!is_q) {
        const float* vs = proj + (size_t)row * ldp + H * dim + G * dim + g * vdim;
        float vinv = 1.0f;
        if (op.v_unit) {
            float vv = 0.f;
            for (int j = lane; j < vdim; j += 64) vv = fmaf(vs[j], vs[j], vv);
            vinv = 1.0f / sqrtf(hb_wave_sum(vv) / (float)vdim + eps);
        }
        for (int j = lane; j < vdim; j += 64) hb_st(cache + v_base + tok * (size_t)(G * vdim) + g * vdim + j, vs[j] * vinv);
        // steps with one row per request (pool != NULL): the pooled entry of a block this token closes, here instead of in a launch
        // of its own — the block's other tokens were cached by earlier steps; this row's own values enter as the cache rounds them,
        // last, which is k_hb_pool_update's arithmetic
        const int pi = pos[row];
        if (pool && (pi + 1) % P == 0) {
            const int* pt = ptab + (size_t)row_req[row] * pts;
            float* dst = pool + (((size_t)pt[pi / ps] * ppp + (pi % ps) / P) * G + g) * (size_t)(dim + vdim);
#pragma unroll
            for (int e = 0; e < HB_MAX_DPL; ++e) {
                const int d = lane + e * 64;
                if (d < dim) {
                    float sum = 0.f;
                    for (int j = pi - P + 1; j < pi; ++j) sum += hb_ld(cache + ((size_t)pt[j / ps] * ps + j % ps) * (size_t)(G * dim) + g * dim + d);
                    sum += hb_operand<T>(y[e] * inv);
                    dst[d] = sum / (float)P;
                }
            }
            for (int j2 = lane; j2 < vdim; j2 += 64) {
                float sum = 0.f;
                for (int j = pi - P + 1; j < pi; ++j)
                    sum += hb_ld(cache + v_base + ((size_t)pt[j / ps] * ps + j % ps) * (size_t)(G * vdim) + g * vdim + j2);
                sum += hb_operand<T>(vs[j2]);
                dst[dim + j2] = sum / (float)P;
            }
        }
    }
}

// The plain causal form behind a short convolution.  proj row = [q (H*dim) | k (G*dim) | v (G*vdim) | convolved q | k | v at off_y |
// processed q at off_qc | per block of 256 channels its sums of squares over the q and over the k channels at off_ss].
// First launch, one thread per (row, channel): the convolution (hb_conv_taps; the history is the whole state slot), and the block's
// share of the two sums of squares (block order fixed by the channel count).
__global__ __launch_bounds__(256) void k_hb_attn_conv(float* proj, long ldp, const float* cw, const float* state, long per_slot, const int* pos,
                                                      const int* row_req, const int* req_rows, const int* req_state, int nq, int nk, int C, int taps,
                                                      int off_y, int off_ss) {
    __shared__ float red[2][4];
    const int row = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    float v = 0.f;
    if (c < C) {
        const int r = row_req[row], rs = req_rows[r];
        v = hb_conv_taps(proj, ldp, cw, state + (size_t)req_state[r] * per_slot, row, rs, pos[row], pos[rs], c, C, taps);
        proj[(size_t)row * ldp + off_y + c] = v;
    }
    const float sq = hb_block_sum256(c < nq ? v * v : 0.f, red[0]), sk = hb_block_sum256(c >= nq && c < nq + nk ? v * v : 0.f, red[1]);
    if (threadIdx.x == 0) {
        proj[(size_t)row * ldp + off_ss + 2 * blockIdx.y] = sq;
        proj[(size_t)row * ldp + off_ss + 2 * blockIdx.y + 1] = sk;
    }
}
// Second launch, one wave per (row, head of q | k | v): q and k RMS-normed -- whole: over the entire projection (the blocks' sums added in
// block order) with weights [H*dim] / [G*dim]; else per head with weights [dim] shared by heads (NULL: none) --, then the first `rot`
// dims of the head rotated (interleaved pairs).  q goes to off_qc, k and v into the cache.  Blocks (row, H + 2G + j) of a request's
// last row: the convolution's history of 64 channels moves on.
template <typename T>
__global__ __launch_bounds__(64) void k_hb_attn_norm_rot(float* proj, long ldp, T* cache, float* state, long per_slot, const float* q_norm,
                                                         const float* k_norm, const float* inv_freq, const int* pos, const int* page,
                                                         const int* slot, const int* row_req, const int* req_rows, const int* req_state, int H,
                                                         int G, int dim, int vdim, int rot, int taps, int ps, long v_base, float eps, int off_y,
                                                         int off_qc, int off_ss, int whole) {
    const int row = blockIdx.x, hb = blockIdx.y, lane = threadIdx.x;
    const int nq = H * dim, nk = G * dim, nv = G * vdim, C = nq + nk + nv;
    if (hb >= H + 2 * G) {
        const int r = row_req[row], rs = req_rows[r], re = req_rows[r + 1], c = (hb - H - 2 * G) * 64 + lane;
        if (row != re - 1 || c >= C) return;
        hb_conv_hist_update(proj, ldp, state + (size_t)req_state[r] * per_slot, rs, re, pos[rs], c, C, taps);
        return;
    }
    const float* yr = proj + (size_t)row * ldp + off_y;
    const size_t tok = (size_t)page[row] * ps + slot[row];
    if (hb >= H + G) {
        const int g = hb - H - G;
        for (int j = lane; j < vdim; j += 64) hb_st(cache + v_base + tok * (size_t)nv + g * vdim + j, yr[nq + nk + g * vdim + j]);
        return;
    }
    const bool is_q = hb < H;
    const int c0 = is_q ? hb * dim : nq + (hb - H) * dim;       // the head's first channel
    float inv;
    if (whole) {
        const float* ss = proj + (size_t)row * ldp + off_ss + (is_q ? 0 : 1);
        float sum = 0.f;
        for (int b = 0; b < (C + 255) / 256; ++b) sum += ss[2 * b];
        inv = 1.0f / sqrtf(sum / (float)(is_q ? nq : nk) + eps);
    } else {
        float s2 = 0.f;
        for (int d = lane; d < dim; d += 64) s2 = fmaf(yr[c0 + d], yr[c0 + d], s2);
        inv = 1.0f / sqrtf(hb_wave_sum(s2) / (float)dim + eps);
    }
    const float* nw = is_q ? q_norm : k_norm;
    const int w0 = whole ? (is_q ? hb * dim : (hb - H) * dim) : 0;
    const float pf = (float)pos[row];
    for (int d = lane; d < dim; d += 64) {
        float v = yr[c0 + d] * inv * (nw ? nw[w0 + d] : 1.0f);
        if (d < rot) {
            const int dp = d ^ 1;
            const float other = yr[c0 + dp] * inv * (nw ? nw[w0 + dp] : 1.0f);
            float sn, cs;
            sincosf(pf * inv_freq[d >> 1], &sn, &cs);
            v = (d & 1) ? fmaf(v, cs, other * sn) : fmaf(v, cs, -(other * sn));
        }
        if (is_q) proj[(size_t)row * ldp + off_qc + c0 + d] = v;
        else hb_st(cache + tok * (size_t)nk + (c0 - nq) + d, v);
    }
}

// mean key / value of a block of `P` tokens, taken from the cache as stored, when the row's token closes the block.
// pool entry of block b sits with the page of the block's last token t: pool[(page(t) * ppp + (t % ps) / P)][G][dim + vdim].
template <typename T>
__global__ __launch_bounds__(64) void k_hb_pool_update(const T* cache, float* pool, const int* pos, const int* row_req, const int* ptab,
                                                       int pts, int G, int dim, int vdim, int P, int ps, int ppp, long v_base) {
    const int row = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
    const int p = pos[row];
    if ((p + 1) % P != 0) return;
    const int* pt = ptab + (size_t)row_req[row] * pts;
    const size_t entry = (size_t)pt[p / ps] * ppp + (p % ps) / P;
    float* dst = pool + (entry * G + g) * (size_t)(dim + vdim);
    for (int d = lane; d < dim + vdim; d += 64) {
        float s = 0.f;
        for (int j = p - P + 1; j <= p; ++j) {
            const size_t tok = (size_t)pt[j / ps] * ps + j % ps;
            s += d < dim ? hb_ld(cache + tok * (size_t)(G * dim) + g * dim + d)
                         : hb_ld(cache + v_base + tok * (size_t)(G * vdim) + g * vdim + (d - dim));
        }
        dst[d] = s / (float)P;
    }
}

// One block per (row, kv head).  Keys of a row at position p: the pooled blocks 0 .. nb-1 (nb = floor((p - window + 1) / P), those
// wholly before the window) and then the tokens max(0, p-window+1) .. p.  The block has SPLIT waves per query head of the group; wave
// (head, s) takes the 64-key chunks s, s + SPLIT, ... in ascending order: lane = key for the scores, lane = value column for the
// weighted sum, running maximum and sum across its chunks; the SPLIT partial results of a head are merged in split order.  SPLIT is a
// property of the layer (its group size), so a row's arithmetic does not depend on the step it is part of.
#define HB_MAX_VPL 8   // value columns per lane: vdim <= 512
#define HB_ATTN_SEG 4        // 64-key chunks per block of a segmented launch
#define HB_ATTN_SEG_ROWS 32  // steps of at most this many rows are segmented
__device__ __forceinline__ float hb_dot_row(const float* q, const float* k, int dim, bool vec) {
    float dot = 0.f;
    if (vec) {
        for (int d = 0; d < dim; d += 4) {
            const float4 a = *(const float4*)(q + d), b = *(const float4*)(k + d);
            dot = fmaf(a.x, b.x, dot); dot = fmaf(a.y, b.y, dot); dot = fmaf(a.z, b.z, dot); dot = fmaf(a.w, b.w, dot);
        }
    } else {
        for (int d = 0; d < dim; ++d) dot = fmaf(q[d], k[d], dot);
    }
    return dot;
}
__device__ __forceinline__ float hb_dot_row(const float* q, const bf16_t* k, int dim, bool vec) {
    float dot = 0.f;
    if (vec) {
        for (int d = 0; d < dim; d += 8) {
            const uint4 u = *(const uint4*)(k + d);
            const float4 a = *(const float4*)(q + d), b = *(const float4*)(q + d + 4);
            dot = fmaf(a.x, bflo(u.x), dot); dot = fmaf(a.y, bfhi(u.x), dot); dot = fmaf(a.z, bflo(u.y), dot); dot = fmaf(a.w, bfhi(u.y), dot);
            dot = fmaf(b.x, bflo(u.z), dot); dot = fmaf(b.y, bfhi(u.z), dot); dot = fmaf(b.z, bflo(u.w), dot); dot = fmaf(b.w, bfhi(u.w), dot);
        }
    } else {
        for (int d = 0; d < dim; ++d) dot = fmaf(q[d], bf2f(k[d]), dot);
    }
    return dot;
}
// one lane's share of a key row under the sixteen-lanes-per-key split: dims [sub*8, sub*8+8) of every 128
__device__ __forceinline__ float hb_dot_slices(const float* q, const float* k, int dim, int sub) {
    float part = 0.f;
    for (int d = sub * 8; d < dim; d += 128) {
        const float4 k0 = *(const float4*)(k + d), k1 = *(const float4*)(k + d + 4);
        const float4 a = *(const float4*)(q + d), b = *(const float4*)(q + d + 4);
        part = fmaf(a.x, k0.x, part); part = fmaf(a.y, k0.y, part); part = fmaf(a.z, k0.z, part); part = fmaf(a.w, k0.w, part);
        part = fmaf(b.x, k1.x, part); part = fmaf(b.y, k1.y, part); part = fmaf(b.z, k1.z, part); part = fmaf(b.w, k1.w, part);
    }
    return part;
}
__device__ __forceinline__ float hb_dot_slices(const float* q, const bf16_t* k, int dim, int sub) {
    float part = 0.f;
    for (int d = sub * 8; d < dim; d += 128) {
        const uint4 u = *(const uint4*)(k + d);
        const float4 a = *(const float4*)(q + d), b = *(const float4*)(q + d + 4);
        part = fmaf(a.x, bflo(u.x), part); part = fmaf(a.y, bfhi(u.x), part); part = fmaf(a.z, bflo(u.y), part); part = fmaf(a.w, bfhi(u.y), part);
        part = fmaf(b.x, bflo(u.z), part); part = fmaf(b.y, bfhi(u.z), part); part = fmaf(b.z, bflo(u.w), part); part = fmaf(b.w, bfhi(u.w), part);
    }
    return part;
}
template <typename T>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(1, 4))) void k_hb_attn(const float* proj, long ldp, const T* cache, const float* pool, float* out, long ldo, const int* pos,
                          const int* row_req, const int* ptab, int pts, int H, int G, int dim, int vdim, int window, int P, int ps, int ppp,
                          long v_base, float scale, int split, int seg_chunks, float* part, const float* gate, long ldg, float out_scale,
                          int Gc, long v_ld, int sink) {
    extern __shared__ float sm[];
    const int QG = H / G, NWV = QG * split;
    const int dimp = (dim + 3) & ~3;
    long* loc = (long*)sm;                  // [NWV][64]  (>= 0: token index in the cache, < 0: -(pool entry) - 1)
    float* pr = sm + NWV * 128;             // [NWV][64]
    float* qs = pr + NWV * 64;              // [QG][dimp]
    float* mo = qs + QG * dimp;             // [NWV][vdim + 2]: partial output, maximum, sum of each wave
    const int row = blockIdx.x, g = blockIdx.y, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int qh = wv % QG, sp = wv / QG, hq = g * QG + qh;
    // Gc heads per cached row; the grid's G groups of query heads divide evenly over them (Gc = G: one group per cached head; Gc < G:
    // G / Gc consecutive groups read the same cached head), value rows v_ld apart
    const int gk = g / (G / Gc);
    const size_t kld = (size_t)Gc * dim;
    const int p = pos[row];
    const int* pt = ptab + (size_t)row_req[row] * pts;
    const int first = p - window + 1;
    const int lo = first > 0 ? first : 0;
    const int nb = first > 0 ? first / P : 0;
    const int total = nb + (p - lo + 1);
    // few-row steps: block z takes the chunks [z * seg_chunks, (z + 1) * seg_chunks) and leaves an unnormalised partial result
    const int nchunks = (total + 63) >> 6;
    const int c0 = seg_chunks > 0 ? blockIdx.z * seg_chunks : 0;
    const int c1 = seg_chunks > 0 && c0 + seg_chunks < nchunks ? c0 + seg_chunks : nchunks;
    if (c0 >= nchunks) return;
    for (int i = threadIdx.x; i < QG * dimp; i += blockDim.x) {
        const int hh = i / dimp, d = i % dimp;
        qs[i] = d < dim ? proj[(size_t)row * ldp + (g * QG + hh) * dim + d] : 0.f;
    }
    __syncthreads();
    const float* q = qs + qh * dimp;
    const int pw = dim + vdim;
    const bool kvec = (dim % (sizeof(T) == 2 ? 8 : 4)) == 0, pvec = (dim % 4 == 0) && (pw % 4 == 0);
    const bool pair = sizeof(T) == 2 && (vdim % 2 == 0) && (dim % 2 == 0);
    const bool coop = (dim % 8 == 0) && (pw % 4 == 0);
    float m = -INFINITY, l = 0.f, acc[HB_MAX_VPL];
#pragma unroll
    for (int e = 0; e < HB_MAX_VPL; ++e) acc[e] = 0.f;
    long* wloc = loc + wv * 64;
    float* wpr = pr + wv * 64;
    for (int base = (c0 + sp) * 64; base < c1 * 64; base += split * 64) {
        const int u = base + lane;
        const int cnt = total - base < 64 ? total - base : 64;
        // where each lane's own key lives: >= 0 a token of the cache, < 0 a pooled entry
        long where = 0;
        if (u < total) {
            if (u < nb) {
                const int t = u * P + P - 1;
                where = -(long)(((size_t)pt[t / ps] * ppp + (t % ps) / P) * G + g) - 1;
            } else {
                const int j = lo + (u - nb);
                where = (long)((size_t)pt[j / ps] * ps + j % ps);
            }
        }
        __builtin_amdgcn_wave_barrier();
        wloc[lane] = where;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        float dot = 0.f;
        const int npool_c = nb - base < 0 ? 0 : (nb - base < cnt ? nb - base : cnt);
        if (coop && sizeof(T) == 2 && dim <= 128 && npool_c == 0) {
            // a chunk of cached tokens only, one 128-dim slice: all sixteen row requests of the wave go out before the first is used
            const int sub = lane & 15, grp = lane >> 4;
            const bool mine_ok = sub * 8 < dim;
            const bf16_t* kb = (const bf16_t*)cache + gk * dim + (mine_ok ? sub * 8 : 0);
            float4 qa = make_float4(0.f, 0.f, 0.f, 0.f), qb = qa;
            if (mine_ok) { qa = *(const float4*)(q + sub * 8); qb = *(const float4*)(q + sub * 8 + 4); }
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                uint4 kreg[8];
#pragma unroll
                for (int i8 = 0; i8 < 8; ++i8) {
                    const int it = half * 8 + i8;
                    const int kk = it * 4 + grp < cnt ? it * 4 + grp : cnt - 1;
                    kreg[i8] = *(const uint4*)(kb + (size_t)wloc[kk] * kld);
                }
#pragma unroll
                for (int i8 = 0; i8 < 8; ++i8) {
                    const int it = half * 8 + i8;
                    const uint4 u4 = kreg[i8];
                    float part = 0.f;
                    part = fmaf(qa.x, bflo(u4.x), part); part = fmaf(qa.y, bfhi(u4.x), part); part = fmaf(qa.z, bflo(u4.y), part); part = fmaf(qa.w, bfhi(u4.y), part);
                    part = fmaf(qb.x, bflo(u4.z), part); part = fmaf(qb.y, bfhi(u4.z), part); part = fmaf(qb.z, bflo(u4.w), part); part = fmaf(qb.w, bfhi(u4.w), part);
                    part += __shfl_xor(part, 8, 64);
                    part += __shfl_xor(part, 4, 64);
                    part += __shfl_xor(part, 2, 64);
                    part += __shfl_xor(part, 1, 64);
                    const float got = __shfl(part, (lane & 3) * 16, 64);
                    if ((lane >> 2) == it) dot = got;
                }
            }
        } else if (coop) {
            // sixteen lanes per key: each takes 8 dims of every 128 (one 16-byte request of a bf16 row), so a wave's request covers
            // four whole key rows instead of 64 scattered ones; the 16 partial dots are added by a butterfly, then lane L takes key L's
            const int sub = lane & 15, grp = lane >> 4;
            for (int it = 0; it * 4 < cnt; ++it) {
                const int kk = it * 4 + grp < cnt ? it * 4 + grp : cnt - 1;
                const long w = wloc[kk];
                float part = 0.f;
                if (w < 0) {
                    const float* kp = pool + (size_t)(-w - 1) * pw;
                    for (int d = sub * 8; d < dim; d += 128) {
                        const float4 k0 = *(const float4*)(kp + d), k1 = *(const float4*)(kp + d + 4);
                        const float4 a = *(const float4*)(q + d), b2 = *(const float4*)(q + d + 4);
                        part = fmaf(a.x, k0.x, part); part = fmaf(a.y, k0.y, part); part = fmaf(a.z, k0.z, part); part = fmaf(a.w, k0.w, part);
                        part = fmaf(b2.x, k1.x, part); part = fmaf(b2.y, k1.y, part); part = fmaf(b2.z, k1.z, part); part = fmaf(b2.w, k1.w, part);
                    }
                } else {
                    part = hb_dot_slices(q, cache + (size_t)w * kld + gk * dim, dim, sub);
                }
                part += __shfl_xor(part, 8, 64);
                part += __shfl_xor(part, 4, 64);
                part += __shfl_xor(part, 2, 64);
                part += __shfl_xor(part, 1, 64);
                const float got = __shfl(part, (lane & 3) * 16, 64);
                if ((lane >> 2) == it) dot = got;
            }
        } else if (u < total) {
            dot = where < 0 ? hb_dot_row(q, pool + (size_t)(-where - 1) * pw, dim, pvec)
                            : hb_dot_row(q, cache + (size_t)where * kld + gk * dim, dim, kvec);
        }
        const float sc = u < total ? dot * scale : -INFINITY;
        const float mn = fmaxf(m, hb_wave_max(sc));
        const float alpha = expf(m - mn);
        const float e = u < total ? expf(sc - mn) : 0.f;
        l = l * alpha + hb_wave_sum(e);
        m = mn;
        wpr[lane] = e;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        // pooled keys come first in the key order: two loops without a per-key branch, many independent requests in flight each.
        // acc[e] belongs to value column hb_vcol(e): with a bf16 cache and an even vdim a lane owns two adjacent columns of each
        // 128-column group (one 4-byte request per key), else one column of each 64-column group.
        const int npool = nb - base < 0 ? 0 : (nb - base < cnt ? nb - base : cnt);
        const size_t gv = (size_t)v_ld;
        if (pair) {
#pragma unroll
            for (int c = 0; c < HB_MAX_VPL / 2; ++c) {
                if (c * 128 < vdim) {
                    const int j = c * 128 + 2 * lane;
                    const int jj = j < vdim ? j : vdim - 2;
                    const float* pbase = pool + dim + jj;
                    const T* vbase = cache + v_base + gk * vdim + jj;
                    float a0 = acc[2 * c] * alpha, a1 = acc[2 * c + 1] * alpha;
                    for (int k0 = 0; k0 < npool; k0 += 8) {
                        float pv[8];
                        float2 vv[8];
#pragma unroll
                        for (int x = 0; x < 8; ++x) {
                            const int kk = k0 + x < npool ? k0 + x : npool - 1;
                            pv[x] = k0 + x < npool ? wpr[kk] : 0.f;
                            vv[x] = *(const float2*)(pbase + (size_t)(-wloc[kk] - 1) * pw);
                        }
#pragma unroll
                        for (int x = 0; x < 8; ++x) { a0 = fmaf(pv[x], vv[x].x, a0); a1 = fmaf(pv[x], vv[x].y, a1); }
                    }
                    for (int k0 = npool; k0 < cnt; k0 += 16) {
                        float pv[16];
                        u32 vv[16];
#pragma unroll
                        for (int x = 0; x < 16; ++x) {
                            const int kk = k0 + x < cnt ? k0 + x : cnt - 1;
                            pv[x] = k0 + x < cnt ? wpr[kk] : 0.f;
                            vv[x] = *(const u32*)(vbase + (size_t)wloc[kk] * gv);
                        }
#pragma unroll
                        for (int x = 0; x < 16; ++x) { a0 = fmaf(pv[x], bflo(vv[x]), a0); a1 = fmaf(pv[x], bfhi(vv[x]), a1); }
                    }
                    acc[2 * c] = a0;
                    acc[2 * c + 1] = a1;
                }
            }
        } else {
#pragma unroll
        for (int c = 0; c < HB_MAX_VPL; ++c) {
            const int j = lane + c * 64;
            if (c * 64 < vdim) {
                const int jj = j < vdim ? j : vdim - 1;
                const float* pbase = pool + dim + jj;
                const T* vbase = cache + v_base + gk * vdim + jj;
                float a = acc[c] * alpha;
                for (int k0 = 0; k0 < npool; k0 += 8) {
                    float pv[8], vv[8];
#pragma unroll
                    for (int x = 0; x < 8; ++x) {
                        const int kk = k0 + x < npool ? k0 + x : npool - 1;
                        pv[x] = k0 + x < npool ? wpr[kk] : 0.f;
                        vv[x] = pbase[(size_t)(-wloc[kk] - 1) * pw];
                    }
#pragma unroll
                    for (int x = 0; x < 8; ++x) a = fmaf(pv[x], vv[x], a);
                }
                for (int k0 = npool; k0 < cnt; k0 += 16) {
                    float pv[16], vv[16];
#pragma unroll
                    for (int x = 0; x < 16; ++x) {
                        const int kk = k0 + x < cnt ? k0 + x : cnt - 1;
                        pv[x] = k0 + x < cnt ? wpr[kk] : 0.f;
                        vv[x] = hb_ld(vbase + (size_t)wloc[kk] * gv);
                    }
#pragma unroll
                    for (int x = 0; x < 16; ++x) a = fmaf(pv[x], vv[x], a);
                }
                acc[c] = a;
            }
        }
        }
        __builtin_amdgcn_wave_barrier();
    }
    // merge the splits of each head in split order
    float* mine = mo + (size_t)wv * (vdim + 2);
#pragma unroll
    for (int c = 0; c < HB_MAX_VPL; ++c) {
        const int j = pair ? (c >> 1) * 128 + 2 * lane + (c & 1) : lane + c * 64;
        if (j < vdim) mine[j] = acc[c];
    }
    if (lane == 0) { mine[vdim] = m; mine[vdim + 1] = l; }
    __syncthreads();
    if (sp == 0) {
        // sink: a key of score 0 without a value joins the softmax of the whole row (a segmented launch adds it in the merge)
        float mm = sink && !part ? 0.f : -INFINITY;
        for (int s2 = 0; s2 < split; ++s2) mm = fmaxf(mm, mo[(size_t)(s2 * QG + qh) * (vdim + 2) + vdim]);
        float lt = 0.f;
        for (int s2 = 0; s2 < split; ++s2) {
            const float* o2 = mo + (size_t)(s2 * QG + qh) * (vdim + 2);
            lt += o2[vdim + 1] * expf(o2[vdim] - mm);
        }
        if (sink && !part) lt += expf(-mm);
        if (part) {
            float* dst = part + ((size_t)(row * H + hq) * gridDim.z + blockIdx.z) * (vdim + 2);
            for (int j = lane; j < vdim; j += 64) {
                float a = 0.f;
                for (int s2 = 0; s2 < split; ++s2) {
                    const float* o2 = mo + (size_t)(s2 * QG + qh) * (vdim + 2);
                    a += o2[j] * expf(o2[vdim] - mm);
                }
                dst[j] = a;
            }
            if (lane == 0) { dst[vdim] = mm; dst[vdim + 1] = lt; }
            return;
        }
        const float gmul = (gate ? hb_sigmoid(gate[(size_t)row * ldg + hq]) : 1.0f) * out_scale;
        for (int j = lane; j < vdim; j += 64) {
            float a = 0.f;
            for (int s2 = 0; s2 < split; ++s2) {
                const float* o2 = mo + (size_t)(s2 * QG + qh) * (vdim + 2);
                a += o2[j] * expf(o2[vdim] - mm);
            }
            out[(size_t)row * ldo + hq * vdim + j] = a / lt * gmul;
        }
    }
}

// few-row steps: the segments' partial results of a (row, head), merged in segment order; output gate applied here
__global__ __launch_bounds__(64) void k_hb_attn_merge(const float* part, int nseg_grid, float* out, long ldo, const int* pos, int H, int vdim,
                                                      int window, int P, int seg_chunks, const float* gate, long ldg, float out_scale, int chunk,
                                                      int sink) {
    const int row = blockIdx.x, hq = blockIdx.y, lane = threadIdx.x;
    const int p = pos[row];
    const int first = p - window + 1;
    const int total = (first > 0 ? first / P : 0) + (p - (first > 0 ? first : 0) + 1);
    const int nseg = ((total + chunk - 1) / chunk + seg_chunks - 1) / seg_chunks;
    const float* src = part + (size_t)(row * H + hq) * nseg_grid * (vdim + 2);
    // lane s of each 64 segments fetches segment s's maximum and sum; the total is added in segment order
    float mm = sink ? 0.f : -INFINITY;      // sink: a key of score 0 without a value
    for (int s0 = 0; s0 < nseg; s0 += 64) mm = fmaxf(mm, s0 + lane < nseg ? src[(size_t)(s0 + lane) * (vdim + 2) + vdim] : -INFINITY);
    mm = hb_wave_max(mm);
    const float gmul = (gate ? hb_sigmoid(gate[(size_t)row * ldg + hq]) : 1.0f) * out_scale;
    float lt = 0.f;
    float acc[HB_MAX_VPL];
#pragma unroll
    for (int e = 0; e < HB_MAX_VPL; ++e) acc[e] = 0.f;
    for (int s0 = 0; s0 < nseg; s0 += 64) {
        const bool mine = s0 + lane < nseg;
        const float wmine = mine ? expf(src[(size_t)(s0 + lane) * (vdim + 2) + vdim] - mm) : 0.f;
        const float lmine = mine ? src[(size_t)(s0 + lane) * (vdim + 2) + vdim + 1] * wmine : 0.f;
        const int ns = nseg - s0 < 64 ? nseg - s0 : 64;
        for (int s2 = 0; s2 < ns; s2 += 4) {
            // four segments' values on their way before the first is used
            float v[4][HB_MAX_VPL];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const float* sp = src + (size_t)(s0 + (s2 + u < ns ? s2 + u : ns - 1)) * (vdim + 2);
#pragma unroll
                for (int e = 0; e < HB_MAX_VPL; ++e) {
                    const int j = lane + e * 64;
                    v[u][e] = j < vdim ? sp[j] : 0.f;
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (s2 + u >= ns) break;
                const float w = __shfl(wmine, s2 + u, 64);
                lt += __shfl(lmine, s2 + u, 64);
#pragma unroll
                for (int e = 0; e < HB_MAX_VPL; ++e) acc[e] += v[u][e] * w;
            }
        }
    }
    if (sink) lt += expf(-mm);
#pragma unroll
    for (int e = 0; e < HB_MAX_VPL; ++e) {
        const int j = lane + e * 64;
        if (j < vdim) out[(size_t)row * ldo + hq * vdim + j] = acc[e] / lt * gmul;
    }
}

// ---- latent attention, steps of few rows: one block per (row, segment of keys), every head against a key tile held in LDS ------
// All heads read the same cached rows [R latent | r rotated key part]; the first R values are also the value.  The block stages KT
// keys at a time in LDS (as the cache holds them), every thread takes one key and HPT heads for the scores (fp32 sums over the dims in
// ascending order), the weights of a (head, tile) come from one running softmax per head, then every thread owns two value columns of
// all heads of the group.  Heads are taken in groups of 16.  part != NULL: the block leaves an unnormalised partial result per head
// (k_hb_attn_merge's layout) for its `cpb` tiles; else it covers all keys and writes o / l * sigmoid(gate) * out_scale.
#define HB_LAT_HG 16
// KT keys per tile; NT threads per block: NT / KT thread groups share the 16 heads of a group for the scores (NT <= 16 * KT), and
// NT / 256 thread groups share them for the weighted sums (every 256 threads cover the value columns two by two)
template <typename T> struct hb_lat_tile {
    static constexpr int KT = sizeof(T) == 2 ? 64 : 32;
    static constexpr int NT = sizeof(T) == 2 ? 1024 : 512;
};
template <typename T>
__global__ __launch_bounds__(hb_lat_tile<T>::NT) void k_hb_latent_attn_rows(const float* qa, long ldq, const T* cache, float* out, long ldo, const int* pos,
                                                             const int* row_req, const int* ptab, int pts, int H, int R, int r, int window,
                                                             int ps, float scale, int cpb, float* part, const float* gate, long ldg,
                                                             float out_scale, int DP) {
    constexpr int KT = hb_lat_tile<T>::KT, NT = hb_lat_tile<T>::NT, NS = NT / KT, HPT = HB_LAT_HG / NS, PVH = HB_LAT_HG / (NT / 256);
    extern __shared__ float sm[];
    const int D = R + r, Dq = (D + 3) & ~3;
    T* Kt = (T*)sm;                                                    // [KT][DP]
    float* qs = sm + (((size_t)KT * DP * sizeof(T) + 15) / 16) * 4;    // [16][Dq]
    float* pw = qs + HB_LAT_HG * Dq;                                   // [KT][16] weights of the tile
    float* al = pw + KT * HB_LAT_HG;                                   // [16] rescale factors of the tile
    float* ml = al + HB_LAT_HG;                                        // [16][2] final maximum and sum
    const int row = blockIdx.x, seg = blockIdx.y, tid = threadIdx.x;
    const int p = pos[row];
    const int* pt = ptab + (size_t)row_req[row] * pts;
    const int lo = p - window + 1 > 0 ? p - window + 1 : 0;
    const int total = p - lo + 1, nchunks = (total + KT - 1) / KT;
    const int c0 = seg * cpb, c1 = c0 + cpb < nchunks ? c0 + cpb : nchunks;
    if (c0 >= nchunks) return;
    const int j = tid % KT, hs = tid / KT;
    constexpr int VE = 16 / sizeof(T);
    const bool vec = (D % VE == 0) && ((((size_t)cache) & 15) == 0);
    const bool quad = (D % 4 == 0);
    for (int h0 = 0; h0 < H; h0 += HB_LAT_HG) {
        const int hg = H - h0 < HB_LAT_HG ? H - h0 : HB_LAT_HG;
        __syncthreads();
        const float* qrow = qa + (size_t)row * ldq + (size_t)h0 * D;
        if (quad && (ldq % 4 == 0) && ((((size_t)qa) & 15) == 0)) {
            // the group's queries are one contiguous run of hg * D floats (Dq = D): 16-byte requests, several in flight per thread
            const int nv = HB_LAT_HG * D / 4, have = hg * D / 4;
            constexpr int U = 5;
            for (int i0 = tid; i0 < nv; i0 += NT * U) {
                float4 u[U];
#pragma unroll
                for (int k = 0; k < U; ++k) {
                    const int idx = i0 + NT * k;
                    u[k] = idx < have ? *(const float4*)(qrow + 4 * (size_t)idx) : make_float4(0.f, 0.f, 0.f, 0.f);
                }
#pragma unroll
                for (int k = 0; k < U; ++k) {
                    const int idx = i0 + NT * k;
                    if (idx < nv) *(float4*)(qs + 4 * (size_t)idx) = u[k];
                }
            }
        } else {
            for (int i = tid; i < HB_LAT_HG * Dq; i += NT) {
                const int h = i / Dq, d = i - h * Dq;
                qs[i] = (h < hg && d < D) ? qrow[(size_t)h * D + d] : 0.f;
            }
        }
        float m[HPT], l[HPT], acc[PVH][2];
        const int ct = tid & 255, hb = (tid >> 8) * PVH;      // the thread's column pair (2 ct, 2 ct + 1) and first head of the weighted sums
#pragma unroll
        for (int i = 0; i < HPT; ++i) { m[i] = -INFINITY; l[i] = 0.f; }
#pragma unroll
        for (int h = 0; h < PVH; ++h) acc[h][0] = acc[h][1] = 0.f;
        for (int c = c0; c < c1; ++c) {
            const int base = c * KT, cnt = total - base < KT ? total - base : KT;
            __syncthreads();
            // the tile: key jj of the tile is the token at position lo + base + jj; rows behind the last key are zero
            if (vec) {
                // 16-byte requests, six in flight per thread before the first is stored
                const int per = D / VE, nv = KT * per;
                constexpr int U = 6;
                for (int i0 = tid; i0 < nv; i0 += NT * U) {
                    uint4 u[U];
#pragma unroll
                    for (int k = 0; k < U; ++k) {
                        const int idx = i0 + NT * k, jj = idx / per, v = idx - jj * per;
                        u[k] = make_uint4(0, 0, 0, 0);
                        if (idx < nv && jj < cnt) {
                            const int t = lo + base + jj;
                            u[k] = *(const uint4*)(cache + ((size_t)pt[t / ps] * ps + t % ps) * (size_t)D + (size_t)v * VE);
                        }
                    }
#pragma unroll
                    for (int k = 0; k < U; ++k) {
                        const int idx = i0 + NT * k, jj = idx / per, v = idx - jj * per;
                        if (idx < nv) {
                            u32* dst = (u32*)(Kt + (size_t)jj * DP + (size_t)v * VE);
                            dst[0] = u[k].x; dst[1] = u[k].y; dst[2] = u[k].z; dst[3] = u[k].w;
                        }
                    }
                }
            } else {
                for (int idx = tid; idx < KT * D; idx += NT) {
                    const int jj = idx / D, d = idx - jj * D;
                    T v = (T)0;
                    if (jj < cnt) {
                        const int t = lo + base + jj;
                        v = cache[((size_t)pt[t / ps] * ps + t % ps) * (size_t)D + d];
                    }
                    Kt[(size_t)jj * DP + d] = v;
                }
            }
            __syncthreads();
            float dot[HPT];
#pragma unroll
            for (int i = 0; i < HPT; ++i) dot[i] = 0.f;
            const T* kr = Kt + (size_t)j * DP;
            int d = 0;
            if (quad) {
#pragma unroll 4
                for (; d < D; d += 4) {
                    float k0, k1, k2, k3;
                    if (sizeof(T) == 2) {
                        const u32 a = *(const u32*)(kr + d), b = *(const u32*)(kr + d + 2);
                        k0 = bflo(a); k1 = bfhi(a); k2 = bflo(b); k3 = bfhi(b);
                    } else {
                        k0 = hb_ld(kr + d); k1 = hb_ld(kr + d + 1); k2 = hb_ld(kr + d + 2); k3 = hb_ld(kr + d + 3);
                    }
#pragma unroll
                    for (int i = 0; i < HPT; ++i) {
                        const float4 q4 = *(const float4*)(qs + (hs + NS * i) * Dq + d);
                        dot[i] = fmaf(q4.x, k0, dot[i]); dot[i] = fmaf(q4.y, k1, dot[i]);
                        dot[i] = fmaf(q4.z, k2, dot[i]); dot[i] = fmaf(q4.w, k3, dot[i]);
                    }
                }
            } else {
                for (; d < D; ++d) {
                    const float kv = hb_ld(kr + d);
#pragma unroll
                    for (int i = 0; i < HPT; ++i) dot[i] = fmaf(qs[(hs + NS * i) * Dq + d], kv, dot[i]);
                }
            }
            const bool valid = j < cnt;
#pragma unroll
            for (int i = 0; i < HPT; ++i) {
                const float sc = valid ? dot[i] * scale : -INFINITY;
                float mx = sc;
#pragma unroll
                for (int o = KT / 2; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
                const float mn = fmaxf(m[i], mx);
                const float alpha = expf(m[i] - mn);
                const float e = valid ? expf(sc - mn) : 0.f;
                float sum = e;
#pragma unroll
                for (int o = KT / 2; o >= 1; o >>= 1) sum += __shfl_xor(sum, o, 64);
                l[i] = l[i] * alpha + sum;
                m[i] = mn;
                pw[j * HB_LAT_HG + hs + NS * i] = e;
                if (j == 0) al[hs + NS * i] = alpha;
            }
            __syncthreads();
            if (2 * ct < R) {
                const bool two = 2 * ct + 1 < R;
#pragma unroll
                for (int h = 0; h < PVH; ++h) { const float a = al[hb + h]; acc[h][0] *= a; acc[h][1] *= a; }
#pragma unroll 4
                for (int jj = 0; jj < cnt; ++jj) {
                    float v0, v1 = 0.f;
                    if (sizeof(T) == 2) {
                        const u32 u = *(const u32*)(Kt + (size_t)jj * DP + 2 * ct);      // (DP is even and > 2 * ct: the pair lies in the row)
                        v0 = bflo(u); v1 = bfhi(u);
                    } else {
                        v0 = hb_ld(Kt + (size_t)jj * DP + 2 * ct);
                        if (two) v1 = hb_ld(Kt + (size_t)jj * DP + 2 * ct + 1);
                    }
#pragma unroll
                    for (int h4 = 0; h4 < PVH; h4 += 4) {
                        const float4 p4 = *(const float4*)(pw + jj * HB_LAT_HG + hb + h4);
                        acc[h4][0] = fmaf(p4.x, v0, acc[h4][0]); acc[h4][1] = fmaf(p4.x, v1, acc[h4][1]);
                        acc[h4 + 1][0] = fmaf(p4.y, v0, acc[h4 + 1][0]); acc[h4 + 1][1] = fmaf(p4.y, v1, acc[h4 + 1][1]);
                        acc[h4 + 2][0] = fmaf(p4.z, v0, acc[h4 + 2][0]); acc[h4 + 2][1] = fmaf(p4.z, v1, acc[h4 + 2][1]);
                        acc[h4 + 3][0] = fmaf(p4.w, v0, acc[h4 + 3][0]); acc[h4 + 3][1] = fmaf(p4.w, v1, acc[h4 + 3][1]);
                    }
                }
            }
        }
        if (j == 0)
#pragma unroll
            for (int i = 0; i < HPT; ++i) { ml[2 * (hs + NS * i)] = m[i]; ml[2 * (hs + NS * i) + 1] = l[i]; }
        __syncthreads();
        if (2 * ct < R) {
            const bool two = 2 * ct + 1 < R;
#pragma unroll
            for (int h = 0; h < PVH; ++h) {
                if (hb + h >= hg) break;
                const int hq = h0 + hb + h;
                if (part) {
                    float* dst = part + ((size_t)(row * H + hq) * gridDim.y + seg) * (R + 2);
                    dst[2 * ct] = acc[h][0];
                    if (two) dst[2 * ct + 1] = acc[h][1];
                    if (ct == 0) { dst[R] = ml[2 * (hb + h)]; dst[R + 1] = ml[2 * (hb + h) + 1]; }
                } else {
                    const float gmul = (gate ? hb_sigmoid(gate[(size_t)row * ldg + hq]) : 1.0f) * out_scale;
                    float* dst = out + (size_t)row * ldo + (size_t)hq * R;
                    dst[2 * ct] = acc[h][0] / ml[2 * (hb + h) + 1] * gmul;
                    if (two) dst[2 * ct + 1] = acc[h][1] / ml[2 * (hb + h) + 1] * gmul;
                }
            }
        }
    }
}
// row length of the key tile in LDS, in elements: 4-byte aligned rows whose stride in 4-byte words is odd (no two of a wave's rows
// start in the same bank)
template <typename T> static int hb_lat_dp(int D) {
    if (sizeof(T) == 4) return D | 1;
    int dp = (D + 1) & ~1;
    return (dp / 2) % 2 ? dp : dp + 2;
}

// ---- latent attention, steps of many rows, bf16 cache: the matrix-core form -------------------------------------------------------
// A block takes four consecutive rows of one request, one wave per row, and a group of up to 16 heads; the heads are the 16 columns of
// every product, so all 16 x 16 entries of a tile share the row's window.  Tiles of 64 keys are staged in LDS twice: as the cache
// holds them (Kt[key][dim]) and the value part transposed (Vt[value column][key]).  Per tile and wave:
//   S^T[key][head] = sum_dim Kt[key][dim] Q[head][dim]     v_mfma_f32_16x16x32_bf16, A = Kt rows from LDS, B = the row's query in
//                                                          registers (fp32 split in two bf16 parts, hi + lo: two products)
//   running softmax per head over the lane's 16 scores and the four lane groups
//   O^T[col][head] += sum_key Vt[col][key] P[head][key]    A = Vt rows from LDS; B = the weights as they sit in the lanes after the first
//                                                          product (lane group g holds keys 4g..4g+3 of each 16-key tile: the k index of
//                                                          the product is laid out to match, so no weight leaves its lane), hi + lo
// Scores, maxima, sums and weights are fp32; the two-part operands keep 16 bits of mantissa of the queries and weights.
// Tile t of the launch is found by walking the requests' row counts (ceil(rows / 4) tiles each); blocks beyond the last tile leave.
#define HB_LM_VLD 72      // keys per row of the transposed value tile (64 + 8: rows 16 bytes apart in banks)
__device__ __forceinline__ void hb_split_bf16x8(const float* v, uint4& hi, uint4& lo) {
    float h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = bfround(v[i]);
    hi = make_uint4(pack_bf2(h[0], h[1]), pack_bf2(h[2], h[3]), pack_bf2(h[4], h[5]), pack_bf2(h[6], h[7]));
    lo = make_uint4(pack_bf2(v[0] - h[0], v[1] - h[1]), pack_bf2(v[2] - h[2], v[3] - h[3]), pack_bf2(v[4] - h[4], v[5] - h[5]),
                    pack_bf2(v[6] - h[6], v[7] - h[7]));
}
__device__ __forceinline__ hb_f32x4 hb_mfma_bf16(uint4 a, uint4 b, hb_f32x4 c) {
    union { uint4 u; hb_bf16x8 v; } x, y;
    x.u = a; y.u = b;
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x.v, y.v, c, 0, 0, 0);
}
template <int KS, int CT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void k_hb_latent_attn_mfma(
    const float* qa, long ldq, const bf16_t* cache, float* out, long ldo, const int* pos, const int* req_rows, int n_req, const int* ptab, int pts,
    int H, int R, int r, int window, int ps, float scale, const float* gate, long ldg, float out_scale, int ks_n, int ct_n) {
    extern __shared__ float sm[];
    const int D = R + r, DPK = ks_n * 32 + 8;
    long* tokoff = (long*)sm;                      // [64] where the tile's keys start in the cache
    bf16_t* Kt = (bf16_t*)(sm + 128);              // [64][DPK]
    bf16_t* Vt = Kt + 64 * DPK;                    // [ct_n * 16][HB_LM_VLD]
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, col = lane & 15, g = lane >> 4;
    int t = blockIdx.x, rq = -1, rs = 0, re = 0;
    for (int q = 0; q < n_req; ++q) {
        const int a = req_rows[q], b = req_rows[q + 1], nt = (b - a + 3) >> 2;
        if (t < nt) { rq = q; rs = a + 4 * t; re = b; break; }
        t -= nt;
    }
    if (rq < 0) return;
    const int nrows = re - rs < 4 ? re - rs : 4;
    const bool active = wv < nrows;
    const int row = rs + (active ? wv : 0);
    const int p0 = pos[rs], pl = pos[rs + nrows - 1], p = pos[row];
    const int lo_t = p0 - window + 1 > 0 ? p0 - window + 1 : 0, lo_r = p - window + 1 > 0 ? p - window + 1 : 0;
    const int nchunks = (pl - lo_t + 64) >> 6;
    const int* pt = ptab + (size_t)rq * pts;
    const int h0 = blockIdx.y * 16, hg = H - h0 < 16 ? H - h0 : 16;
    // the row's query: head `col`, dims ks*32 + g*8 .. +8 of every 32-dim step
    uint4 qh[KS], ql[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = 0.f;
        const int d0 = ks * 32 + g * 8;
        if (ks < ks_n && active && col < hg && d0 < D) {
            const float* src = qa + (size_t)row * ldq + (size_t)(h0 + col) * D + d0;
            const float4 a = *(const float4*)src, b = *(const float4*)(src + 4);
            v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
        }
        hb_split_bf16x8(v, qh[ks], ql[ks]);
    }
    // value-tile rows behind the last value column are never written again: zero once
    for (int i = R * HB_LM_VLD + tid; i < ct_n * 16 * HB_LM_VLD; i += 256) Vt[i] = (bf16_t)0;
    float m = -INFINITY, l = 0.f;
    hb_f32x4 oacc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) oacc[ct] = hb_f32x4{0.f, 0.f, 0.f, 0.f};
    const int per = D >> 3, pv = ks_n * 4, nv = 64 * pv;
    // idx / pv as a multiplication (exact for idx * pv < 2^32): the tile loop has no integer division
    const unsigned pv_magic = (unsigned)((0x100000000ull + (unsigned)pv - 1) / (unsigned)pv);
    for (int c = 0; c < nchunks; ++c) {
        const int base = lo_t + c * 64, cnt = pl - base + 1 < 64 ? pl - base + 1 : 64;
        __syncthreads();
        if (tid < 64 && tid < cnt) {
            const int tk = base + tid;
            tokoff[tid] = ((long)pt[tk / ps] * ps + tk % ps) * (long)D;
        }
        __syncthreads();
        // the tile as the cache holds it: consecutive lanes take consecutive 16-byte pieces of a key's row (whole cache lines per request)
        constexpr int U = 9;      // requests in flight per thread: a tile of 64 keys x 576 dims is two such rounds
        for (int i0 = tid; i0 < nv; i0 += 256 * U) {
            uint4 u[U];
#pragma unroll
            for (int k = 0; k < U; ++k) {
                const int idx = i0 + 256 * k, jj = (int)__umulhi((unsigned)idx, pv_magic), v = idx - jj * pv;
                u[k] = make_uint4(0, 0, 0, 0);
                if (idx < nv && jj < cnt && v < per) u[k] = *(const uint4*)(cache + tokoff[jj] + v * 8);
            }
#pragma unroll
            for (int k = 0; k < U; ++k) {
                const int idx = i0 + 256 * k, jj = (int)__umulhi((unsigned)idx, pv_magic), v = idx - jj * pv;
                if (idx < nv) *(uint4*)(Kt + jj * DPK + v * 8) = u[k];
            }
        }
        __syncthreads();
        // the value part transposed, from LDS to LDS: lane = key, so the four 2-byte stores of a wave each fall into one row of Vt
        // (stores of consecutive columns of one key would all hit two banks)
        {
            const int jj = tid & 63;
            for (int c4 = (tid >> 6) * 4; c4 < R; c4 += 16) {
                const uint2 w = *(const uint2*)(Kt + (size_t)jj * DPK + c4);
                bf16_t* dst = Vt + (size_t)c4 * HB_LM_VLD + jj;
                dst[0] = (bf16_t)(w.x & 0xffffu);
                if (c4 + 1 < R) dst[HB_LM_VLD] = (bf16_t)(w.x >> 16);
                if (c4 + 2 < R) dst[2 * HB_LM_VLD] = (bf16_t)(w.y & 0xffffu);
                if (c4 + 3 < R) dst[3 * HB_LM_VLD] = (bf16_t)(w.y >> 16);
            }
        }
        __syncthreads();
        if (!active) continue;
        hb_f32x4 st[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) st[kt] = hb_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks < ks_n) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt) {
                    const uint4 a = *(const uint4*)(Kt + (size_t)(kt * 16 + col) * DPK + ks * 32 + g * 8);
                    st[kt] = hb_mfma_bf16(a, qh[ks], st[kt]);
                    st[kt] = hb_mfma_bf16(a, ql[ks], st[kt]);
                }
            }
        }
        // lane (col, g) holds the scores of head `col` against keys base + kt*16 + g*4 + i
        float sc[4][4], mx = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = base + kt * 16 + g * 4 + i;
                sc[kt][i] = (key >= lo_r && key <= p) ? st[kt][i] * scale : -INFINITY;
                mx = fmaxf(mx, sc[kt][i]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(m, mx);
        const float alpha = mn == -INFINITY ? 1.0f : expf(m - mn);
        float sum = 0.f, pr[4][4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pr[kt][i] = sc[kt][i] == -INFINITY ? 0.f : expf(sc[kt][i] - mn);
                sum += pr[kt][i];
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        l = l * alpha + sum;
        m = mn;
        uint4 ph[2], plo[2];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const float v[8] = {pr[2 * kk][0], pr[2 * kk][1], pr[2 * kk][2], pr[2 * kk][3], pr[2 * kk + 1][0], pr[2 * kk + 1][1], pr[2 * kk + 1][2],
                                pr[2 * kk + 1][3]};
            hb_split_bf16x8(v, ph[kk], plo[kk]);
        }
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (ct < ct_n) {
                hb_f32x4 o = oacc[ct];
                o[0] *= alpha; o[1] *= alpha; o[2] *= alpha; o[3] *= alpha;
#pragma unroll
                for (int kk = 0; kk < 2; ++kk) {
                    const bf16_t* vr = Vt + (size_t)(ct * 16 + col) * HB_LM_VLD + kk * 32 + g * 4;
                    const uint2 a0 = *(const uint2*)vr, a1 = *(const uint2*)(vr + 16);
                    const uint4 a = make_uint4(a0.x, a0.y, a1.x, a1.y);
                    o = hb_mfma_bf16(a, ph[kk], o);
                    o = hb_mfma_bf16(a, plo[kk], o);
                }
                oacc[ct] = o;
            }
        }
    }
    if (!active || col >= hg) return;
    const int hq = h0 + col;
    const float gmul = (gate ? hb_sigmoid(gate[(size_t)row * ldg + hq]) : 1.0f) * out_scale;
    float* dst = out + (size_t)row * ldo + (size_t)hq * R;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
        if (ct < ct_n)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int cc = ct * 16 + g * 4 + i;
                if (cc < R) dst[cc] = oacc[ct][i] / l * gmul;
            }
}

// ---- routed feed-forward --------------------------------------------------------------------------------------------------
// One block per row: router logits z_j = router[j] . h in fp32 (lane-strided sums over four waves and a butterfly: an order fixed by
// the width, the same for every step shape), then one wave: s = softmax(z) over all nE router outputs, choice = s + correction, the `top` largest choices (first
// index wins a tie) in descending order; weights = their s / (sum + 1e-20).  sel[row*top + k] = router output index, wgt likewise.
// sigmoid != 0: s_j = sigmoid(z_j) instead of the softmax; renorm == 0: the weights are the chosen s as they are.
// bias != NULL: added to the logits before the scores are formed.
__global__ __launch_bounds__(256) void k_hb_moe_router(const float* h, long ldh, const float* router, const float* corr, int W, int nE, int top,
                                                       int* sel, float* wgt, int sigmoid, int renorm, const float* bias) {
    extern __shared__ float sm[];
    float* sc = sm;                    // [nE] logits, then scores
    float* ch = sm + nE;               // [nE] choice values
    int* pick = (int*)(sm + 2 * nE);   // [top]
    float* part = sm + 2 * nE + top;   // [4][nE] the waves' partial logits
    const int row = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const float* x = h + (size_t)row * ldh;
    const bool vec = (W % 4 == 0) && (ldh % 4 == 0) && ((((size_t)h) & 15) == 0) && ((((size_t)router) & 15) == 0);
    // wave w sums the k-chunks w, w + 4, ... (64 lanes x 4 values, or 64 values); a logit = the four waves' sums added in wave order
    for (int j0 = 0; j0 < nE; j0 += 8) {
        float acc[8];
        const float* r[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) { acc[j] = 0.f; r[j] = router + (size_t)(j0 + j < nE ? j0 + j : nE - 1) * W; }
        if (vec) {
            for (int k = (wv * 64 + lane) * 4; k < W; k += 1024) {
                const float4 xv = *(const float4*)(x + k);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float4 rv = *(const float4*)(r[j] + k);
                    acc[j] = fmaf(rv.x, xv.x, acc[j]); acc[j] = fmaf(rv.y, xv.y, acc[j]);
                    acc[j] = fmaf(rv.z, xv.z, acc[j]); acc[j] = fmaf(rv.w, xv.w, acc[j]);
                }
            }
        } else {
            for (int k = wv * 64 + lane; k < W; k += 256) {
                const float xv = x[k];
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] = fmaf(r[j][k], xv, acc[j]);
            }
        }
        // eight sums over the wave with 10 exchanges instead of 48: each of the first three exchanges halves the values a lane
        // carries (lanes with the partner bit clear keep the lower half and receive the partner's), three more finish the one left;
        // the lane whose low three bits are clear ends up with the sum of value (bit 5, bit 4, bit 3 of its number)
        {
            const bool hi5 = lane & 32, hi4 = lane & 16, hi3 = lane & 8;
            float b4[4], b2[2];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float mine = hi5 ? acc[i + 4] : acc[i], give = hi5 ? acc[i] : acc[i + 4];
                b4[i] = mine + __shfl_xor(give, 32, 64);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const float mine = hi4 ? b4[i + 2] : b4[i], give = hi4 ? b4[i] : b4[i + 2];
                b2[i] = mine + __shfl_xor(give, 16, 64);
            }
            const float mine = hi3 ? b2[1] : b2[0], give = hi3 ? b2[0] : b2[1];
            float v = mine + __shfl_xor(give, 8, 64);
            v += __shfl_xor(v, 4, 64);
            v += __shfl_xor(v, 2, 64);
            v += __shfl_xor(v, 1, 64);
            const int j = (hi5 ? 4 : 0) + (hi4 ? 2 : 0) + (hi3 ? 1 : 0);
            if ((lane & 7) == 0 && j0 + j < nE) part[wv * nE + j0 + j] = v;
        }
    }
    __syncthreads();
    if (wv != 0) return;
    for (int i = lane; i < nE; i += 64) sc[i] = (((part[i] + part[nE + i]) + part[2 * nE + i]) + part[3 * nE + i]) + (bias ? bias[i] : 0.f);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    if (sigmoid) {
        for (int i = lane; i < nE; i += 64) {
            const float v = hb_sigmoid(sc[i]);
            sc[i] = v;
            ch[i] = v + (corr ? corr[i] : 0.f);
        }
    } else {
        float mx = -INFINITY;
        for (int i = lane; i < nE; i += 64) mx = fmaxf(mx, sc[i]);
        mx = hb_wave_max(mx);
        float sum = 0.f;
        for (int i = lane; i < nE; i += 64) {
            const float e = expf(sc[i] - mx);
            sc[i] = e;
            sum += e;
        }
        sum = hb_wave_sum(sum);
        for (int i = lane; i < nE; i += 64) {
            const float v = sc[i] / sum;
            sc[i] = v;
            ch[i] = v + (corr ? corr[i] : 0.f);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    // one wave from here on: every lane follows the same picks; lane 0 retires a pick in LDS before the next search reads it
    float wsum = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int i = lane; i < nE; i += 64) {
            const float v = ch[i];
            if (v > best || (v == best && i < at)) { best = v; at = i; }
        }
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) {
            const float ov = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(at, o, 64);
            if (ov > best || (ov == best && oi < at)) { best = ov; at = oi; }
        }
        if (at == 0x7fffffff) at = 0;
        const float sv = sc[at];
        wsum += sv;
        if (lane == (k & 63)) { pick[k] = at; }
        __builtin_amdgcn_wave_barrier();
        if (lane == 0) ch[at] = -INFINITY;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_wave_barrier();
    }
    const float den = wsum + 1e-20f;
    for (int k = lane; k < top; k += 64) {
        sel[(size_t)row * top + k] = pick[k];
        wgt[(size_t)row * top + k] = renorm ? sc[pick[k]] / den : sc[pick[k]];
    }
}
// Block e lists the entries (row*top + k) routed to expert e, ascending: list[e*cap + 0 .. count[e]).
__global__ __launch_bounds__(256) void k_hb_moe_group(const int* sel, int n_entries, int cap, int* list, int* count) {
    __shared__ int wsum[4];
    __shared__ int base;
    const int e = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    if (threadIdx.x == 0) base = 0;
    __syncthreads();
    for (int i0 = 0; i0 < n_entries; i0 += 256) {
        const int i = i0 + threadIdx.x;
        const bool hit = i < n_entries && sel[i] == e;
        const unsigned long long bal = __ballot(hit);
        const int before = __popcll(bal & ((1ull << lane) - 1ull));
        if (lane == 0) wsum[wv] = __popcll(bal);
        __syncthreads();
        int off = base;
        for (int w = 0; w < wv; ++w) off += wsum[w];
        if (hit) list[(size_t)e * cap + off + before] = i;
        __syncthreads();
        if (threadIdx.x == 0) base += wsum[0] + wsum[1] + wsum[2] + wsum[3];
        __syncthreads();
    }
    if (threadIdx.x == 0) count[e] = base;
}
// y = act(g) * (u + up_offset), g = min(gate, limit), u = clamp(up, -limit, limit); act(g) = g * sigmoid(alpha g), or the tanh form
// of gelu (gelu != 0); gu row = [gate (ff) | up (ff)].
// sel != NULL: rows are routed entries, those of identity outputs (sel >= experts) are skipped.
__device__ __forceinline__ float hb_glu(float g0, float u0, float limit, float alpha, float up_offset, int gelu) {
    const float g = fminf(g0, limit), u = fminf(fmaxf(u0, -limit), limit);
    return (gelu ? hb_gelu_tanh(g) : g * hb_sigmoid(alpha * g)) * (u + up_offset);
}
// the activation of an up / down unit: the square of relu, or g * sigmoid(alpha g)
__device__ __forceinline__ float hb_unit_act(float g, int relu2, float alpha) {
    if (relu2) { const float r = fmaxf(g, 0.f); return r * r; }
    return g * hb_sigmoid(alpha * g);
}
// up_down != 0: gu row = [up (ff)] and y = act(up) (relu2 != 0: the square of relu, else g * sigmoid(alpha g)), nothing clamped.
__global__ __launch_bounds__(256) void k_hb_glu_clamp(const float* gu, float* y, int ff, float limit, float alpha, const int* sel, int experts,
                                                      float up_offset, int gelu, int up_down, int relu2) {
    const int row = blockIdx.x;
    if (sel && sel[row] >= experts) return;
    if (up_down) {
        for (int j = blockIdx.y * 256 + threadIdx.x; j < ff; j += gridDim.y * 256) y[(size_t)row * ff + j] = hb_unit_act(gu[(size_t)row * ff + j], relu2, alpha);
        return;
    }
    for (int j = blockIdx.y * 256 + threadIdx.x; j < ff; j += gridDim.y * 256)
        y[(size_t)row * ff + j] = hb_glu(gu[(size_t)row * 2 * ff + j], gu[(size_t)row * 2 * ff + ff + j], limit, alpha, up_offset, gelu);
}
// Few-row steps.  Entries per row: its `top` routed choices, then (shared_ff > 0) the shared expert.
struct hb_moe_small {
    const int* sel;
    const float* wgt;
    int top, experts, ff, shared_ff, ld_act;
    float limit, shared_limit, alpha, up_offset;
    int scale_input;        // the routing weight multiplies the expert's input instead of its output
    const float* shared_bias;   // [2 * shared_ff] gate, then up biases of the shared unit, or NULL
    int shared_gelu;            // the shared unit's activation is the tanh form of gelu
    int up_down, relu2;         // units are down(act(up h)): the matrices hold up rows only; act = the square of relu (else swish)
    const float* out_scale;     // [W] layer scale of what joins the residual sum, or NULL
};
// gate / up products + activation of every entry: block (column tile, entry); a wave takes gate row n and up row ff + n of the
// entry's expert and stores g * sigmoid(alpha g) * (u + 1) with the clamps of that expert.  act row of an entry: ld_act floats.
template <typename T>
__global__ __launch_bounds__(256) void k_hb_moe_gate_up(const float* h, long ldh, const T* w_gate_up, const T* shared_gate_up, float* act, int W,
                                                        hb_moe_small q) {
    const int per = q.top + (q.shared_ff > 0 ? 1 : 0);
    const int entry = blockIdx.y, row = entry / per, slot = entry - row * per, lane = threadIdx.x & 63, n = blockIdx.x * 4 + (threadIdx.x >> 6);
    const T* wg;
    int N;
    float limit, xs = 1.0f;
    const float* gb = nullptr;
    int gelu = 0;
    if (slot < q.top) {
        const int e = q.sel[(size_t)row * q.top + slot];
        if (e >= q.experts) return;
        wg = w_gate_up + (size_t)e * (q.up_down ? 1 : 2) * q.ff * W;
        N = q.ff;
        limit = q.limit;
        if (q.scale_input) xs = q.wgt[(size_t)row * q.top + slot];
    } else {
        wg = shared_gate_up;
        N = q.shared_ff;
        limit = q.shared_limit;
        gb = q.shared_bias;
        gelu = q.shared_gelu;
    }
    if (n >= N) return;
    constexpr int CH = sizeof(T) == 2 ? 8 : 4;
    const float* x = h + (size_t)row * ldh;
    const bool vec = (W % CH == 0) && ((((size_t)wg) & 15) == 0) && (ldh % 4 == 0) && ((((size_t)h) & 15) == 0);
    if (q.up_down) {
        const float u1 = hb_dot_wave<T>(wg + (size_t)n * W, x, W, vec, lane, xs);
        if (lane == 0) act[(size_t)entry * q.ld_act + n] = hb_unit_act(u1, q.relu2, q.alpha);
        return;
    }
    const float g0 = hb_dot_wave<T>(wg + (size_t)n * W, x, W, vec, lane, xs), u0 = hb_dot_wave<T>(wg + (size_t)(N + n) * W, x, W, vec, lane, xs);
    if (lane == 0) act[(size_t)entry * q.ld_act + n] = hb_glu(g0 + (gb ? gb[n] : 0.f), u0 + (gb ? gb[N + n] : 0.f), limit, q.alpha, q.up_offset, gelu);
}
// down products of a row's entries, weighted and added to the residual stream: a wave per (row, output column):
// x[row][c] += sum_k wgt_k * (identity ? h[row][c] : down_{e_k}[c] . act_k)  +  shared_down[c] . act_shared, k ascending.
template <typename T>
__global__ __launch_bounds__(256) void k_hb_moe_down_combine(const float* h, long ldh, const T* w_down, const T* shared_down, const float* act,
                                                             float* x, long ldx, int W, hb_moe_small q) {
    const int per = q.top + (q.shared_ff > 0 ? 1 : 0);
    const int row = blockIdx.y, lane = threadIdx.x & 63, c = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (c >= W) return;
    constexpr int CH = sizeof(T) == 2 ? 8 : 4;
    const bool avec = (q.ld_act % 4 == 0) && ((((size_t)act) & 15) == 0);
    float acc = 0.f;
    for (int k = 0; k < q.top; ++k) {
        const int e = q.sel[(size_t)row * q.top + k];
        const float wk0 = q.wgt[(size_t)row * q.top + k];
        if (e >= q.experts) { acc = fmaf(wk0, h[(size_t)row * ldh + c], acc); continue; }
        const float wk = q.scale_input ? 1.0f : wk0;
        const T* wd = w_down + ((size_t)e * W + c) * q.ff;
        const bool vec = avec && (q.ff % CH == 0) && ((((size_t)w_down) & 15) == 0);
        acc = fmaf(wk, hb_dot_wave<T>(wd, act + (size_t)(row * per + k) * q.ld_act, q.ff, vec, lane), acc);
    }
    if (q.shared_ff > 0) {
        const bool vec = avec && (q.shared_ff % CH == 0) && ((((size_t)shared_down) & 15) == 0);
        acc += hb_dot_wave<T>(shared_down + (size_t)c * q.shared_ff, act + (size_t)(row * per + q.top) * q.ld_act, q.shared_ff, vec, lane);
    }
    if (lane == 0) x[(size_t)row * ldx + c] += q.out_scale ? acc * q.out_scale[c] : acc;
}
// x[row] += sum_k wgt[row*top + k] * (identity output ? h[row] : expert_out[row*top + k]), k ascending
// (scale_input: an expert's output enters with weight 1, its input was scaled instead)
__global__ __launch_bounds__(256) void k_hb_moe_combine(float* x, long ldx, const float* h, long ldh, const float* eo, const int* sel,
                                                        const float* wgt, int top, int experts, int W, int scale_input, const float* out_scale) {
    const int row = blockIdx.x;
    for (int i = threadIdx.x; i < W; i += 256) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const size_t en = (size_t)row * top + k;
            const bool ident = sel[en] >= experts;
            acc = fmaf(scale_input && !ident ? 1.0f : wgt[en], ident ? h[(size_t)row * ldh + i] : eo[en * W + i], acc);
        }
        x[(size_t)row * ldx + i] += out_scale ? acc * out_scale[i] : acc;
    }
}

__global__ void k_hb_copy_rows(const float* src, long lds_, float* dst, long ldd, int W) {
    const int row = blockIdx.x;
    for (int i = threadIdx.x; i < W; i += blockDim.x) dst[(size_t)row * ldd + i] = src[(size_t)row * lds_ + i];
}
__global__ void k_hb_logits_bf16(const float* src, bf16_t* dst, long n) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = f2bf(src[i]);
}
// greedy pick on the fp32 logits: first maximum of each row
__global__ __launch_bounds__(1024) void k_hb_argmax(const float* logits, int V, int* out_ids) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    const int row = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const float* p = logits + (size_t)row * V;
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += 1024) {
        const float v = p[i];
        if (v > best || (v == best && i < at)) { best = v; at = i; }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(at, o, 64);
        if (ov > best || (ov == best && oi < at)) { best = ov; at = oi; }
    }
    if (lane == 0) { bv[wv] = best; bi[wv] = at; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w)
            if (bv[w] > best || (bv[w] == best && bi[w] < at)) { best = bv[w]; at = bi[w]; }
        out_ids[row] = at == 0x7fffffff ? 0 : at;
    }
}
__global__ void k_hb_feedback(const int* out_ids, int* input_ids, uint64_t* rng, int B, int feedback) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (feedback && b < B) input_ids[b] = out_ids[b];
    if (b == 0 && rng) *rng += 1;
}

}  // namespace

#define HB_LAT_MAX_SEG 64     // blocks that share the keys of one row in the few-row latent attention
#define HB_MOE_GEMV_ROWS 8    // steps of at most this many rows run the routed feed-forward entry by entry
#define HB_SCAN_CHUNK 64       // rows per chunk of the chunked matrix-state scan; steps of more rows take that form
#define HB_LRU_SEQ_ROWS 64    // steps of at most this many rows run the gated linear recurrent unit token by token
#define HB_DELTA_CHUNK 128     // rows per chunk of the chunked delta-rule scan (every chunk costs a dim x dim x vdim product in the carry)
#define HB_DELTA_CHUNK_DIM 128 // key dims up to which the delta rule's long portions run in chunks (the carry kernel gives every key row a thread)

struct vox_hybrid {
    vox_ctx* ctx;
    vox_hybrid_config cfg;
    std::vector<vox_hybrid_layer> layers;
    std::vector<vox_hybrid_moe> moes;      // copies of the layers' routed feed-forwards (layers[i].moe points into this)
    std::vector<vox_hybrid_run> runs;
    vox_hybrid_weights w;
    float *xa = nullptr, *xb = nullptr, *h = nullptr, *h2 = nullptr, *proj = nullptr, *mix = nullptr, *ff = nullptr, *hout = nullptr;
    float *ff_act = nullptr;                // [max_rows][max gated dense width]: activation output of the gated dense feed-forward
    int max_gated = 0;
    float *shift = nullptr;                 // [5][max_rows][width]: token-shift mixes
    float *scan_ws = nullptr;               // chunk states and decay products of the chunked matrix-state scan
    size_t scan_ws_floats = 0;
    float *moe_wgt = nullptr, *moe_act = nullptr, *moe_out = nullptr;
    int *moe_sel = nullptr, *moe_list = nullptr, *moe_count = nullptr;
    bf16_t* logits16 = nullptr;
    float* attn_ws = nullptr;
    size_t attn_ws_bytes = 0;
    int max_in = 0, max_mix = 0, max_ff = 0;
    int max_ne = 0, max_top = 0, max_eff = 0, max_experts = 0;
    bool any_shift = false;
    bool attn_big_lds = false;              // the attention kernel was given the right to more than 64 KB of LDS
    bool lat_big_lds = false;               // the same for the few-row latent attention
};

static bool hb_is_attn(int kind) { return kind == VOX_MIXER_POOLED_WINDOW_ATTN || kind == VOX_MIXER_CAUSAL_ATTN || kind == VOX_MIXER_LATENT_ATTN; }
static inline int hb_up4(int v) { return (v + 3) & ~3; }
// Where a latent-attention row keeps what it derives from the fused projection [query latent | kv latent | rotated key | gate]:
// q = per head [plain | rotated] at off_q, the query against the cached rows (per head [R | r]) at off_qa, the weighted sum of cached
// latents per head at off_o.  Every part starts on a 16-byte boundary.
struct hb_latent_layout {
    int n_in, off_q, off_qa, off_o, n_proj;
};
static hb_latent_layout hb_latent(const vox_hybrid_layer& L) {
    hb_latent_layout y;
    y.n_in = L.q_rank + L.kv_rank + L.rot_dim + L.heads;
    y.off_q = hb_up4(y.n_in);
    y.off_qa = y.off_q + hb_up4(L.heads * (L.dim + L.rot_dim));
    y.off_o = y.off_qa + hb_up4(L.heads * (L.kv_rank + L.rot_dim));
    y.n_proj = y.off_o + hb_up4(L.heads * L.kv_rank);
    return y;
}
// query heads per block of the latent attention: all heads read the one cached row; at most 16 share a block
static int hb_latent_groups(int H) {
    for (int g = 1; g <= H; ++g)
        if (H % g == 0 && H / g <= 16) return g;
    return H;
}
// Columns of a delta-rule row: the fused projection, then (each part on a 16-byte boundary) the pre-activations of the bottleneck
// forms, the convolved q | k | v, the decays and q . k per key head.
static hb_delta_layout hb_delta(const vox_hybrid_layer& L) {
    hb_delta_layout y;
    const int nv = L.heads * L.vdim;
    y.nq = L.kv_heads * L.dim;
    y.nqkv = 2 * y.nq + nv;
    y.off_b = y.nqkv;
    y.off_din = y.off_b + L.heads;
    y.ndec = L.decay_channels ? L.heads * L.dim : L.heads;
    y.off_gin = y.off_din + (L.lora > 0 ? L.lora : y.ndec);
    y.n_in = y.off_gin + (L.gate_rank > 0 ? L.gate_rank : nv);
    int next = hb_up4(y.n_in);
    y.off_dec = y.off_din;
    if (L.lora > 0) { y.off_dec = next; next += hb_up4(y.ndec); }
    y.off_gate = y.off_gin;
    if (L.gate_rank > 0) { y.off_gate = next; next += hb_up4(nv); }
    y.off_c = next; next += hb_up4(y.nqkv);
    y.off_g = next; next += hb_up4(y.ndec);
    y.off_kq = next; next += hb_up4(L.kv_heads);
    y.n_proj = next;
    return y;
}
// a causal attention layer whose q | k | v pass a convolution first
static bool hb_conv_attn(const vox_hybrid_layer& L) { return L.kind == VOX_MIXER_CAUSAL_ATTN && L.conv_taps > 0; }
// Columns of such a layer's row behind the fused projection [q | k | v] (C values): the convolved q | k | v, the processed query, and
// per block of 256 channels the sums of squares over its q and its k channels.
struct hb_conv_attn_layout {
    int off_y, off_qc, off_ss, n_proj;
};
static hb_conv_attn_layout hb_conv_attn_cols(const vox_hybrid_layer& L) {
    const int C = L.heads * L.dim + L.kv_heads * (L.dim + L.vdim);
    hb_conv_attn_layout y;
    y.off_y = hb_up4(C);
    y.off_qc = y.off_y + hb_up4(C);
    y.off_ss = y.off_qc + hb_up4(L.heads * L.dim);
    y.n_proj = y.off_ss + hb_up4(2 * ((C + 255) / 256));
    return y;
}
// rows of the fused input projection
static int hb_layer_in(const vox_hybrid_layer& L) {
    switch (L.kind) {
        case VOX_MIXER_HGRN2: return 2 * L.heads * L.dim + L.heads * L.vdim;
        case VOX_MIXER_POOLED_WINDOW_ATTN: return L.heads * L.dim + L.kv_heads * (L.dim + L.vdim) + L.heads;
        case VOX_MIXER_MLSTM: return 2 * L.heads * L.dim + 2 * L.heads * L.vdim + 2 * L.heads;
        case VOX_MIXER_RGLRU: return 2 * L.heads * L.dim;
        case VOX_MIXER_CAUSAL_ATTN: return L.heads * L.dim + L.kv_heads * (L.dim + L.vdim);
        case VOX_MIXER_SHIFT_DECAY: return 4 * L.heads * L.dim + L.lora;
        case VOX_MIXER_LATENT_ATTN: return L.q_rank + L.kv_rank + L.rot_dim + L.heads;
        case VOX_MIXER_RETENTION: return 2 * L.heads * L.dim + 2 * L.heads * L.vdim;
        case VOX_MIXER_DELTA: return L.kv_heads > 0 ? hb_delta(L).n_in : -1;
    }
    return -1;
}
// floats per row of the projection buffer: the projection's outputs and what the mixer derives from them
static int hb_layer_proj(const vox_hybrid_layer& L) {
    if (L.kind == VOX_MIXER_RGLRU) return 5 * L.heads * L.dim;                           // + conv output, 2 gates
    if (L.kind == VOX_MIXER_SHIFT_DECAY) return 5 * L.heads * L.dim + L.lora;            // + decay pre-activation
    if (L.kind == VOX_MIXER_LATENT_ATTN) return hb_latent(L).n_proj;
    if (L.kind == VOX_MIXER_DELTA) return hb_delta(L).n_proj;
    if (hb_conv_attn(L)) return hb_conv_attn_cols(L).n_proj;
    return hb_layer_in(L);
}

static void hb_norm(const vox_hybrid* m, hipStream_t st, int n, const float* x, long ldx, const int* rows, const float* w1, float* y1,
                    const float* w2, float* y2, long ldy) {
    const vox_hybrid_config& c = m->cfg;
    if (c.norm_kind == VOX_NORM_RMS_GROUPS && c.norm_groups == 1) {
        hipLaunchKernelGGL(k_hb_rms_row, dim3(n), dim3(256), 0, st, x, ldx, rows, w1, y1, w2, y2, ldy, c.width, c.eps);
    } else if (c.norm_kind == VOX_NORM_RMS_GROUPS) {
        hipLaunchKernelGGL(k_hb_rms_groups, dim3(n, (c.norm_groups + 3) / 4 < 8 ? (c.norm_groups + 3) / 4 : 8), dim3(256), 0, st, x, ldx, rows, w1, y1,
                           w2, y2, ldy, c.width, c.norm_groups, c.eps);
    } else {
        hb_layernorm(st, n, x, ldx, rows, w1, y1, ldy, c.width, c.eps);
        if (w2) hb_layernorm(st, n, x, ldx, rows, w2, y2, ldy, c.width, c.eps);
    }
}
// the fused one-row norm + GEMV exists for the layer norm and for the RMS norm over one slice
template <typename T>
static bool hb_try_norm_gemv(const vox_hybrid* m, hipStream_t st, int epi, const float* X, long ldx, const int* rows, const float* nw, const T* W,
                             const float* bias, float* C, int N, int K, float epi_arg = 0.f) {
    const bool rms = m->cfg.norm_kind == VOX_NORM_RMS_GROUPS && m->cfg.norm_groups == 1;
    return (m->cfg.norm_kind == VOX_NORM_LAYER || rms) && hb_try_ln_gemv<T>(st, epi, X, ldx, rows, nw, m->cfg.eps, W, bias, C, N, K, rms ? 1 : 0, epi_arg);
}

// The matrix-core latent attention for steps of many rows over a bf16 cache.  false: the shapes do not fit it (rows of the cache that are
// no multiple of 16 bytes, a latent beyond 512 values or keys beyond 576) and the caller takes the general kernel.
static bool hb_try_latent_mfma(vox_hybrid* m, hipStream_t st, const vox_hybrid_io* io, const vox_hybrid_layer& L, const bf16_t* cache, const float* qa,
                               float* o, long ldp, const float* gate, int n, int n_req, int window, int ps) {
    const int R = L.kv_rank, r = L.rot_dim, D = R + r;
    if ((D & 7) || R > 512 || D > 576 || (ldp & 3)) return false;
    const int ks_n = (D + 31) / 32, ct_n = (R + 15) / 16;
    const size_t lds = 512 + (size_t)64 * (ks_n * 32 + 8) * 2 + (size_t)ct_n * 16 * HB_LM_VLD * 2;
    const dim3 grid((n + 3) / 4 + n_req, (L.heads + 15) / 16), block(256);
#define HB_LM(KS_, CT_) \
    do { \
        if (lds > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k_hb_latent_attn_mfma<KS_, CT_>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
        hipLaunchKernelGGL((k_hb_latent_attn_mfma<KS_, CT_>), grid, block, lds, st, qa, ldp, cache, o, ldp, io->pos, io->req_rows, n_req, io->page_table, \
                           io->pt_stride, L.heads, R, r, window, ps, L.scale, gate, ldp, L.out_scale, ks_n, ct_n); \
    } while (0)
    if (ks_n <= 10 && ct_n <= 16) HB_LM(10, 16);
    else if (ct_n <= 16) HB_LM(18, 16);
    else HB_LM(18, 32);
#undef HB_LM
    (void)m;
    return true;
}
static bool hb_try_latent_mfma(vox_hybrid*, hipStream_t, const vox_hybrid_io*, const vox_hybrid_layer&, const float*, const float*, float*, long,
                               const float*, int, int, int, int) { return false; }

// cur += (A . W^T + bias) [* scale column by column]
template <typename T>
static int hb_gemm_resid(hipStream_t st, const float* A, long lda, const T* W, const float* bias, float* cur, long ldx, int n, int N, int K,
                         const float* scale) {
    hb_rowmap rm = hb_plain();
    rm.col_scale = scale;
    return hb_gemm<T>(st, scale ? HB_EPI_RESID_SCALED : HB_EPI_RESID, A, lda, W, bias, cur, ldx, n, N, K, rm);
}
// One mixer: reads the normed rows (hn != NULL) or norms `cur` itself with L.norm1, adds out_scale * mixer(.) [* ls1] to cur.
template <typename T>
static int hb_mixer(vox_hybrid* m, hipStream_t st, const vox_hybrid_io* io, const vox_hybrid_layer& L, void* cache, float* pool, float* state,
                    const float* hn, float* cur, long ldx, int n, int n_req, int max_kvlen) {
    const vox_hybrid_config& c = m->cfg;
    const int W = c.width, ps = c.page_size;
    const int n_in = hb_layer_in(L), n_proj = hb_layer_proj(L), n_mix = L.heads * L.vdim;
    if (L.kind == VOX_MIXER_SHIFT_DECAY) {
        // five token-shift mixes of the normed input, each with its own projection
        if (!hn) { hb_norm(m, st, n, cur, ldx, nullptr, L.norm1, m->h, nullptr, nullptr, (long)W); hn = m->h; }
        const int HD = L.heads * L.dim;
        const long per_slot = (long)HD * L.dim + W, rows_stride = (long)c.max_rows * W;
        const T* wi = (const T*)L.w_in;
        if (n == 1) {
            // one row: mixes and the five projections in one launch
            const dim3 g((4 * HD + L.lora + 3) / 4), b(256);
#define HB_SHIFT(MR_) \
    hipLaunchKernelGGL((k_hb_shift_gemv<T, MR_>), g, b, 0, st, hn, (long)W, L.shift_mu, wi, L.b_in, m->proj, (long)n_proj, state, per_slot, \
                       (long)HD * L.dim, io->pos, io->row_req, io->req_rows, io->req_state, n, 4 * HD + L.lora, HD, W)
            if (n == 1) HB_SHIFT(1);
            else if (n == 2) HB_SHIFT(2);
            else if (n <= 4) HB_SHIFT(4);
            else HB_SHIFT(8);
#undef HB_SHIFT
        } else {
            hipLaunchKernelGGL(k_hb_shift_mix, dim3(n, n <= 64 ? (W + 255) / 256 : 1), dim3(256), 0, st, hn, (long)W, L.shift_mu, m->shift, rows_stride,
                               state, per_slot, (long)HD * L.dim, io->pos, io->row_req, io->req_rows, io->req_state, W);
            // r, k, v, g: four products of one shape, each on its own mix, in one launch
            VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, m->shift, W, wi, L.b_in, m->proj, n_proj, n, HD, W,
                               hb_rowmap{nullptr, nullptr, 0, 1, (long)HD * W, rows_stride, (long)HD, (long)HD}, 4));
            VOX_TRY(hb_gemm<T>(st, HB_EPI_TANH, m->shift + 4 * rows_stride, W, wi + (size_t)4 * HD * W, nullptr, m->proj + 4 * HD, n_proj, n, L.lora, W));
        }
        VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, m->proj + 4 * HD, n_proj, (const T*)L.w_decay2, L.decay0, m->proj + 4 * HD + L.lora, n_proj, n, HD, L.lora));
        const int dpw = L.dim <= 16 * HB_SCAN_MAX_WAVES ? 16 : (L.dim <= 32 * HB_SCAN_MAX_WAVES ? 32 : 64);
        const int nwv = (L.dim + dpw - 1) / dpw, dpad = nwv * dpw;
        const int tt = 4096 / dpad >= 16 ? 16 : (4096 / dpad >= 1 ? 4096 / dpad : 1);
        auto kern = dpw == 16 ? k_hb_shift_decay_scan<16> : (dpw == 32 ? k_hb_shift_decay_scan<32> : k_hb_shift_decay_scan<64>);
        const size_t lds = (size_t)(3 * tt * dpad + tt * 64 + 2 * nwv * 64) * 4;
        // few-row steps with heads of at most 64 dims (one block holds a head): the scan also applies the head norm, the gate and the
        // scale (per token that is a reduction inside the sequential loop, which long portions leave to a launch of its own)
        const bool fused_norm = L.dim <= 64 && n <= HB_MOE_GEMV_ROWS;
        const int vt = (L.dim + 63) / 64;
        if (n > HB_SCAN_CHUNK && m->scan_ws) {
            // steps of many rows: every request's rows in chunks of HB_SCAN_CHUNK side by side — each chunk reduced from a zero state,
            // the carries pushed through in order, each chunk replayed from its carry (rounding aside the token-by-token form)
            const int nch = (n + HB_SCAN_CHUNK - 1) / HB_SCAN_CHUNK;
            hipLaunchKernelGGL(kern, dim3(n_req, L.heads, vt * nch), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, L.bonus,
                               state, per_slot, hn, (long)W, W, io->req_rows, io->req_state, io->pos, L.heads, L.dim, L.lora, tt,
                               (const float*)nullptr, c.eps, L.out_scale, (int)HB_SCAN_REDUCE, HB_SCAN_CHUNK, m->scan_ws);
            hipLaunchKernelGGL(k_hb_shift_decay_carry, dim3(n_req, L.heads, (L.dim * L.dim + 255) / 256 < 64 ? (L.dim * L.dim + 255) / 256 : 64), dim3(256), 0, st, m->scan_ws, state, per_slot, hn, (long)W, W,
                               io->req_rows, io->req_state, io->pos, L.heads, L.dim, HB_SCAN_CHUNK);
            hipLaunchKernelGGL(kern, dim3(n_req, L.heads, vt * nch), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, L.bonus,
                               state, per_slot, hn, (long)W, W, io->req_rows, io->req_state, io->pos, L.heads, L.dim, L.lora, tt,
                               (const float*)nullptr, c.eps, L.out_scale, (int)HB_SCAN_REPLAY, HB_SCAN_CHUNK, m->scan_ws);
        } else {
            hipLaunchKernelGGL(kern, dim3(n_req, L.heads, vt), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, L.bonus,
                               state, per_slot, hn, (long)W, W, io->req_rows, io->req_state, io->pos, L.heads, L.dim, L.lora, tt,
                               fused_norm ? L.head_norm : (const float*)nullptr, c.eps, L.out_scale, (int)HB_SCAN_WHOLE, 0, (float*)nullptr);
        }
        if (!fused_norm)
            hipLaunchKernelGGL(k_hb_head_norm, dim3(n, L.heads), dim3(64), 0, st, m->mix, (long)n_mix, L.head_norm, 1, m->proj, (long)n_proj, 3 * HD,
                               (int)HB_GATE_SILU, L.vdim, c.eps, L.out_scale);
        return hb_gemm_resid<T>(st, m->mix, n_mix, (const T*)L.w_out, nullptr, cur, ldx, n, W, n_mix, L.ls1);
    }
    if (!hn && !(n == 1 && hb_try_norm_gemv<T>(m, st, HB_EPI_STORE, cur, ldx, nullptr, L.norm1, (const T*)L.w_in, L.b_in, m->proj, n_in, W))) {
        hb_norm(m, st, n, cur, ldx, nullptr, L.norm1, m->h, nullptr, nullptr, (long)W);
        hn = m->h;
    }
    if (hn) VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, hn, W, (const T*)L.w_in, L.b_in, m->proj, n_proj, n, n_in, W));
    const int vt = (L.vdim + 63) / 64;
    // dims per wave of the scans: the smallest of 16 / 32 / 64 that covers dim with at most 16 waves
    const int dpw = L.dim <= 16 * HB_SCAN_MAX_WAVES ? 16 : (L.dim <= 32 * HB_SCAN_MAX_WAVES ? 32 : 64);
    const int nwv = (L.dim + dpw - 1) / dpw;
    // tokens staged per tile: as many as fit 4096 staged floats per array, at most 16
    const int dpad = nwv * dpw;
    const int tt = 4096 / dpad >= 16 ? 16 : (4096 / dpad >= 1 ? 4096 / dpad : 1);
    if (L.kind == VOX_MIXER_HGRN2) {
        auto kern = dpw == 16 ? k_hb_hgrn2_scan<16> : (dpw == 32 ? k_hb_hgrn2_scan<32> : k_hb_hgrn2_scan<64>);
        const size_t lds = (size_t)(2 * tt * dpad + tt * 64 + 2 * nwv * 64) * 4;
        hipLaunchKernelGGL(kern, dim3(n_req, L.heads, vt), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, L.lower,
                           state, io->req_rows, io->req_state, io->pos, L.heads, L.dim, L.vdim, tt);
        hipLaunchKernelGGL(k_hb_head_norm, dim3(n, L.heads), dim3(64), 0, st, m->mix, (long)n_mix, L.head_norm, 0, m->proj, (long)n_proj, -1,
                           (int)HB_GATE_NONE, L.vdim, c.eps, L.out_scale);
    } else if (L.kind == VOX_MIXER_MLSTM) {
        auto kern = dpw == 16 ? k_hb_mlstm_scan<16> : (dpw == 32 ? k_hb_mlstm_scan<32> : k_hb_mlstm_scan<64>);
        const size_t lds = (size_t)(2 * tt * dpad + tt * 64 + tt * 2 + 2 * nwv * 65) * 4;
        hipLaunchKernelGGL(kern, dim3(n_req, L.heads, vt), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, state,
                           io->req_rows, io->req_state, io->pos, L.heads, L.dim, L.vdim, L.gate_cap, tt);
        hipLaunchKernelGGL(k_hb_head_norm, dim3(n, L.heads), dim3(64), 0, st, m->mix, (long)n_mix, L.head_norm, 1, m->proj, (long)n_proj,
                           2 * L.heads * L.dim + L.heads * L.vdim, (int)HB_GATE_SIGMOID, L.vdim, c.eps, L.out_scale);
    } else if (L.kind == VOX_MIXER_RETENTION) {
        auto kern = dpw == 16 ? k_hb_retention_scan<16> : (dpw == 32 ? k_hb_retention_scan<32> : k_hb_retention_scan<64>);
        const size_t lds = (size_t)(2 * tt * dpad + tt * 64 + 2 * nwv * 64) * 4;
        const float kscale = 1.0f / sqrtf((float)L.dim);
        if (n > HB_SCAN_CHUNK && m->scan_ws) {
            // steps of many rows: chunks of HB_SCAN_CHUNK rows side by side (reduce from zero, carries in order, replay)
            const int nch = (n + HB_SCAN_CHUNK - 1) / HB_SCAN_CHUNK;
            const int per = L.dim * L.vdim;
            hipLaunchKernelGGL(kern, dim3(n_req, L.heads, vt * nch), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, L.decay,
                               L.inv_freq, state, io->req_rows, io->req_state, io->pos, L.heads, L.dim, L.vdim, L.rot_dims, kscale, tt, 1,
                               HB_SCAN_CHUNK, m->scan_ws);
            hipLaunchKernelGGL(k_hb_retention_carry, dim3(n_req, L.heads, (per + 255) / 256 < 64 ? (per + 255) / 256 : 64), dim3(256), 0, st,
                               m->scan_ws, state, L.decay, io->req_rows, io->req_state, io->pos, L.heads, L.dim, L.vdim, HB_SCAN_CHUNK);
            hipLaunchKernelGGL(kern, dim3(n_req, L.heads, vt * nch), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, L.decay,
                               L.inv_freq, state, io->req_rows, io->req_state, io->pos, L.heads, L.dim, L.vdim, L.rot_dims, kscale, tt, 2,
                               HB_SCAN_CHUNK, m->scan_ws);
        } else {
            hipLaunchKernelGGL(kern, dim3(n_req, L.heads, vt), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, L.decay,
                               L.inv_freq, state, io->req_rows, io->req_state, io->pos, L.heads, L.dim, L.vdim, L.rot_dims, kscale, tt, 0, 0,
                               (float*)nullptr);
        }
        hipLaunchKernelGGL(k_hb_head_norm, dim3(n, L.heads), dim3(64), 0, st, m->mix, (long)n_mix, L.head_norm, 1, m->proj, (long)n_proj,
                           2 * L.heads * L.dim + L.heads * L.vdim, (int)HB_GATE_SILU, L.vdim, c.eps, L.out_scale);
    } else if (L.kind == VOX_MIXER_DELTA) {
        const hb_delta_layout y = hb_delta(L);
        const int H = L.heads, G = L.kv_heads, nv = H * L.vdim;
        const long per_slot = (long)H * L.dim * L.vdim + (long)(L.conv_taps - 1) * y.nqkv, hist_off = (long)H * L.dim * L.vdim;
        if (L.lora > 0)
            VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, m->proj + y.off_din, n_proj, (const T*)L.w_decay2, nullptr, m->proj + y.off_dec, n_proj, n, y.ndec, L.lora));
        if (L.gate_rank > 0)
            VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, m->proj + y.off_gin, n_proj, (const T*)L.w_gate2, nullptr, m->proj + y.off_gate, n_proj, n, nv, L.gate_rank));
        hipLaunchKernelGGL(k_hb_delta_conv, dim3(n, (y.nqkv + y.ndec + H + 255) / 256), dim3(256), 0, st, m->proj, (long)n_proj, L.conv_w, state,
                           per_slot, hist_off, L.a_log, L.dt_bias, io->pos, io->row_req, io->req_rows, io->req_state, y, H, L.dim, L.conv_taps,
                           L.decay_channels);
        hipLaunchKernelGGL(k_hb_delta_unit, dim3(n, G + (L.conv_taps > 1 ? (y.nqkv + 127) / 128 : 0)), dim3(128), 0, st, m->proj, (long)n_proj,
                           state, per_slot, hist_off, io->pos, io->row_req, io->req_rows, io->req_state, y, G, L.dim, L.conv_taps);
        const bool chunked = n > HB_DELTA_CHUNK && m->scan_ws && L.dim <= HB_DELTA_CHUNK_DIM;
        const int gate_mode = L.gate_act == VOX_GATE_SILU ? (int)HB_GATE_SILU : (L.gate_act == VOX_GATE_SIGMOID ? (int)HB_GATE_SIGMOID : (int)HB_GATE_NONE);
        // few-row steps with heads of at most 64 value columns (one block holds a head): the scan also applies the head norm, the gate
        // and the scale (per token that is a reduction inside the sequential loop, which long portions leave to a launch of its own)
        const bool fused_norm = L.vdim <= 64 && n <= HB_MOE_GEMV_ROWS;
        auto kern = dpw == 16 ? k_hb_delta_scan<16> : (dpw == 32 ? k_hb_delta_scan<32> : k_hb_delta_scan<64>);
        // three staged arrays per token here: fewer tokens per tile at the widest heads, so that the tile stays within 64 KB of LDS
        const int tt = 3072 / dpad >= 16 ? 16 : (3072 / dpad >= 1 ? 3072 / dpad : 1);
        const size_t lds = (size_t)(3 * tt * dpad + tt * 64 + tt * 2 + 2 * nwv * 128) * 4;
        if (chunked) {
            // steps of many rows: chunks of HB_DELTA_CHUNK rows side by side (each chunk's transition and offset from the identity and
            // from zero, the carries pushed through in order, each chunk replayed from its carry)
            const int nch = (n + HB_DELTA_CHUNK - 1) / HB_DELTA_CHUNK, at = (L.dim + 63) / 64;
            hipLaunchKernelGGL(kern, dim3(n_req, H, (vt + at) * nch), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, state,
                               per_slot, io->req_rows, io->req_state, io->pos, H, G, L.dim, L.vdim, y, L.decay_channels, tt, (int)HB_SCAN_REDUCE,
                               HB_DELTA_CHUNK, m->scan_ws, (const float*)nullptr, 0, c.eps, L.out_scale);
            hipLaunchKernelGGL(L.dim <= 64 ? k_hb_delta_carry<64> : k_hb_delta_carry<128>, dim3(n_req, H, (L.vdim + HB_DC_COLS - 1) / HB_DC_COLS),
                               dim3(256), 0, st, m->scan_ws, state, per_slot, io->req_rows, io->req_state, io->pos, H, L.dim, L.vdim, HB_DELTA_CHUNK);
            hipLaunchKernelGGL(kern, dim3(n_req, H, vt * nch), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, state,
                               per_slot, io->req_rows, io->req_state, io->pos, H, G, L.dim, L.vdim, y, L.decay_channels, tt, (int)HB_SCAN_REPLAY,
                               HB_DELTA_CHUNK, m->scan_ws, (const float*)nullptr, 0, c.eps, L.out_scale);
        } else {
            hipLaunchKernelGGL(kern, dim3(n_req, H, vt), dim3(64 * nwv), lds, st, m->proj, (long)n_proj, m->mix, (long)n_mix, state, per_slot,
                               io->req_rows, io->req_state, io->pos, H, G, L.dim, L.vdim, y, L.decay_channels, tt, (int)HB_SCAN_WHOLE, 0,
                               (float*)nullptr, fused_norm ? L.head_norm : (const float*)nullptr, gate_mode, c.eps, L.out_scale);
        }
        if (!fused_norm)
            hipLaunchKernelGGL(k_hb_head_norm, dim3(n, H), dim3(64), 0, st, m->mix, (long)n_mix, L.head_norm, 0, m->proj, (long)n_proj, y.off_gate,
                               gate_mode, L.vdim, c.eps, L.out_scale);
    } else if (L.kind == VOX_MIXER_LATENT_ATTN) {
        const hb_latent_layout y = hb_latent(L);
        const int H = L.heads, R = L.kv_rank, r = L.rot_dim, D = R + r, dq = L.dim + r;
        float* q = m->proj + y.off_q;
        float* qa = m->proj + y.off_qa;
        float* o = m->proj + y.off_o;
        hipLaunchKernelGGL((k_hb_latent_prep<T>), dim3(n, 2), dim3(256), 0, st, m->proj, (long)n_proj, (T*)cache, L.q_lat_norm, L.kv_lat_norm,
                           L.inv_freq, io->pos, io->page, io->slot, L.q_rank, R, r, L.rot_dims, ps, c.eps);
        VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, m->proj, n_proj, (const T*)L.w_uq, nullptr, q, n_proj, n, H * dq, L.q_rank));
        // every head's plain query part times its key expansion: the query against the cached latent
        VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, q, n_proj, (const T*)L.w_ukT, nullptr, qa, n_proj, n, R, L.dim,
                           hb_rowmap{nullptr, nullptr, 0, 1, (long)R * L.dim, (long)dq, (long)D, 0, nullptr, 0.f}, H));
        if (r > 0)
            hipLaunchKernelGGL(k_hb_latent_qrot, dim3(n, H), dim3(64), 0, st, q, (long)n_proj, qa, (long)n_proj, L.inv_freq, io->pos, L.dim, R, r,
                               L.rot_dims);
        // attention of all heads over one cached head of D key dims whose first R dims are also the value
        const int G = hb_latent_groups(H), QG = H / G;
        const int window = L.window > 0 ? L.window : c.max_seq_len, P = 0x7fffffff;
        const int split = 16 / QG >= 4 ? 4 : (16 / QG >= 1 ? 16 / QG : 1);
        const int nwv2 = QG * split, dimp = (D + 3) & ~3;
        const size_t lds = (size_t)nwv2 * 64 * 8 + (size_t)nwv2 * 64 * 4 + (size_t)QG * dimp * 4 + (size_t)nwv2 * (R + 2) * 4;
        const int max_keys = max_kvlen < window ? max_kvlen : window;
        const float* gate = m->proj + L.q_rank + D;
        if (n <= HB_ATTN_SEG_ROWS) {
            // few rows: a block per (row, key tiles), all heads against the tile in LDS; the tiles of a row spread over up to
            // HB_LAT_MAX_SEG blocks whose partial results are merged
            constexpr int KT = hb_lat_tile<T>::KT;
            const int nchunks = (max_keys + KT - 1) / KT;
            int cpb = n <= 8 ? 1 : (n <= 16 ? 2 : 4);
            if ((nchunks + cpb - 1) / cpb > HB_LAT_MAX_SEG) cpb = (nchunks + HB_LAT_MAX_SEG - 1) / HB_LAT_MAX_SEG;
            const int nseg2 = (nchunks + cpb - 1) / cpb;
            const bool seg2 = nseg2 > 1;
            if (seg2 && (size_t)n * H * nseg2 * (R + 2) * 4 > m->attn_ws_bytes) return vox_fail(VOX_ERR_INVALID, "hybrid_step: attention workspace");
            const int DP = hb_lat_dp<T>(D), Dq = (D + 3) & ~3;
            const size_t lds2 = (((size_t)KT * DP * sizeof(T) + 15) / 16) * 16 + (size_t)(HB_LAT_HG * Dq + KT * HB_LAT_HG + HB_LAT_HG * 3) * 4;
            if (lds2 > 64 * 1024 && !m->lat_big_lds) {
                VOX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_hb_latent_attn_rows<T>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
                m->lat_big_lds = true;
            }
            hipLaunchKernelGGL((k_hb_latent_attn_rows<T>), dim3(n, nseg2), dim3(hb_lat_tile<T>::NT), lds2, st, qa, (long)n_proj, (const T*)cache, o, (long)n_proj,
                               io->pos, io->row_req, io->page_table, io->pt_stride, H, R, r, window, ps, L.scale, cpb,
                               seg2 ? m->attn_ws : (float*)nullptr, gate, (long)n_proj, L.out_scale, DP);
            if (seg2)
                hipLaunchKernelGGL(k_hb_attn_merge, dim3(n, H), dim3(64), 0, st, m->attn_ws, nseg2, o, (long)n_proj, io->pos, H, R, window, P, cpb,
                                   gate, (long)n_proj, L.out_scale, KT, 0);
        } else if (hb_try_latent_mfma(m, st, io, L, (const T*)cache, qa, o, (long)n_proj, gate, n, n_req, window, ps)) {
        } else {
        const int nseg = 1;
        const bool segmented = false;
        if (lds > 64 * 1024 && !m->attn_big_lds) {
            VOX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_hb_attn<T>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            m->attn_big_lds = true;
        }
        hipLaunchKernelGGL((k_hb_attn<T>), dim3(n, G, segmented ? nseg : 1), dim3(64 * nwv2), lds, st, qa, (long)n_proj, (const T*)cache,
                           (const float*)nullptr, o, (long)n_proj, io->pos, io->row_req, io->page_table, io->pt_stride, H, G, D, R, window, P, ps, 1,
                           0L, L.scale, split, segmented ? HB_ATTN_SEG : 0, segmented ? m->attn_ws : (float*)nullptr, gate, (long)n_proj,
                           L.out_scale, 1, (long)D, 0);
        if (segmented)
            hipLaunchKernelGGL(k_hb_attn_merge, dim3(n, H), dim3(64), 0, st, m->attn_ws, nseg, o, (long)n_proj, io->pos, H, R, window, P,
                               HB_ATTN_SEG, gate, (long)n_proj, L.out_scale, 64, 0);
        }
        // every head's weighted latent times its value expansion
        VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, o, n_proj, (const T*)L.w_uv, nullptr, m->mix, n_mix, n, L.vdim, R,
                           hb_rowmap{nullptr, nullptr, 0, 1, (long)L.vdim * R, (long)R, (long)L.vdim, 0, nullptr, 0.f}, H));
    } else if (L.kind == VOX_MIXER_RGLRU) {
        const int C = L.heads * L.dim, bs = L.dim;
        hipLaunchKernelGGL(k_hb_conv_causal, dim3(n, (C + 255) / 256), dim3(256), 0, st, m->proj, (long)n_proj, L.conv_w, L.conv_b, state, io->pos,
                           io->row_req, io->req_rows, io->req_state, C, L.conv_taps);
        // block-diagonal gates: block b's 2*bs outputs (r rows, then i rows) from its bs channels of the convolution's output
        VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, m->proj + 2 * C, n_proj, (const T*)L.w_gates, L.b_gates, m->proj + 3 * C, n_proj, n, 2 * bs, bs,
                           hb_rowmap{nullptr, nullptr, 0, 1, (long)2 * bs * bs, (long)bs, (long)2 * bs, (long)2 * bs}, L.heads));
        // steps of many rows cut every request's rows into chunks that run side by side; the chunked form replays the same recurrence
        // from carries that were pushed through whole chunks, which differs from the plain form by rounding only
        if (n > HB_LRU_SEQ_ROWS)
            hipLaunchKernelGGL(k_hb_rglru_scan_chunked, dim3(n_req, (C + 31) / 32), dim3(1024), 0, st, m->proj, (long)n_proj, m->mix, (long)n_mix,
                               L.lam, state, io->req_rows, io->req_state, io->pos, C, bs, L.conv_taps, L.rec_scale, L.out_scale);
        else
            hipLaunchKernelGGL(k_hb_rglru_scan, dim3(n_req, (C + 63) / 64), dim3(64), 0, st, m->proj, (long)n_proj, m->mix, (long)n_mix, L.lam, state,
                               io->req_rows, io->req_state, io->pos, C, bs, L.conv_taps, L.rec_scale, L.out_scale);
    } else {
        const bool causal = L.kind == VOX_MIXER_CAUSAL_ATTN, conv = hb_conv_attn(L);
        // query heads per block: the whole group of a key / value head, or (groups of more than 16) its largest divisor up to 16
        int QG = L.heads / L.kv_heads;
        if (causal)
            for (int q2 = QG < 16 ? QG : 16; q2 >= 1; --q2)
                if ((L.heads / L.kv_heads) % q2 == 0) { QG = q2; break; }
        const int H = L.heads, G = L.kv_heads, GG = H / QG;
        const int window = causal ? c.max_seq_len : L.window, P = causal ? 1 : L.pool;
        const long v_base = (long)c.max_pages * ps * G * L.dim;
        const int ppp = (ps - 1) / P + 1;
        const bool one_row_each = n == n_req;      // decode steps: every block a row closes was filled by earlier steps
        const hb_qkv_opts op = causal ? hb_qkv_opts{L.q_norm, L.k_norm, L.q_temp_coef, L.q_temp_every > 0 ? L.q_temp_every : 1, L.v_unit_rms}
                                      : hb_qkv_opts{nullptr, nullptr, 0.f, 1, 0};
        const float* qrows = m->proj;
        if (conv) {
            const hb_conv_attn_layout y = hb_conv_attn_cols(L);
            const int C = n_in;
            const long per_slot = (long)(L.conv_taps - 1) * C;
            hipLaunchKernelGGL(k_hb_attn_conv, dim3(n, (C + 255) / 256), dim3(256), 0, st, m->proj, (long)n_proj, L.conv_w, state, per_slot, io->pos,
                               io->row_req, io->req_rows, io->req_state, H * L.dim, G * L.dim, C, L.conv_taps, y.off_y, y.off_ss);
            hipLaunchKernelGGL((k_hb_attn_norm_rot<T>), dim3(n, H + 2 * G + (L.conv_taps > 1 ? (C + 63) / 64 : 0)), dim3(64), 0, st, m->proj,
                               (long)n_proj, (T*)cache, state, per_slot, L.q_norm, L.k_norm, L.inv_freq, io->pos, io->page, io->slot, io->row_req,
                               io->req_rows, io->req_state, H, G, L.dim, L.vdim, L.rot_dims, L.conv_taps, ps, v_base, c.eps, y.off_y, y.off_qc,
                               y.off_ss, L.qk_norm_whole);
            const int off_qc = y.off_qc;
            qrows = m->proj + off_qc;
        } else
        hipLaunchKernelGGL((k_hb_attn_prep<T>), dim3(n, H + G), dim3(64), 0, st, m->proj, (long)n_proj, (T*)cache, L.inv_freq, io->pos,
                           io->page, io->slot, H, G, L.dim, L.vdim, causal ? 0 : L.rot_dims, ps, v_base, c.eps,
                           one_row_each && !causal ? pool : (float*)nullptr, io->row_req, io->page_table, io->pt_stride, P, ppp, op);
        if (!one_row_each && !causal)
            hipLaunchKernelGGL((k_hb_pool_update<T>), dim3(n, G), dim3(64), 0, st, (const T*)cache, pool, io->pos, io->row_req,
                               io->page_table, io->pt_stride, G, L.dim, L.vdim, P, ps, ppp, v_base);
        const int split = 16 / QG >= 4 ? 4 : (16 / QG >= 1 ? 16 / QG : 1);      // up to 16 waves per block, at most 4 per head
        const int nwv2 = QG * split, dimp = (L.dim + 3) & ~3;
        const size_t lds = (size_t)nwv2 * 64 * 8 + (size_t)nwv2 * 64 * 4 + (size_t)QG * dimp * 4 + (size_t)nwv2 * (L.vdim + 2) * 4;
        // steps of few rows: 4-chunk key segments on separate blocks + a merge pass (more blocks than rows x kv heads); a row's
        // result differs from the one-block form by the rounding of the merge only
        const int max_keys = causal ? max_kvlen : (max_kvlen < window ? max_kvlen : window) + max_kvlen / P + 1;
        const int nseg = ((max_keys + 63) / 64 + HB_ATTN_SEG - 1) / HB_ATTN_SEG;
        const bool segmented = n <= HB_ATTN_SEG_ROWS && nseg > 1 && (size_t)n * H * nseg * (L.vdim + 2) * 4 <= m->attn_ws_bytes;
        const float* gate = causal ? (const float*)nullptr : m->proj + H * L.dim + G * L.dim + G * L.vdim;      // one logit per query head
        const int sink = causal && L.sink ? 1 : 0;
        hipLaunchKernelGGL((k_hb_attn<T>), dim3(n, GG, segmented ? nseg : 1), dim3(64 * nwv2), lds, st, qrows, (long)n_proj, (const T*)cache,
                           pool, m->mix, (long)n_mix, io->pos, io->row_req, io->page_table, io->pt_stride, H, GG, L.dim, L.vdim, window,
                           P, ps, ppp, v_base, L.scale, split, segmented ? HB_ATTN_SEG : 0, segmented ? m->attn_ws : (float*)nullptr,
                           gate, (long)n_proj, L.out_scale, G, (long)G * L.vdim, sink);
        if (segmented)
            hipLaunchKernelGGL(k_hb_attn_merge, dim3(n, H), dim3(64), 0, st, m->attn_ws, nseg, m->mix, (long)n_mix, io->pos, H, L.vdim, window, P,
                               HB_ATTN_SEG, gate, (long)n_proj, L.out_scale, 64, sink);
    }
    return hb_gemm_resid<T>(st, m->mix, n_mix, (const T*)L.w_out, nullptr, cur, ldx, n, W, n_mix, L.ls1);
}

// Routed feed-forward of the normed rows h2, added to cur.  Few rows: one GEMV pair per routed entry; more: the entries are
// listed per expert and every expert multiplies its own rows in one tile launch.
template <typename T>
static int hb_moe(vox_hybrid* m, hipStream_t st, const vox_hybrid_moe& E, const float* h2, float* cur, long ldx, int n, const float* ls) {
    const int W = m->cfg.width, nE = E.experts + E.identity, top = E.top, ne = n * top, ff = E.ff;
    const int up_down = E.expert_form == VOX_EXPERT_UP_DOWN ? 1 : 0, relu2 = E.expert_act == VOX_ACT_RELU2 ? 1 : 0, nf = up_down ? 1 : 2;
    hipLaunchKernelGGL(k_hb_moe_router, dim3(n), dim3(256), (size_t)(6 * nE + top) * 4, st, h2, (long)W, E.router, E.correction, W, nE, top,
                       m->moe_sel, m->moe_wgt, E.score_kind == VOX_ROUTER_SIGMOID ? 1 : 0, E.renorm, E.router_bias);
    if (n <= HB_MOE_GEMV_ROWS) {
        const int per = top + (E.shared_ff > 0 ? 1 : 0), maxf = ff > E.shared_ff ? ff : E.shared_ff;
        const hb_moe_small q{m->moe_sel, m->moe_wgt, top, E.experts, ff, E.shared_ff, m->max_eff, E.limit, E.shared_limit, E.act_alpha, E.up_offset,
                             E.scale_input, nullptr, 0, up_down, relu2, ls};
        if (maxf > 0 && per > 0 && (E.experts > 0 || E.shared_ff > 0))
            hipLaunchKernelGGL((k_hb_moe_gate_up<T>), dim3((maxf + 3) / 4, n * per), dim3(256), 0, st, h2, (long)W, (const T*)E.w_gate_up,
                               (const T*)E.shared_gate_up, m->moe_act, W, q);
        hipLaunchKernelGGL((k_hb_moe_down_combine<T>), dim3((W + 3) / 4, n), dim3(256), 0, st, h2, (long)W, (const T*)E.w_down,
                           (const T*)E.shared_down, m->moe_act, cur, ldx, W, q);
        return VOX_OK;
    }
    if (E.experts > 0) {
        const int cap = m->cfg.max_rows;
        hipLaunchKernelGGL(k_hb_moe_group, dim3(E.experts), dim3(256), 0, st, m->moe_sel, ne, cap, m->moe_list, m->moe_count);
        VOX_TRY(hb_gemm_tiles<HB_EPI_STORE>(st, h2, (long)W, (const T*)E.w_gate_up, nullptr, m->ff, (long)nf * ff, n, nf * ff, W,
                                            hb_rowmap{m->moe_count, m->moe_list, cap, top, (long)nf * ff * W, 0, 0, 0,
                                                      E.scale_input ? m->moe_wgt : (const float*)nullptr, 0.f}, E.experts));
        hipLaunchKernelGGL(k_hb_glu_clamp, dim3(ne, (ff + 1023) / 1024), dim3(256), 0, st, m->ff, m->moe_act, ff, E.limit, E.act_alpha,
                           m->moe_sel, E.experts, E.up_offset, 0, up_down, relu2);
        VOX_TRY(hb_gemm_tiles<HB_EPI_STORE>(st, m->moe_act, (long)ff, (const T*)E.w_down, nullptr, m->moe_out, (long)W, n, W, ff,
                                            hb_rowmap{m->moe_count, m->moe_list, cap, 1, (long)W * ff, 0, 0, 0}, E.experts));
    }
    hipLaunchKernelGGL(k_hb_moe_combine, dim3(n), dim3(256), 0, st, cur, ldx, h2, (long)W, m->moe_out, m->moe_sel, m->moe_wgt, top, E.experts, W,
                       E.scale_input, ls);
    if (E.shared_ff > 0) {
        const int sf = E.shared_ff;
        VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, h2, W, (const T*)E.shared_gate_up, nullptr, m->ff, nf * sf, n, nf * sf, W));
        hipLaunchKernelGGL(k_hb_glu_clamp, dim3(n, (sf + 1023) / 1024), dim3(256), 0, st, m->ff, m->moe_act, sf, E.shared_limit, E.act_alpha,
                           (const int*)nullptr, 0, E.up_offset, 0, up_down, relu2);
        VOX_TRY(hb_gemm_resid<T>(st, m->moe_act, sf, (const T*)E.shared_down, nullptr, cur, ldx, n, W, sf, ls));
    }
    return VOX_OK;
}

template <typename T>
static int hb_step(vox_hybrid* m, hipStream_t st, const vox_hybrid_io* io, const int32_t* ids, int n, int n_req, int n_out, int max_kvlen) {
    const vox_hybrid_config& c = m->cfg;
    const int W = c.width;
    const long ldx = 2L * W;
    const bool bigram = c.bigram_buckets > 0 && m->w.bigram && m->w.prev_token;
    const hb_bigram bg{bigram ? m->w.bigram : nullptr, m->w.prev_token, c.bigram_buckets, c.bigram_mul_prev, c.bigram_mul_cur, n == n_req ? 1 : 0};
    hipLaunchKernelGGL((k_hb_embed<T>), dim3(n), dim3(256), 0, st, (const T*)m->w.embedding, ids, 1, m->xa, m->xb, W, c.vocab, c.embed_scale, bg,
                       io->pos, io->row_req, io->req_rows, io->req_state);
    if (bigram && n != n_req)
        hipLaunchKernelGGL(k_hb_store_prev, dim3((n_req + 63) / 64), dim3(64), 0, st, ids, 1, c.vocab, io->req_rows, io->req_state, m->w.prev_token, n_req);
    float *cur = m->xa, *other = m->xb;
    for (int ri = 0; ri < c.n_runs; ++ri) {
        const vox_hybrid_run& run = m->runs[ri];
        const vox_hybrid_layer& L = m->layers[run.layer];
        if (run.loop_in) {
            VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, cur, ldx, (const T*)m->w.loop_in, nullptr, other, ldx, n, W, 2 * W));
            float* t = cur; cur = other; other = t;
        }
        const bool has_ff = L.ff > 0 || L.moe;
        const bool one_norm = L.block == VOX_BLOCK_PARALLEL_ONE_NORM;
        const bool parallel = L.block == VOX_BLOCK_PARALLEL || one_norm;
        // a parallel layer norms x once for both branches before anything is added; a mixer with a sibling needs the normed rows twice
        const float* hn = nullptr;
        if (parallel || L.sibling >= 0) {
            hb_norm(m, st, n, cur, ldx, nullptr, L.norm1, m->h, parallel && has_ff && !one_norm ? L.norm2 : nullptr, m->h2, (long)W);
            hn = m->h;
        }
        const float* hf = one_norm ? m->h : m->h2;      // what the feed-forward of a parallel layer reads
        VOX_TRY(hb_mixer<T>(m, st, io, L, run.cache, run.pool, run.state, hn, cur, ldx, n, n_req, max_kvlen));
        if (L.sibling >= 0)
            VOX_TRY(hb_mixer<T>(m, st, io, m->layers[L.sibling], run.side_cache, run.side_pool, run.side_state, hn, cur, ldx, n, n_req, max_kvlen));
        if (L.moe) {
            if (!parallel) hb_norm(m, st, n, cur, ldx, nullptr, L.norm2, m->h2, nullptr, nullptr, (long)W);
            VOX_TRY(hb_moe<T>(m, st, *L.moe, hf, cur, ldx, n, L.ls2));
        } else if (L.ff > 0 && L.ff_kind == VOX_FF_GATED) {
            // down(act(gate h + b) * (up h + b)) + b: gate and up rows in one product, the activation in place behind it
            if (!parallel) hb_norm(m, st, n, cur, ldx, nullptr, L.norm2, m->h2, nullptr, nullptr, (long)W);
            const float* hd = parallel ? hf : m->h2;
            if (n == 1) {
                // one row: gate and up rows of a column by one wave, biases and activation in its epilogue (the routed feed-forward's
                // kernel with the dense unit in the place of the shared expert and nothing routed); more rows would stream the matrix
                // once per row
                const hb_moe_small q{nullptr, nullptr, 0, 0, 0, L.ff, L.ff, INFINITY, INFINITY, 1.0f, 0.0f, 0, L.b_up, L.ff_act == VOX_ACT_GELU_TANH ? 1 : 0,
                                     0, 0, nullptr};
                hipLaunchKernelGGL((k_hb_moe_gate_up<T>), dim3((L.ff + 3) / 4, n), dim3(256), 0, st, hd, (long)W, (const T*)nullptr, (const T*)L.w_up,
                                   m->ff_act, W, q);
            } else {
                VOX_TRY(hb_gemm<T>(st, HB_EPI_STORE, hd, W, (const T*)L.w_up, L.b_up, m->ff, 2 * L.ff, n, 2 * L.ff, W));
                hipLaunchKernelGGL(k_hb_glu_clamp, dim3(n, (L.ff + 1023) / 1024), dim3(256), 0, st, m->ff, m->ff_act, L.ff, INFINITY, 1.0f,
                                   (const int*)nullptr, 0, 0.0f, L.ff_act == VOX_ACT_GELU_TANH ? 1 : 0, 0, 0);
            }
            VOX_TRY(hb_gemm_resid<T>(st, m->ff_act, L.ff, (const T*)L.w_down, L.b_down, cur, ldx, n, W, L.ff, L.ls2));
        } else if (L.ff > 0) {
            if (parallel) {
                VOX_TRY(hb_gemm<T>(st, HB_EPI_GELU, hf, W, (const T*)L.w_up, nullptr, m->ff, L.ff, n, L.ff, W));
            } else if (!(n == 1 && hb_try_norm_gemv<T>(m, st, HB_EPI_GELU, cur, ldx, nullptr, L.norm2, (const T*)L.w_up, nullptr, m->ff, L.ff, W))) {
                hb_norm(m, st, n, cur, ldx, nullptr, L.norm2, m->h, nullptr, nullptr, (long)W);
                VOX_TRY(hb_gemm<T>(st, HB_EPI_GELU, m->h, W, (const T*)L.w_up, nullptr, m->ff, L.ff, n, L.ff, W));
            }
            VOX_TRY(hb_gemm_resid<T>(st, m->ff, L.ff, (const T*)L.w_down, nullptr, cur, ldx, n, W, L.ff, L.ls2));
        }
        if (io->trace)
            hipLaunchKernelGGL(k_hb_copy_rows, dim3(n), dim3(256), 0, st, cur, ldx, io->trace + (size_t)ri * c.max_rows * W, (long)W, W);
    }
    if (n_out > 0) {
        const bool scaled = c.logit_scale != 0.f && c.logit_scale != 1.0f;
        if (!(n_out == 1 && !(c.logit_softcap > 0.f) &&
              hb_try_norm_gemv<T>(m, st, scaled ? HB_EPI_SCALE : HB_EPI_STORE, cur, ldx, io->out_rows, m->w.final_norm, (const T*)m->w.head, nullptr,
                                  io->logits, c.vocab, W, c.logit_scale))) {
            hb_norm(m, st, n_out, cur, ldx, io->out_rows, m->w.final_norm, m->hout, nullptr, nullptr, (long)W);
            hb_rowmap rm = hb_plain();
            rm.epi_arg = c.logit_softcap > 0.f ? c.logit_softcap : c.logit_scale;
            VOX_TRY(hb_gemm<T>(st, c.logit_softcap > 0.f ? HB_EPI_SOFTCAP : (scaled ? HB_EPI_SCALE : HB_EPI_STORE), m->hout, W, (const T*)m->w.head,
                               nullptr, io->logits, c.vocab, n_out, c.vocab, W, rm));
        }
    }
    VOX_HIP(hipGetLastError());
    return VOX_OK;
}

extern "C" {

int vox_hybrid_create(vox_ctx* ctx, const vox_hybrid_config* cfg, const vox_hybrid_weights* w, vox_hybrid** out) {
    if (!ctx || !cfg || !w || !out || !w->layers || !w->runs) return vox_fail(VOX_ERR_INVALID, "hybrid_create: NULL argument");
    if (cfg->dtype != VOX_HYBRID_BF16 && cfg->dtype != VOX_HYBRID_F32) return vox_fail(VOX_ERR_INVALID, "hybrid_create: dtype %d", cfg->dtype);
    if (cfg->width < 1 || cfg->vocab < 1 || cfg->page_size < 1 || cfg->max_rows < 1 || cfg->max_batch < 1 || cfg->max_out < 1 || cfg->max_seq_len < 1)
        return vox_fail(VOX_ERR_INVALID, "hybrid_create: bad sizes");
    if (cfg->norm_kind != VOX_NORM_LAYER && cfg->norm_kind != VOX_NORM_RMS_GROUPS) return vox_fail(VOX_ERR_INVALID, "hybrid_create: norm kind %d", cfg->norm_kind);
    if (cfg->logit_softcap > 0.f && cfg->logit_scale != 0.f && cfg->logit_scale != 1.0f)
        return vox_fail(VOX_ERR_INVALID, "hybrid_create: a logit scale beside a soft cap");
    if (cfg->norm_kind == VOX_NORM_RMS_GROUPS && (cfg->norm_groups < 1 || cfg->width % cfg->norm_groups != 0))
        return vox_fail(VOX_ERR_INVALID, "hybrid_create: %d norm groups do not divide width %d", cfg->norm_groups, cfg->width);
    vox_hybrid* m = new vox_hybrid();
    m->ctx = ctx; m->cfg = *cfg; m->w = *w;
    m->layers.assign(w->layers, w->layers + cfg->n_layers);
    m->runs.assign(w->runs, w->runs + cfg->n_runs);
    m->w.layers = nullptr; m->w.runs = nullptr;
    m->moes.reserve(m->layers.size());
    for (vox_hybrid_layer& L : m->layers)
        if (L.moe) { m->moes.push_back(*L.moe); L.moe = &m->moes.back(); }
    for (const vox_hybrid_layer& L : m->layers) {
        const int n_in = hb_layer_in(L);
        const char* bad = nullptr;
        if (n_in < 0) bad = "unknown mixer kind";
        else if (L.heads < 1 || L.dim < 1 || L.vdim < 1) bad = "heads / dim / vdim";
        else if (L.vdim > 64 * HB_MAX_VPL && L.kind != VOX_MIXER_RGLRU) bad = "vdim above 512";
        else if (!L.norm1 || !L.w_in || !L.w_out) bad = "missing weights";
        else if (L.ff > 0 && ((!L.norm2 && L.block != VOX_BLOCK_PARALLEL_ONE_NORM) || !L.w_up || !L.w_down)) bad = "missing feed-forward weights";
        else if (L.ff > 0 && L.ff_kind != VOX_FF_UP_DOWN && L.ff_kind != VOX_FF_GATED) bad = "feed-forward form";
        else if (L.block != VOX_BLOCK_SEQUENTIAL && L.block != VOX_BLOCK_PARALLEL && L.block != VOX_BLOCK_PARALLEL_ONE_NORM) bad = "block form";
        else if (L.sibling >= cfg->n_layers || (L.sibling >= 0 && m->layers[L.sibling].sibling >= 0)) bad = "sibling index";
        else if (L.kind == VOX_MIXER_HGRN2 && (!L.lower || !L.head_norm)) bad = "hgrn2 needs lower and head_norm";
        else if (L.kind == VOX_MIXER_MLSTM && (!L.head_norm || !(L.gate_cap > 0.f))) bad = "mlstm needs head_norm and gate_cap";
        else if (L.kind == VOX_MIXER_RETENTION && (!L.decay || L.rot_dims < 0 || L.rot_dims > L.dim || (L.rot_dims & 1) || (L.rot_dims > 0 && !L.inv_freq)))
            bad = "retention needs decay and an even rot_dims <= dim";
        else if (L.kind == VOX_MIXER_LATENT_ATTN) {
            if (L.q_rank < 1 || L.kv_rank < 1 || L.rot_dim < 0 || !L.w_uq || !L.w_ukT || !L.w_uv || !L.q_lat_norm || !L.kv_lat_norm) bad = "latent attention: ranks / expansions / norms";
            else if (L.kv_rank > 64 * HB_MAX_VPL) bad = "latent attention: kv_rank above 512";
            else if (L.kv_rank + L.rot_dim > 768) bad = "latent attention: kv_rank + rot_dim above 768 (a key tile and 16 queries have to fit the LDS)";
            else if (L.rot_dims < 0 || L.rot_dims > L.rot_dim || (L.rot_dims & 1) || (L.rot_dims > 0 && !L.inv_freq)) bad = "latent attention: rot_dims";
            else if (L.window < 0) bad = "latent attention: window";
        }
        else if ((L.kind == VOX_MIXER_HGRN2 || L.kind == VOX_MIXER_MLSTM || L.kind == VOX_MIXER_SHIFT_DECAY || L.kind == VOX_MIXER_RETENTION ||
                  L.kind == VOX_MIXER_DELTA) && L.dim > 64 * HB_SCAN_MAX_WAVES)
            bad = "recurrent dim above 1024";
        else if (L.kind == VOX_MIXER_DELTA) {
            if (L.kv_heads < 1 || L.heads % L.kv_heads != 0) bad = "delta: heads / kv_heads";
            else if (L.conv_taps < 1 || !L.conv_w) bad = "delta: convolution";
            else if (!L.a_log || !L.dt_bias || !L.head_norm) bad = "delta: a_log / dt_bias / head_norm";
            else if (L.lora < 0 || (L.lora > 0 && !L.w_decay2)) bad = "delta: decay bottleneck";
            else if (L.gate_rank < 0 || (L.gate_rank > 0 && !L.w_gate2)) bad = "delta: gate bottleneck";
            else if (L.gate_act != VOX_GATE_NONE && L.gate_act != VOX_GATE_SIGMOID && L.gate_act != VOX_GATE_SILU) bad = "delta: gate activation";
        }
        else if (L.kind == VOX_MIXER_RGLRU && (L.dim != L.vdim || L.conv_taps < 1 || !L.conv_w || !L.w_gates || !L.lam)) bad = "rglru needs conv, gates and lam";
        else if (L.kind == VOX_MIXER_SHIFT_DECAY && (L.dim != L.vdim || L.lora < 1 || !L.shift_mu || !L.w_decay2 || !L.decay0 || !L.bonus || !L.head_norm))
            bad = "shift-decay needs mu, decay and bonus tensors";
        else if (hb_is_attn(L.kind) && L.kind != VOX_MIXER_LATENT_ATTN) {
            if (L.kv_heads < 1 || L.heads % L.kv_heads != 0 || (L.heads / L.kv_heads > 16 && L.kind != VOX_MIXER_CAUSAL_ATTN))
                bad = "heads / kv_heads (group of at most 16)";
            else if (hb_conv_attn(L) && (!L.conv_w || (L.qk_norm_whole && (!L.q_norm || !L.k_norm)))) bad = "attention behind a convolution: conv_w / q_norm / k_norm";
            else if (hb_conv_attn(L) && (L.rot_dims < 0 || L.rot_dims > L.dim || (L.rot_dims & 1) || (L.rot_dims > 0 && !L.inv_freq))) bad = "rot_dims";
            else if (hb_conv_attn(L) && (L.q_temp_coef != 0.f || L.v_unit_rms)) bad = "attention behind a convolution: no query temperature / unit values";
            else if (L.dim > 64 * HB_MAX_DPL) bad = "dim above 512";
            else if (L.kind == VOX_MIXER_POOLED_WINDOW_ATTN && (L.window < 1 || L.pool < 1)) bad = "window / pool";
            else if (L.kind == VOX_MIXER_POOLED_WINDOW_ATTN && (L.rot_dims < 0 || L.rot_dims > L.dim || (L.rot_dims & 1) || (L.rot_dims > 0 && !L.inv_freq))) bad = "rot_dims";
        }
        if (!bad && L.moe) {
            const vox_hybrid_moe& E = *L.moe;
            if (E.experts < 0 || E.identity < 0 || E.top < 1 || E.top > E.experts + E.identity) bad = "moe: experts / identity / top";
            else if (E.expert_form != VOX_EXPERT_GATED && E.expert_form != VOX_EXPERT_UP_DOWN) bad = "moe: expert form";
            else if (E.expert_form == VOX_EXPERT_UP_DOWN && E.expert_act != VOX_ACT_RELU2 && E.expert_act != VOX_ACT_SWISH) bad = "moe: expert activation";
            else if (!E.router || (!L.norm2 && L.block != VOX_BLOCK_PARALLEL_ONE_NORM)) bad = "moe: router or norm2 missing";
            else if (E.score_kind != VOX_ROUTER_SOFTMAX && E.score_kind != VOX_ROUTER_SIGMOID) bad = "moe: score kind";
            else if (E.experts > 0 && (E.ff < 1 || !E.w_gate_up || !E.w_down)) bad = "moe: expert weights";
            else if (E.shared_ff > 0 && (!E.shared_gate_up || !E.shared_down)) bad = "moe: shared expert weights";
        }
        if (bad) { delete m; return vox_fail(VOX_ERR_INVALID, "hybrid_create: layer: %s", bad); }
        const int n_proj = hb_layer_proj(L);
        if (n_proj > m->max_in) m->max_in = n_proj;
        if (L.heads * L.vdim > m->max_mix) m->max_mix = L.heads * L.vdim;
        if ((L.ff_kind == VOX_FF_GATED ? 2 : 1) * L.ff > m->max_ff) m->max_ff = (L.ff_kind == VOX_FF_GATED ? 2 : 1) * L.ff;
        if (L.ff_kind == VOX_FF_GATED && L.ff > m->max_gated) m->max_gated = L.ff;
        if (L.kind == VOX_MIXER_RETENTION) {
            const size_t f = ((size_t)cfg->max_rows / HB_SCAN_CHUNK + cfg->max_batch + 1) * L.heads * ((size_t)L.dim * L.vdim);
            if (f > m->scan_ws_floats) m->scan_ws_floats = f;
        }
        if (L.kind == VOX_MIXER_DELTA && L.dim <= HB_DELTA_CHUNK_DIM) {
            const size_t f = ((size_t)cfg->max_rows / HB_DELTA_CHUNK + cfg->max_batch + 1) * L.heads * ((size_t)L.dim * (L.vdim + L.dim));
            if (f > m->scan_ws_floats) m->scan_ws_floats = f;
        }
        if (L.kind == VOX_MIXER_SHIFT_DECAY) {
            m->any_shift = true;
            const size_t f = ((size_t)cfg->max_rows / HB_SCAN_CHUNK + cfg->max_batch + 1) * L.heads * ((size_t)L.dim * L.dim + L.dim);
            if (f > m->scan_ws_floats) m->scan_ws_floats = f;
        }
        if (L.moe) {
            const vox_hybrid_moe& E = *L.moe;
            if (E.experts + E.identity > m->max_ne) m->max_ne = E.experts + E.identity;
            if (E.experts > m->max_experts) m->max_experts = E.experts;
            if (E.top > m->max_top) m->max_top = E.top;
            if (E.top * 2 * E.ff > m->max_ff) m->max_ff = E.top * 2 * E.ff;
            if (2 * E.shared_ff > m->max_ff) m->max_ff = 2 * E.shared_ff;
            if (E.top * E.ff > m->max_eff) m->max_eff = E.top * E.ff;
            if (E.shared_ff > m->max_eff) m->max_eff = E.shared_ff;
        }
    }
    for (const vox_hybrid_run& r : m->runs) {
        const char* bad = nullptr;
        if (r.layer < 0 || r.layer >= cfg->n_layers) bad = "layer index";
        else {
            const vox_hybrid_layer& L = m->layers[r.layer];
            if (hb_is_attn(L.kind) ? (!r.cache || (L.kind == VOX_MIXER_POOLED_WINDOW_ATTN && !r.pool) || (hb_conv_attn(L) && L.conv_taps > 1 && !r.state))
                                   : !r.state) bad = "missing cache / state";
            else if (cfg->bigram_buckets > 0 && (!w->bigram || !w->prev_token)) bad = "bigram table / previous-token state";
            else if (L.sibling >= 0) {
                const vox_hybrid_layer& S2 = m->layers[L.sibling];
                if (hb_is_attn(S2.kind) ? (!r.side_cache || (S2.kind == VOX_MIXER_POOLED_WINDOW_ATTN && !r.side_pool)) : !r.side_state)
                    bad = "missing cache / state of the sibling mixer";
            }
            if (!bad && r.loop_in && !w->loop_in) bad = "loop_in weight";
        }
        if (bad) { delete m; return vox_fail(VOX_ERR_INVALID, "hybrid_create: run: %s", bad); }
    }
    const size_t R = cfg->max_rows, W = cfg->width;
    bool ok = hipMalloc((void**)&m->xa, R * 2 * W * 4) == hipSuccess && hipMalloc((void**)&m->xb, R * 2 * W * 4) == hipSuccess &&
              hipMalloc((void**)&m->h, R * W * 4) == hipSuccess && hipMalloc((void**)&m->h2, R * W * 4) == hipSuccess &&
              hipMalloc((void**)&m->proj, R * (size_t)m->max_in * 4) == hipSuccess &&
              hipMalloc((void**)&m->mix, R * (size_t)m->max_mix * 4) == hipSuccess &&
              hipMalloc((void**)&m->ff, R * (size_t)(m->max_ff > 0 ? m->max_ff : 1) * 4) == hipSuccess &&
              hipMalloc((void**)&m->hout, (size_t)cfg->max_out * W * 4) == hipSuccess &&
              hipMalloc((void**)&m->logits16, (size_t)cfg->max_batch * cfg->vocab * 2) == hipSuccess;
    if (ok && m->any_shift) ok = hipMalloc((void**)&m->shift, 5 * R * W * 4) == hipSuccess;
    if (ok && m->max_gated) ok = hipMalloc((void**)&m->ff_act, R * (size_t)m->max_gated * 4) == hipSuccess;
    if (ok && m->scan_ws_floats && cfg->max_rows > HB_SCAN_CHUNK) ok = hipMalloc((void**)&m->scan_ws, m->scan_ws_floats * 4) == hipSuccess;
    if (ok && m->max_top > 0) {
        const size_t ne = R * (size_t)m->max_top;
        ok = hipMalloc((void**)&m->moe_wgt, ne * 4) == hipSuccess &&
             hipMalloc((void**)&m->moe_sel, ne * 4) == hipSuccess &&
             hipMalloc((void**)&m->moe_act, (R > HB_MOE_GEMV_ROWS * (size_t)(m->max_top + 1) ? R : HB_MOE_GEMV_ROWS * (size_t)(m->max_top + 1)) *
                                                (size_t)(m->max_eff > 0 ? m->max_eff : 1) * 4) == hipSuccess &&
             hipMalloc((void**)&m->moe_out, ne * W * 4) == hipSuccess &&
             hipMalloc((void**)&m->moe_list, (size_t)(m->max_experts > 0 ? m->max_experts : 1) * R * 4) == hipSuccess &&
             hipMalloc((void**)&m->moe_count, (size_t)(m->max_experts > 0 ? m->max_experts : 1) * 4) == hipSuccess;
    }
    // partial results of segmented attention launches: few rows x heads x segments of the longest sequence
    for (const vox_hybrid_layer& L : m->layers)
        if (hb_is_attn(L.kind)) {
            const bool causal = L.kind == VOX_MIXER_CAUSAL_ATTN, latent = L.kind == VOX_MIXER_LATENT_ATTN;
            const int max_keys = causal || (latent && L.window < 1) ? cfg->max_seq_len
                                 : (cfg->max_seq_len < L.window ? cfg->max_seq_len : L.window) + (latent ? 0 : cfg->max_seq_len / L.pool + 1);
            size_t nseg = ((max_keys + 63) / 64 + HB_ATTN_SEG - 1) / HB_ATTN_SEG;
            if (latent) nseg = (size_t)(max_keys + 31) / 32 < HB_LAT_MAX_SEG ? (size_t)(max_keys + 31) / 32 : HB_LAT_MAX_SEG;
            const size_t b = (size_t)HB_ATTN_SEG_ROWS * L.heads * nseg * ((latent ? L.kv_rank : L.vdim) + 2) * 4;
            if (b > m->attn_ws_bytes) m->attn_ws_bytes = b;
        }
    if (ok && m->attn_ws_bytes) ok = hipMalloc((void**)&m->attn_ws, m->attn_ws_bytes) == hipSuccess;
    if (!ok) { vox_hybrid_destroy(m); return vox_fail(VOX_ERR_NOMEM, "hybrid_create: hipMalloc failed"); }
    *out = m;
    return VOX_OK;
}

void vox_hybrid_destroy(vox_hybrid* m) {
    if (!m) return;
    (void)hipFree(m->xa); (void)hipFree(m->xb); (void)hipFree(m->h); (void)hipFree(m->h2); (void)hipFree(m->proj); (void)hipFree(m->mix);
    (void)hipFree(m->ff); (void)hipFree(m->ff_act); (void)hipFree(m->hout); (void)hipFree(m->logits16); (void)hipFree(m->attn_ws); (void)hipFree(m->shift); (void)hipFree(m->scan_ws);
    (void)hipFree(m->moe_wgt); (void)hipFree(m->moe_sel); (void)hipFree(m->moe_act); (void)hipFree(m->moe_out);
    (void)hipFree(m->moe_list); (void)hipFree(m->moe_count);
    delete m;
}

int vox_hybrid_step(vox_hybrid* m, void* stream, const vox_hybrid_io* io, const int32_t* ids, int n_rows, int n_req, int n_out,
                    int max_kvlen, const vox_sampling_config* sc, uint64_t seed, int feedback) {
    if (!m || !io || !ids) return vox_fail(VOX_ERR_INVALID, "hybrid_step: NULL");
    const vox_hybrid_config& c = m->cfg;
    if (n_rows < 1 || n_rows > c.max_rows || n_req < 1 || n_req > c.max_batch || n_req > n_rows || n_out < 0 || n_out > c.max_out)
        return vox_fail(VOX_ERR_INVALID, "hybrid_step: rows %d / requests %d / outputs %d out of range", n_rows, n_req, n_out);
    if (!io->pos || !io->row_req || !io->page || !io->slot || !io->req_rows || !io->req_state || !io->page_table || (n_out && (!io->out_rows || !io->logits)))
        return vox_fail(VOX_ERR_INVALID, "hybrid_step: missing plan arrays");
    if (max_kvlen < 1 || max_kvlen > c.max_seq_len) max_kvlen = c.max_seq_len;
    hipStream_t st = (hipStream_t)stream;
    VOX_TRY(c.dtype == VOX_HYBRID_F32 ? hb_step<float>(m, st, io, ids, n_rows, n_req, n_out, max_kvlen) : hb_step<bf16_t>(m, st, io, ids, n_rows, n_req, n_out, max_kvlen));
    if (!sc) return VOX_OK;
    // sampling: one pick per request from the first n_req output rows (the caller lists each request's last row first)
    if (n_out < n_req || n_req > c.max_batch || !io->out_ids) return vox_fail(VOX_ERR_INVALID, "hybrid_step: sampling needs one output row per request");
    if (sc->greedy) {
        hipLaunchKernelGGL(k_hb_argmax, dim3(n_req), dim3(1024), 0, st, io->logits, c.vocab, io->out_ids);
        if (feedback || io->rng_offset)
            hipLaunchKernelGGL(k_hb_feedback, dim3((n_req + 63) / 64), dim3(64), 0, st, io->out_ids, io->input_ids, io->rng_offset, n_req,
                               feedback && io->input_ids ? 1 : 0);
        return VOX_OK;
    }
    // stochastic modes: the library's sampler (bf16 logits, Philox stream keyed by seed and the engine's step counter)
    const long nl = (long)n_req * c.vocab;
    hipLaunchKernelGGL(k_hb_logits_bf16, dim3((unsigned)((nl + 255) / 256)), dim3(256), 0, st, io->logits, m->logits16, nl);
    SampleCall s;
    s.logits = m->logits16; s.B = n_req; s.V = c.vocab; s.cfg = *sc; s.cfg.repetition_penalty = 1.0f; s.seed = seed; s.offset = 0;
    s.offset_dev = io->rng_offset; s.offset_mul = 1; s.out_ids = io->out_ids; s.out_stride = 1; s.out_col = 0;
    s.ws = m->ctx->samp_ws;
    VOX_TRY(vox_launch_sample(st, s));
    if (feedback || io->rng_offset)
        hipLaunchKernelGGL(k_hb_feedback, dim3((n_req + 63) / 64), dim3(64), 0, st, io->out_ids, io->input_ids, io->rng_offset, n_req,
                           feedback && io->input_ids ? 1 : 0);
    return VOX_OK;
}

}  // extern "C"
