// Several residual streams ("hyper-connections") and the token embedding with a hashed pair table.
//
// Streams: the residual state of a token is S float32 rows x_0 .. x_(S-1) of width d, laid out [S, T, d].
// A sublayer reads u = sum_s in[s] x_s and, when its result y is there, every stream is rewritten from the old ones:
//     x_t <- sum_s mix[s, t] x_s + out[t] y.
// ic_hc_step does the write that the sublayer before still owes (optional), the read for the next sublayer
// (optional) and the RMS norm of what was read (optional), one block per token, the row read once.
//
// Pair table: beside table[token] the embedding adds pair[(prev * mul_prev + token * mul_cur) mod buckets], where prev
// is the token before in the same sequence; the first token of a sequence takes row `buckets`.  The token before
// a step's first one is kept per sequence in an int32 state.
#include "common.h"

constexpr int kHcMaxStreams = 8;

// four consecutive values as floats
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16* p) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    return float4{bf16_bits_to_f32((uint16_t)(v.x & 0xffff)), bf16_bits_to_f32((uint16_t)(v.x >> 16)),
                  bf16_bits_to_f32((uint16_t)(v.y & 0xffff)), bf16_bits_to_f32((uint16_t)(v.y >> 16))};
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16* p, float4 v) {
    uint2 o;
    o.x = (uint32_t)f32_to_bf16_bits(v.x) | ((uint32_t)f32_to_bf16_bits(v.y) << 16);
    o.y = (uint32_t)f32_to_bf16_bits(v.z) | ((uint32_t)f32_to_bf16_bits(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = o;
}

__global__ void pair_rows_kernel(const int* __restrict__ tokens, const int* __restrict__ positions,
                                 const int* __restrict__ token_req, const int* __restrict__ state_slots,
                                 const int* __restrict__ prev_state, int* __restrict__ rows, int T, long long buckets,
                                 long long mul_prev, long long mul_cur) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= T) return;
    if (positions[t] == 0) {
        rows[t] = (int)buckets;
        return;
    }
    const int r = token_req[t];
    const bool first = t == 0 || token_req[t - 1] != r;
    const long long prev = first ? prev_state[state_slots[r]] : tokens[t - 1];
    rows[t] = (int)((prev * mul_prev + (long long)tokens[t] * mul_cur) % buckets);
}

IC_EXPORT int ic_pair_rows(const int* tokens, const int* positions, const int* token_req, const int* state_slots,
                           const int* prev_state, int* rows, int T, int buckets, int mul_prev, int mul_cur,
                           hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (buckets <= 0 || mul_prev < 0 || mul_cur < 0) return IC_ERR_ARG;
    hipLaunchKernelGGL(pair_rows_kernel, dim3((T + 255) / 256), dim3(256), 0, stream, tokens, positions, token_req,
                       state_slots, prev_state, rows, T, (long long)buckets, (long long)mul_prev, (long long)mul_cur);
    return ic_launch_status();
}

// out[s, t, :] = table[tokens[t]] + pair[rows[t]] for every stream s; the last token of every request's share
// of the step becomes the request's remembered token.
template <typename T>
__global__ void __launch_bounds__(256)
embed_streams_kernel(const int* __restrict__ tokens, const int* __restrict__ rows, const T* __restrict__ table,
                     const T* __restrict__ pair, float* __restrict__ out, int n_streams, int n_tokens, int d,
                     const int* __restrict__ token_req, const int* __restrict__ state_slots,
                     int* __restrict__ prev_state) {
    const int t = blockIdx.x;
    const int tok = tokens[t];
    const T* e = table + (size_t)tok * d;
    const T* p = pair ? pair + (size_t)rows[t] * d : nullptr;
    if (d % 4 == 0) {
#pragma unroll 4
        for (int j = 4 * threadIdx.x; j < d; j += 4 * blockDim.x) {
            float4 v = load4(e + j);
            if (p) {
                const float4 w = load4(p + j);
                v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
            }
            for (int s = 0; s < n_streams; ++s) store4(out + ((size_t)s * n_tokens + t) * d + j, v);
        }
    } else {
        for (int j = threadIdx.x; j < d; j += blockDim.x) {
            float v = to_f32(e[j]);
            if (p) v += to_f32(p[j]);
            for (int s = 0; s < n_streams; ++s) out[((size_t)s * n_tokens + t) * d + j] = v;
        }
    }
    if (prev_state && threadIdx.x == 0) {
        const int r = token_req[t];
        if (t == n_tokens - 1 || token_req[t + 1] != r) prev_state[state_slots[r]] = tok;
    }
}

IC_EXPORT int ic_embed_streams(const int* tokens, const int* rows, const void* table, const void* pair, int dtype,
                               float* out, int n_streams, int T, int d, const int* token_req, const int* state_slots,
                               int* prev_state, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (n_streams <= 0 || d <= 0 || (pair && !rows) || (prev_state && (!token_req || !state_slots))) return IC_ERR_ARG;
    if (dtype == IC_F32)
        hipLaunchKernelGGL(embed_streams_kernel<float>, dim3(T), dim3(256), 0, stream, tokens, rows, (const float*)table,
                           (const float*)pair, out, n_streams, T, d, token_req, state_slots, prev_state);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(embed_streams_kernel<bf16>, dim3(T), dim3(256), 0, stream, tokens, rows, (const bf16*)table,
                           (const bf16*)pair, out, n_streams, T, d, token_req, state_slots, prev_state);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// One block per token.  y (nullable): the write owed, with mix [S, S] indexed [from, to] and out_w [S].
// in_w (nullable): the read u = sum_s in_w[s] x_s; norm_w (nullable): h = u * rsqrt(mean(u^2) + eps) * norm_w,
// else h = u.  h is TH (the compute dtype, or float32 for a plain sum).
template <int S, typename TY, typename TH>
__global__ void __launch_bounds__(256)
hc_step_kernel(float* __restrict__ x, int n_tokens, int d, const TY* __restrict__ y,
               const float* __restrict__ mix, const float* __restrict__ out_w, const float* __restrict__ in_w,
               const float* __restrict__ norm_w, float eps, TH* __restrict__ h) {
    extern __shared__ float u_row[];          // d floats
    __shared__ float red[8];
    const int t = blockIdx.x;
    float m[S * S], ow[S], iw[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        ow[s] = y ? out_w[s] : 0.f;
        iw[s] = in_w ? in_w[s] : 0.f;
#pragma unroll
        for (int q = 0; q < S; ++q) m[s * S + q] = y ? mix[s * S + q] : 0.f;
    }
    float ss = 0.f;
    const int width = (d % 4 == 0) ? 4 : 1;          // four columns per thread and round where rows allow 16-byte accesses
#pragma unroll 2
    for (int j0 = width * threadIdx.x; j0 < d; j0 += width * blockDim.x) {
        float xs[S][4], yv[4] = {0.f, 0.f, 0.f, 0.f};
        if (width == 4) {
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const float4 v = load4(x + ((size_t)s * n_tokens + t) * d + j0);
                xs[s][0] = v.x; xs[s][1] = v.y; xs[s][2] = v.z; xs[s][3] = v.w;
            }
            if (y) {
                const float4 v = load4(y + (size_t)t * d + j0);
                yv[0] = v.x; yv[1] = v.y; yv[2] = v.z; yv[3] = v.w;
            }
        } else {
#pragma unroll
            for (int s = 0; s < S; ++s) xs[s][0] = x[((size_t)s * n_tokens + t) * d + j0];
            if (y) yv[0] = to_f32(y[(size_t)t * d + j0]);
        }
        if (y) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (e >= width) break;
                float nx[S];
#pragma unroll
                for (int q = 0; q < S; ++q) {
                    float a = 0.f;
#pragma unroll
                    for (int s = 0; s < S; ++s) a += m[s * S + q] * xs[s][e];
                    nx[q] = a + ow[q] * yv[e];
                }
#pragma unroll
                for (int q = 0; q < S; ++q) xs[q][e] = nx[q];
            }
#pragma unroll
            for (int q = 0; q < S; ++q) {
                float* dst = x + ((size_t)q * n_tokens + t) * d + j0;
                if (width == 4) store4(dst, float4{xs[q][0], xs[q][1], xs[q][2], xs[q][3]});
                else dst[0] = xs[q][0];
            }
        }
        if (in_w) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (e >= width) break;
                float u = 0.f;
#pragma unroll
                for (int s = 0; s < S; ++s) u += iw[s] * xs[s][e];
                u_row[j0 + e] = u;
                ss += u * u;
            }
        }
    }
    if (!in_w) return;
    float r = 1.f;
    if (norm_w) r = 1.0f / sqrtf(block_sum(ss, red) / (float)d + eps);
    if (width == 4) {
#pragma unroll 2
        for (int j0 = 4 * threadIdx.x; j0 < d; j0 += 4 * blockDim.x) {     // a thread reads back what it wrote itself
            float4 u = *reinterpret_cast<const float4*>(u_row + j0);
            if (norm_w) {
                const float4 w = load4(norm_w + j0);
                u = float4{u.x * r * w.x, u.y * r * w.y, u.z * r * w.z, u.w * r * w.w};
            }
            store4(h + (size_t)t * d + j0, u);
        }
    } else {
        for (int j = threadIdx.x; j < d; j += blockDim.x) {
            const float u = u_row[j];
            h[(size_t)t * d + j] = from_f32<TH>(norm_w ? u * r * norm_w[j] : u);
        }
    }
}

template <typename TY, typename TH>
static void hc_launch(float* x, int S, int T, int d, const void* y, const float* mix, const float* out_w,
                      const float* in_w, const float* norm_w, float eps, void* h, hipStream_t stream) {
    const size_t lds = (size_t)d * sizeof(float);
#define IC_HC(N)                                                                                                  \
    case N:                                                                                                       \
        hipLaunchKernelGGL((hc_step_kernel<N, TY, TH>), dim3(T), dim3(256), lds, stream, x, T, d, (const TY*)y, mix, \
                           out_w, in_w, norm_w, eps, (TH*)h);                                                     \
        break;
    switch (S) { IC_HC(1) IC_HC(2) IC_HC(3) IC_HC(4) IC_HC(5) IC_HC(6) IC_HC(7) IC_HC(8) }
#undef IC_HC
}

IC_EXPORT int ic_hc_step(float* x, int S, int T, int d, const void* y, int y_dtype, const float* mix,
                         const float* out_w, const float* in_w, const float* norm_w, float eps, void* h, int h_dtype,
                         hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (S <= 0 || S > kHcMaxStreams || d <= 0 || d > 16128 || (y && (!mix || !out_w)) || (in_w && !h)) return IC_ERR_ARG;
    const int yd = y ? y_dtype : (h_dtype == IC_F32 ? IC_F32 : IC_BF16);
    if (yd == IC_F32 && h_dtype == IC_F32) hc_launch<float, float>(x, S, T, d, y, mix, out_w, in_w, norm_w, eps, h, stream);
    else if (yd == IC_BF16 && h_dtype == IC_BF16) hc_launch<bf16, bf16>(x, S, T, d, y, mix, out_w, in_w, norm_w, eps, h, stream);
    else if (yd == IC_BF16 && h_dtype == IC_F32) hc_launch<bf16, float>(x, S, T, d, y, mix, out_w, in_w, norm_w, eps, h, stream);
    else return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}
