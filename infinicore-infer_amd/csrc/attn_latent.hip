// Attention through a latent: what is cached per token is ONE row [c | k_rot] of R + E values, shared by all
// heads: c (R values) is the normed latent that keys and values are made from, k_rot (E values) the rotated key
// part.  A head's key is W_uk c and its value W_uv c, so with q' = W_uk^T q_plain the score is
//     s = scale * (q' . c + q_rot . k_rot)
// and the head's result is W_uv (sum_j p_j c_j): the kernels here walk the latent rows only, every head against
// the same rows, and leave the two small products per head to the caller.
//
// Cache plane: [pages, 1, page_size, R + E].  Rotation: entries (2i, 2i+1) of the first `rot_dims` entries of a
// rotated part turn by the angle position * freq[i]; the rest pass unchanged.  Angles, scores and the running
// softmax are float32.
#include "common.h"

constexpr int kLatentMaxRank = 512;    // R: a lane holds R / 64 sums per head
constexpr int kLatentHeads = 4;        // heads that share one walk over the rows

// ---- per token: the query latent's norm, the key latent's norm, the rotated key part, the cache write -----------
// row[t] = [dq: Rq | dkv: R + E | ...].  cq[t] = rms(dq) * qn_w; cache[slot] = [rms(dkv[:R]) * kvn_w | rot(dkv[R:])].
template <typename T>
__global__ void __launch_bounds__(256)
latent_prep_kernel(const T* __restrict__ rows, int ld, int Rq, int R, int E, const float* __restrict__ qn_w,
                   const float* __restrict__ kvn_w, float eps, const float* __restrict__ freq, int rot_dims,
                   const int* __restrict__ positions, T* __restrict__ cq, T* __restrict__ cache,
                   const int* __restrict__ slots) {
    __shared__ float red[8];
    const int t = blockIdx.x;
    const T* row = rows + (size_t)t * ld;
    float ss = 0.f;
    for (int j = threadIdx.x; j < Rq; j += blockDim.x) {
        const float v = to_f32(row[j]);
        ss += v * v;
    }
    float r = 1.0f / sqrtf(block_sum(ss, red) / (float)Rq + eps);
    for (int j = threadIdx.x; j < Rq; j += blockDim.x) cq[(size_t)t * Rq + j] = from_f32<T>(to_f32(row[j]) * r * qn_w[j]);
    if (!slots) return;
    const T* kv = row + Rq;
    T* dst = cache + (size_t)slots[t] * (R + E);
    ss = 0.f;
    for (int j = threadIdx.x; j < R; j += blockDim.x) {
        const float v = to_f32(kv[j]);
        ss += v * v;
    }
    r = 1.0f / sqrtf(block_sum(ss, red) / (float)R + eps);
    for (int j = threadIdx.x; j < R; j += blockDim.x) dst[j] = from_f32<T>(to_f32(kv[j]) * r * kvn_w[j]);
    const float pos = (float)positions[t];
    for (int i = threadIdx.x; i < rot_dims / 2; i += blockDim.x) {
        const float a = pos * freq[i];
        const float c = cosf(a), s = sinf(a);
        const float u = to_f32(kv[R + 2 * i]), v = to_f32(kv[R + 2 * i + 1]);
        dst[R + 2 * i] = from_f32<T>(u * c - v * s);
        dst[R + 2 * i + 1] = from_f32<T>(v * c + u * s);
    }
    for (int j = rot_dims + threadIdx.x; j < E; j += blockDim.x) dst[R + j] = kv[R + j];
}

IC_EXPORT int ic_latent_prep(const void* rows, int ld, int dtype, int Rq, int R, int E, const float* qn_w,
                             const float* kvn_w, float eps, const float* freq, int rot_dims, const int* positions,
                             void* cq, void* cache, const int* slots, int T, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (Rq <= 0 || R <= 0 || E < 0 || rot_dims < 0 || rot_dims > E || rot_dims % 2) return IC_ERR_ARG;
    if (dtype == IC_F32)
        hipLaunchKernelGGL(latent_prep_kernel<float>, dim3(T), dim3(256), 0, stream, (const float*)rows, ld, Rq, R, E, qn_w,
                           kvn_w, eps, freq, rot_dims, positions, (float*)cq, (float*)cache, slots);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(latent_prep_kernel<bf16>, dim3(T), dim3(256), 0, stream, (const bf16*)rows, ld, Rq, R, E, qn_w,
                           kvn_w, eps, freq, rot_dims, positions, (bf16*)cq, (bf16*)cache, slots);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---- the queries' rotated parts: q[t, h, dim:dim+E] rotated into qa[t, h, R:R+E] -----------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
latent_q_rotate_kernel(const T* __restrict__ q, int q_stride, int dim, int E, int R, int H, const float* __restrict__ freq,
                       int rot_dims, const int* __restrict__ positions, T* __restrict__ qa, int qa_stride) {
    const int t = blockIdx.x;
    const float pos = (float)positions[t];
    const int half = rot_dims / 2, rest = E - rot_dims, per = half + rest;
    for (int e = threadIdx.x; e < H * per; e += blockDim.x) {
        const int h = e / per, i = e % per;
        const T* src = q + (size_t)t * q_stride + (size_t)h * (dim + E) + dim;
        T* dst = qa + (size_t)t * qa_stride + (size_t)h * (R + E) + R;
        if (i < half) {
            const float a = pos * freq[i];
            const float c = cosf(a), s = sinf(a);
            const float u = to_f32(src[2 * i]), v = to_f32(src[2 * i + 1]);
            dst[2 * i] = from_f32<T>(u * c - v * s);
            dst[2 * i + 1] = from_f32<T>(v * c + u * s);
        } else {
            dst[rot_dims + i - half] = src[rot_dims + i - half];
        }
    }
}

IC_EXPORT int ic_latent_q_rotate(const void* q, int q_stride, int dtype, int dim, int E, int R, int H, const float* freq,
                                 int rot_dims, const int* positions, void* qa, int qa_stride, int T, hipStream_t stream) {
    if (T <= 0 || E == 0) return IC_OK;
    if (dim < 0 || E < 0 || R <= 0 || H <= 0 || rot_dims < 0 || rot_dims > E || rot_dims % 2) return IC_ERR_ARG;
    if (dtype == IC_F32)
        hipLaunchKernelGGL(latent_q_rotate_kernel<float>, dim3(T), dim3(256), 0, stream, (const float*)q, q_stride, dim, E,
                           R, H, freq, rot_dims, positions, (float*)qa, qa_stride);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(latent_q_rotate_kernel<bf16>, dim3(T), dim3(256), 0, stream, (const bf16*)q, q_stride, dim, E, R,
                           H, freq, rot_dims, positions, (bf16*)qa, qa_stride);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---- the walk over the latent rows ----------------------------------------------------------------------------------
// One wave per (token, group of up to kLatentHeads heads, split of the keys).  Scores: a lane owns one of 64 keys
// and reads its row in pieces of VEC values (16 bytes where the sizes allow), against the queries in LDS.
// Weighted sum: a lane owns pieces of the R columns and reads every key's row there.  With n_split > 1 each split
// leaves (max, sum, unnormalised row) in scratch memory and ic_attn_latent_merge finishes.
template <typename T, int VEC>
__global__ void __launch_bounds__(64)
attn_latent_kernel(const T* __restrict__ qa, int qa_stride, T* __restrict__ out, int out_stride,
                   const T* __restrict__ cache, const int* __restrict__ block_tables, int bt_stride,
                   const int* __restrict__ token_req, const int* __restrict__ positions,
                   const int* __restrict__ row_list, int H, int R, int E,
                   int page_size, float scale, int n_split, float* __restrict__ part_acc, float* __restrict__ part_ml) {
    constexpr int HG = kLatentHeads, NP = kLatentMaxRank / 64 / VEC;   // pieces of VEC columns a lane owns
    extern __shared__ float qs[];                 // HG * (R + E) floats
    __shared__ float ps[HG][64];
    __shared__ long long krow[64];
    const int D = R + E, lane = threadIdx.x;
    const int n_groups = (H + HG - 1) / HG;
    const int hg = blockIdx.x % n_groups, split = blockIdx.y;
    const int t = row_list ? row_list[blockIdx.x / n_groups] : blockIdx.x / n_groups;
    const int h0 = hg * HG, nh = (H - h0 < HG) ? H - h0 : HG;
    const int pos = positions[t];
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;
    for (int e = lane; e < HG * D; e += 64) {
        const int g = e / D, d = e % D;
        qs[e] = g < nh ? to_f32(qa[(size_t)t * qa_stride + (size_t)(h0 + g) * D + d]) : 0.f;
    }
    __syncthreads();
    // this split's share of the keys 0..pos, in whole chunks of 64
    const int n_chunks = (pos + 64) / 64;
    const int per = (n_chunks + n_split - 1) / n_split;
    const int c_lo = split * per, c_hi = (c_lo + per < n_chunks) ? c_lo + per : n_chunks;

    float acc[HG][NP][VEC];
#pragma unroll
    for (int g = 0; g < HG; ++g)
#pragma unroll
        for (int i = 0; i < NP; ++i)
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[g][i][v] = 0.f;
    float m[HG], l[HG];
#pragma unroll
    for (int g = 0; g < HG; ++g) { m[g] = -INFINITY; l[g] = 0.f; }

    for (int ch = c_lo; ch < c_hi; ++ch) {
        const int key = ch * 64 + lane;
        const bool valid = key <= pos;
        float s[HG];
#pragma unroll
        for (int g = 0; g < HG; ++g) s[g] = 0.f;
        long long base = 0;
        if (valid) {
            base = ((long long)bt[key / page_size] * page_size + key % page_size) * D;
            const T* kp = cache + base;
            for (int d = 0; d < D; d += VEC) {
                alignas(16) T kv[VEC];
                if (VEC == 1) kv[0] = kp[d];
                else *reinterpret_cast<uint4*>(kv) = *reinterpret_cast<const uint4*>(kp + d);
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    const float kf = to_f32(kv[v]);
#pragma unroll
                    for (int g = 0; g < HG; ++g) s[g] += qs[g * D + d + v] * kf;
                }
            }
        }
        float corr[HG];
#pragma unroll
        for (int g = 0; g < HG; ++g) {
            const float sv = valid ? s[g] * scale : -INFINITY;
            const float m_new = fmaxf(m[g], wave_max(sv));      // the chunk's first key is always visible
            const float p = valid ? expf(sv - m_new) : 0.f;
            corr[g] = expf(m[g] - m_new);
            l[g] = l[g] * corr[g] + wave_sum(p);
            m[g] = m_new;
            ps[g][lane] = p;
        }
        krow[lane] = base;
        __syncthreads();
        const int nk = (pos - ch * 64 + 1 < 64) ? pos - ch * 64 + 1 : 64;
#pragma unroll
        for (int g = 0; g < HG; ++g)
#pragma unroll
            for (int i = 0; i < NP; ++i)
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[g][i][v] *= corr[g];
        for (int kk = 0; kk < nk; ++kk) {
            const T* cp = cache + krow[kk];
            float pk[HG];
#pragma unroll
            for (int g = 0; g < HG; ++g) pk[g] = ps[g][kk];
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int col = (lane + 64 * i) * VEC;
                if (col < R) {
                    alignas(16) T cv[VEC];
                    if (VEC == 1) cv[0] = cp[col];
                    else *reinterpret_cast<uint4*>(cv) = *reinterpret_cast<const uint4*>(cp + col);
#pragma unroll
                    for (int v = 0; v < VEC; ++v) {
                        const float cf = to_f32(cv[v]);
#pragma unroll
                        for (int g = 0; g < HG; ++g) acc[g][i][v] += pk[g] * cf;
                    }
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int g = 0; g < HG; ++g) {
        if (g >= nh) continue;
        const int h = h0 + g;
        if (n_split == 1) {
            const float inv = 1.0f / l[g];
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int col = (lane + 64 * i) * VEC;
                if (col < R) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v)
                        out[(size_t)t * out_stride + (size_t)h * R + col + v] = from_f32<T>(acc[g][i][v] * inv);
                }
            }
        } else {
            const size_t pi = ((size_t)t * H + h) * n_split + split;
            if (lane == 0) { part_ml[2 * pi] = m[g]; part_ml[2 * pi + 1] = l[g]; }
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int col = (lane + 64 * i) * VEC;
                if (col < R) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v) part_acc[pi * R + col + v] = acc[g][i][v];
                }
            }
        }
    }
}

// Merge of the splits: one block per (token, head).
template <typename T>
__global__ void __launch_bounds__(256)
attn_latent_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml, int n_split, int H, int R,
                         T* __restrict__ out, int out_stride, const int* __restrict__ row_list) {
    const int h = blockIdx.x % H, t = row_list ? row_list[blockIdx.x / H] : blockIdx.x / H;
    const size_t p0 = ((size_t)t * H + h) * n_split;
    float m = -INFINITY;
    for (int s = 0; s < n_split; ++s) m = fmaxf(m, part_ml[2 * (p0 + s)]);
    float l = 0.f;
    for (int s = 0; s < n_split; ++s) {
        const float ms = part_ml[2 * (p0 + s)];
        if (ms > -INFINITY) l += part_ml[2 * (p0 + s) + 1] * expf(ms - m);
    }
    const float inv = 1.0f / l;
    for (int j = threadIdx.x; j < R; j += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < n_split; ++s) {
            const float ms = part_ml[2 * (p0 + s)];
            if (ms > -INFINITY) a += part_acc[(p0 + s) * R + j] * expf(ms - m);
        }
        out[(size_t)t * out_stride + (size_t)h * R + j] = from_f32<T>(a * inv);
    }
}

IC_EXPORT int ic_attn_latent(const void* qa, int qa_stride, void* out, int out_stride, int dtype, const void* cache,
                             const int* block_tables, int bt_stride, const int* token_req, const int* positions,
                             const int* row_list, int T, int H, int R, int E, int page_size, float scale, int n_split,
                             float* part_acc, float* part_ml, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (H <= 0 || R <= 0 || R > kLatentMaxRank || E < 0 || page_size <= 0 || n_split < 1 || n_split > 64) return IC_ERR_ARG;
    if (n_split > 1 && (!part_acc || !part_ml)) return IC_ERR_ARG;
    const int D = R + E;
    const size_t lds = (size_t)kLatentHeads * D * sizeof(float);
    if (lds > 60 * 1024) return IC_ERR_TOO_LARGE;
    const int n_groups = (H + kLatentHeads - 1) / kLatentHeads;
    if ((long long)T * n_groups > 0x7fffffffLL) return IC_ERR_ARG;
    dim3 grid((unsigned)(T * n_groups), n_split), block(64);
#define IC_LAT(TT, VV)                                                                                                 \
    hipLaunchKernelGGL((attn_latent_kernel<TT, VV>), grid, block, lds, stream, (const TT*)qa, qa_stride, (TT*)out,     \
                       out_stride, (const TT*)cache, block_tables, bt_stride, token_req, positions, row_list, H, R, E,  \
                       page_size, scale, n_split, part_acc, part_ml)
    if (dtype == IC_F32) {
        if (R % 4 == 0 && E % 4 == 0) IC_LAT(float, 4); else IC_LAT(float, 1);
    } else if (dtype == IC_BF16) {
        if (R % 8 == 0 && E % 8 == 0) IC_LAT(bf16, 8); else IC_LAT(bf16, 1);
    } else
        return IC_ERR_UNSUPPORTED;
#undef IC_LAT
    if (n_split > 1) {
        if (dtype == IC_F32)
            hipLaunchKernelGGL(attn_latent_merge_kernel<float>, dim3(T * H), dim3(256), 0, stream, part_acc, part_ml, n_split,
                               H, R, (float*)out, out_stride, row_list);
        else
            hipLaunchKernelGGL(attn_latent_merge_kernel<bf16>, dim3(T * H), dim3(256), 0, stream, part_acc, part_ml, n_split,
                               H, R, (bf16*)out, out_stride, row_list);
    }
    return ic_launch_status();
}

// ---- prompt portions through matrix products -------------------------------------------------------------------------
// For a portion of several tokens the walk is two products over all heads at once, rows = (token, head):
// scores = Q' C^T and result = P C[:, :R].  The request's latent rows are gathered out of their pages into one
// matrix (and its first R columns transposed, for the second product), the scores pass a masked softmax.

// rows[j] = cache row of key j (j < L), zeros for L <= j < L_pad; rows_t[c, j] = rows[j, c] for c < R.
template <typename T>
__global__ void __launch_bounds__(256)
latent_gather_kernel(const T* __restrict__ cache, const int* __restrict__ table, int page_size, int D, int R, int L,
                     int L_pad, T* __restrict__ rows, T* __restrict__ rows_t) {
    __shared__ T tile[64][65];
    const int j0 = blockIdx.x * 64;
    for (int jj = threadIdx.x / 64; jj < 64; jj += 4) {
        const int j = j0 + jj;
        if (j >= L_pad) break;
        const T* src = j < L ? cache + ((long long)table[j / page_size] * page_size + j % page_size) * D : nullptr;
        for (int c = threadIdx.x % 64; c < D; c += 64) rows[(size_t)j * D + c] = src ? src[c] : from_f32<T>(0.f);
    }
    __syncthreads();
    for (int c0 = 0; c0 < R; c0 += 64) {
        for (int jj = threadIdx.x / 64; jj < 64; jj += 4) {
            const int j = j0 + jj, c = c0 + threadIdx.x % 64;
            tile[jj][threadIdx.x % 64] = (j < L_pad && c < R) ? rows[(size_t)j * D + c] : from_f32<T>(0.f);
        }
        __syncthreads();
        for (int cc = threadIdx.x / 64; cc < 64; cc += 4) {
            const int c = c0 + cc, j = j0 + threadIdx.x % 64;
            if (c < R && j < L_pad) rows_t[(size_t)c * L_pad + j] = tile[threadIdx.x % 64][cc];
        }
        __syncthreads();
    }
}

IC_EXPORT int ic_latent_gather(const void* cache, int dtype, const int* table, int page_size, int D, int R, int L, int L_pad,
                               void* rows, void* rows_t, hipStream_t stream) {
    if (L <= 0) return IC_OK;
    if (page_size <= 0 || D <= 0 || R <= 0 || R > D || L_pad < L) return IC_ERR_ARG;
    dim3 grid((L_pad + 63) / 64), block(256);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(latent_gather_kernel<float>, grid, block, 0, stream, (const float*)cache, table, page_size, D, R, L,
                           L_pad, (float*)rows, (float*)rows_t);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(latent_gather_kernel<bf16>, grid, block, 0, stream, (const bf16*)cache, table, page_size, D, R, L,
                           L_pad, (bf16*)rows, (bf16*)rows_t);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// Row m belongs to token m / H of the portion, which sees keys 0 .. first_limit + m / H.  p = softmax(scale * s) over
// them, zero beyond (up to n_cols).  One block per row; the scores are float32.
template <typename T>
__global__ void __launch_bounds__(256)
latent_softmax_kernel(const float* __restrict__ s, int lds, T* __restrict__ p, int ldp, int H, int n_cols, int first_limit,
                      float scale) {
    __shared__ float red[8];
    const int m = blockIdx.x;
    const int n = min(first_limit + m / H + 1, n_cols);
    const float* row = s + (size_t)m * lds;
    float mx = -INFINITY;
    for (int j = threadIdx.x; j < n; j += blockDim.x) mx = fmaxf(mx, row[j]);
    mx = block_max(mx, red) * scale;
    float sum = 0.f;
    for (int j = threadIdx.x; j < n; j += blockDim.x) sum += expf(row[j] * scale - mx);
    const float inv = 1.0f / block_sum(sum, red);
    T* out = p + (size_t)m * ldp;
    for (int j = threadIdx.x; j < n_cols; j += blockDim.x)
        out[j] = from_f32<T>(j < n ? expf(row[j] * scale - mx) * inv : 0.f);
}

IC_EXPORT int ic_latent_softmax(const float* s, int lds, void* p, int ldp, int dtype, int M, int H, int n_cols,
                                int first_limit, float scale, hipStream_t stream) {
    if (M <= 0) return IC_OK;
    if (H <= 0 || n_cols <= 0 || first_limit < 0 || scale <= 0.f) return IC_ERR_ARG;
    if (dtype == IC_F32)
        hipLaunchKernelGGL(latent_softmax_kernel<float>, dim3(M), dim3(256), 0, stream, s, lds, (float*)p, ldp, H, n_cols,
                           first_limit, scale);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(latent_softmax_kernel<bf16>, dim3(M), dim3(256), 0, stream, s, lds, (bf16*)p, ldp, H, n_cols,
                           first_limit, scale);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}
