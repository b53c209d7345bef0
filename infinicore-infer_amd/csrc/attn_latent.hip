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

// ---- the same walk on the matrix cores (bfloat16) --------------------------------------------------------------------
// One block per (token, group of up to 32 heads, split of the keys); the heads are the 32 "queries" of
// v_mfma_f32_32x32x16_bf16.  A step of 32 keys is loaded once into LDS as padded rows.  Scores are computed
// transposed, S^T = K Q^T (A = 32 key rows x 16 values out of LDS, B = the heads' queries, held in registers), so a
// lane holds 16 keys of ONE head, its partner lane (l ^ 32) the other 16, and the probabilities are already the B
// operand of O^T = V^T P^T, whose A operand (the first R values of the same LDS rows, transposed) comes out of LDS
// through the transposing read.  Operand layout (lane l, h = l / 32): A[i = l % 32][k = 8h..8h+7],
// B[k = 8h..8h+7][j = l % 32], D[i = 8(r / 4) + 4h + r % 4][j = l % 32] for the 16 accumulators r.
// A key beyond the token's position is replaced by the position's own row when loaded, and masked.
typedef __bf16 lat_bf16x8 __attribute__((ext_vector_type(8)));
typedef float lat_v16f __attribute__((ext_vector_type(16)));
typedef float lat_v8f __attribute__((ext_vector_type(8)));
typedef short lat_v4s __attribute__((ext_vector_type(4)));

template <int R, int E>
__global__ void __launch_bounds__(64 * (R >= 128 ? 4 : R / 32))
attn_latent_mfma_kernel(const bf16* __restrict__ qa, int qa_stride, bf16* __restrict__ out, int out_stride,
                        const bf16* __restrict__ cache, const int* __restrict__ block_tables, int bt_stride,
                        const int* __restrict__ token_req, const int* __restrict__ positions,
                        const int* __restrict__ row_list, int H, int page_size, float scale, int n_split,
                        float* __restrict__ part_acc, float* __restrict__ part_ml) {
    // The block's waves share a step's rows in LDS; each computes the (same) scores and owns ND / WAVES of the
    // 32-column tiles of the result.
    constexpr int D = R + E, NC = D / 16, ND = R / 32, PK = D + 8, PIECES = D / 8;
    constexpr int WAVES = ND >= 4 ? 4 : ND, NDW = ND / WAVES, THREADS = 64 * WAVES;
    constexpr int NL = (32 * PIECES + THREADS - 1) / THREADS;       // 16-byte pieces of a step a thread loads
    constexpr bool QLDS = NC > 20;         // long rows: the queries wait in LDS (in registers they would halve the waves a unit holds)
    __shared__ __attribute__((aligned(16))) uint16_t Ks[32 * PK];
    __shared__ __attribute__((aligned(16))) uint16_t Qs[QLDS ? 32 * PK : 8];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, lq = lane & 31, half = lane >> 5;
    const int n_groups = (H + 31) / 32;
    const int hg = blockIdx.x % n_groups, split = blockIdx.y;
    const int t = row_list ? row_list[blockIdx.x / n_groups] : blockIdx.x / n_groups;
    const int head = hg * 32 + lq;
    const bool row_ok = head < H;
    const int pos = positions[t];
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;

    lat_bf16x8 qf[QLDS ? 1 : NC];
    {
        const bf16* qp = qa + (size_t)t * qa_stride + (size_t)(row_ok ? head : 0) * D + 8 * half;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            if (QLDS && c % WAVES != wave) continue;          // the waves write the queries' pieces in turn
            uint4 v = *reinterpret_cast<const uint4*>(qp + 16 * c);
            if (!row_ok) v = uint4{0u, 0u, 0u, 0u};
            if (QLDS) *reinterpret_cast<uint4*>(Qs + lq * PK + 16 * c + 8 * half) = v;
            else qf[c] = __builtin_bit_cast(lat_bf16x8, v);
        }
    }
    const int n_steps = pos / 32 + 1;
    const int per = (n_steps + n_split - 1) / n_split;
    const int s_lo = split * per, s_hi = (s_lo + per < n_steps) ? s_lo + per : n_steps;

    lat_v16f oacc[NDW];
#pragma unroll
    for (int i = 0; i < NDW; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m = -INFINITY, l = 0.f;
    const float scale_log2e = scale * 1.4426950408889634f;
    const int vrow = 4 * half + ((lane & 15) >> 2);
    const int vcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    // A step's rows are asked for one step ahead: while this step is computed out of LDS the next one's loads are in flight.
    uint4 got[NL];
    auto fetch = [&](int step) {
        const int kb = 32 * step;
#pragma unroll
        for (int k = 0; k < NL; ++k) {
            const int e = threadIdx.x + THREADS * k;
            if (e < 32 * PIECES) {
                const int row = e / PIECES, piece = e % PIECES;
                const int key = (kb + row < pos) ? kb + row : pos;
                got[k] = *reinterpret_cast<const uint4*>(cache + ((long long)bt[key / page_size] * page_size + key % page_size) * D + piece * 8);
            }
        }
    };
    if (s_lo < s_hi) fetch(s_lo);
    for (int s = s_lo; s < s_hi; ++s) {
        const int kb = 32 * s;
#pragma unroll
        for (int k = 0; k < NL; ++k) {
            const int e = threadIdx.x + THREADS * k;
            if (e < 32 * PIECES) *reinterpret_cast<uint4*>(Ks + (e / PIECES) * PK + (e % PIECES) * 8) = got[k];
        }
        __syncthreads();
        if (s + 1 < s_hi) fetch(s + 1);
        lat_v16f sacc, sacc2;                  // two chains of dependent products instead of one
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[r] = sacc2[r] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const lat_bf16x8 a = *reinterpret_cast<const lat_bf16x8*>(Ks + lq * PK + 16 * c + 8 * half);
            const lat_bf16x8 q = QLDS ? *reinterpret_cast<const lat_bf16x8*>(Qs + lq * PK + 16 * c + 8 * half) : qf[c];
            if (c & 1) sacc2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, q, sacc2, 0, 0, 0);
            else sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, q, sacc, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[r] += sacc2[r];
        if (kb + 31 > pos) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (kb + 8 * (r >> 2) + 4 * half + (r & 3) > pos) sacc[r] = -INFINITY;
        }
        float mloc = sacc[0];
#pragma unroll
        for (int r = 1; r < 16; ++r) mloc = fmaxf(mloc, sacc[r]);
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave));
        const float m_new = fmaxf(m, mloc);                     // finite: the step's first key is visible
        const float mc = m_new * scale_log2e;
        const float corr = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m * scale_log2e - mc);
        float rs = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float p = __builtin_amdgcn_exp2f(fmaf(sacc[r], scale_log2e, -mc));
            sacc[r] = p;
            rs += p;
        }
        rs += __shfl_xor(rs, 32, kWave);
        l = l * corr + rs;
        m = m_new;
#pragma unroll
        for (int i = 0; i < NDW; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] *= corr;
#pragma unroll
        for (int kc = 0; kc < 2; ++kc) {
            lat_v8f pf;
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = sacc[8 * kc + e];
            const lat_bf16x8 b = __builtin_convertvector(pf, lat_bf16x8);
#pragma unroll
            for (int dt = 0; dt < NDW; ++dt) {
                const uint16_t* vp = Ks + (16 * kc + vrow) * PK + 32 * (wave * NDW + dt) + vcol;
                const lat_v4s lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lat_v4s __attribute__((address_space(3)))*)vp);
                const lat_v4s hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lat_v4s __attribute__((address_space(3)))*)(vp + 8 * PK));
                const lat_bf16x8 a = __builtin_bit_cast(lat_bf16x8, __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
                oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, oacc[dt], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    if (!row_ok) return;
    if (n_split == 1) {
        const float inv = 1.0f / l;
        bf16* op = out + (size_t)t * out_stride + (size_t)head * R + 32 * wave * NDW;
#pragma unroll
        for (int dt = 0; dt < NDW; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) op[32 * dt + 8 * (r >> 2) + 4 * half + (r & 3)] = __float2bfloat16(oacc[dt][r] * inv);
    } else {
        const size_t pi = ((size_t)t * H + head) * n_split + split;
        if (half == 0 && wave == 0) { part_ml[2 * pi] = m * scale; part_ml[2 * pi + 1] = l; }
#pragma unroll
        for (int dt = 0; dt < NDW; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                part_acc[pi * R + 32 * (wave * NDW + dt) + 8 * (r >> 2) + 4 * half + (r & 3)] = oacc[dt][r];
    }
}

template <int R, int E>
static void latent_mfma_launch(dim3 grid, hipStream_t stream, const void* qa, int qa_stride, void* out, int out_stride,
                               const void* cache, const int* block_tables, int bt_stride, const int* token_req,
                               const int* positions, const int* row_list, int H, int page_size, float scale, int n_split,
                               float* part_acc, float* part_ml) {
    hipLaunchKernelGGL((attn_latent_mfma_kernel<R, E>), grid, dim3(64 * (R >= 128 ? 4 : R / 32)), 0, stream, (const bf16*)qa, qa_stride, (bf16*)out,
                       out_stride, (const bf16*)cache, block_tables, bt_stride, token_req, positions, row_list, H, page_size,
                       scale, n_split, part_acc, part_ml);
}

// Sizes the matrix-core walk is built for: the latent 64, 128, 256 or 512 wide, the rotated part 16, 32 or 64.
IC_EXPORT int ic_attn_latent_on_matrix_cores(int dtype, int R, int E) {
    return dtype == IC_BF16 && (R == 64 || R == 128 || R == 256 || R == 512) && (E == 16 || E == 32 || E == 64);
}

// Merge of the splits: one block per (token, head).
template <typename T>
__global__ void __launch_bounds__(256)
attn_latent_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml, int n_split, int H, int R,
                         T* __restrict__ out, int out_stride, const int* __restrict__ row_list) {
    const int h = blockIdx.x % H, t = row_list ? row_list[blockIdx.x / H] : blockIdx.x / H;
    const size_t p0 = ((size_t)t * H + h) * n_split;
    __shared__ float wgt[64];                 // a split's share of the result: exp(m_s - m) / l
    if (threadIdx.x < 64) {
        const int sp = threadIdx.x;
        const float ms = sp < n_split ? part_ml[2 * (p0 + sp)] : -INFINITY;
        const float ls = sp < n_split ? part_ml[2 * (p0 + sp) + 1] : 0.f;
        const float m = wave_max(ms);
        const float e = ms > -INFINITY ? expf(ms - m) : 0.f;
        const float l = wave_sum(ls * e);
        wgt[sp] = e / l;
    }
    __syncthreads();
    for (int j = threadIdx.x; j < R; j += blockDim.x) {
        float a = 0.f;
#pragma unroll 4
        for (int sp = 0; sp < n_split; ++sp) a += part_acc[(p0 + sp) * R + j] * wgt[sp];     // (an empty split left zeros)
        out[(size_t)t * out_stride + (size_t)h * R + j] = from_f32<T>(a);
    }
}

IC_EXPORT int ic_attn_latent(const void* qa, int qa_stride, void* out, int out_stride, int dtype, const void* cache,
                             const int* block_tables, int bt_stride, const int* token_req, const int* positions,
                             const int* row_list, int T, int H, int R, int E, int page_size, float scale, int n_split,
                             float* part_acc, float* part_ml, int force_vector, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (H <= 0 || R <= 0 || R > kLatentMaxRank || E < 0 || page_size <= 0 || n_split < 1 || n_split > 64) return IC_ERR_ARG;
    if (n_split > 1 && (!part_acc || !part_ml)) return IC_ERR_ARG;
    const int D = R + E;
    const size_t lds = (size_t)kLatentHeads * D * sizeof(float);
    if (lds > 60 * 1024) return IC_ERR_TOO_LARGE;
    if (ic_attn_latent_on_matrix_cores(dtype, R, E) && scale > 0.f && !force_vector) {
        const int wide_groups = (H + 31) / 32;
        if ((long long)T * wide_groups > 0x7fffffffLL) return IC_ERR_ARG;
        dim3 wide((unsigned)(T * wide_groups), n_split);
#define IC_LATM(RR, EE)                                                                                                  \
    if (R == RR && E == EE)                                                                                              \
        latent_mfma_launch<RR, EE>(wide, stream, qa, qa_stride, out, out_stride, cache, block_tables, bt_stride, token_req, \
                                   positions, row_list, H, page_size, scale, n_split, part_acc, part_ml);
        IC_LATM(64, 16) IC_LATM(64, 32) IC_LATM(64, 64) IC_LATM(128, 16) IC_LATM(128, 32) IC_LATM(128, 64)
        IC_LATM(256, 16) IC_LATM(256, 32) IC_LATM(256, 64) IC_LATM(512, 16) IC_LATM(512, 32) IC_LATM(512, 64)
#undef IC_LATM
        if (n_split > 1)
            hipLaunchKernelGGL(attn_latent_merge_kernel<bf16>, dim3(T * H), dim3(256), 0, stream, part_acc, part_ml, n_split, H,
                               R, (bf16*)out, out_stride, row_list);
        return ic_launch_status();
    }
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
    // blockIdx.y == 0: 64 keys' rows as they are; blockIdx.y = 1 + i: columns 64 i .. 64 i + 63 of the same keys, transposed
    __shared__ T tile[64][65];
    const int j0 = blockIdx.x * 64, lane = threadIdx.x % 64, w = threadIdx.x / 64;
    if (blockIdx.y == 0) {
        for (int jj = w; jj < 64; jj += 4) {
            const int j = j0 + jj;
            if (j >= L_pad) break;
            const T* src = j < L ? cache + ((long long)table[j / page_size] * page_size + j % page_size) * D : nullptr;
            for (int c = lane; c < D; c += 64) rows[(size_t)j * D + c] = src ? src[c] : from_f32<T>(0.f);
        }
        return;
    }
    const int c0 = 64 * (blockIdx.y - 1);
    for (int jj = w; jj < 64; jj += 4) {
        const int j = j0 + jj, c = c0 + lane;
        T v = from_f32<T>(0.f);
        if (j < L && c < R) v = cache[((long long)table[j / page_size] * page_size + j % page_size) * D + c];
        tile[jj][lane] = v;
    }
    __syncthreads();
    for (int cc = w; cc < 64; cc += 4) {
        const int c = c0 + cc, j = j0 + lane;
        if (c < R && j < L_pad) rows_t[(size_t)c * L_pad + j] = tile[lane][cc];
    }
}

IC_EXPORT int ic_latent_gather(const void* cache, int dtype, const int* table, int page_size, int D, int R, int L, int L_pad,
                               void* rows, void* rows_t, hipStream_t stream) {
    if (L <= 0) return IC_OK;
    if (page_size <= 0 || D <= 0 || R <= 0 || R > D || L_pad < L) return IC_ERR_ARG;
    dim3 grid((L_pad + 63) / 64, 1 + (R + 63) / 64), block(256);
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
    T* out = p + (size_t)m * ldp;
    if (n_cols <= 16 * 256) {                 // the row is read once and waits in registers
        float v[16];
        float mx = -INFINITY;
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const int j = threadIdx.x + 256 * k;
            v[k] = j < n ? row[j] : -INFINITY;
            mx = fmaxf(mx, v[k]);
        }
        mx = block_max(mx, red) * scale;
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            v[k] = expf(v[k] * scale - mx);       // exp(-inf) = 0 beyond the visible keys
            sum += v[k];
        }
        const float inv = 1.0f / block_sum(sum, red);
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const int j = threadIdx.x + 256 * k;
            if (j < n_cols) out[j] = from_f32<T>(v[k] * inv);
        }
        return;
    }
    float mx = -INFINITY;
    for (int j = threadIdx.x; j < n; j += blockDim.x) mx = fmaxf(mx, row[j]);
    mx = block_max(mx, red) * scale;
    float sum = 0.f;
    for (int j = threadIdx.x; j < n; j += blockDim.x) sum += expf(row[j] * scale - mx);
    const float inv = 1.0f / block_sum(sum, red);
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
