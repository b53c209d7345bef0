// Attention over the paged cache for mixers whose keys and values have different sizes per head and
// whose queries see a SPAN of the keys: the last `window` keys (window 0: all earlier keys) plus the
// first `keep_first` keys of the sequence, which are never dropped.  Query at position i sees key j when
//     j <= i  and  (window == 0  or  i - j < window  or  j < keep_first).
// `sink` adds one term exp(0) to the softmax's denominator that has no value:
//     p_j = exp(s_j) / (sink + sum_j exp(s_j)).
// `gate` (nullable): the result is multiplied element by element with sigmoid(gate[t, h * dv + d]).
// Scores, the running softmax and the sums are float32.
//
// Cache layout of one layer: K plane [num_pages, n_kv_heads, page_size, dk], V plane [.., dv].
//
// This file holds the general kernel (any sizes, float32 or bfloat16), which is also the yardstick of
// the tiled ones.
#include "common.h"

constexpr int kSpanMaxDim = 512;

// The visible keys of a query at `pos` as two runs: [0, n_kept) and [lo, pos].
struct SpanRuns {
    int n_kept;   // keys 0 .. n_kept-1 (the kept first keys that lie before the window)
    int lo;       // first key of the window
    int total;    // number of visible keys
};
__device__ __forceinline__ SpanRuns span_runs(int pos, int window, int keep_first) {
    SpanRuns r;
    r.lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    r.n_kept = keep_first < r.lo ? keep_first : r.lo;
    if (r.n_kept < 0) r.n_kept = 0;
    r.total = r.n_kept + (pos - r.lo + 1);
    return r;
}
__device__ __forceinline__ int span_key(const SpanRuns& r, int i) { return i < r.n_kept ? i : r.lo + (i - r.n_kept); }

// One wave per (token, head): walks the visible keys 64 at a time.
template <typename T>
__global__ void __launch_bounds__(64)
attn_span_generic_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
                         const T* __restrict__ gate, int gate_stride,
                         const T* __restrict__ kcache, const T* __restrict__ vcache,
                         const int* __restrict__ block_tables, int bt_stride,
                         const int* __restrict__ token_req, const int* __restrict__ positions,
                         int nh, int nkvh, int dk, int dv, int page_size, float scale, int window, int keep_first,
                         int sink) {
    __shared__ float qs[kSpanMaxDim];
    __shared__ float ps[64];
    __shared__ long long vrow[64];

    const int h = blockIdx.x % nh, t = blockIdx.x / nh, lane = threadIdx.x;
    const int kvh = h / (nh / nkvh);
    const int pos = positions[t];
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;
    const T* qp = q + (size_t)t * q_stride + (size_t)h * dk;
    for (int d = lane; d < dk; d += 64) qs[d] = to_f32(qp[d]);
    __syncthreads();

    const SpanRuns runs = span_runs(pos, window, keep_first);
    const int nd = (dv + 63) / 64;
    float acc[kSpanMaxDim / 64];
#pragma unroll
    for (int i = 0; i < kSpanMaxDim / 64; ++i) acc[i] = 0.f;
    float m = -INFINITY, l = 0.f;

    for (int ib = 0; ib < runs.total; ib += 64) {
        const int idx = ib + lane;
        const bool valid = idx < runs.total;
        float s = -INFINITY;
        long long vbase = 0;
        if (valid) {
            const int key = span_key(runs, idx);
            const int pg = bt[key / page_size];
            const int off = key % page_size;
            const long long rowi = ((long long)pg * nkvh + kvh) * page_size + off;
            vbase = rowi * dv;
            const T* kp = kcache + rowi * dk;
            float dot = 0.f;
            for (int d = 0; d < dk; ++d) dot += qs[d] * to_f32(kp[d]);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));       // lane 0 of every chunk is valid: m_new is finite
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);               // exp(-inf) = 0 on the first chunk
        l = l * corr + wave_sum(p);
        m = m_new;
        __syncthreads();
        ps[lane] = p;
        vrow[lane] = vbase;
        __syncthreads();
        const int nk = (runs.total - ib < 64) ? runs.total - ib : 64;
#pragma unroll
        for (int i = 0; i < kSpanMaxDim / 64; ++i) {
            if (i < nd) {
                const int d = lane + 64 * i;
                float a = acc[i] * corr;
                if (d < dv)
                    for (int kk = 0; kk < nk; ++kk) a += ps[kk] * to_f32(vcache[vrow[kk] + d]);
                acc[i] = a;
            }
        }
    }
    if (sink) {                                           // the term exp(0 - m) joins the denominator
        const float m_new = fmaxf(m, 0.f);
        const float corr = expf(m - m_new);
        l = l * corr + expf(-m_new);
#pragma unroll
        for (int i = 0; i < kSpanMaxDim / 64; ++i) acc[i] *= corr;
    }
    T* op = out + (size_t)t * out_stride + (size_t)h * dv;
    const T* gp = gate ? gate + (size_t)t * gate_stride + (size_t)h * dv : nullptr;
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < kSpanMaxDim / 64; ++i) {
        const int d = lane + 64 * i;
        if (i < nd && d < dv) {
            float o = acc[i] * inv;
            if (gp) o *= 1.0f / (1.0f + expf(-to_f32(gp[d])));
            op[d] = from_f32<T>(o);
        }
    }
}

IC_EXPORT int ic_attn_span_generic(const void* q, int q_stride, void* out, int out_stride, const void* gate,
                                   int gate_stride, int dtype, const void* kcache, const void* vcache,
                                   const int* block_tables, int bt_stride, const int* token_req, const int* positions,
                                   int T, int nh, int nkvh, int dk, int dv, int page_size, float scale, int window,
                                   int keep_first, int sink, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || dk <= 0 || dk > kSpanMaxDim || dv <= 0 || dv > kSpanMaxDim ||
        page_size <= 0 || window < 0 || keep_first < 0)
        return IC_ERR_ARG;
    if ((long long)T * nh > 0x7fffffffLL) return IC_ERR_ARG;
    dim3 grid((unsigned)(T * nh)), block(64);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(attn_span_generic_kernel<float>, grid, block, 0, stream, (const float*)q, q_stride, (float*)out,
                           out_stride, (const float*)gate, gate_stride, (const float*)kcache, (const float*)vcache,
                           block_tables, bt_stride, token_req, positions, nh, nkvh, dk, dv, page_size, scale, window,
                           keep_first, sink);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(attn_span_generic_kernel<bf16>, grid, block, 0, stream, (const bf16*)q, q_stride, (bf16*)out,
                           out_stride, (const bf16*)gate, gate_stride, (const bf16*)kcache, (const bf16*)vcache,
                           block_tables, bt_stride, token_req, positions, nh, nkvh, dk, dv, page_size, scale, window,
                           keep_first, sink);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}
