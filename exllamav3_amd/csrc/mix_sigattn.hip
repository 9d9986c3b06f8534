// Causal attention WITHOUT softmax: a visible key weighs sigmoid(scale q.k + bias_head), weights are not normalised over keys, positions do not enter
// the scores.  Nothing bounds how far back a row looks, so keys and values live in PAGES: pools [pages][page][kv_heads * dim] / [..][kv_heads * vdim]
// shared by all sequences, and a table [slots][max pages] that says which pages a sequence owns, in order.
// This file: the store of a step's keys and values into the pages, and the exact float32-score form of prompt steps (keys of the step's own rows)
// and decode steps (keys through the page table) -- one workgroup per (row, query head), a key per lane, the waves' partial sums merged through LDS.
// The matrix-core form of prompt steps for bfloat16 is mix_sigattn_mfma.hip.
#include "mix_common.cuh"

template <typename T> struct sg_vec;
template <> struct sg_vec<bf16_t> { static constexpr int N = 8; };
template <> struct sg_vec<float> { static constexpr int N = 4; };

__device__ __forceinline__ int64_t paged_row(const int32_t* __restrict__ table, int page, int j)
{
    return (int64_t) table[j / page] * page + (j % page);
}

template <typename T>
__global__ __launch_bounds__(256) void paged_store_kernel(T* __restrict__ k_pages, T* __restrict__ v_pages, const T* __restrict__ k, int64_t k_ld, const T* __restrict__ v, int64_t v_ld,
                                                          const int32_t* __restrict__ table, int64_t table_ld, int page, const int32_t* __restrict__ tok_seq,
                                                          const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ slots, int kw, int vw)
{
    const int n = blockIdx.x;
    const int64_t row = paged_row(table + (int64_t) slots[tok_seq[n]] * table_ld, page, tok_pos[n]);
    for (int i = threadIdx.x; i < kw; i += 256) k_pages[row * kw + i] = k[(int64_t) n * k_ld + i];
    for (int i = threadIdx.x; i < vw; i += 256) v_pages[row * vw + i] = v[(int64_t) n * v_ld + i];
}

// The row worker.  Keys j < count: PAGED ? row paged_row(table, page, j) of the pools : row j behind kb / vb (row strides k_step / v_step, the head's offset
// already applied in both cases).  MAXV = ceil(vdim / 64) accumulators per lane.
template <typename T, int MAXV, int NW, bool PAGED>
__device__ __forceinline__ void sig_row(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kb, int64_t k_step, const T* __restrict__ vb, int64_t v_step,
                                        const int32_t* __restrict__ table, int page, int count, int dim, int vdim, float scale, float bias, bool k_vec, float* smem)
{
    float* qs = smem;                                   // [dim]
    float* ps = qs + ((dim + 1) & ~1);                 // [NW][64] weights (the 8-byte entries behind them stay aligned for odd dim)
    int64_t* rs = (int64_t*) (ps + NW * 64);            // [NW][64] value rows
    float* mg = (float*) (rs + NW * 64);                // [NW][MAXV * 64]
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < dim; i += 64 * NW) qs[i] = to_f(q[i]);
    __syncthreads();
    float acc[MAXV];
    #pragma unroll
    for (int i = 0; i < MAXV; ++i) acc[i] = 0.f;
    float* pw = ps + w * 64;
    int64_t* rw = rs + w * 64;
    constexpr int VN = sg_vec<T>::N;
    for (int j0 = w * 64; j0 < count; j0 += 64 * NW)
    {
        const int j = j0 + lane;
        float p = 0.f;
        int64_t row = 0;
        if (j < count)
        {
            row = PAGED ? paged_row(table, page, j) : (int64_t) j;
            const T* kr = kb + row * k_step;
            float d = 0.f;
            if (k_vec)
            {
                for (int c = 0; c < dim; c += VN)
                {
                    union { uint4 v; T e[VN]; } t;
                    t.v = *(const uint4*) (kr + c);
                    #pragma unroll
                    for (int e = 0; e < VN; ++e) d += qs[c + e] * to_f(t.e[e]);
                }
            }
            else
                for (int c = 0; c < dim; ++c) d += qs[c] * to_f(kr[c]);
            p = sigmoid_f(d * scale + bias);
        }
        pw[lane] = p;
        rw[lane] = row;
        __builtin_amdgcn_wave_barrier();                    // LDS serves a wave's accesses in order: its own stores are visible to the reads below
        const int cnt = min(64, count - j0);
        #pragma unroll
        for (int i = 0; i < MAXV; ++i)
        {
            const int c = lane + 64 * i;
            float a = acc[i];
            if (c < vdim)
            {
                int jj = 0;
                for (; jj + 8 <= cnt; jj += 8)                // eight value rows in flight, then the sums
                {
                    float vv[8];
                    #pragma unroll
                    for (int e = 0; e < 8; ++e) vv[e] = to_f(vb[rw[jj + e] * v_step + c]);
                    #pragma unroll
                    for (int e = 0; e < 8; ++e) a += pw[jj + e] * vv[e];
                }
                for (; jj < cnt; ++jj) a += pw[jj] * to_f(vb[rw[jj] * v_step + c]);
            }
            acc[i] = a;
        }
        __builtin_amdgcn_wave_barrier();
    }
    float* mine = mg + w * (MAXV * 64);
    #pragma unroll
    for (int i = 0; i < MAXV; ++i) mine[i * 64 + lane] = acc[i];
    __syncthreads();
    if (w != 0) return;
    #pragma unroll
    for (int i = 0; i < MAXV; ++i)
    {
        float s = 0.f;
        #pragma unroll
        for (int ww = 0; ww < NW; ++ww) s += mg[ww * (MAXV * 64) + i * 64 + lane];
        const int c = lane + 64 * i;
        if (c < vdim) out[c] = from_f<T>(s);
    }
}

template <typename T>
__device__ __forceinline__ bool sg_rows_16_byte(const T* base, int64_t step, int dim)
{
    return ((uintptr_t) base % 16 == 0) && ((step * (int64_t) sizeof(T)) % 16 == 0) && (dim % sg_vec<T>::N == 0);
}

template <typename T, int MAXV, int NW>
__global__ __launch_bounds__(64 * NW) void sigattn_prefill_kernel(T* __restrict__ out, const T* __restrict__ q, int64_t q_ld, const T* __restrict__ k, int64_t k_ld,
                                                                  const T* __restrict__ v, int64_t v_ld, const float* __restrict__ bias, const int32_t* __restrict__ cu,
                                                                  const int32_t* __restrict__ tok_seq, int heads, int kv_heads, int dim, int vdim, float scale)
{
    extern __shared__ float smem[];
    const int n = blockIdx.x, h = blockIdx.y, g = h / (heads / kv_heads);
    const int first = cu[tok_seq[n]];
    const T* kb = k + (int64_t) first * k_ld + (int64_t) g * dim;
    sig_row<T, MAXV, NW, false>(out + ((int64_t) n * heads + h) * vdim, q + (int64_t) n * q_ld + (int64_t) h * dim, kb, k_ld, v + (int64_t) first * v_ld + (int64_t) g * vdim, v_ld,
                                nullptr, 1, n - first + 1, dim, vdim, scale, bias ? bias[h] : 0.f, sg_rows_16_byte(kb, k_ld, dim), smem);
}

template <typename T, int MAXV, int NW>
__global__ __launch_bounds__(64 * NW) void sigattn_decode_kernel(T* __restrict__ out, const T* __restrict__ q, int64_t q_ld, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                                                                 const float* __restrict__ bias, const int32_t* __restrict__ table, int64_t table_ld, int page,
                                                                 const int32_t* __restrict__ slots, const int32_t* __restrict__ len_after, int heads, int kv_heads, int dim, int vdim,
                                                                 float scale)
{
    extern __shared__ float smem[];
    const int n = blockIdx.x, h = blockIdx.y, g = h / (heads / kv_heads);
    const T* kb = k_pages + (int64_t) g * dim;
    const int64_t k_step = (int64_t) kv_heads * dim;
    sig_row<T, MAXV, NW, true>(out + ((int64_t) n * heads + h) * vdim, q + (int64_t) n * q_ld + (int64_t) h * dim, kb, k_step, v_pages + (int64_t) g * vdim, (int64_t) kv_heads * vdim,
                               table + (int64_t) slots[n] * table_ld, page, len_after[n], dim, vdim, scale, bias ? bias[h] : 0.f, sg_rows_16_byte(kb, k_step, dim), smem);
}

#define SIG_LAUNCH_NW(KERNEL, NWV, ...) \
    do { \
        const size_t sm = (size_t) (dim + 2 + NWV * 64 + NWV * 128 + NWV * mvt * 64) * sizeof(float); \
        if (mvt == 1)      hipLaunchKernelGGL((KERNEL<T, 1, NWV>), dim3(n, heads), dim3(64 * NWV), sm, (hipStream_t) stream, (T*) out, __VA_ARGS__); \
        else if (mvt == 2) hipLaunchKernelGGL((KERNEL<T, 2, NWV>), dim3(n, heads), dim3(64 * NWV), sm, (hipStream_t) stream, (T*) out, __VA_ARGS__); \
        else if (mvt == 4) hipLaunchKernelGGL((KERNEL<T, 4, NWV>), dim3(n, heads), dim3(64 * NWV), sm, (hipStream_t) stream, (T*) out, __VA_ARGS__); \
        else               hipLaunchKernelGGL((KERNEL<T, 8, NWV>), dim3(n, heads), dim3(64 * NWV), sm, (hipStream_t) stream, (T*) out, __VA_ARGS__); \
    } while (0)
#define SIG_LAUNCH(KERNEL, ...) \
    do { \
        const int mv = (vdim + 63) / 64; \
        const int mvt = mv == 1 ? 1 : (mv == 2 ? 2 : (mv <= 4 ? 4 : 8)); \
        MIX_DISPATCH_T(dtype, if (wide) SIG_LAUNCH_NW(KERNEL, 16, __VA_ARGS__); else SIG_LAUNCH_NW(KERNEL, 4, __VA_ARGS__)); \
    } while (0)

static int sig_check(const char* what, int n, int heads, int kv_heads, int dim, int vdim)
{
    MIX_CHECK(n >= 0 && heads > 0 && heads <= 65535 && kv_heads > 0 && heads % kv_heads == 0, "%s: heads %d must be a multiple of kv_heads %d", what, heads, kv_heads);
    MIX_CHECK(dim > 0 && dim <= 4096 && vdim > 0 && vdim <= 512, "%s: dim %d (<= 4096) / vdim %d (<= 512) out of range", what, dim, vdim);
    return EXL3_MIX_OK;
}

extern "C" int exl3_mix_paged_store(void* k_pages, void* v_pages, const void* k, int64_t k_ld, const void* v, int64_t v_ld, const int32_t* table, int64_t table_ld, int page,
                                    const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, int n, int kw, int vw, int dtype, void* stream)
{
    MIX_CHECK(k_pages && v_pages && k && v && table && tok_seq && tok_pos && slots, "mix_paged_store: null pointer");
    MIX_CHECK(n >= 0 && kw > 0 && vw > 0 && page > 0 && table_ld > 0 && k_ld >= kw && v_ld >= vw, "mix_paged_store: bad sizes");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(paged_store_kernel<T>, dim3(n), dim3(256), 0, (hipStream_t) stream, (T*) k_pages, (T*) v_pages, (const T*) k, k_ld, (const T*) v, v_ld,
                                             table, table_ld, page, tok_seq, tok_pos, slots, kw, vw));
    return mix_check_launch("mix_paged_store");
}

extern "C" int exl3_mix_sigattn_prefill(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld, const float* bias,
                                        const int32_t* cu, const int32_t* tok_seq, int n, int heads, int kv_heads, int dim, int vdim, float scale, int dtype, void* stream)
{
    MIX_CHECK(out && q && k && v && cu && tok_seq, "mix_sigattn_prefill: null pointer");
    if (int rc = sig_check("mix_sigattn_prefill", n, heads, kv_heads, dim, vdim)) return rc;
    MIX_CHECK(q_ld >= (int64_t) heads * dim && k_ld >= (int64_t) kv_heads * dim && v_ld >= (int64_t) kv_heads * vdim, "mix_sigattn_prefill: bad row strides");
    if (n == 0) return EXL3_MIX_OK;
    const bool wide = false;
    SIG_LAUNCH(sigattn_prefill_kernel, (const T*) q, q_ld, (const T*) k, k_ld, (const T*) v, v_ld, bias, cu, tok_seq, heads, kv_heads, dim, vdim, scale);
    return mix_check_launch("mix_sigattn_prefill");
}

extern "C" int exl3_mix_sigattn_decode(void* out, const void* q, int64_t q_ld, const void* k_pages, const void* v_pages, const float* bias, const int32_t* table, int64_t table_ld,
                                       int page, const int32_t* slots, const int32_t* len_after, int n, int heads, int kv_heads, int dim, int vdim, float scale, int dtype, void* stream)
{
    MIX_CHECK(out && q && k_pages && v_pages && table && slots && len_after, "mix_sigattn_decode: null pointer");
    if (int rc = sig_check("mix_sigattn_decode", n, heads, kv_heads, dim, vdim)) return rc;
    MIX_CHECK(q_ld >= (int64_t) heads * dim && page > 0 && table_ld > 0, "mix_sigattn_decode: bad row stride or page size");
    if (n == 0) return EXL3_MIX_OK;
    const bool wide = (int64_t) n * heads <= 512 && vdim <= 256;       // few rows over long caches: the chain of key chunks a wave walks bounds the step, not bytes
    SIG_LAUNCH(sigattn_decode_kernel, (const T*) q, q_ld, (const T*) k_pages, (const T*) v_pages, bias, table, table_ld, page, slots, len_after, heads, kv_heads, dim, vdim, scale);
    return mix_check_launch("mix_sigattn_decode");
}
