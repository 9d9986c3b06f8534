// Prefill of differential attention on the matrix cores (bfloat16 activations): both attention maps of a head in ONE workgroup, and the combination
// of the maps in the epilogue.  The layout of the work is that of mix_attn_mfma.hip -- 128 query rows of one sequence and one head per workgroup, eight
// waves of 16 rows, scores transposed (S^T = K Q^T) so that a lane holds the scores of one query and the probabilities never pass through LDS -- with
// these differences:
//   * a key tile holds the keys of both maps side by side ([key][map][dim]) and the value tile, which both maps read, is staged (transposed) once: the
//     transposing stores are the costly part of staging, and here they are paid once for twice the matrix work;
//   * every wave keeps two online softmaxes (maximum, sum, value accumulators per map) and walks the maps one after the other inside a tile;
//   * scores may be soft-capped, cap tanh(scale s / cap), before the running maximum (tanh is increasing: the largest raw score is the largest score);
//   * the mask gives every row a first visible key lo(i) that never decreases with i (a chunk's start, or i - window + 1);
//   * epilogue: o = a1 / l1 - lambda a2 / l2 in float32, divided by its root mean square over the value dim, times (1 - diff), times the sigmoid of the
//     head's gate; written in bfloat16 as [row][head][vdim].  The two maps' outputs never leave the registers.
#include "mix_common.cuh"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

#define AD_ROWS 128
#define AD_THREADS 512
#define AD_PAD 8
#define AD_LOG2E 1.4426950408889634f

__device__ __forceinline__ int ad_first_visible(int i, int window, int mask) { return mask == EXL3_MIX_MASK_CHUNK ? (i / window) * window : i - window + 1; }

// KD: contraction steps of 32 over the (zero-padded) head dim; NV: 16-column tiles of the (padded) value dim; KT: keys per tile.
template <int KD, int NV, int KT, bool CAP>
__global__ __launch_bounds__(AD_THREADS) void attn_prefill_mfma_diff_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int64_t q_ld, const bf16_t* __restrict__ k,
                                                                     int64_t k_ld, const bf16_t* __restrict__ v, int64_t v_ld, const bf16_t* __restrict__ gate, int64_t gate_ld,
                                                                     const int32_t* __restrict__ cu, int heads, int kv_heads, int dim, int vdim, float scale, float softcap,
                                                                     int window, int mask, float lambda, float diff, float eps, int k_vec, int v_vec)
{
    constexpr int DP = KD * 32, KS = 2 * DP + AD_PAD, VS = KT + AD_PAD, NS = KT / 16;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t* k_lds = (uint16_t*) smem_raw;                       // [KT][KS]: map 0 in columns 0 .. DP-1, map 1 in DP .. 2 DP - 1
    uint16_t* vt_lds = k_lds + KT * KS;                           // [NV * 16][VS]   (value column, key)

    const int b = blockIdx.y, h = blockIdx.z;
    const int first = cu[b], len = cu[b + 1] - first;
    const int q0 = blockIdx.x * AD_ROWS;
    if (q0 >= len) return;
    const int vh = h / (heads / kv_heads);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;

    // this wave's 16 query rows of both maps as B operands of S^T = K Q^T (rows beyond the sequence read row len-1: computed and never stored)
    const int qrow_a = min(q0 + w * 16 + c, len - 1);
    bf16x8 qf[2][KD];
    #pragma unroll
    for (int m = 0; m < 2; ++m)
    {
        #pragma unroll
        for (int s = 0; s < KD; ++s)
        {
            union { bf16x8 v; uint16_t u[8]; } t;
            #pragma unroll
            for (int e = 0; e < 8; ++e)
            {
                const int col = s * 32 + g * 8 + e;
                t.u[e] = col < dim ? q[(int64_t) (first + qrow_a) * q_ld + (int64_t) (h * 2 + m) * dim + col].u : (uint16_t) 0;
            }
            qf[m][s] = t.v;
        }
    }
    const int wq_lo = q0 + w * 16, wq_hi = min(q0 + w * 16 + 15, len - 1);           // this wave's rows
    const bool wave_live = wq_lo < len;
    const int qi = q0 + w * 16 + c;                                                   // per lane: query c of the wave
    float mrun[2] = {-1e30f, -1e30f}, lsum[2] = {0.f, 0.f};                           // running maximum (the same in a query's four lanes), this lane's share of the sum
    f32x4 acc[2][NV];                                                                 // O^T tiles per map: value rows 4g .. 4g+3 of tile t, query c
    #pragma unroll
    for (int m = 0; m < 2; ++m)
    {
        #pragma unroll
        for (int t = 0; t < NV; ++t) acc[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const int blk_hi = min(q0 + AD_ROWS - 1, len - 1);
    const int j_begin = (max(0, ad_first_visible(q0, window, mask)) / KT) * KT;
    const int wave_lo = ad_first_visible(wq_lo, window, mask), wave_hi_lo = ad_first_visible(wq_hi, window, mask);
    const int my_lo = ad_first_visible(qi, window, mask);
    for (int j0 = j_begin; j0 <= blk_hi; j0 += KT)
    {
        __syncthreads();                                           // the previous tile's operand reads are over
        for (int idx = threadIdx.x; idx < KT * 2 * (DP / 8); idx += AD_THREADS)
        {
            const int r = idx / (2 * (DP / 8)), rest = idx - r * (2 * (DP / 8)), m = rest / (DP / 8), cg = rest - m * (DP / 8);
            const int j = j0 + r;
            const bf16_t* src = k + (int64_t) (first + min(j, len - 1)) * k_ld + (int64_t) (vh * 2 + m) * dim + cg * 8;
            union { uint4 v; uint16_t u[8]; } t;
            if (k_vec && j < len && cg * 8 + 8 <= dim) t.v = *(const uint4*) src;          // 16-byte rows (host-checked alignment)
            else
            {
                #pragma unroll
                for (int e = 0; e < 8; ++e) t.u[e] = (j < len && cg * 8 + e < dim) ? src[e].u : (uint16_t) 0;
            }
            *(uint4*) (k_lds + r * KS + m * DP + cg * 8) = t.v;
        }
        for (int idx = threadIdx.x; idx < KT * NV * 2; idx += AD_THREADS)
        {
            const int cg = idx / KT, r = idx - cg * KT;                       // consecutive lanes: consecutive keys of one column group (LDS stores side by side)
            const int j = j0 + r;
            const bf16_t* src = v + (int64_t) (first + min(j, len - 1)) * v_ld + (int64_t) vh * vdim + cg * 8;
            union { uint4 v; uint16_t u[8]; } t;
            if (v_vec && j < len && cg * 8 + 8 <= vdim) t.v = *(const uint4*) src;
            else
            {
                #pragma unroll
                for (int e = 0; e < 8; ++e) t.u[e] = (j < len && cg * 8 + e < vdim) ? src[e].u : (uint16_t) 0;
            }
            #pragma unroll
            for (int e = 0; e < 8; ++e) vt_lds[(cg * 8 + e) * VS + r] = t.u[e];
        }
        __syncthreads();
        // tiles wholly outside this wave's rows' visible keys: nothing to add (uniform per wave; the barriers above are still met)
        const bool skip = !wave_live || j0 > wq_hi || j0 + KT - 1 < wave_lo;
        if (skip) continue;
        const bool interior = j0 + KT - 1 <= wq_lo && j0 >= wave_hi_lo && q0 + w * 16 + 15 < len;
        #pragma unroll
        for (int m = 0; m < 2; ++m)
        {
            f32x4 sc[NS];
            #pragma unroll
            for (int u = 0; u < NS; ++u) sc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            #pragma unroll
            for (int s = 0; s < KD; ++s)
            {
                #pragma unroll
                for (int u = 0; u < NS; ++u)
                {
                    const bf16x8 kf = *(const bf16x8*) (k_lds + (u * 16 + c) * KS + m * DP + s * 32 + g * 8);
                    sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[m][s], sc[u], 0, 0, 0);
                }
            }
            // sc[u][i] = raw score of key j0 + 16u + 4g + i against query qi
            if (CAP)
            {
                // score <- cap tanh(scale raw / cap), tanh(x) = 1 - 2 / (1 + e^(2x)): one v_exp_f32 and one reciprocal per key
                const float a = 2.0f * AD_LOG2E * scale / softcap;
                #pragma unroll
                for (int u = 0; u < NS; ++u)
                {
                    #pragma unroll
                    for (int i = 0; i < 4; ++i) sc[u][i] = softcap - 2.0f * softcap * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(sc[u][i] * a));
                }
            }
            const float s_scale = CAP ? 1.0f : scale;                          // what is left to multiply the held scores with
            float mx = -INFINITY;
            if (interior)
            {
                #pragma unroll
                for (int u = 0; u < NS; ++u)
                {
                    #pragma unroll
                    for (int i = 0; i < 4; ++i) mx = fmaxf(mx, sc[u][i]);
                }
            }
            else
            {
                #pragma unroll
                for (int u = 0; u < NS; ++u)
                {
                    #pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        const int j = j0 + u * 16 + g * 4 + i;
                        const bool ok = j <= qi && j >= my_lo && qi < len;
                        sc[u][i] = ok ? sc[u][i] : -INFINITY;
                        mx = fmaxf(mx, sc[u][i]);
                    }
                }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float mn = fmaxf(mrun[m], mx * s_scale);                     // scale > 0 (host-checked)
            const float corr = __builtin_amdgcn_exp2f((mrun[m] - mn) * AD_LOG2E);
            mrun[m] = mn;
            const float c2 = s_scale * AD_LOG2E, off = -mn * AD_LOG2E;
            float sum = 0.f;
            #pragma unroll
            for (int u = 0; u < NS; ++u)
            {
                #pragma unroll
                for (int i = 0; i < 4; ++i) { sc[u][i] = __builtin_amdgcn_exp2f(sc[u][i] * c2 + off); sum += sc[u][i]; }      // masked: 2^(-inf) = 0
            }
            lsum[m] = lsum[m] * corr + sum;
            #pragma unroll
            for (int t = 0; t < NV; ++t) acc[m][t] *= corr;
            #pragma unroll
            for (int kk = 0; kk < NS / 2; ++kk)
            {
                bf16x8 pb;
                #pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    pb[i] = (__bf16) sc[2 * kk][i];
                    pb[4 + i] = (__bf16) sc[2 * kk + 1][i];
                }
                #pragma unroll
                for (int t = 0; t < NV; ++t)
                {
                    union { bf16x8 v; bf16x4 h[2]; } va;
                    va.h[0] = *(const bf16x4*) (vt_lds + (t * 16 + c) * VS + (2 * kk) * 16 + g * 4);
                    va.h[1] = *(const bf16x4*) (vt_lds + (t * 16 + c) * VS + (2 * kk + 1) * 16 + g * 4);
                    acc[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va.v, pb, acc[m][t], 0, 0, 0);
                }
            }
        }
    }
    if (!wave_live) return;
    float f[2];
    #pragma unroll
    for (int m = 0; m < 2; ++m)
    {
        float l = lsum[m];
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        f[m] = l > 0.f ? 1.0f / l : 0.f;
    }
    // o = a1 - lambda a2 over the value dim of query c: this lane holds rows 4g .. 4g+3 of every tile, the query's other rows are in the lanes g' != g
    float ss = 0.f;
    #pragma unroll
    for (int t = 0; t < NV; ++t)
    {
        #pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            const float o = acc[0][t][i] * f[0] - lambda * (acc[1][t][i] * f[1]);       // padded value rows hold zeros
            acc[0][t][i] = o;
            ss += o * o;
        }
    }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if (qi >= len) return;
    const int64_t n = first + qi;
    float fo = (1.0f - diff) / sqrtf(ss / (float) vdim + eps);
    if (gate) fo *= sigmoid_f(to_f(gate[n * gate_ld + h]));
    #pragma unroll
    for (int t = 0; t < NV; ++t)
    {
        #pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            const int col = t * 16 + g * 4 + i;
            if (col < vdim) out[(n * heads + h) * vdim + col] = from_f<bf16_t>(acc[0][t][i] * fo);
        }
    }
}

extern "C" int exl3_mix_attn_prefill_mfma_diff(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                                               const void* gate, int64_t gate_ld, const int32_t* cu, int batch, int max_rows, int heads, int kv_heads, int dim, int vdim,
                                               float scale, float softcap, int window, int mask, float lambda, float diff, float eps, void* stream)
{
    MIX_CHECK(out && q && k && v && cu, "mix_attn_prefill_mfma_diff: null pointer");
    MIX_CHECK(batch >= 0 && max_rows >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && heads <= 65535 && batch <= 65535,
              "mix_attn_prefill_mfma_diff: heads %d / kv_heads %d / batch %d", heads, kv_heads, batch);
    MIX_CHECK(dim > 0 && dim <= 128 && vdim > 0 && vdim <= 256 && window > 0, "mix_attn_prefill_mfma_diff: dim %d must be <= 128 and vdim %d <= 256", dim, vdim);
    MIX_CHECK(scale > 0.f && softcap >= 0.f && (mask == EXL3_MIX_MASK_WINDOW || mask == EXL3_MIX_MASK_CHUNK),
              "mix_attn_prefill_mfma_diff: the score scale must be positive (the running maximum is taken over raw scores), softcap >= 0, mask %d", mask);
    MIX_CHECK(q_ld >= (int64_t) heads * 2 * dim && k_ld >= (int64_t) kv_heads * 2 * dim && v_ld >= (int64_t) kv_heads * vdim && (!gate || gate_ld >= heads),
              "mix_attn_prefill_mfma_diff: bad row strides");
    if (batch == 0 || max_rows == 0) return EXL3_MIX_OK;
    const dim3 grid((max_rows + AD_ROWS - 1) / AD_ROWS, batch, heads);
    const int k_vec = ((uintptr_t) k % 16 == 0) && (k_ld % 8 == 0) && (dim % 8 == 0);
    const int v_vec = ((uintptr_t) v % 16 == 0) && (v_ld % 8 == 0) && (vdim % 8 == 0);
    #define AD_LDS(KDV, NVV, KTV) ((size_t) (KTV * (2 * KDV * 32 + AD_PAD) + NVV * 16 * (KTV + AD_PAD)) * sizeof(uint16_t))
    #define AD_LAUNCH_C(KDV, NVV, KTV, CAPV) \
        hipLaunchKernelGGL((attn_prefill_mfma_diff_kernel<KDV, NVV, KTV, CAPV>), grid, dim3(AD_THREADS), AD_LDS(KDV, NVV, KTV), (hipStream_t) stream, (bf16_t*) out, \
                           (const bf16_t*) q, q_ld, (const bf16_t*) k, k_ld, (const bf16_t*) v, v_ld, (const bf16_t*) gate, gate_ld, cu, heads, kv_heads, dim, vdim, scale, softcap, \
                           window, mask, lambda, diff, eps, k_vec, v_vec)
    #define AD_LAUNCH(KDV, NVV, KTV) do { \
        static_assert(AD_LDS(KDV, NVV, KTV) <= 65536, "tile does not fit the LDS"); \
        if (softcap > 0.f) AD_LAUNCH_C(KDV, NVV, KTV, true); else AD_LAUNCH_C(KDV, NVV, KTV, false); } while (0)
    const int kd = (dim + 31) / 32, nv = (vdim + 15) / 16;
    if (kd <= 1)      { if (nv <= 4) AD_LAUNCH(1, 4, 64); else if (nv <= 8) AD_LAUNCH(1, 8, 64); else AD_LAUNCH(1, 16, 64); }
    else if (kd <= 2) { if (nv <= 4) AD_LAUNCH(2, 4, 64); else if (nv <= 8) AD_LAUNCH(2, 8, 64); else AD_LAUNCH(2, 16, 32); }
    else              { if (nv <= 4) AD_LAUNCH(4, 4, 64); else if (nv <= 8) AD_LAUNCH(4, 8, 64); else AD_LAUNCH(4, 16, 32); }
    #undef AD_LDS
    #undef AD_LAUNCH
    #undef AD_LAUNCH_C
    return mix_check_launch("mix_attn_prefill_mfma_diff");
}
