// Prefill of the sliding-window sink attention on the matrix cores (bfloat16 activations): scores = Q K^T and the weighted sum P V with
// v_mfma_f32_16x16x32_bf16, scores, running maximum, exponentials and sums in float32; the softmax starts from the sink, so the sink is one
// more term of the denominator and nothing else.
//
// One workgroup = 128 query rows of one sequence and one head, 8 waves of 16 rows.  Key tiles of KT = 64 rows (32 for the largest heads, where
// 64 would not fit 64 KB of LDS) are staged in LDS once for the eight waves: K as stored, V transposed (value column, key).
//
// MFMA operand lane (g = lane / 16, c = lane % 16) holds row / column c and contraction slots 8g .. 8g+7; result lane (g, c) holds rows
// 4g .. 4g+3 of column c.  The scores are computed TRANSPOSED, S^T = K Q^T (keys are rows, the wave's 16 queries are columns): a lane then
// holds scores of ONE query (column c), so the running maximum, the sum and the rescale factor are per-lane scalars (two cross-lane steps
// per tile for the maximum, the sum is reduced once at the end), and the result registers of two 16-key tiles are, as they stand, the B
// operand of O^T = V^T P^T when contraction slot (g, e) is read as key 4g + e of the first tile (e < 4) or of the second (e >= 4); the A operand
// V^T is read from LDS in the same key order (two 8-byte reads).  No probability goes through LDS.  Only the key tiles that intersect the
// window of the block's rows are visited, and a wave skips the tiles outside its own rows' windows.
//
// Variants of the same kernel: `maps` attention maps per head (queries [head][map][dim], keys [kv head][map][dim], every map reads the values of the
// head's key/value head; result [row][head][map][vdim]); a chunk mask (a row sees the positions of its own chunk of `window` positions) beside the
// sliding window -- both give every row a first visible key lo(i) that never decreases with i, which is all the tile logic uses; a soft cap on the
// scores, cap tanh(score / cap), applied to the scaled scores before the running maximum (tanh is increasing, so the largest raw score still is the
// largest score); and a float32 result.
#include "mix_common.cuh"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

#define AM_ROWS 128
#define AM_THREADS 512
#define AM_PAD 8
#define LOG2E 1.4426950408889634f

// KD: contraction steps of 32 over the (zero-padded) head dim; NV: 16-column tiles of the (padded) value dim.
__device__ __forceinline__ int first_visible(int i, int window, int mask) { return mask == EXL3_MIX_MASK_CHUNK ? (i / window) * window : i - window + 1; }

template <int KD, int NV, int AM_KEYS, bool CAP>
__global__ __launch_bounds__(AM_THREADS) void attn_prefill_mfma_kernel(void* __restrict__ out_any, int out_f32, const bf16_t* __restrict__ q, int64_t q_ld, const bf16_t* __restrict__ k,
                                                                int64_t k_ld, const bf16_t* __restrict__ v_norm, int64_t v_ld, const bf16_t* __restrict__ gate, int64_t gate_ld,
                                                                const float* __restrict__ sink, const int32_t* __restrict__ cu,
                                                                int heads, int kv_heads, int maps, int dim, int vdim, float scale, float softcap, int window, int mask,
                                                                int k_vec, int v_vec)
{
    constexpr int DP = KD * 32, KS = DP + AM_PAD, VS = AM_KEYS + AM_PAD;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t* k_lds = (uint16_t*) smem_raw;                       // [AM_KEYS][KS]
    uint16_t* vt_lds = k_lds + AM_KEYS * KS;                      // [NV * 16][VS]   (value column, key)

    const int b = blockIdx.y, h = blockIdx.z;
    const int first = cu[b], len = cu[b + 1] - first;
    const int q0 = blockIdx.x * AM_ROWS;
    if (q0 >= len) return;
    const int hh = h / maps;                                      // h counts (head, map)
    const int vh = hh / (heads / kv_heads), kvh = vh * maps + (h - hh * maps);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;

    // this wave's 16 query rows as B operands of S^T = K Q^T (rows beyond the sequence read row len-1: computed and never stored)
    const int qrow_a = min(q0 + w * 16 + c, len - 1);
    bf16x8 qf[KD];
    #pragma unroll
    for (int s = 0; s < KD; ++s)
    {
        union { bf16x8 v; uint16_t u[8]; } t;
        #pragma unroll
        for (int e = 0; e < 8; ++e)
        {
            const int col = s * 32 + g * 8 + e;
            t.u[e] = col < dim ? q[(int64_t) (first + qrow_a) * q_ld + (int64_t) h * dim + col].u : (uint16_t) 0;
        }
        qf[s] = t.v;
    }
    const int wq_lo = q0 + w * 16, wq_hi = min(q0 + w * 16 + 15, len - 1);           // this wave's rows
    const bool wave_live = wq_lo < len;

    // per lane: query c of the wave.  m: running maximum (the same in the four lanes of a query), l: this lane's share of the sum
    const int qi = q0 + w * 16 + c;
    float m = sink ? sink[h] : -1e30f;
    float l = (sink && g == 0) ? 1.0f : 0.0f;
    f32x4 acc[NV];                                                 // O^T tiles: value rows 4g .. 4g+3 of tile t, query c
    #pragma unroll
    for (int t = 0; t < NV; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int blk_hi = min(q0 + AM_ROWS - 1, len - 1);
    const int j_begin = (max(0, first_visible(q0, window, mask)) / AM_KEYS) * AM_KEYS;
    const int wave_lo = first_visible(wq_lo, window, mask), wave_hi_lo = first_visible(wq_hi, window, mask);      // first visible key of the wave's first / last row
    const int my_lo = first_visible(qi, window, mask);
    for (int j0 = j_begin; j0 <= blk_hi; j0 += AM_KEYS)
    {
        __syncthreads();                                           // the previous tile's operand reads are over
        // stage K [32][DP] (zero beyond dim / len) and V^T [vdim][32]
        for (int idx = threadIdx.x; idx < AM_KEYS * (DP / 8); idx += AM_THREADS)
        {
            const int r = idx / (DP / 8), cg = idx - r * (DP / 8);
            const int j = j0 + r;
            const bf16_t* src = k + (int64_t) (first + min(j, len - 1)) * k_ld + (int64_t) kvh * dim + cg * 8;
            union { uint4 v; uint16_t u[8]; } t;
            if (k_vec && j < len && cg * 8 + 8 <= dim) t.v = *(const uint4*) src;          // 16-byte rows (host-checked alignment)
            else
            {
                #pragma unroll
                for (int e = 0; e < 8; ++e) t.u[e] = (j < len && cg * 8 + e < dim) ? src[e].u : (uint16_t) 0;
            }
            *(uint4*) (k_lds + r * KS + cg * 8) = t.v;
        }
        for (int idx = threadIdx.x; idx < AM_KEYS * NV * 2; idx += AM_THREADS)
        {
            const int cg = idx / AM_KEYS, r = idx - cg * AM_KEYS;               // consecutive lanes: consecutive keys of one column group (LDS stores side by side)
            const int j = j0 + r;
            const bf16_t* src = v_norm + (int64_t) (first + min(j, len - 1)) * v_ld + (int64_t) vh * vdim + cg * 8;
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
        // tiles wholly outside this wave's windows: nothing to add (uniform per wave; the barriers above are still met)
        const bool skip = !wave_live || j0 > wq_hi || j0 + AM_KEYS - 1 < wave_lo;
        if (!skip)
        {
            constexpr int NS = AM_KEYS / 16;                                   // 16-key score tiles
            f32x4 sc[NS];
            #pragma unroll
            for (int u = 0; u < NS; ++u) sc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            #pragma unroll
            for (int s = 0; s < KD; ++s)
            {
                #pragma unroll
                for (int u = 0; u < NS; ++u)
                {
                    const bf16x8 kf = *(const bf16x8*) (k_lds + (u * 16 + c) * KS + s * 32 + g * 8);
                    sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[s], sc[u], 0, 0, 0);
                }
            }
            // sc[u][i] = raw score of key j0 + 16u + 4g + i against query qi.  A tile whose keys all lie inside the window of every row of the wave
            // needs no mask (wave-uniform branch; with a window of many tiles that is most of them).
            const bool interior = j0 + AM_KEYS - 1 <= wq_lo && j0 >= wave_hi_lo && q0 + w * 16 + 15 < len;
            if (CAP)
            {
                // score <- cap tanh(scale raw / cap), tanh(x) = 1 - 2 / (1 + e^(2x)): one v_exp_f32 and one reciprocal per key
                const float a = 2.0f * LOG2E * scale / softcap;
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
            const float mn = fmaxf(m, mx * s_scale);                           // scale > 0 (host-checked): the largest raw score is the largest score
            const float corr = __builtin_amdgcn_exp2f((m - mn) * LOG2E);
            m = mn;
            // weight = exp(score * scale - m) = 2^(score * c2 - m * log2 e): one multiply-add and one v_exp_f32 per key
            const float c2 = s_scale * LOG2E, off = -mn * LOG2E;
            float sum = 0.f;
            #pragma unroll
            for (int u = 0; u < NS; ++u)
            {
                #pragma unroll
                for (int i = 0; i < 4; ++i) { sc[u][i] = __builtin_amdgcn_exp2f(sc[u][i] * c2 + off); sum += sc[u][i]; }      // masked: 2^(-inf) = 0
            }
            l = l * corr + sum;
            #pragma unroll
            for (int t = 0; t < NV; ++t) acc[t] *= corr;
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
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va.v, pb, acc[t], 0, 0, 0);
                }
            }
        }
    }
    if (!wave_live) return;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (qi >= len) return;
    const int64_t n = first + qi;
    const float gt = gate ? sigmoid_f(to_f(gate[n * gate_ld + h])) : 1.0f;
    const float f = (l > 0.f ? 1.0f / l : 0.f) * gt;
    const int64_t o0 = (n * heads * maps + h) * vdim;
    #pragma unroll
    for (int t = 0; t < NV; ++t)
    {
        #pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            const int col = t * 16 + g * 4 + i;
            if (col < vdim)
            {
                if (out_f32) ((float*) out_any)[o0 + col] = acc[t][i] * f;
                else         ((bf16_t*) out_any)[o0 + col] = from_f<bf16_t>(acc[t][i] * f);
            }
        }
    }
}

extern "C" int exl3_mix_attn_prefill_mfma(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v_norm,
                                          const void* gate, int64_t gate_ld, const float* sink, const int32_t* cu,
                                          int batch, int max_rows, int heads, int kv_heads, int dim, int vdim, float scale, int window, void* stream)
{
    return exl3_mix_attn_prefill_mfma_ex(out, 0, q, q_ld, k, k_ld, v_norm, (int64_t) kv_heads * vdim, gate, gate_ld, sink, cu, batch, max_rows, heads, kv_heads, 1, dim, vdim,
                                         scale, 0.f, window, EXL3_MIX_MASK_WINDOW, stream);
}

extern "C" int exl3_mix_attn_prefill_mfma_ex(void* out, int out_f32, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v_norm, int64_t v_ld,
                                             const void* gate, int64_t gate_ld, const float* sink, const int32_t* cu,
                                             int batch, int max_rows, int heads, int kv_heads, int maps, int dim, int vdim, float scale, float softcap, int window, int mask,
                                             void* stream)
{
    MIX_CHECK(out && q && k && v_norm && cu, "mix_attn_prefill_mfma: null pointer");
    MIX_CHECK(batch >= 0 && max_rows >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && maps >= 1 && heads * maps <= 65535 && batch <= 65535,
              "mix_attn_prefill_mfma: heads %d / kv_heads %d / batch %d", heads, kv_heads, batch);
    MIX_CHECK((maps == 1 || !gate) && softcap >= 0.f && (mask == EXL3_MIX_MASK_WINDOW || mask == EXL3_MIX_MASK_CHUNK),
              "mix_attn_prefill_mfma: a gate per head applies to one map only; softcap >= 0; mask %d", mask);
    MIX_CHECK(dim > 0 && dim <= 256 && vdim > 0 && vdim <= 256 && window > 0, "mix_attn_prefill_mfma: dim %d and vdim %d must be <= 256", dim, vdim);
    MIX_CHECK(scale > 0.f, "mix_attn_prefill_mfma: the score scale must be positive (the running maximum is taken over raw scores)");
    MIX_CHECK(q_ld >= (int64_t) heads * maps * dim && k_ld >= (int64_t) kv_heads * maps * dim && v_ld >= (int64_t) kv_heads * vdim && (!gate || gate_ld >= heads),
              "mix_attn_prefill_mfma: bad row strides");
    if (batch == 0 || max_rows == 0) return EXL3_MIX_OK;
    const dim3 grid((max_rows + AM_ROWS - 1) / AM_ROWS, batch, heads * maps);
    const int k_vec = ((uintptr_t) k % 16 == 0) && (k_ld % 8 == 0) && (dim % 8 == 0);
    const int v_vec = ((uintptr_t) v_norm % 16 == 0) && (v_ld % 8 == 0) && (vdim % 8 == 0);
    #define AM_LDS(KDV, NVV, KTV) ((size_t) (KTV * (KDV * 32 + AM_PAD) + NVV * 16 * (KTV + AM_PAD)) * sizeof(uint16_t))
    #define AM_LAUNCH_C(KDV, NVV, KTV, CAPV) \
        hipLaunchKernelGGL((attn_prefill_mfma_kernel<KDV, NVV, KTV, CAPV>), grid, dim3(AM_THREADS), AM_LDS(KDV, NVV, KTV), (hipStream_t) stream, out, out_f32, (const bf16_t*) q, q_ld, \
                           (const bf16_t*) k, k_ld, (const bf16_t*) v_norm, v_ld, (const bf16_t*) gate, gate_ld, sink, cu, heads, kv_heads, maps, dim, vdim, scale, softcap, window, mask, \
                           k_vec, v_vec)
    #define AM_LAUNCH(KDV, NVV, KTV) do { \
        static_assert(AM_LDS(KDV, NVV, KTV) <= 65536, "tile does not fit the LDS"); \
        if (softcap > 0.f) AM_LAUNCH_C(KDV, NVV, KTV, true); else AM_LAUNCH_C(KDV, NVV, KTV, false); } while (0)
    const int kd = (dim + 31) / 32, nv = (vdim + 15) / 16;
    if (kd <= 2)      { if (nv <= 4) AM_LAUNCH(2, 4, 64); else if (nv <= 8) AM_LAUNCH(2, 8, 64); else AM_LAUNCH(2, 16, 64); }
    else if (kd <= 4) { if (nv <= 4) AM_LAUNCH(4, 4, 64); else if (nv <= 8) AM_LAUNCH(4, 8, 64); else AM_LAUNCH(4, 16, 64); }
    else              { if (nv <= 4) AM_LAUNCH(8, 4, 64); else if (nv <= 8) AM_LAUNCH(8, 8, 64); else AM_LAUNCH(8, 16, 32); }
    #undef AM_LDS
    #undef AM_LAUNCH
    #undef AM_LAUNCH_C
    return mix_check_launch("mix_attn_prefill_mfma");
}
