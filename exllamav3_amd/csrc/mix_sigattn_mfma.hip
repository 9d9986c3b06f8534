// Prompt steps of the causal attention without softmax on the matrix cores (bfloat16 activations): scores = Q K^T and the weighted sum P V with
// v_mfma_f32_16x16x32_bf16; scores and the weights sigmoid(scale score + bias_head) are float32, the weights are rounded to bfloat16 only as operands of
// the second product, whose sums are float32 again.  There is no running maximum, no sum of weights and nothing to rescale: a tile's weights go straight
// into the accumulators.
//
// One workgroup = 128 query rows of one sequence and one head, 8 waves of 16 rows.  Key tiles of 64 rows (32 for the largest heads) are staged in LDS
// once for the eight waves: K as stored, V transposed (value column, key).  The scores are computed TRANSPOSED, S^T = K Q^T (keys are rows, the wave's 16
// queries are columns), so the result registers of two 16-key tiles are, as they stand, the B operand of O^T = V^T P^T when contraction slot (g, e) is
// read as key 4g + e of the first tile (e < 4) or of the second (e >= 4); the A operand V^T is read from LDS in the same key order.  No weight goes
// through LDS.  Every row sees the keys from the sequence's start, so a block visits the tiles 0 .. its last row, and only the tile on the diagonal
// needs a mask.
#include "mix_common.cuh"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

#define SM_ROWS 128
#define SM_THREADS 512
#define SM_PAD 8
#define SM_LOG2E 1.4426950408889634f

// KD: contraction steps of 32 over the (zero-padded) head dim; NV: 16-column tiles of the (padded) value dim.
template <int KD, int NV, int SM_KEYS>
__global__ __launch_bounds__(SM_THREADS) void sigattn_prefill_mfma_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int64_t q_ld, const bf16_t* __restrict__ k,
                                                                          int64_t k_ld, const bf16_t* __restrict__ v, int64_t v_ld, const float* __restrict__ bias,
                                                                          const int32_t* __restrict__ cu, int heads, int kv_heads, int dim, int vdim, float scale, int k_vec, int v_vec)
{
    constexpr int DP = KD * 32, KS = DP + SM_PAD, VS = SM_KEYS + SM_PAD;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t* k_lds = (uint16_t*) smem_raw;                       // [SM_KEYS][KS]
    uint16_t* vt_lds = k_lds + SM_KEYS * KS;                      // [NV * 16][VS]   (value column, key)

    const int b = blockIdx.y, h = blockIdx.z;
    const int first = cu[b], len = cu[b + 1] - first;
    const int q0 = ((int) gridDim.x - 1 - (int) blockIdx.x) * SM_ROWS;      // the blocks with the most keys start first
    if (q0 >= len) return;
    const int vh = h / (heads / kv_heads);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;

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
    const int wq_lo = q0 + w * 16, wq_hi = min(q0 + w * 16 + 15, len - 1);
    const bool wave_live = wq_lo < len;
    const int qi = q0 + w * 16 + c;
    // weight = 1 / (1 + 2^(-(scale s + bias) log2 e)): one multiply-add, one v_exp_f32 and one reciprocal per key
    const float c2 = -scale * SM_LOG2E, off = -(bias ? bias[h] : 0.f) * SM_LOG2E;
    f32x4 acc[NV];
    #pragma unroll
    for (int t = 0; t < NV; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int blk_hi = min(q0 + SM_ROWS - 1, len - 1);
    for (int j0 = 0; j0 <= blk_hi; j0 += SM_KEYS)
    {
        __syncthreads();
        for (int idx = threadIdx.x; idx < SM_KEYS * (DP / 8); idx += SM_THREADS)
        {
            const int r = idx / (DP / 8), cg = idx - r * (DP / 8);
            const int j = j0 + r;
            const bf16_t* src = k + (int64_t) (first + min(j, len - 1)) * k_ld + (int64_t) vh * dim + cg * 8;
            union { uint4 v; uint16_t u[8]; } t;
            if (k_vec && j < len && cg * 8 + 8 <= dim) t.v = *(const uint4*) src;
            else
            {
                #pragma unroll
                for (int e = 0; e < 8; ++e) t.u[e] = (j < len && cg * 8 + e < dim) ? src[e].u : (uint16_t) 0;
            }
            *(uint4*) (k_lds + r * KS + cg * 8) = t.v;
        }
        for (int idx = threadIdx.x; idx < SM_KEYS * NV * 2; idx += SM_THREADS)
        {
            const int cg = idx / SM_KEYS, r = idx - cg * SM_KEYS;
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
        const bool skip = !wave_live || j0 > wq_hi;                 // keys behind every row of the wave
        if (!skip)
        {
            constexpr int NS = SM_KEYS / 16;
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
            // sc[u][i] = raw score of key j0 + 16u + 4g + i against query qi
            const bool interior = j0 + SM_KEYS - 1 <= wq_lo && q0 + w * 16 + 15 < len;
            #pragma unroll
            for (int u = 0; u < NS; ++u)
            {
                #pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    const float p = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(sc[u][i] * c2 + off));
                    const int j = j0 + u * 16 + g * 4 + i;
                    sc[u][i] = (interior || (j <= qi && qi < len)) ? p : 0.f;
                }
            }
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
    if (!wave_live || qi >= len) return;
    const int64_t o0 = ((int64_t) (first + qi) * heads + h) * vdim;
    #pragma unroll
    for (int t = 0; t < NV; ++t)
    {
        #pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            const int col = t * 16 + g * 4 + i;
            if (col < vdim) out[o0 + col] = from_f<bf16_t>(acc[t][i]);
        }
    }
}

extern "C" int exl3_mix_sigattn_prefill_mfma(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld, const float* bias,
                                             const int32_t* cu, int batch, int max_rows, int heads, int kv_heads, int dim, int vdim, float scale, void* stream)
{
    MIX_CHECK(out && q && k && v && cu, "mix_sigattn_prefill_mfma: null pointer");
    MIX_CHECK(batch >= 0 && max_rows >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && heads <= 65535 && batch <= 65535,
              "mix_sigattn_prefill_mfma: heads %d / kv_heads %d / batch %d", heads, kv_heads, batch);
    MIX_CHECK(dim > 0 && dim <= 256 && vdim > 0 && vdim <= 256, "mix_sigattn_prefill_mfma: dim %d and vdim %d must be <= 256", dim, vdim);
    MIX_CHECK(q_ld >= (int64_t) heads * dim && k_ld >= (int64_t) kv_heads * dim && v_ld >= (int64_t) kv_heads * vdim, "mix_sigattn_prefill_mfma: bad row strides");
    if (batch == 0 || max_rows == 0) return EXL3_MIX_OK;
    const dim3 grid((max_rows + SM_ROWS - 1) / SM_ROWS, batch, heads);
    const int k_vec = ((uintptr_t) k % 16 == 0) && (k_ld % 8 == 0) && (dim % 8 == 0);
    const int v_vec = ((uintptr_t) v % 16 == 0) && (v_ld % 8 == 0) && (vdim % 8 == 0);
    #define SM_LDS(KDV, NVV, KTV) ((size_t) (KTV * (KDV * 32 + SM_PAD) + NVV * 16 * (KTV + SM_PAD)) * sizeof(uint16_t))
    #define SM_LAUNCH(KDV, NVV, KTV) do { \
        static_assert(SM_LDS(KDV, NVV, KTV) <= 65536, "tile does not fit the LDS"); \
        hipLaunchKernelGGL((sigattn_prefill_mfma_kernel<KDV, NVV, KTV>), grid, dim3(SM_THREADS), SM_LDS(KDV, NVV, KTV), (hipStream_t) stream, (bf16_t*) out, (const bf16_t*) q, q_ld, \
                           (const bf16_t*) k, k_ld, (const bf16_t*) v, v_ld, bias, cu, heads, kv_heads, dim, vdim, scale, k_vec, v_vec); } while (0)
    const int kd = (dim + 31) / 32, nv = (vdim + 15) / 16;
    if (kd <= 2)      { if (nv <= 4) SM_LAUNCH(2, 4, 64); else if (nv <= 8) SM_LAUNCH(2, 8, 64); else SM_LAUNCH(2, 16, 64); }
    else if (kd <= 4) { if (nv <= 4) SM_LAUNCH(4, 4, 64); else if (nv <= 8) SM_LAUNCH(4, 8, 64); else SM_LAUNCH(4, 16, 64); }
    else              { if (nv <= 4) SM_LAUNCH(8, 4, 64); else if (nv <= 8) SM_LAUNCH(8, 8, 64); else SM_LAUNCH(8, 16, 32); }
    #undef SM_LDS
    #undef SM_LAUNCH
    return mix_check_launch("mix_sigattn_prefill_mfma");
}
