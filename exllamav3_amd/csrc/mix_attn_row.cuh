// The row worker of the lane-per-key attention kernels (exact float32 scores and softmax): shared by the sliding-window kernels of mix_attn.hip
// and the latent-cache decode kernel of mix_latent.hip.
#pragma once
#include "mix_common.cuh"

// One workgroup of NW waves (AT_WAVES unless the caller asks for more: few rows, long caches) per (row, query head).  Keys kb + j * k_step, values vb + j * v_step, j < count: wave w takes the 64-key chunks
// w, w + NW, ... (one key per lane, its row read in 16-byte pieces when the layout allows), keeps its own running maximum, sum and
// value accumulators (MAXV = ceil(vdim / 64) per lane), and the waves are merged through LDS at the end.  Wave 0 starts from the sink.
// The query's first dim1 elements are read from q, the rest from q2 (dim1 = dim: one part).  softcap > 0: score <- softcap tanh(score / softcap).
// TO: the element type of the result (float keeps the weighted sum unrounded for a caller that combines several maps).
#define AT_WAVES 4

template <typename T> struct kvec;
template <> struct kvec<bf16_t> { static constexpr int N = 8; };
template <> struct kvec<float> { static constexpr int N = 4; };

template <typename T, int MAXV, typename TO = T, int NW = AT_WAVES>
__device__ __forceinline__ void attn_row(TO* __restrict__ out, const T* __restrict__ q, const T* q2, int dim1, const T* __restrict__ kb, int64_t k_step, const T* __restrict__ vb,
                                         int64_t v_step, int count, int dim, int vdim, float scale, bool has_sink, float sink, float gate, bool k_vec,
                                         float* smem, float softcap = 0.f)
{
    float* qs = smem;                                   // [dim]
    float* ps = qs + dim;                               // [NW][64]
    float* mg = ps + NW * 64;                     // [NW][2 + MAXV * 64]: m, l, accumulators
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < dim; i += 64 * NW) qs[i] = to_f(i < dim1 ? q[i] : q2[i - dim1]);      // the query may come in two parts
    __syncthreads();
    const bool seeded = has_sink && w == 0;
    float m = seeded ? sink : -INFINITY, l = seeded ? 1.0f : 0.0f;
    float acc[MAXV];
    #pragma unroll
    for (int i = 0; i < MAXV; ++i) acc[i] = 0.f;
    float* pw = ps + w * 64;
    constexpr int VN = kvec<T>::N;
    for (int j0 = w * 64; j0 < count; j0 += 64 * NW)
    {
        const int j = j0 + lane;
        float s = -INFINITY;
        if (j < count)
        {
            const T* kr = kb + (int64_t) j * k_step;
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
            s = d * scale;
            if (softcap > 0.f) s = softcap * tanhf(s / softcap);
        }
        const float m_new = fmaxf(m, wave_max(s));          // finite: j0 < count, so lane 0 of the chunk holds a score
        const float p = (j < count) ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);                 // m = -inf (nothing yet): 0
        l = l * corr + wave_sum(p);
        m = m_new;
        pw[lane] = p;
        __builtin_amdgcn_wave_barrier();                    // LDS serves a wave's accesses in order: its own stores are visible to the reads below
        const int cnt = min(64, count - j0);
        #pragma unroll
        for (int i = 0; i < MAXV; ++i)
        {
            const int c = lane + 64 * i;
            float a = acc[i] * corr;
            if (c < vdim)
            {
                int jj = 0;
                for (; jj + 8 <= cnt; jj += 8)                // eight value rows in flight, then the sums
                {
                    float vv[8];
                    #pragma unroll
                    for (int e = 0; e < 8; ++e) vv[e] = to_f(vb[(int64_t) (j0 + jj + e) * v_step + c]);
                    #pragma unroll
                    for (int e = 0; e < 8; ++e) a += pw[jj + e] * vv[e];
                }
                for (; jj < cnt; ++jj) a += pw[jj] * to_f(vb[(int64_t) (j0 + jj) * v_step + c]);
            }
            acc[i] = a;
        }
        __builtin_amdgcn_wave_barrier();
    }
    // merge the waves: wave 0 rescales every wave's partial to the common maximum
    float* mine = mg + w * (2 + MAXV * 64);
    if (lane == 0) { mine[0] = m; mine[1] = l; }
    #pragma unroll
    for (int i = 0; i < MAXV; ++i) mine[2 + i * 64 + lane] = acc[i];
    __syncthreads();
    if (w != 0) return;
    float mt = -INFINITY;
    #pragma unroll
    for (int ww = 0; ww < NW; ++ww) mt = fmaxf(mt, mg[ww * (2 + MAXV * 64)]);
    float lt = 0.f;
    #pragma unroll
    for (int i = 0; i < MAXV; ++i) acc[i] = 0.f;
    #pragma unroll
    for (int ww = 0; ww < NW; ++ww)
    {
        const float* o = mg + ww * (2 + MAXV * 64);
        const float f = (o[0] == -INFINITY) ? 0.f : expf(o[0] - mt);
        lt += o[1] * f;
        #pragma unroll
        for (int i = 0; i < MAXV; ++i) acc[i] += o[2 + i * 64 + lane] * f;
    }
    const float f = (lt > 0.f ? 1.0f / lt : 0.f) * gate;
    #pragma unroll
    for (int i = 0; i < MAXV; ++i)
    {
        const int c = lane + 64 * i;
        if (c < vdim) out[c] = from_f<TO>(acc[i] * f);
    }
}

template <typename T>
__device__ __forceinline__ bool rows_are_16_byte(const T* base, int64_t step, int dim)
{
    return ((uintptr_t) base % 16 == 0) && ((step * (int64_t) sizeof(T)) % 16 == 0) && (dim % kvec<T>::N == 0);
}

