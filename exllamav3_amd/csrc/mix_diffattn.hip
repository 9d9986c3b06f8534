// Around the attention core of heads that carry normed, rotated queries and keys and several attention maps per head:
//   qk_prep        per row, for every (head, map): RMS norm of the query / key over its dim with a weight shared by all heads, rotary positions on the first
//                  rot_dims entries (pairs (i, i + rot_dims/2), or interleaved pairs), in place; keys and values of the rows a sequence keeps go into
//                  the slot's rings.
//   diff_combine   differential attention: o = a1 - lambda a2 of a head's two maps, divided by its root mean square over the value dim, times
//                  (1 - diff), times the sigmoid of the head's gate.
// Sums of squares, angles, cos / sin and the combination are float32.
#include "mix_common.cuh"

// One workgroup of QP_WAVES waves per row: cos / sin of the row's position are computed once into LDS, then the waves take the row's items -- q_heads
// query vectors, k_heads key vectors, v_heads value vectors -- in turn.  q [n][q_heads][dim], k [n][k_heads][dim], v [n][v_heads][vdim] are column blocks
// of wider matrices (row strides); q_heads and k_heads count (head, map).  ring_k [slots][window][k_heads][dim], ring_v [slots][window][v_heads][vdim],
// entry = position % window, written for the rows with position >= len_after - window.
#define QP_WAVES 4
template <typename T>
__global__ __launch_bounds__(64 * QP_WAVES) void qk_prep_kernel(T* __restrict__ q, int64_t q_ld, T* __restrict__ k, int64_t k_ld, const T* __restrict__ v, int64_t v_ld,
                                                     const float* __restrict__ q_norm, const float* __restrict__ k_norm, const float* __restrict__ freq, int rot_dims,
                                                     float mag, int interleaved, float eps, T* __restrict__ ring_k, T* __restrict__ ring_v,
                                                     const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ slots,
                                                     const int32_t* __restrict__ len_after, int q_heads, int k_heads, int v_heads, int dim, int vdim, int window)
{
    extern __shared__ float smem[];                           // cos [rot_dims / 2] | sin [rot_dims / 2] | per wave: a vector [dim]
    const int n = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int half = freq ? rot_dims >> 1 : 0;
    float* cs = smem;
    float* sn = smem + half;
    float* buf = smem + 2 * half + wv * dim;
    const int b = tok_seq[n], pos = tok_pos[n];
    const bool keep = pos >= len_after[b] - window;
    const int64_t ring_row = (int64_t) slots[b] * window + (pos % window);
    for (int p = threadIdx.x; p < half; p += 64 * QP_WAVES)
    {
        const float a = (float) pos * freq[p];
        cs[p] = cosf(a) * mag; sn[p] = sinf(a) * mag;
    }
    __syncthreads();
    const int items = q_heads + k_heads + (keep ? v_heads : 0);
    for (int item = wv; item < items; item += QP_WAVES)
    {
        if (item >= q_heads + k_heads)
        {
            const int g = item - q_heads - k_heads;
            const T* vr = v + (int64_t) n * v_ld + (int64_t) g * vdim;
            T* rv = ring_v + (ring_row * v_heads + g) * vdim;
            for (int i = lane; i < vdim; i += 64) rv[i] = vr[i];
            continue;
        }
        const bool is_q = item < q_heads;
        const int head = is_q ? item : item - q_heads;
        T* vec = is_q ? q + (int64_t) n * q_ld + (int64_t) head * dim : k + (int64_t) n * k_ld + (int64_t) head * dim;
        const float* nw = is_q ? q_norm : k_norm;
        float ss = 0.f;
        for (int i = lane; i < dim; i += 64) { const float x = to_f(vec[i]); buf[i] = x; ss += x * x; }
        if (nw)
        {
            ss = wave_sum(ss);
            const float inv = 1.0f / sqrtf(ss / (float) dim + eps);
            for (int i = lane; i < dim; i += 64) buf[i] = buf[i] * inv * nw[i];
        }
        __builtin_amdgcn_wave_barrier();                      // LDS serves a wave's accesses in order: the stores above are visible to the reads below
        for (int p = lane; p < half; p += 64)
        {
            const int i0 = interleaved ? 2 * p : p, i1 = interleaved ? 2 * p + 1 : p + half;
            const float u = buf[i0], w = buf[i1], c = cs[p], s = sn[p];
            buf[i0] = u * c - w * s;
            buf[i1] = w * c + u * s;
        }
        __builtin_amdgcn_wave_barrier();
        T* rk = (!is_q && keep) ? ring_k + (ring_row * k_heads + head) * dim : nullptr;
        for (int i = lane; i < dim; i += 64)
        {
            const T o = from_f<T>(buf[i]);
            vec[i] = o;
            if (rk) rk[i] = o;
        }
        __builtin_amdgcn_wave_barrier();                      // the next item overwrites buf
    }
}

// The same for rows that fit the LDS and allow 16-byte accesses (dim and vdim multiples of VN = 16 / sizeof(T) elements, 16-byte aligned blocks and rings):
// the workgroup loads the row's queries and keys with 16 bytes per lane into LDS (float32), a wave per vector norms and rotates there, and the
// workgroup stores 16 bytes per lane -- queries and keys in place, keys and values into the rings.  LDS: (q_heads + k_heads) * dim + rot_dims floats.
template <typename T> struct qvec;
template <> struct qvec<bf16_t> { static constexpr int N = 8; };
template <> struct qvec<float> { static constexpr int N = 4; };

template <typename T, int QR_WAVES>
__global__ __launch_bounds__(64 * QR_WAVES) void qk_prep_row_kernel(T* __restrict__ q, int64_t q_ld, T* __restrict__ k, int64_t k_ld, const T* __restrict__ v, int64_t v_ld,
                                                         const float* __restrict__ q_norm, const float* __restrict__ k_norm, const float* __restrict__ freq, int rot_dims,
                                                         float mag, int interleaved, float eps, T* __restrict__ ring_k, T* __restrict__ ring_v,
                                                         const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ slots,
                                                         const int32_t* __restrict__ len_after, int q_heads, int k_heads, int v_heads, int dim, int vdim, int window)
{
    constexpr int VN = qvec<T>::N;
    extern __shared__ float smem[];                           // cos [rot_dims / 2] | sin [rot_dims / 2] | the row: q_heads * dim, k_heads * dim
    const int n = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int half = freq ? rot_dims >> 1 : 0;
    float* cs = smem;
    float* sn = smem + half;
    float* row = smem + 2 * half;
    const int b = tok_seq[n], pos = tok_pos[n];
    const bool keep = pos >= len_after[b] - window;
    const int64_t ring_row = (int64_t) slots[b] * window + (pos % window);
    const int nq = q_heads * dim, nk = k_heads * dim, nv = v_heads * vdim;
    T* qr = q + (int64_t) n * q_ld;
    T* kr = k + (int64_t) n * k_ld;
    for (int i = threadIdx.x * VN; i < nq + nk; i += 64 * QR_WAVES * VN)
    {
        union { uint4 v; T e[VN]; } t;
        t.v = *(const uint4*) (i < nq ? qr + i : kr + (i - nq));
        #pragma unroll
        for (int e = 0; e < VN; ++e) row[i + e] = to_f(t.e[e]);
    }
    if (keep)                                                 // values: straight into the ring
    {
        const T* vr = v + (int64_t) n * v_ld;
        T* rv = ring_v + ring_row * nv;
        for (int i = threadIdx.x * VN; i < nv; i += 64 * QR_WAVES * VN) *(uint4*) (rv + i) = *(const uint4*) (vr + i);
    }
    for (int p = threadIdx.x; p < half; p += 64 * QR_WAVES)
    {
        float sv, cv;
        sincosf((float) pos * freq[p], &sv, &cv);
        cs[p] = cv * mag; sn[p] = sv * mag;
    }
    __syncthreads();
    for (int item = wv; item < q_heads + k_heads; item += QR_WAVES)
    {
        float* buf = row + item * dim;
        const float* nw = item < q_heads ? q_norm : k_norm;
        if (nw)
        {
            float ss = 0.f;
            for (int i = lane; i < dim; i += 64) { const float x = buf[i]; ss += x * x; }
            ss = wave_sum(ss);
            const float inv = 1.0f / sqrtf(ss / (float) dim + eps);
            for (int i = lane; i < dim; i += 64) buf[i] = buf[i] * inv * nw[i];
            __builtin_amdgcn_wave_barrier();                  // LDS serves a wave's accesses in order: the stores above are visible to the reads below
        }
        for (int p = lane; p < half; p += 64)
        {
            const int i0 = interleaved ? 2 * p : p, i1 = interleaved ? 2 * p + 1 : p + half;
            const float u = buf[i0], w = buf[i1], c = cs[p], s = sn[p];
            buf[i0] = u * c - w * s;
            buf[i1] = w * c + u * s;
        }
    }
    __syncthreads();
    T* rk = keep ? ring_k + ring_row * nk : nullptr;
    for (int i = threadIdx.x * VN; i < nq + nk; i += 64 * QR_WAVES * VN)
    {
        union { uint4 v; T e[VN]; } t;
        #pragma unroll
        for (int e = 0; e < VN; ++e) t.e[e] = from_f<T>(row[i + e]);
        if (i < nq) *(uint4*) (qr + i) = t.v;
        else
        {
            *(uint4*) (kr + (i - nq)) = t.v;
            if (rk) *(uint4*) (rk + (i - nq)) = t.v;
        }
    }
}

// a [n][heads][2][vdim] (float32): out[n][h * vdim + c] = o_c / sqrt(mean_c(o^2) + eps) * (1 - diff) * sigmoid(gate[n][h]), o = a[.,0] - lambda a[.,1]
template <typename T>
__global__ __launch_bounds__(64) void diff_combine_kernel(T* __restrict__ out, const float* __restrict__ a, float lambda, float diff, float eps, const T* __restrict__ gate,
                                                          int64_t gate_ld, int heads, int vdim)
{
    const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* a1 = a + ((int64_t) n * heads + h) * 2 * vdim;
    const float* a2 = a1 + vdim;
    float ss = 0.f;
    for (int c = lane; c < vdim; c += 64) { const float o = a1[c] - lambda * a2[c]; ss += o * o; }
    ss = wave_sum(ss);
    float f = (1.0f - diff) / sqrtf(ss / (float) vdim + eps);
    if (gate) f *= sigmoid_f(to_f(gate[(int64_t) n * gate_ld + h]));
    T* o_row = out + ((int64_t) n * heads + h) * vdim;
    for (int c = lane; c < vdim; c += 64) o_row[c] = from_f<T>((a1[c] - lambda * a2[c]) * f);
}

extern "C" int exl3_mix_qk_prep(void* q, int64_t q_ld, void* k, int64_t k_ld, const void* v, int64_t v_ld, const float* q_norm, const float* k_norm,
                                const float* freq, int rot_dims, float mag, int interleaved, float eps, void* ring_k, void* ring_v,
                                const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* len_after,
                                int n, int q_heads, int k_heads, int v_heads, int dim, int vdim, int window, int dtype, void* stream)
{
    MIX_CHECK(q && k && v && ring_k && ring_v && tok_seq && tok_pos && slots && len_after, "mix_qk_prep: null pointer");
    MIX_CHECK(n >= 0 && q_heads > 0 && k_heads > 0 && v_heads > 0 && dim > 0 && dim <= 2048 && vdim > 0 && window > 0,
              "mix_qk_prep: bad sizes");
    MIX_CHECK(q_ld >= (int64_t) q_heads * dim && k_ld >= (int64_t) k_heads * dim && v_ld >= (int64_t) v_heads * vdim, "mix_qk_prep: bad row strides");
    MIX_CHECK(!freq || (rot_dims >= 2 && rot_dims % 2 == 0 && rot_dims <= dim), "mix_qk_prep: %d rotated entries of %d", rot_dims, dim);
    if (n == 0) return EXL3_MIX_OK;
    const int vn = dtype == EXL3_MIX_BF16 ? 8 : 4;
    const size_t sm_row = (size_t) ((freq ? rot_dims : 0) + (int64_t) (q_heads + k_heads) * dim) * sizeof(float);
    const bool by16 = dim % vn == 0 && vdim % vn == 0 && q_ld % vn == 0 && k_ld % vn == 0 && v_ld % vn == 0 && (uintptr_t) q % 16 == 0 && (uintptr_t) k % 16 == 0 &&
                      (uintptr_t) v % 16 == 0 && (uintptr_t) ring_k % 16 == 0 && (uintptr_t) ring_v % 16 == 0 && sm_row <= 48 * 1024;
    if (by16)
    {
        // few rows (steps of one row per sequence): sixteen waves share a row's vectors, the step is bound by the chain a wave walks; many rows: four
        #define QR_LAUNCH(NWV) \
            MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((qk_prep_row_kernel<T, NWV>), dim3(n), dim3(64 * NWV), sm_row, (hipStream_t) stream, \
                                                     (T*) q, q_ld, (T*) k, k_ld, (const T*) v, v_ld, q_norm, k_norm, freq, rot_dims, mag, interleaved, eps, (T*) ring_k, (T*) ring_v, \
                                                     tok_seq, tok_pos, slots, len_after, q_heads, k_heads, v_heads, dim, vdim, window))
        if (n <= 64) QR_LAUNCH(16); else QR_LAUNCH(4);
        #undef QR_LAUNCH
        return mix_check_launch("mix_qk_prep");
    }
    const size_t sm = (size_t) ((freq ? rot_dims : 0) + QP_WAVES * dim) * sizeof(float);
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(qk_prep_kernel<T>, dim3(n), dim3(64 * QP_WAVES), sm, (hipStream_t) stream,
                                             (T*) q, q_ld, (T*) k, k_ld, (const T*) v, v_ld, q_norm, k_norm, freq, rot_dims, mag, interleaved, eps, (T*) ring_k, (T*) ring_v,
                                             tok_seq, tok_pos, slots, len_after, q_heads, k_heads, v_heads, dim, vdim, window));
    return mix_check_launch("mix_qk_prep");
}

extern "C" int exl3_mix_diff_combine(void* out, const float* a, float lambda, float diff, float eps, const void* gate, int64_t gate_ld,
                                     int n, int heads, int vdim, int dtype, void* stream)
{
    MIX_CHECK(out && a && n >= 0 && heads > 0 && heads <= 65535 && vdim > 0 && (!gate || gate_ld >= heads), "mix_diff_combine: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(diff_combine_kernel<T>, dim3(n, heads), dim3(64), 0, (hipStream_t) stream, (T*) out, a, lambda, diff, eps, (const T*) gate, gate_ld,
                                             heads, vdim));
    return mix_check_launch("mix_diff_combine");
}
