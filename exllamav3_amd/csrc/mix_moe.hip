// Unquantized experts.  A few rows (decode, short prompts): one wave per output element streams the chosen expert's weight row, sums in
// float32.  Many rows (prompts): the host sorts the rows by expert and runs one vendor matrix product per expert and projection; the
// activation between them and the weighted un-sort are the two small kernels at the end of this file.
#include "mix_common.cuh"

template <typename T> struct vecn;
template <> struct vecn<bf16_t> { static constexpr int N = 8; };
template <> struct vecn<float> { static constexpr int N = 4; };

// dot products of one activation row with up to two weight rows, 16 bytes per lane and load (rows 16-byte aligned, length a multiple of the vector)
template <typename T, bool TWO>
__device__ __forceinline__ void dot_rows(const T* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b, int len, bool vec, float& ra, float& rb)
{
    constexpr int VN = vecn<T>::N;
    const int lane = threadIdx.x & 63;
    float sa = 0.f, sb = 0.f;
    if (vec)
    {
        for (int c = lane * VN; c < len; c += 64 * VN)
        {
            union { uint4 v; T e[VN]; } tx, ta, tb;
            tx.v = *(const uint4*) (x + c); ta.v = *(const uint4*) (a + c);
            if (TWO) tb.v = *(const uint4*) (b + c);
            #pragma unroll
            for (int e = 0; e < VN; ++e)
            {
                const float xv = to_f(tx.e[e]);
                sa += xv * to_f(ta.e[e]);
                if (TWO) sb += xv * to_f(tb.e[e]);
            }
        }
    }
    else
    {
        for (int c = lane; c < len; c += 64)
        {
            const float xv = to_f(x[c]);
            sa += xv * to_f(a[c]);
            if (TWO) sb += xv * to_f(b[c]);
        }
    }
    ra = wave_sum(sa);
    if (TWO) rb = wave_sum(sb);
}

// GATED: hid = glu(Wg h, Wu h) (EXL3_MIX_GLU_*); otherwise hid = act(Wu h) (EXL3_MIX_ACT_*), wg unused.  A choice that names no stored expert
// (idx outside 0 .. experts-1: an expert without weights, handled by the caller) is skipped.
template <typename T, bool GATED>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(T* __restrict__ hid, const T* __restrict__ h, const T* __restrict__ wg, const T* __restrict__ wu,
                                                          const int32_t* __restrict__ idx, int experts, int ff, int width, int top, int vec, int act, float limit)
{
    const int row = blockIdx.x;                              // n * top + r
    const int j = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (j >= ff) return;
    const int lane = threadIdx.x & 63;
    const int e = idx[row];
    if (e < 0 || e >= experts) return;
    const T* x = h + (int64_t) (row / top) * width;
    const T* u = wu + ((int64_t) e * ff + j) * width;
    const T* g = GATED ? wg + ((int64_t) e * ff + j) * width : u;
    float ag = 0.f, au;
    if (GATED) dot_rows<T, true>(x, g, u, width, vec != 0, ag, au);
    else       dot_rows<T, false>(x, u, u, width, vec != 0, au, ag);
    // the projections leave the matrix product in the activation type before the activation, like any other linear of the model
    if (lane == 0)
        hid[(int64_t) row * ff + j] = from_f<T>(GATED ? glu_act_f(to_f(from_f<T>(ag)), to_f(from_f<T>(au)), act, limit) : act_f(to_f(from_f<T>(au)), act));
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(T* __restrict__ y, const T* __restrict__ hid, const T* __restrict__ wd, const int32_t* __restrict__ idx,
                                                       const float* __restrict__ wts, int experts, int ff, int width, int top, int vec,
                                                       const T* __restrict__ h_id, const float* __restrict__ idw)
{
    const int n = blockIdx.x;
    const int col = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (col >= width) return;
    const int lane = threadIdx.x & 63;
    float acc = 0.f;
    for (int r = 0; r < top; ++r)
    {
        const int e = idx[(int64_t) n * top + r];
        if (e < 0 || e >= experts) continue;
        const T* hr = hid + ((int64_t) n * top + r) * ff;
        const T* wr = wd + ((int64_t) e * width + col) * ff;
        float a, unused;
        dot_rows<T, false>(hr, wr, wr, ff, vec != 0, a, unused);
        acc += wts[(int64_t) n * top + r] * a;
    }
    if (idw) acc += idw[n] * to_f(h_id[(int64_t) n * width + col]);         // experts that return their input, with the sum of their weights
    if (lane == 0) y[(int64_t) n * width + col] = from_f<T>(acc);
}

template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ g, const T* __restrict__ u, int64_t count)
{
    for (int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t) gridDim.x * 256)
        out[i] = from_f<T>(silu_f(to_f(g[i])) * to_f(u[i]));
}

// y[n] = sum_r wts[n][r] * sorted[where[n*top + r]]: the rows of the expert-sorted result back in token order, weighted.  With idx, choices outside
// 0 .. experts-1 have no row in `sorted` and are left out; with idw, y[n] += idw[n] * h_id[n] (experts that return their input).
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(T* __restrict__ y, const T* __restrict__ sorted, const int32_t* __restrict__ where,
                                                          const float* __restrict__ wts, int top, int width, const int32_t* __restrict__ idx, int experts,
                                                          const T* __restrict__ h_id, const float* __restrict__ idw)
{
    const int n = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += 256)
    {
        float acc = 0.f;
        for (int r = 0; r < top; ++r)
        {
            if (idx) { const int e = idx[(int64_t) n * top + r]; if (e < 0 || e >= experts) continue; }
            acc += wts[(int64_t) n * top + r] * to_f(sorted[(int64_t) where[(int64_t) n * top + r] * width + c]);
        }
        if (idw) acc += idw[n] * to_f(h_id[(int64_t) n * width + c]);
        y[(int64_t) n * width + c] = from_f<T>(acc);
    }
}

// Expert-major form for a handful to a few dozen rows: one workgroup per (expert, four outputs).  The rows that chose the expert are listed in
// LDS first; a wave then reads each 16-byte piece of ITS weight row(s) once and multiplies it with the same piece of up to EM_ROWS listed
// rows (their activations come from L1 / L2), so an expert's weights are streamed once however many rows use it.  Needs the 16-byte layout.
#define EM_ROWS 8

__device__ __forceinline__ int em_list_rows(int* list, const int32_t* __restrict__ idx, int n_rows, int e)
{
    // wave 0 compacts the matching (row, choice) indices in order; every thread gets the count
    __shared__ int cnt_s;
    const int lane = threadIdx.x & 63;
    if ((threadIdx.x >> 6) == 0)
    {
        int c = 0;
        for (int base = 0; base < n_rows; base += 64)
        {
            const int r = base + lane;
            const bool hit = r < n_rows && idx[r] == e;
            const unsigned long long mask = __ballot(hit);
            if (hit) list[c + __popcll(mask & ((1ull << lane) - 1ull))] = r;
            c += __popcll(mask);
        }
        if (lane == 0) cnt_s = c;
    }
    __syncthreads();
    return cnt_s;
}

template <typename T, bool GATED>
__global__ __launch_bounds__(256) void moe_gate_up_em_kernel(T* __restrict__ hid, const T* __restrict__ h, const T* __restrict__ wg, const T* __restrict__ wu,
                                                             const int32_t* __restrict__ idx, int n_rows, int ff, int width, int top, int act, float limit)
{
    extern __shared__ int em_list[];
    constexpr int VN = vecn<T>::N;
    const int e = blockIdx.x, j = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int cnt = em_list_rows(em_list, idx, n_rows, e);
    if (cnt == 0 || j >= ff) return;
    const T* u = wu + ((int64_t) e * ff + j) * width;
    const T* g = GATED ? wg + ((int64_t) e * ff + j) * width : u;
    for (int r0 = blockIdx.z * EM_ROWS; r0 < cnt; r0 += gridDim.z * EM_ROWS)      // a long list is shared by the workgroups along z
    {
        float sa[EM_ROWS], sb[EM_ROWS];
        #pragma unroll
        for (int m = 0; m < EM_ROWS; ++m) { sa[m] = 0.f; sb[m] = 0.f; }
        for (int c = lane * VN; c < width; c += 64 * VN)
        {
            union { uint4 v; T e[VN]; } tg, tu;
            tu.v = *(const uint4*) (u + c);
            if (GATED) tg.v = *(const uint4*) (g + c); else tg.v = tu.v;
            #pragma unroll
            for (int m = 0; m < EM_ROWS; ++m)
            {
                if (r0 + m < cnt)
                {
                    union { uint4 v; T e[VN]; } tx;
                    tx.v = *(const uint4*) (h + (int64_t) (em_list[r0 + m] / top) * width + c);
                    #pragma unroll
                    for (int q = 0; q < VN; ++q)
                    {
                        const float xv = to_f(tx.e[q]);
                        if (GATED) sa[m] += xv * to_f(tg.e[q]);
                        sb[m] += xv * to_f(tu.e[q]);
                    }
                }
            }
        }
        #pragma unroll
        for (int m = 0; m < EM_ROWS; ++m)
        {
            if (r0 + m < cnt)
            {
                const float ag = GATED ? wave_sum(sa[m]) : 0.f, au = wave_sum(sb[m]);
                if (lane == 0)
                    hid[(int64_t) em_list[r0 + m] * ff + j] = from_f<T>(GATED ? glu_act_f(to_f(from_f<T>(ag)), to_f(from_f<T>(au)), act, limit) : act_f(to_f(from_f<T>(au)), act));
            }
        }
    }
}

// per[(row, choice)][col] = Wd[expert][col] . hid[(row, choice)] (unweighted; exl3_mix_moe_combine adds the choices with their weights)
template <typename T>
__global__ __launch_bounds__(256) void moe_down_em_kernel(T* __restrict__ per, const T* __restrict__ hid, const T* __restrict__ wd, const int32_t* __restrict__ idx,
                                                          int n_rows, int ff, int width)
{
    extern __shared__ int em_list[];
    constexpr int VN = vecn<T>::N;
    const int e = blockIdx.x, col = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int cnt = em_list_rows(em_list, idx, n_rows, e);
    if (cnt == 0 || col >= width) return;
    const T* wr = wd + ((int64_t) e * width + col) * ff;
    for (int r0 = blockIdx.z * EM_ROWS; r0 < cnt; r0 += gridDim.z * EM_ROWS)      // a long list is shared by the workgroups along z
    {
        float sa[EM_ROWS];
        #pragma unroll
        for (int m = 0; m < EM_ROWS; ++m) sa[m] = 0.f;
        for (int c = lane * VN; c < ff; c += 64 * VN)
        {
            union { uint4 v; T e[VN]; } tw;
            tw.v = *(const uint4*) (wr + c);
            #pragma unroll
            for (int m = 0; m < EM_ROWS; ++m)
            {
                if (r0 + m < cnt)
                {
                    union { uint4 v; T e[VN]; } tx;
                    tx.v = *(const uint4*) (hid + (int64_t) em_list[r0 + m] * ff + c);
                    #pragma unroll
                    for (int q = 0; q < VN; ++q) sa[m] += to_f(tx.e[q]) * to_f(tw.e[q]);
                }
            }
        }
        #pragma unroll
        for (int m = 0; m < EM_ROWS; ++m)
        {
            if (r0 + m < cnt)
            {
                const float a = wave_sum(sa[m]);
                if (lane == 0) per[(int64_t) em_list[r0 + m] * width + col] = from_f<T>(a);
            }
        }
    }
}

static int moe_expert_major(void* per, void* hid, const void* h, const void* wg, const void* wu, const void* wd, const int32_t* idx,
                            int n, int top, int experts, int ff, int width, bool gated, int act, float limit, int dtype, void* stream)
{
    if (gated) MIX_CHECK(act == EXL3_MIX_GLU_SILU || act == EXL3_MIX_GLU_CLAMPED_SWISH, "mix_moe_expert_major: unknown gated activation %d", act);
    else       MIX_CHECK(act >= EXL3_MIX_ACT_RELU2 && act <= EXL3_MIX_ACT_SILU, "mix_moe_expert_major: unknown activation %d", act);
    if (!gated) wg = wu;
    MIX_CHECK(per && hid && h && wg && wu && wd && idx && n >= 0 && top > 0 && experts > 0 && ff > 0 && width > 0, "mix_moe_expert_major: bad arguments");
    const int vn = dtype == EXL3_MIX_BF16 ? 8 : 4;
    MIX_CHECK(width % vn == 0 && ff % vn == 0 && (uintptr_t) h % 16 == 0 && (uintptr_t) wg % 16 == 0 && (uintptr_t) wu % 16 == 0 && (uintptr_t) wd % 16 == 0 &&
              (uintptr_t) hid % 16 == 0, "mix_moe_expert_major: rows must be 16-byte aligned multiples of %d elements", vn);
    MIX_CHECK((int64_t) n * top <= 8192, "mix_moe_expert_major: at most 8192 (row, choice) pairs");
    if (n == 0) return EXL3_MIX_OK;
    const int n_rows = n * top;
    const size_t sm = (size_t) n_rows * sizeof(int);
    const int gz = (n_rows + 2 * EM_ROWS - 1) / (2 * EM_ROWS);          // enough workgroups along z that a list of all rows is walked in two turns
    if (gated)
        MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((moe_gate_up_em_kernel<T, true>), dim3(experts, (ff + 3) / 4, gz), dim3(256), sm, (hipStream_t) stream, (T*) hid, (const T*) h,
                                                 (const T*) wg, (const T*) wu, idx, n_rows, ff, width, top, act, limit));
    else
        MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((moe_gate_up_em_kernel<T, false>), dim3(experts, (ff + 3) / 4, gz), dim3(256), sm, (hipStream_t) stream, (T*) hid, (const T*) h,
                                                 (const T*) wg, (const T*) wu, idx, n_rows, ff, width, top, act, limit));
    if (int rc = mix_check_launch("mix_moe_expert_major (gate, up)")) return rc;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(moe_down_em_kernel<T>, dim3(experts, (width + 3) / 4, gz), dim3(256), sm, (hipStream_t) stream, (T*) per, (const T*) hid,
                                             (const T*) wd, idx, n_rows, ff, width));
    return mix_check_launch("mix_moe_expert_major (down)");
}

extern "C" int exl3_mix_moe_expert_major_act(void* per, void* hid, const void* h, const void* wg, const void* wu, const void* wd, const int32_t* idx,
                                             int n, int top, int experts, int ff, int width, int act, float limit, int dtype, void* stream)
{
    return moe_expert_major(per, hid, h, wg, wu, wd, idx, n, top, experts, ff, width, true, act, limit, dtype, stream);
}

extern "C" int exl3_mix_moe_expert_major_plain(void* per, void* hid, const void* h, const void* wu, const void* wd, const int32_t* idx,
                                               int n, int top, int experts, int ff, int width, int act, int dtype, void* stream)
{
    return moe_expert_major(per, hid, h, nullptr, wu, wd, idx, n, top, experts, ff, width, false, act, 0.f, dtype, stream);
}

extern "C" int exl3_mix_moe_expert_major(void* per, void* hid, const void* h, const void* wg, const void* wu, const void* wd, const int32_t* idx,
                                         int n, int top, int experts, int ff, int width, int dtype, void* stream)
{
    return exl3_mix_moe_expert_major_act(per, hid, h, wg, wu, wd, idx, n, top, experts, ff, width, EXL3_MIX_GLU_SILU, 0.f, dtype, stream);
}

extern "C" int exl3_mix_silu_mul(void* out, const void* g, const void* u, int64_t count, int dtype, void* stream)
{
    MIX_CHECK(out && g && u && count >= 0, "mix_silu_mul: bad arguments");
    if (count == 0) return EXL3_MIX_OK;
    const int blocks = (int) ((count + 255) / 256 > 8192 ? 8192 : (count + 255) / 256);
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(silu_mul_kernel<T>, dim3(blocks), dim3(256), 0, (hipStream_t) stream, (T*) out, (const T*) g, (const T*) u, count));
    return mix_check_launch("mix_silu_mul");
}

extern "C" int exl3_mix_moe_combine_id(void* y, const void* sorted, const int32_t* where, const float* wts, const int32_t* idx, int experts, const void* h_id,
                                       const float* idw, int n, int top, int width, int dtype, void* stream)
{
    MIX_CHECK(y && sorted && where && wts && n >= 0 && top > 0 && width > 0 && (!idw || h_id) && (!idx || experts > 0), "mix_moe_combine: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(moe_combine_kernel<T>, dim3(n), dim3(256), 0, (hipStream_t) stream, (T*) y, (const T*) sorted, where, wts, top, width,
                                             idx, experts, (const T*) h_id, idw));
    return mix_check_launch("mix_moe_combine");
}

extern "C" int exl3_mix_moe_combine(void* y, const void* sorted, const int32_t* where, const float* wts, int n, int top, int width, int dtype, void* stream)
{
    return exl3_mix_moe_combine_id(y, sorted, where, wts, nullptr, 0, nullptr, nullptr, n, top, width, dtype, stream);
}

extern "C" int exl3_mix_moe_gate_up_act(void* hid, const void* h, const void* wg, const void* wu, const int32_t* idx, int n, int top, int experts, int ff, int width,
                                        int act, float limit, int dtype, void* stream)
{
    MIX_CHECK(act == EXL3_MIX_GLU_SILU || act == EXL3_MIX_GLU_CLAMPED_SWISH, "mix_moe_gate_up: unknown activation %d", act);
    MIX_CHECK(hid && h && wg && wu && idx && n >= 0 && top > 0 && experts > 0 && ff > 0 && width > 0, "mix_moe_gate_up: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    const int vn = dtype == EXL3_MIX_BF16 ? 8 : 4;
    const int vec = width % vn == 0 && (uintptr_t) h % 16 == 0 && (uintptr_t) wg % 16 == 0 && (uintptr_t) wu % 16 == 0;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((moe_gate_up_kernel<T, true>), dim3(n * top, (ff + 3) / 4), dim3(256), 0, (hipStream_t) stream, (T*) hid, (const T*) h,
                                             (const T*) wg, (const T*) wu, idx, experts, ff, width, top, vec, act, limit));
    return mix_check_launch("mix_moe_gate_up");
}

extern "C" int exl3_mix_moe_up_act(void* hid, const void* h, const void* wu, const int32_t* idx, int n, int top, int experts, int ff, int width, int act, int dtype, void* stream)
{
    MIX_CHECK(act >= EXL3_MIX_ACT_RELU2 && act <= EXL3_MIX_ACT_SILU, "mix_moe_up_act: unknown activation %d", act);
    MIX_CHECK(hid && h && wu && idx && n >= 0 && top > 0 && experts > 0 && ff > 0 && width > 0, "mix_moe_up_act: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    const int vn = dtype == EXL3_MIX_BF16 ? 8 : 4;
    const int vec = width % vn == 0 && (uintptr_t) h % 16 == 0 && (uintptr_t) wu % 16 == 0;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((moe_gate_up_kernel<T, false>), dim3(n * top, (ff + 3) / 4), dim3(256), 0, (hipStream_t) stream, (T*) hid, (const T*) h,
                                             (const T*) wu, (const T*) wu, idx, experts, ff, width, top, vec, act, 0.f));
    return mix_check_launch("mix_moe_up_act");
}

extern "C" int exl3_mix_moe_gate_up(void* hid, const void* h, const void* wg, const void* wu, const int32_t* idx, int n, int top, int experts, int ff, int width,
                                    int dtype, void* stream)
{
    return exl3_mix_moe_gate_up_act(hid, h, wg, wu, idx, n, top, experts, ff, width, EXL3_MIX_GLU_SILU, 0.f, dtype, stream);
}

extern "C" int exl3_mix_moe_down(void* y, const void* hid, const void* wd, const int32_t* idx, const float* wts, int n, int top, int experts, int ff, int width,
                                 int dtype, void* stream)
{
    return exl3_mix_moe_down_id(y, hid, wd, idx, wts, nullptr, nullptr, n, top, experts, ff, width, dtype, stream);
}

extern "C" int exl3_mix_moe_down_id(void* y, const void* hid, const void* wd, const int32_t* idx, const float* wts, const void* h_id, const float* idw,
                                    int n, int top, int experts, int ff, int width, int dtype, void* stream)
{
    MIX_CHECK(y && hid && wd && idx && wts && n >= 0 && top > 0 && experts > 0 && ff > 0 && width > 0 && (!idw || h_id), "mix_moe_down: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    const int vn = dtype == EXL3_MIX_BF16 ? 8 : 4;
    const int vec = ff % vn == 0 && (uintptr_t) hid % 16 == 0 && (uintptr_t) wd % 16 == 0;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(moe_down_kernel<T>, dim3(n, (width + 3) / 4), dim3(256), 0, (hipStream_t) stream, (T*) y, (const T*) hid, (const T*) wd,
                                             idx, wts, experts, ff, width, top, vec, (const T*) h_id, idw));
    return mix_check_launch("mix_moe_down");
}
