// Pre-norm blocks whose sublayers read a short causal convolution of the normed stream: the residual update fused with the RMS norm of the
// next sublayer, and the per-channel input convolution h_t + sum_j w[c][j] h_(t - taps + 1 + j) over time with the last taps - 1 normed rows of
// every sequence kept in a per-slot ring.  Prompt steps run two kernels (every row's norm, then the convolution over the step's own rows);
// steps of one row per sequence run ONE kernel (update, norm, convolution against the ring, ring store).  The residual, the sums of squares
// and the convolution's sum are float32; the normed rows and the ring are held in the activation type.
#include "mix_common.cuh"

#define CN_THREADS 256
#define CN_WAVES 4
#define CN_MAX_TAPS 16

// four consecutive elements at once (rows of a multiple of four elements, 16-byte aligned for float32 / 8-byte for bfloat16)
template <typename T> struct raw4;
template <> struct raw4<bf16_t> { typedef uint2 type; };
template <> struct raw4<float> { typedef uint4 type; };
template <typename T> __device__ __forceinline__ void load4(const T* p, float (&o)[4])
{
    union { typename raw4<T>::type v; T e[4]; } t;
    t.v = *(const typename raw4<T>::type*) p;
    #pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = to_f(t.e[e]);
}
template <typename T> __device__ __forceinline__ void store4(T* p, const float (&o)[4])
{
    union { typename raw4<T>::type v; T e[4]; } t;
    #pragma unroll
    for (int e = 0; e < 4; ++e) t.e[e] = from_f<T>(o[e]);
    *(typename raw4<T>::type*) p = t.v;
}
// the value a T holds after rounding
template <typename T> __device__ __forceinline__ float rounded(float v) { return to_f(from_f<T>(v)); }

// mode 0: x stays; 1: x += y; 2: x = y.  Then hn = x / sqrt(mean(x^2) + eps) * w.  With conv_w [taps][width] (one row per sequence, predecessors in the
// ring): h = hn + sum_j conv_w[j][c] * (j == taps - 1 ? hn : ring[(pos - (taps - 1 - j)) % (taps - 1)]), positions below 0 count as zero rows, and hn goes
// into the ring at pos % (taps - 1).  Without conv_w, h = hn.  V: elements per thread and access (4 when the rows allow it).
// CENTER: the norm is a layer norm, (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + bias, the mean taken first and the deviations squared after it.
// y2 (optional): a second addend, y' = (y + y2) * y_scale (the two sublayers of a parallel block and the block's residual factor); without it y' = y * y_scale.
// hn_out (optional): the normed row itself, for a consumer that reads it without the convolution.
template <typename T, int V, bool CENTER>
__global__ __launch_bounds__(CN_THREADS) void residual_rms_kernel(float* __restrict__ x, const T* __restrict__ y, int64_t y_ld, const T* __restrict__ y2, int64_t y2_ld, float y_scale,
                                                                  int mode, const float* __restrict__ w, const float* __restrict__ bias, float eps,
                                                                  T* __restrict__ h, int64_t h_ld, T* __restrict__ hn_out, int64_t hn_ld,
                                                                  const float* __restrict__ conv_w, int taps, T* __restrict__ ring,
                                                                  const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                                                  const int32_t* __restrict__ slots, int width)
{
    __shared__ float red[CN_WAVES];
    const int n = blockIdx.x;
    float* xr = x + (int64_t) n * width;
    const T* yr = y + (int64_t) n * y_ld;
    const T* y2r = y2 ? y2 + (int64_t) n * y2_ld : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x * V; i < width; i += CN_THREADS * V)
    {
        float v[V];
        if constexpr (V == 4) { const float4 t = *(const float4*) (xr + i); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[V - 1] = t.w; } else v[0] = xr[i];
        if (mode != 0)
        {
            float a[V];
            if constexpr (V == 4) load4<T>(yr + i, (float (&)[4]) a); else a[0] = to_f(yr[i]);
            if (y2r)
            {
                float a2[V];
                if constexpr (V == 4) load4<T>(y2r + i, (float (&)[4]) a2); else a2[0] = to_f(y2r[i]);
                #pragma unroll
                for (int e = 0; e < V; ++e) a[e] += a2[e];
            }
            #pragma unroll
            for (int e = 0; e < V; ++e) v[e] = mode == 1 ? v[e] + a[e] * y_scale : a[e] * y_scale;
            if constexpr (V == 4) *(float4*) (xr + i) = make_float4(v[0], v[1], v[2], v[V - 1]); else xr[i] = v[0];
        }
        #pragma unroll
        for (int e = 0; e < V; ++e) ss += CENTER ? v[e] : v[e] * v[e];
    }
    if (!h && !hn_out) return;
    ss = block_sum<CN_WAVES>(ss, red);
    float mean = 0.f;
    if constexpr (CENTER)
    {
        mean = ss / (float) width;
        float dd = 0.f;
        for (int i = threadIdx.x * V; i < width; i += CN_THREADS * V)                 // the thread's own part of x once more
        {
            #pragma unroll
            for (int e = 0; e < V; ++e) { const float d = xr[i + e] - mean; dd += d * d; }
        }
        ss = block_sum<CN_WAVES>(dd, red);
    }
    const float inv = 1.0f / sqrtf(ss / (float) width + eps);
    T* hr = h + (int64_t) n * h_ld;
    const int pos = conv_w ? tok_pos[n] : 0, keep = taps - 1;
    T* rg = conv_w ? ring + (int64_t) slots[tok_seq[n]] * (keep > 0 ? keep : 1) * width : nullptr;
    for (int i = threadIdx.x * V; i < width; i += CN_THREADS * V)                     // a thread reads back the part of x that it wrote itself
    {
        float hn[V], wv[V];
        if constexpr (V == 4)
        {
            const float4 t = *(const float4*) (xr + i), u = *(const float4*) (w + i);
            hn[0] = t.x; hn[1] = t.y; hn[2] = t.z; hn[V - 1] = t.w; wv[0] = u.x; wv[1] = u.y; wv[2] = u.z; wv[V - 1] = u.w;
        }
        else { hn[0] = xr[i]; wv[0] = w[i]; }
        if constexpr (CENTER)
        {
            #pragma unroll
            for (int e = 0; e < V; ++e) hn[e] = rounded<T>((hn[e] - mean) * inv * wv[e] + (bias ? bias[i + e] : 0.f));
        }
        else
        {
            #pragma unroll
            for (int e = 0; e < V; ++e) hn[e] = rounded<T>(hn[e] * inv * wv[e]);        // the normed row is held in the activation type wherever it is kept
        }
        if (hn_out)
        {
            T* dsth = hn_out + (int64_t) n * hn_ld + i;
            if constexpr (V == 4) store4<T>(dsth, (const float (&)[4]) hn); else dsth[0] = from_f<T>(hn[0]);
        }
        if (!h) continue;
        if (!conv_w)
        {
            if constexpr (V == 4) store4<T>(hr + i, (const float (&)[4]) hn); else hr[i] = from_f<T>(hn[0]);
            continue;
        }
        float acc[V], c[V];
        if constexpr (V == 4) { const float4 t = *(const float4*) (conv_w + (int64_t) keep * width + i); c[0] = t.x; c[1] = t.y; c[2] = t.z; c[V - 1] = t.w; }
        else c[0] = conv_w[(int64_t) keep * width + i];
        #pragma unroll
        for (int e = 0; e < V; ++e) acc[e] = hn[e] + c[e] * hn[e];
        for (int j = 0; j < keep; ++j)
        {
            const int p = pos - (keep - j);
            if (p < 0) continue;
            float r[V];
            const T* src = rg + (int64_t) (p % keep) * width + i;
            if constexpr (V == 4)
            {
                const float4 t = *(const float4*) (conv_w + (int64_t) j * width + i); c[0] = t.x; c[1] = t.y; c[2] = t.z; c[V - 1] = t.w;
                load4<T>(src, (float (&)[4]) r);
            }
            else { c[0] = conv_w[(int64_t) j * width + i]; r[0] = to_f(src[0]); }
            #pragma unroll
            for (int e = 0; e < V; ++e) acc[e] += c[e] * r[e];
        }
        if (keep > 0)                                                                    // after the reads: this entry held position pos - keep
        {
            T* dst = rg + (int64_t) (pos % keep) * width + i;
            if constexpr (V == 4) store4<T>(dst, (const float (&)[4]) hn); else dst[0] = from_f<T>(hn[0]);
        }
        if constexpr (V == 4) store4<T>(hr + i, (const float (&)[4]) acc); else hr[i] = from_f<T>(acc[0]);
    }
}

// The convolution of a prompt step: row n of a sequence reads its predecessors among the step's own rows (a sequence's rows lie one behind the
// other) where they are in the step (position >= pos0 of the sequence), and from the ring otherwise; the rows at the last taps - 1 positions of
// a sequence go into the ring.  One thread per (row, V channels); conv_w [taps][width].
template <typename T, int V>
__global__ __launch_bounds__(CN_THREADS) void canon_kernel(T* __restrict__ out, int64_t out_ld, const T* __restrict__ hn, int64_t hn_ld, const float* __restrict__ conv_w, int taps,
                                                           T* __restrict__ ring, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                                           const int32_t* __restrict__ slots, const int32_t* __restrict__ pos0, const int32_t* __restrict__ len_after, int width)
{
    const int n = blockIdx.y;
    const int i = (blockIdx.x * CN_THREADS + threadIdx.x) * V;
    if (i >= width) return;
    const int b = tok_seq[n], pos = tok_pos[n], keep = taps - 1, start = pos0[b];
    T* rg = ring + (int64_t) slots[b] * (keep > 0 ? keep : 1) * width;
    float hv[V], c[V], acc[V];
    if constexpr (V == 4)
    {
        load4<T>(hn + (int64_t) n * hn_ld + i, (float (&)[4]) hv);
        const float4 t = *(const float4*) (conv_w + (int64_t) keep * width + i); c[0] = t.x; c[1] = t.y; c[2] = t.z; c[V - 1] = t.w;
    }
    else { hv[0] = to_f(hn[(int64_t) n * hn_ld + i]); c[0] = conv_w[(int64_t) keep * width + i]; }
    #pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = hv[e] + c[e] * hv[e];
    for (int j = 0; j < keep; ++j)
    {
        const int back = keep - j, p = pos - back;
        if (p < 0) continue;
        const T* src = p >= start ? hn + (int64_t) (n - back) * hn_ld + i : rg + (int64_t) (p % keep) * width + i;
        float r[V];
        if constexpr (V == 4)
        {
            const float4 t = *(const float4*) (conv_w + (int64_t) j * width + i); c[0] = t.x; c[1] = t.y; c[2] = t.z; c[V - 1] = t.w;
            load4<T>(src, (float (&)[4]) r);
        }
        else { c[0] = conv_w[(int64_t) j * width + i]; r[0] = to_f(src[0]); }
        #pragma unroll
        for (int e = 0; e < V; ++e) acc[e] += c[e] * r[e];
    }
    if constexpr (V == 4) store4<T>(out + (int64_t) n * out_ld + i, (const float (&)[4]) acc); else out[(int64_t) n * out_ld + i] = from_f<T>(acc[0]);
    // The rows at the last `keep` positions go into the ring.  A step that starts its sequences reads nothing from the ring; a step of one row per
    // sequence overwrites the entry of position pos - keep, which this same thread has read above.
    if (keep > 0 && pos >= len_after[b] - keep)
    {
        T* dst = rg + (int64_t) (pos % keep) * width + i;
        if constexpr (V == 4) store4<T>(dst, (const float (&)[4]) hv); else dst[0] = from_f<T>(hv[0]);
    }
}

// rows of a multiple of four elements whose starts are 16-byte aligned (element sizes 2 and 4: a multiple of 4 elements from a 16-byte aligned base with
// a row stride that is a multiple of 8 elements for bfloat16 / 4 for float32 keeps every 4-element access aligned to its size)
static bool rows_by_four(const void* p, int64_t ld, int dtype)
{
    return p == nullptr || ((uintptr_t) p % 16 == 0 && ld % (dtype == EXL3_MIX_BF16 ? 8 : 4) == 0);
}

extern "C" int exl3_mix_residual_norm_conv(float* x, const void* y, int64_t y_ld, const void* y2, int64_t y2_ld, float y_scale, int mode, int center, const float* w,
                                           const float* bias, float eps, void* h, int64_t h_ld, void* hn_out, int64_t hn_ld, const float* conv_w, int taps, void* ring,
                                           const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, int n, int width, int dtype, void* stream)
{
    MIX_CHECK(x && n >= 0 && width > 0 && mode >= 0 && mode <= 2, "mix_residual_norm_conv: bad arguments");
    MIX_CHECK(mode == 0 || (y && y_ld >= width && (!y2 || y2_ld >= width)), "mix_residual_norm_conv: an addend is needed");
    MIX_CHECK((!h && !hn_out) || (w && (!h || h_ld >= width) && (!hn_out || hn_ld >= width)), "mix_residual_norm_conv: the norm needs its weight");
    MIX_CHECK(center || !bias, "mix_residual_norm_conv: a bias goes with the layer norm");
    MIX_CHECK(!conv_w || (h && ring && tok_seq && tok_pos && slots && taps >= 1 && taps <= CN_MAX_TAPS), "mix_residual_norm_conv: the convolution needs 1..%d taps, the ring and the step's rows", CN_MAX_TAPS);
    if (n == 0 || (mode == 0 && !h && !hn_out)) return EXL3_MIX_OK;
    const bool by4 = width % 8 == 0 && (uintptr_t) x % 16 == 0 && rows_by_four(y, y_ld, dtype) && rows_by_four(y2, y2_ld, dtype) && rows_by_four(h, h_ld, dtype) &&
                     rows_by_four(hn_out, hn_ld, dtype) && rows_by_four(ring, 8, dtype) && (uintptr_t) w % 16 == 0 && (uintptr_t) conv_w % 16 == 0;
    #define RN_LAUNCH(VV, CC) hipLaunchKernelGGL((residual_rms_kernel<T, VV, CC>), dim3(n), dim3(CN_THREADS), 0, (hipStream_t) stream, x, (const T*) y, y_ld, (const T*) y2, y2_ld, y_scale, \
                                                 mode, w, bias, eps, (T*) h, h_ld, (T*) hn_out, hn_ld, conv_w, taps, (T*) ring, tok_seq, tok_pos, slots, width)
    MIX_DISPATCH_T(dtype, if (by4) { if (center) RN_LAUNCH(4, true); else RN_LAUNCH(4, false); } else { if (center) RN_LAUNCH(1, true); else RN_LAUNCH(1, false); });
    #undef RN_LAUNCH
    return mix_check_launch("mix_residual_norm_conv");
}

extern "C" int exl3_mix_residual_rms(float* x, const void* y, int64_t y_ld, int mode, const float* w, float eps, void* h, int64_t h_ld,
                                     const float* conv_w, int taps, void* ring, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots,
                                     int n, int width, int dtype, void* stream)
{
    return exl3_mix_residual_norm_conv(x, y, y_ld, nullptr, 0, 1.0f, mode, 0, w, nullptr, eps, h, h_ld, nullptr, 0, conv_w, taps, ring, tok_seq, tok_pos, slots, n, width, dtype, stream);
}

extern "C" int exl3_mix_canon(void* out, int64_t out_ld, const void* hn, int64_t hn_ld, const float* conv_w, int taps, void* ring,
                              const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* pos0, const int32_t* len_after,
                              int n, int width, int dtype, void* stream)
{
    MIX_CHECK(out && hn && conv_w && ring && tok_seq && tok_pos && slots && pos0 && len_after && n >= 0 && n <= 65535 * 1024 && width > 0, "mix_canon: bad arguments");
    MIX_CHECK(taps >= 1 && taps <= CN_MAX_TAPS && out_ld >= width && hn_ld >= width && out != hn, "mix_canon: 1..%d taps, row strides >= width, out apart from hn", CN_MAX_TAPS);
    const bool by4 = width % 8 == 0 && rows_by_four(out, out_ld, dtype) && rows_by_four(hn, hn_ld, dtype) && rows_by_four(ring, 8, dtype) && (uintptr_t) conv_w % 16 == 0;
    for (int r0 = 0; r0 < n; r0 += 65535)
    {
        const int rows = n - r0 < 65535 ? n - r0 : 65535;
        // a row's predecessors may lie before r0: the bases are offset, the kernel's row index counts from there
        if (by4)
            MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((canon_kernel<T, 4>), dim3((width / 4 + CN_THREADS - 1) / CN_THREADS, rows), dim3(CN_THREADS), 0, (hipStream_t) stream,
                                                     (T*) out + (int64_t) r0 * out_ld, out_ld, (const T*) hn + (int64_t) r0 * hn_ld, hn_ld, conv_w, taps, (T*) ring,
                                                     tok_seq + r0, tok_pos + r0, slots, pos0, len_after, width));
        else
            MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((canon_kernel<T, 1>), dim3((width + CN_THREADS - 1) / CN_THREADS, rows), dim3(CN_THREADS), 0, (hipStream_t) stream,
                                                     (T*) out + (int64_t) r0 * out_ld, out_ld, (const T*) hn + (int64_t) r0 * hn_ld, hn_ld, conv_w, taps, (T*) ring,
                                                     tok_seq + r0, tok_pos + r0, slots, pos0, len_after, width));
    }
    return mix_check_launch("mix_canon");
}
