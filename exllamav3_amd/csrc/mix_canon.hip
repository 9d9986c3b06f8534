// Pre-norm blocks whose sublayers read a short causal convolution of the normed stream: the residual update fused with the RMS norm of the
// next sublayer, and the per-channel input convolution h_t + sum_j w[c][j] h_(t - taps + 1 + j) over time with the last taps - 1 normed rows of
// every sequence kept in a per-slot ring.  Prompt steps run two kernels (every row's norm, then the convolution over the step's own rows);
// steps of one row per sequence run ONE kernel (update, norm, convolution against the ring, ring store).  The residual, the sums of squares
// and the convolution's sum are float32; the normed rows and the ring are held in the activation type.
#include "mix_common.cuh"

#define CN_THREADS 256
#define CN_WAVES 4
#define CN_MAX_TAPS 16

// mode 0: x stays; 1: x += y; 2: x = y.  Then hn = x / sqrt(mean(x^2) + eps) * w.  With conv_w (one row per sequence, predecessors in the ring):
// h = hn + sum_j conv_w[c][j] * (j == taps - 1 ? hn : ring[(pos - (taps - 1 - j)) % (taps - 1)]), positions below 0 count as zero rows, and hn goes
// into the ring at pos % (taps - 1).  Without conv_w, h = hn.
template <typename T>
__global__ __launch_bounds__(CN_THREADS) void residual_rms_kernel(float* __restrict__ x, const T* __restrict__ y, int64_t y_ld, int mode, const float* __restrict__ w, float eps,
                                                                  T* __restrict__ h, int64_t h_ld, const float* __restrict__ conv_w, int taps, T* __restrict__ ring,
                                                                  const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                                                  const int32_t* __restrict__ slots, int width)
{
    __shared__ float red[CN_WAVES];
    const int n = blockIdx.x;
    float* xr = x + (int64_t) n * width;
    const T* yr = y + (int64_t) n * y_ld;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += CN_THREADS)
    {
        float v = xr[i];
        if (mode != 0)
        {
            const float a = to_f(yr[i]);
            v = mode == 1 ? v + a : a;
            xr[i] = v;
        }
        ss += v * v;
    }
    if (!h) return;
    ss = block_sum<CN_WAVES>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float) width + eps);
    T* hr = h + (int64_t) n * h_ld;
    if (!conv_w)
    {
        for (int i = threadIdx.x; i < width; i += CN_THREADS) hr[i] = from_f<T>(xr[i] * inv * w[i]);     // a thread reads back what it wrote itself
        return;
    }
    const int pos = tok_pos[n], keep = taps - 1;
    T* rg = ring + (int64_t) slots[tok_seq[n]] * (keep > 0 ? keep : 1) * width;
    for (int i = threadIdx.x; i < width; i += CN_THREADS)
    {
        const T hn = from_f<T>(xr[i] * inv * w[i]);
        const float hf = to_f(hn);
        const float* cw = conv_w + (int64_t) i * taps;
        float acc = hf + cw[taps - 1] * hf;
        for (int j = 0; j < keep; ++j)
        {
            const int p = pos - (keep - j);
            if (p >= 0) acc += cw[j] * to_f(rg[(int64_t) (p % keep) * width + i]);
        }
        if (keep > 0) rg[(int64_t) (pos % keep) * width + i] = hn;        // after the reads: this entry held position pos - keep
        hr[i] = from_f<T>(acc);
    }
}

// The convolution of a prompt step: row n of a sequence reads its predecessors among the step's own rows (a sequence's rows lie one behind the
// other) where they are in the step (position >= pos0 of the sequence), and from the ring otherwise; the rows at the last taps - 1 positions of
// a sequence go into the ring.  One thread per (row, channel group).
template <typename T>
__global__ __launch_bounds__(CN_THREADS) void canon_kernel(T* __restrict__ out, int64_t out_ld, const T* __restrict__ hn, int64_t hn_ld, const float* __restrict__ conv_w, int taps,
                                                           T* __restrict__ ring, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                                           const int32_t* __restrict__ slots, const int32_t* __restrict__ pos0, const int32_t* __restrict__ len_after, int width)
{
    const int n = blockIdx.y;
    const int i = blockIdx.x * CN_THREADS + threadIdx.x;
    if (i >= width) return;
    const int b = tok_seq[n], pos = tok_pos[n], keep = taps - 1, start = pos0[b];
    T* rg = ring + (int64_t) slots[b] * (keep > 0 ? keep : 1) * width;
    const float* cw = conv_w + (int64_t) i * taps;
    const T hv = hn[(int64_t) n * hn_ld + i];
    const float hf = to_f(hv);
    float acc = hf + cw[taps - 1] * hf;
    for (int j = 0; j < keep; ++j)
    {
        const int back = keep - j, p = pos - back;
        if (p < 0) continue;
        acc += cw[j] * to_f(p >= start ? hn[(int64_t) (n - back) * hn_ld + i] : rg[(int64_t) (p % keep) * width + i]);
    }
    out[(int64_t) n * out_ld + i] = from_f<T>(acc);
    // The rows at the last `keep` positions go into the ring.  A step that starts its sequences reads nothing from the ring; a step of one row per
    // sequence overwrites the entry of position pos - keep, which this same thread has read above.
    if (keep > 0 && pos >= len_after[b] - keep) rg[(int64_t) (pos % keep) * width + i] = hv;
}

extern "C" int exl3_mix_residual_rms(float* x, const void* y, int64_t y_ld, int mode, const float* w, float eps, void* h, int64_t h_ld,
                                     const float* conv_w, int taps, void* ring, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots,
                                     int n, int width, int dtype, void* stream)
{
    MIX_CHECK(x && n >= 0 && width > 0 && mode >= 0 && mode <= 2, "mix_residual_rms: bad arguments");
    MIX_CHECK(mode == 0 || (y && y_ld >= width), "mix_residual_rms: an addend is needed");
    MIX_CHECK(!h || (w && h_ld >= width), "mix_residual_rms: the norm needs its weight");
    MIX_CHECK(!conv_w || (h && ring && tok_seq && tok_pos && slots && taps >= 1 && taps <= CN_MAX_TAPS), "mix_residual_rms: the convolution needs 1..%d taps, the ring and the step's rows", CN_MAX_TAPS);
    if (n == 0 || (mode == 0 && !h)) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(residual_rms_kernel<T>, dim3(n), dim3(CN_THREADS), 0, (hipStream_t) stream, x, (const T*) y, y_ld, mode, w, eps, (T*) h, h_ld,
                                             conv_w, taps, (T*) ring, tok_seq, tok_pos, slots, width));
    return mix_check_launch("mix_residual_rms");
}

extern "C" int exl3_mix_canon(void* out, int64_t out_ld, const void* hn, int64_t hn_ld, const float* conv_w, int taps, void* ring,
                              const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* pos0, const int32_t* len_after,
                              int n, int width, int dtype, void* stream)
{
    MIX_CHECK(out && hn && conv_w && ring && tok_seq && tok_pos && slots && pos0 && len_after && n >= 0 && n <= 65535 * 1024 && width > 0, "mix_canon: bad arguments");
    MIX_CHECK(taps >= 1 && taps <= CN_MAX_TAPS && out_ld >= width && hn_ld >= width && out != hn, "mix_canon: 1..%d taps, row strides >= width, out apart from hn", CN_MAX_TAPS);
    for (int r0 = 0; r0 < n; r0 += 65535)
    {
        const int rows = n - r0 < 65535 ? n - r0 : 65535;
        // the kernel indexes rows from the step's first row (a row's predecessors may lie before r0): pass the bases and offset the row index through the pointers
        MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(canon_kernel<T>, dim3((width + CN_THREADS - 1) / CN_THREADS, rows), dim3(CN_THREADS), 0, (hipStream_t) stream,
                                                 (T*) out + (int64_t) r0 * out_ld, out_ld, (const T*) hn + (int64_t) r0 * hn_ld, hn_ld, conv_w, taps, (T*) ring,
                                                 tok_seq + r0, tok_pos + r0, slots, pos0, len_after, width));
    }
    return mix_check_launch("mix_canon");
}
