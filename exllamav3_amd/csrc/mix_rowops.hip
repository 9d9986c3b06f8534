// Row-wise kernels of pre-norm blocks over a float32 residual stream whose norm needs no statistics (Dynamic Tanh), and the small pieces
// between their matrix products: the embedding with a copy in the activation type, the residual update (plain or with the addend divided by
// its root mean square) fused with what the next consumer reads (the next norm, or the stream in the activation type), the last norm on chosen
// rows, element-wise activations (plain and gated, with clamps), a per-token gate from an embedding table, a gate applied across a
// head-major layout, and a router with sigmoid scores.  Sums and the residual are float32.
#include "mix_common.cuh"

#define ROW_THREADS 256
#define ROW_WAVES 4

template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void embed_copy_kernel(float* __restrict__ x, T* __restrict__ xc, int64_t xc_ld, const T* __restrict__ table,
                                                                 const int32_t* __restrict__ tokens, int width, int vocab)
{
    const int n = blockIdx.x;
    int tok = tokens[n];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    const T* src = table + (int64_t) tok * width;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS)
    {
        const T v = src[i];
        x[(int64_t) n * width + i] = to_f(v);
        if (xc) xc[(int64_t) n * xc_ld + i] = v;
    }
}

// x[n] = table[tokens[n]] * scale + P(tok_pos[n]): a sinusoidal position vector, entry 2i = sin(p f_i), entry 2i + 1 = cos(p f_i), f_i = freq[i] (float32;
// the angle is the float32 product of the position and the frequency)
template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void embed_sinusoid_kernel(float* __restrict__ x, const T* __restrict__ table, const int32_t* __restrict__ tokens,
                                                                     const int32_t* __restrict__ tok_pos, const float* __restrict__ freq, float scale, int width, int vocab)
{
    const int n = blockIdx.x;
    int tok = tokens[n];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    const T* src = table + (int64_t) tok * width;
    const float p = (float) tok_pos[n];
    for (int i = threadIdx.x; i < width; i += ROW_THREADS)
    {
        const float a = p * freq[i >> 1];
        x[(int64_t) n * width + i] = to_f(src[i]) * scale + ((i & 1) ? cosf(a) : sinf(a));
    }
}

// h[i] = layer norm of residual row rows[i] (or i): (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b
template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void layer_norm_rows_kernel(T* __restrict__ h, const float* __restrict__ x, const int32_t* __restrict__ rows,
                                                                      const float* __restrict__ w, const float* __restrict__ b, float eps, int width)
{
    __shared__ float red[ROW_WAVES];
    const int n = blockIdx.x;
    const float* xr = x + (int64_t) (rows ? rows[n] : n) * width;
    float s = 0.f;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS) s += xr[i];
    const float mean = block_sum<ROW_WAVES>(s, red) / (float) width;
    float dd = 0.f;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS) { const float d = xr[i] - mean; dd += d * d; }
    dd = block_sum<ROW_WAVES>(dd, red);
    const float inv = 1.0f / sqrtf(dd / (float) width + eps);
    T* hr = h + (int64_t) n * width;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS) hr[i] = from_f<T>((xr[i] - mean) * inv * w[i] + (b ? b[i] : 0.f));
}

// mode 0: x stays; 1: x += y'; 2: x = y'   with y' = y, or y / rms(y) * rms_w when rms_w is given.
// out 0: nothing; 1: h = x in the activation type; 2: h = tanh(alpha x) w + b.
template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void residual_norm_kernel(float* __restrict__ x, const T* __restrict__ y, int64_t y_ld, int mode, const float* __restrict__ rms_w,
                                                                    float eps, int out, float alpha, const float* __restrict__ w, const float* __restrict__ b,
                                                                    T* __restrict__ h, int64_t h_ld, int width)
{
    __shared__ float red[ROW_WAVES];
    const int n = blockIdx.x;
    float* xr = x + (int64_t) n * width;
    const T* yr = y + (int64_t) n * y_ld;
    float inv = 1.0f;
    if (mode != 0 && rms_w)
    {
        float ss = 0.f;
        for (int i = threadIdx.x; i < width; i += ROW_THREADS) { const float v = to_f(yr[i]); ss += v * v; }
        ss = block_sum<ROW_WAVES>(ss, red);
        inv = 1.0f / sqrtf(ss / (float) width + eps);
    }
    T* hr = h + (int64_t) n * h_ld;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS)
    {
        float v = xr[i];
        if (mode != 0)
        {
            float a = to_f(yr[i]);
            if (rms_w) a = a * inv * rms_w[i];
            v = mode == 1 ? v + a : a;
            xr[i] = v;
        }
        if (out == 1) hr[i] = from_f<T>(v);
        else if (out == 2) hr[i] = from_f<T>(tanhf(alpha * v) * w[i] + b[i]);
    }
}

template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void dyn_tanh_rows_kernel(T* __restrict__ h, const float* __restrict__ x, const int32_t* __restrict__ rows, float alpha,
                                                                    const float* __restrict__ w, const float* __restrict__ b, int width)
{
    const int n = blockIdx.x;
    const float* xr = x + (int64_t) (rows ? rows[n] : n) * width;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS) h[(int64_t) n * width + i] = from_f<T>(tanhf(alpha * xr[i]) * w[i] + b[i]);
}

// plain activations: 0 = relu(z)^2, 1 = gelu (tanh form), 2 = silu.  A thread takes VN consecutive elements (16 bytes) when the rows allow it.
template <typename T> struct rvec;
template <> struct rvec<bf16_t> { static constexpr int N = 8; };
template <> struct rvec<float> { static constexpr int N = 4; };

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void act_kernel(T* __restrict__ out, const T* __restrict__ z, int64_t z_ld, int ff, int kind)
{
    constexpr int VN = VEC ? rvec<T>::N : 1;
    const int n = blockIdx.y;
    const int i = (blockIdx.x * 256 + threadIdx.x) * VN;
    if (i >= ff) return;
    if (VEC)
    {
        union { uint4 v; T e[rvec<T>::N]; } a, o;
        a.v = *(const uint4*) (z + (int64_t) n * z_ld + i);
        #pragma unroll
        for (int e = 0; e < rvec<T>::N; ++e) o.e[e] = from_f<T>(act_f(to_f(a.e[e]), kind));
        *(uint4*) (out + (int64_t) n * ff + i) = o.v;
    }
    else out[(int64_t) n * ff + i] = from_f<T>(act_f(to_f(z[(int64_t) n * z_ld + i]), kind));
}

// rg (optional): one number per row; the row's result is multiplied by sigmoid(rg[n]) (a gate on the whole sublayer, applied before its linear down projection)
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void glu_act_kernel(T* __restrict__ out, const T* __restrict__ g, int64_t g_ld, const T* __restrict__ u, int64_t u_ld, int ff, int kind, float limit,
                                                      const T* __restrict__ rg, int64_t rg_ld)
{
    constexpr int VN = VEC ? rvec<T>::N : 1;
    const int n = blockIdx.y;
    const int i = (blockIdx.x * 256 + threadIdx.x) * VN;
    if (i >= ff) return;
    const float rs = rg ? sigmoid_f(to_f(rg[(int64_t) n * rg_ld])) : 1.0f;
    if (VEC)
    {
        union { uint4 v; T e[rvec<T>::N]; } a, b, o;
        a.v = *(const uint4*) (g + (int64_t) n * g_ld + i);
        b.v = *(const uint4*) (u + (int64_t) n * u_ld + i);
        #pragma unroll
        for (int e = 0; e < rvec<T>::N; ++e) { const float r = glu_act_f(to_f(a.e[e]), to_f(b.e[e]), kind, limit); o.e[e] = from_f<T>(rg ? r * rs : r); }
        *(uint4*) (out + (int64_t) n * ff + i) = o.v;
    }
    else
    {
        const float r = glu_act_f(to_f(g[(int64_t) n * g_ld + i]), to_f(u[(int64_t) n * u_ld + i]), kind, limit);
        out[(int64_t) n * ff + i] = from_f<T>(rg ? r * rs : r);
    }
}

// out[n][j] = gelu_tanh(gate[n][j]) * table[tokens[n]][col0 + j]
template <typename T>
__global__ __launch_bounds__(64) void token_gate_kernel(T* __restrict__ out, const T* __restrict__ gate, int64_t gate_ld, const T* __restrict__ table, int64_t table_ld,
                                                        int col0, const int32_t* __restrict__ tokens, int dim, int vocab)
{
    const int n = blockIdx.x;
    int tok = tokens[n];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    const T* e = table + (int64_t) tok * table_ld + col0;
    for (int j = threadIdx.x; j < dim; j += 64)
        out[(int64_t) n * dim + j] = from_f<T>(gelu_tanh_f(to_f(gate[(int64_t) n * gate_ld + j])) * to_f(e[j]));
}

// out[n][h * vdim + v] = a[n * a_row + h * a_head + v] * (gate ? sigmoid(gate[n][h * vdim + v]) : 1)
template <typename T>
__global__ __launch_bounds__(256) void heads_gate_kernel(T* __restrict__ out, const T* __restrict__ a, int64_t a_row, int64_t a_head, const T* __restrict__ gate,
                                                         int64_t gate_ld, int heads, int vdim)
{
    const int n = blockIdx.x;
    for (int t = threadIdx.x; t < heads * vdim; t += 256)
    {
        const int h = t / vdim, v = t - h * vdim;
        float r = to_f(a[(int64_t) n * a_row + (int64_t) h * a_head + v]);
        if (gate) r *= sigmoid_f(to_f(gate[(int64_t) n * gate_ld + t]));
        out[(int64_t) n * heads * vdim + t] = from_f<T>(r);
    }
}

// Router with independent scores: s = sigmoid(z); the `top` experts with the largest s + correction are chosen (ties go to the lower index), and
// their weights are s / (sum of the chosen s + 1e-20) * scale (normalise = 0: s * scale).
__global__ void topk_sigmoid_kernel(int32_t* __restrict__ idx, float* __restrict__ wts, const float* __restrict__ logits, const float* __restrict__ correction,
                                    float scale, int normalise, int n, int experts, int top)
{
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n) return;
    const float* l = logits + (int64_t) t * experts;
    int32_t* id = idx + (int64_t) t * top;
    float* w = wts + (int64_t) t * top;
    float sum = 0.f;
    for (int r = 0; r < top; ++r)
    {
        int best = -1; float bv = 0.f, bs = 0.f;
        for (int e = 0; e < experts; ++e)
        {
            bool taken = false;
            for (int p = 0; p < r; ++p) taken |= (id[p] == e);
            if (taken) continue;
            const float s = sigmoid_f(l[e]);
            const float v = correction ? s + correction[e] : s;
            if (best < 0 || v > bv) { best = e; bv = v; bs = s; }
        }
        id[r] = best; w[r] = bs; sum += bs;
    }
    const float f = normalise ? scale / (sum + 1e-20f) : scale;
    for (int r = 0; r < top; ++r) w[r] = w[r] * f;
}

// Router over `total` outputs of which the first `real` name stored experts and the rest experts that return their input.  One wave per row, the
// outputs across the lanes.  Scores s: softmax over all outputs (kind 0) or independent sigmoids (kind 1).  The choice looks at c = s + correction;
// with groups > 1 the outputs form `groups` equal groups of neighbours, a group counts as its largest c, and only the `keep` best groups can be chosen
// from (the others count as minus infinity).  The `top` largest c are taken one after the other (ties go to the lower index); the weights are the
// chosen s over their sum (+ 1e-20) times `scale` (normalise = 0: s * scale).  Out: idx / wts per choice -- a choice beyond the stored experts is
// written as idx = real with weight 0 -- and idw[n] = the weights of those choices added up.
#define TG_MAX_PER_LANE 8
__global__ __launch_bounds__(64) void topk_grouped_kernel(int32_t* __restrict__ idx, float* __restrict__ wts, float* __restrict__ idw, const float* __restrict__ logits,
                                                          const float* __restrict__ correction, int kind, float scale, int normalise, int groups, int keep,
                                                          int total, int real, int top, int group_top)
{
    __shared__ float gmax[64];
    const int n = blockIdx.x, lane = threadIdx.x;
    const float* l = logits + (int64_t) n * total;
    float s[TG_MAX_PER_LANE], c[TG_MAX_PER_LANE];
    float mx = -INFINITY;
    #pragma unroll
    for (int i = 0; i < TG_MAX_PER_LANE; ++i)
    {
        const int e = lane + 64 * i;
        s[i] = e < total ? l[e] : -INFINITY;
        mx = fmaxf(mx, s[i]);
    }
    if (kind == 0)
    {
        mx = wave_max(mx);
        float den = 0.f;
        #pragma unroll
        for (int i = 0; i < TG_MAX_PER_LANE; ++i) { s[i] = (lane + 64 * i < total) ? expf(s[i] - mx) : 0.f; den += s[i]; }
        den = wave_sum(den);
        #pragma unroll
        for (int i = 0; i < TG_MAX_PER_LANE; ++i) s[i] = s[i] / den;
    }
    else
    {
        #pragma unroll
        for (int i = 0; i < TG_MAX_PER_LANE; ++i) s[i] = (lane + 64 * i < total) ? sigmoid_f(s[i]) : 0.f;
    }
    #pragma unroll
    for (int i = 0; i < TG_MAX_PER_LANE; ++i)
    {
        const int e = lane + 64 * i;
        c[i] = e < total ? (correction ? s[i] + correction[e] : s[i]) : -INFINITY;
    }
    if (groups > 1 && keep < groups)
    {
        const int per = total / groups;
        for (int g = 0; g < groups; ++g)                     // a group's score: the sum of its `group_top` largest choice scores (1: its largest)
        {
            unsigned used = 0u;
            float total_g = 0.f;
            for (int t = 0; t < group_top && t < per; ++t)
            {
                float bv = -INFINITY; int be = 0x7fffffff;
                #pragma unroll
                for (int i = 0; i < TG_MAX_PER_LANE; ++i)
                {
                    const int e = lane + 64 * i;
                    if (e < total && e / per == g && !((used >> i) & 1u) && (c[i] > bv || be == 0x7fffffff)) { bv = c[i]; be = e; }
                }
                #pragma unroll
                for (int o = 32; o > 0; o >>= 1)
                {
                    const float ov = __shfl_xor(bv, o, 64); const int oe = __shfl_xor(be, o, 64);
                    if (oe != 0x7fffffff && (be == 0x7fffffff || ov > bv || (ov == bv && oe < be))) { bv = ov; be = oe; }
                }
                #pragma unroll
                for (int i = 0; i < TG_MAX_PER_LANE; ++i) if (lane + 64 * i == be) used |= 1u << i;
                total_g = t == 0 ? bv : total_g + bv;
            }
            if (lane == 0) gmax[g] = total_g;
        }
        __syncthreads();
        unsigned long long kept = 0ull;                      // every lane picks the same groups: the `keep` largest, ties to the lower index
        for (int r = 0; r < keep; ++r)
        {
            int best = -1; float bv = 0.f;
            for (int g = 0; g < groups; ++g)
            {
                if ((kept >> g) & 1ull) continue;
                if (best < 0 || gmax[g] > bv) { best = g; bv = gmax[g]; }
            }
            kept |= 1ull << best;
        }
        #pragma unroll
        for (int i = 0; i < TG_MAX_PER_LANE; ++i) { const int e = lane + 64 * i; if (e < total && !((kept >> (e / per)) & 1ull)) c[i] = -INFINITY; }
    }
    float sum = 0.f, my_w = 0.f; int my_e = 0;               // lane r keeps choice r
    unsigned taken = 0u;                                     // bit i: this lane's output lane + 64 i is chosen
    for (int r = 0; r < top; ++r)
    {
        float bv = -INFINITY; int be = 0x7fffffff;
        #pragma unroll
        for (int i = 0; i < TG_MAX_PER_LANE; ++i)
        {
            const int e = lane + 64 * i;
            if (e < total && !((taken >> i) & 1u) && (c[i] > bv || be == 0x7fffffff)) { bv = c[i]; be = e; }      // ascending e within a lane: the first of equals stays
        }
        #pragma unroll
        for (int o = 32; o > 0; o >>= 1)
        {
            const float ov = __shfl_xor(bv, o, 64); const int oe = __shfl_xor(be, o, 64);
            if (oe != 0x7fffffff && (be == 0x7fffffff || ov > bv || (ov == bv && oe < be))) { bv = ov; be = oe; }
        }
        float sv = 0.f;
        #pragma unroll
        for (int i = 0; i < TG_MAX_PER_LANE; ++i) if (lane + 64 * i == be) { sv = s[i]; taken |= 1u << i; }
        sv = wave_sum(sv);
        sum += sv;
        if (lane == r) { my_w = sv; my_e = be; }
    }
    const float f = normalise ? scale / (sum + 1e-20f) : scale;
    const bool mine = lane < top;
    const float w = mine ? my_w * f : 0.f;
    const bool ident = mine && my_e >= real;
    if (mine)
    {
        idx[(int64_t) n * top + lane] = ident ? real : my_e;
        wts[(int64_t) n * top + lane] = ident ? 0.f : w;
    }
    const float iw = wave_sum(ident ? w : 0.f);
    if (idw && lane == 0) idw[n] = iw;
}

// x <- cap * tanh(x / cap) over float32 values (logits), in place
__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, int64_t count, float cap)
{
    for (int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t) gridDim.x * 256) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" int exl3_mix_embed_sinusoid(float* x, const void* table, const int32_t* tokens, const int32_t* tok_pos, const float* freq, float scale, int n, int width, int vocab,
                                       int dtype, void* stream)
{
    MIX_CHECK(x && table && tokens && tok_pos && freq && n >= 0 && width > 0 && vocab > 0, "mix_embed_sinusoid: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(embed_sinusoid_kernel<T>, dim3(n), dim3(ROW_THREADS), 0, (hipStream_t) stream, x, (const T*) table, tokens, tok_pos, freq, scale, width, vocab));
    return mix_check_launch("mix_embed_sinusoid");
}

extern "C" int exl3_mix_layer_norm_rows(void* h, const float* x, const int32_t* rows, const float* w, const float* b, float eps, int n, int width, int dtype, void* stream)
{
    MIX_CHECK(h && x && w && n >= 0 && width > 0, "mix_layer_norm_rows: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(layer_norm_rows_kernel<T>, dim3(n), dim3(ROW_THREADS), 0, (hipStream_t) stream, (T*) h, x, rows, w, b, eps, width));
    return mix_check_launch("mix_layer_norm_rows");
}

extern "C" int exl3_mix_embed_copy(float* x, void* xc, int64_t xc_ld, const void* table, const int32_t* tokens, int n, int width, int vocab, int dtype, void* stream)
{
    MIX_CHECK(x && table && tokens && n >= 0 && width > 0 && vocab > 0 && (!xc || xc_ld >= width), "mix_embed_copy: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(embed_copy_kernel<T>, dim3(n), dim3(ROW_THREADS), 0, (hipStream_t) stream, x, (T*) xc, xc_ld, (const T*) table, tokens, width, vocab));
    return mix_check_launch("mix_embed_copy");
}

extern "C" int exl3_mix_residual_norm(float* x, const void* y, int64_t y_ld, int mode, const float* rms_w, float eps, int out, float alpha, const float* w, const float* b,
                                      void* h, int64_t h_ld, int n, int width, int dtype, void* stream)
{
    MIX_CHECK(x && n >= 0 && width > 0 && mode >= 0 && mode <= 2 && out >= 0 && out <= 2, "mix_residual_norm: bad arguments");
    MIX_CHECK(mode == 0 || (y && y_ld >= width), "mix_residual_norm: an addend is needed");
    MIX_CHECK(out == 0 || (h && h_ld >= width), "mix_residual_norm: an output is needed");
    MIX_CHECK(out != 2 || (w && b), "mix_residual_norm: the norm needs its weight and bias");
    if (n == 0 || (mode == 0 && out == 0)) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(residual_norm_kernel<T>, dim3(n), dim3(ROW_THREADS), 0, (hipStream_t) stream, x, (const T*) y, y_ld, mode, rms_w, eps, out, alpha,
                                             w, b, (T*) h, h_ld, width));
    return mix_check_launch("mix_residual_norm");
}

extern "C" int exl3_mix_dyn_tanh_rows(void* h, const float* x, const int32_t* rows, float alpha, const float* w, const float* b, int n, int width, int dtype, void* stream)
{
    MIX_CHECK(h && x && w && b && n >= 0 && width > 0, "mix_dyn_tanh_rows: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(dyn_tanh_rows_kernel<T>, dim3(n), dim3(ROW_THREADS), 0, (hipStream_t) stream, (T*) h, x, rows, alpha, w, b, width));
    return mix_check_launch("mix_dyn_tanh_rows");
}

extern "C" int exl3_mix_act(void* out, const void* z, int64_t z_ld, int n, int ff, int kind, int dtype, void* stream)
{
    MIX_CHECK(out && z && n >= 0 && n <= 65535 * 1024 && ff > 0 && z_ld >= ff && kind >= 0 && kind <= 2, "mix_act: bad arguments");
    const int vn = dtype == EXL3_MIX_BF16 ? 8 : 4;
    const bool vec = ff % vn == 0 && z_ld % vn == 0 && (uintptr_t) out % 16 == 0 && (uintptr_t) z % 16 == 0;
    for (int r0 = 0; r0 < n; r0 += 65535)
    {
        const int rows = n - r0 < 65535 ? n - r0 : 65535;
        if (vec)
            MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((act_kernel<T, true>), dim3((ff / vn + 255) / 256, rows), dim3(256), 0, (hipStream_t) stream, (T*) out + (int64_t) r0 * ff,
                                                     (const T*) z + (int64_t) r0 * z_ld, z_ld, ff, kind));
        else
            MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((act_kernel<T, false>), dim3((ff + 255) / 256, rows), dim3(256), 0, (hipStream_t) stream, (T*) out + (int64_t) r0 * ff,
                                                     (const T*) z + (int64_t) r0 * z_ld, z_ld, ff, kind));
    }
    return mix_check_launch("mix_act");
}

extern "C" int exl3_mix_glu_act(void* out, const void* g, int64_t g_ld, const void* u, int64_t u_ld, int n, int ff, int kind, float limit, int dtype, void* stream)
{
    return exl3_mix_glu_act_rowgate(out, g, g_ld, u, u_ld, nullptr, 0, n, ff, kind, limit, dtype, stream);
}

extern "C" int exl3_mix_glu_act_rowgate(void* out, const void* g, int64_t g_ld, const void* u, int64_t u_ld, const void* rg, int64_t rg_ld, int n, int ff, int kind, float limit,
                                        int dtype, void* stream)
{
    MIX_CHECK(out && g && u && n >= 0 && ff > 0 && g_ld >= ff && u_ld >= ff && kind >= 0 && kind <= 1 && (!rg || rg_ld >= 1), "mix_glu_act: bad arguments");
    const int vn = dtype == EXL3_MIX_BF16 ? 8 : 4;
    const bool vec = ff % vn == 0 && g_ld % vn == 0 && u_ld % vn == 0 && (uintptr_t) out % 16 == 0 && (uintptr_t) g % 16 == 0 && (uintptr_t) u % 16 == 0;
    for (int r0 = 0; r0 < n; r0 += 65535)
    {
        const int rows = n - r0 < 65535 ? n - r0 : 65535;
        if (vec)
            MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((glu_act_kernel<T, true>), dim3((ff / vn + 255) / 256, rows), dim3(256), 0, (hipStream_t) stream, (T*) out + (int64_t) r0 * ff,
                                                     (const T*) g + (int64_t) r0 * g_ld, g_ld, (const T*) u + (int64_t) r0 * u_ld, u_ld, ff, kind, limit,
                                                     rg ? (const T*) rg + (int64_t) r0 * rg_ld : nullptr, rg_ld));
        else
            MIX_DISPATCH_T(dtype, hipLaunchKernelGGL((glu_act_kernel<T, false>), dim3((ff + 255) / 256, rows), dim3(256), 0, (hipStream_t) stream, (T*) out + (int64_t) r0 * ff,
                                                     (const T*) g + (int64_t) r0 * g_ld, g_ld, (const T*) u + (int64_t) r0 * u_ld, u_ld, ff, kind, limit,
                                                     rg ? (const T*) rg + (int64_t) r0 * rg_ld : nullptr, rg_ld));
    }
    return mix_check_launch("mix_glu_act");
}

extern "C" int exl3_mix_token_gate(void* out, const void* gate, int64_t gate_ld, const void* table, int64_t table_ld, int col0, const int32_t* tokens,
                                   int n, int dim, int vocab, int dtype, void* stream)
{
    MIX_CHECK(out && gate && table && tokens && n >= 0 && dim > 0 && vocab > 0 && gate_ld >= dim && col0 >= 0 && table_ld >= col0 + dim, "mix_token_gate: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(token_gate_kernel<T>, dim3(n), dim3(64), 0, (hipStream_t) stream, (T*) out, (const T*) gate, gate_ld, (const T*) table, table_ld,
                                             col0, tokens, dim, vocab));
    return mix_check_launch("mix_token_gate");
}

extern "C" int exl3_mix_heads_gate(void* out, const void* a, int64_t a_row, int64_t a_head, const void* gate, int64_t gate_ld, int n, int heads, int vdim, int dtype, void* stream)
{
    MIX_CHECK(out && a && n >= 0 && heads > 0 && vdim > 0 && (!gate || gate_ld >= (int64_t) heads * vdim), "mix_heads_gate: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(heads_gate_kernel<T>, dim3(n), dim3(256), 0, (hipStream_t) stream, (T*) out, (const T*) a, a_row, a_head, (const T*) gate, gate_ld,
                                             heads, vdim));
    return mix_check_launch("mix_heads_gate");
}

extern "C" int exl3_mix_topk_sigmoid(int32_t* idx, float* wts, const float* logits, const float* correction, float scale, int normalise, int n, int experts, int top, void* stream)
{
    MIX_CHECK(idx && wts && logits && n >= 0 && experts > 0 && top > 0 && top <= experts, "mix_topk_sigmoid: bad arguments (top %d of %d)", top, experts);
    if (n == 0) return EXL3_MIX_OK;
    hipLaunchKernelGGL(topk_sigmoid_kernel, dim3((n + 63) / 64), dim3(64), 0, (hipStream_t) stream, idx, wts, logits, correction, scale, normalise, n, experts, top);
    return mix_check_launch("mix_topk_sigmoid");
}

extern "C" int exl3_mix_topk_grouped(int32_t* idx, float* wts, float* idw, const float* logits, const float* correction, int kind, float scale, int normalise,
                                     int groups, int keep, int n, int total, int real, int top, void* stream)
{
    return exl3_mix_topk_grouped_ex(idx, wts, idw, logits, correction, kind, scale, normalise, groups, keep, 1, n, total, real, top, stream);
}

extern "C" int exl3_mix_topk_grouped_ex(int32_t* idx, float* wts, float* idw, const float* logits, const float* correction, int kind, float scale, int normalise,
                                        int groups, int keep, int group_top, int n, int total, int real, int top, void* stream)
{
    MIX_CHECK(group_top >= 1, "mix_topk_grouped: a group's score is the sum of at least one choice score");
    MIX_CHECK(idx && wts && logits && n >= 0 && total > 0 && real >= 0 && real <= total && (real == total || idw), "mix_topk_grouped: bad arguments");
    MIX_CHECK(total <= 64 * TG_MAX_PER_LANE && top > 0 && top <= 64 && top <= total && (kind == 0 || kind == 1), "mix_topk_grouped: at most %d outputs, top <= 64", 64 * TG_MAX_PER_LANE);
    MIX_CHECK(groups >= 1 && groups <= 64 && total % groups == 0 && keep >= 1 && keep <= groups && top <= keep * (total / groups),
              "mix_topk_grouped: %d groups (keep %d) over %d outputs cannot give %d choices", groups, keep, total, top);
    if (n == 0) return EXL3_MIX_OK;
    hipLaunchKernelGGL(topk_grouped_kernel, dim3(n), dim3(64), 0, (hipStream_t) stream, idx, wts, idw, logits, correction, kind, scale, normalise, groups, keep, total, real, top, group_top);
    return mix_check_launch("mix_topk_grouped");
}

extern "C" int exl3_mix_softcap(float* x, int64_t count, float cap, void* stream)
{
    MIX_CHECK(x && count >= 0 && cap > 0.f, "mix_softcap: bad arguments");
    if (count == 0) return EXL3_MIX_OK;
    const int blocks = (int) ((count + 255) / 256 > 4096 ? 4096 : (count + 255) / 256);
    hipLaunchKernelGGL(softcap_kernel, dim3(blocks), dim3(256), 0, (hipStream_t) stream, x, count, cap);
    return mix_check_launch("mix_softcap");
}
