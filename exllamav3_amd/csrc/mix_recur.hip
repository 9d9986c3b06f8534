// Recurrent mixers whose memory is one float32 matrix per head with a SCALAR decay per head and token: the matrix memory with exponential gating and a
// running maximum (mLSTM), and the gated delta rule.  Both are token-by-token scans that carry the state of a sequence in its slot; decode is the same
// kernel over one token.  Also here: the delta rule's input stage (short causal convolutions with silu, unit vectors, step size and decay), the
// per-head output norm with a gate, and the sum of two RMS-normed branches.
//
// Work split of the scans: one workgroup of 4 waves per (sequence, head, block of 16 value columns).  A wave owns 4 columns; the 16 lanes of a row
// split the key channels of one column (lane kl holds channels kl, kl + 16, ... -- R of them, in registers), so that every product with the state is
// R multiply-adds per lane and one sum over a row of 16 lanes (data-parallel primitives, no LDS).  The state is stored [slot][head][vdim][dim]: a row of
// lanes reads consecutive floats.  A chunk of 16 to 64 tokens is staged in LDS; the waves run it without a barrier and the outputs leave through LDS.
// Everything that enters the recurrences is float32.
#include "mix_common.cuh"

#define RC_COLS 16
// tokens staged per chunk: as many as 32 KB of queries and keys allow (a chunk costs two barriers and, for mLSTM, the gates' transcendentals)
template <int R> struct rc_chunk { static constexpr int TC = R <= 4 ? 64 : (R <= 8 ? 32 : 16); };

// ---------------------------------------------------------------------------------------------------------------------------------------------
// How both scans walk a sequence.  The rows of chunk c + 1 are loaded into REGISTERS before the token loop of chunk c starts and stored to LDS after it ends, so
// the trip to memory runs under the token loop (with fewer workgroups than compute units nothing else would hide it).  Per chunk: registers -> LDS, barrier,
// loads of the next chunk, token loop in groups of four (the tail of a chunk is padded with tokens that change nothing), barrier, outputs from LDS to memory.

// mLSTM.  Per head and token, with log gates i (input) and f (forget) and the running maximum m (m = 0 before the first token):
//   m' = max(f + m, i);  a = exp(f + m - m'), b = exp(i - m');  S <- a S + b k v^T;  n <- a n + b k;  o = S^T q / (max(|n.q|, exp(-m')) + 1e-6)
// i = cap tanh((z_i + bias_i) / cap), f = logsigmoid(cap tanh((z_f + bias_f) / cap)) from the projections z_i, z_f.  q is scaled by q_scale.
// The gates' part of the recurrence stays off the token loop: a token is the map m -> max(m + f, i), maps compose to maps of the same form
// ((f1, i1) then (f2, i2) = (f1 + f2, max(i1 + f2, i2))), so one wave scans a chunk's maps across its lanes in six steps and takes the exponentials of all
// tokens side by side.
template <typename T, int R>
__global__ __launch_bounds__(256) void mlstm_scan_kernel(float* __restrict__ o, float* __restrict__ S_state, float* __restrict__ n_state, float* __restrict__ m_state,
                                                         const T* __restrict__ q, int64_t q_ld, const T* __restrict__ k, int64_t k_ld, const T* __restrict__ v, int64_t v_ld,
                                                         const T* __restrict__ zi, int64_t zi_ld, const T* __restrict__ zf, int64_t zf_ld,
                                                         const float* __restrict__ bias_i, const float* __restrict__ bias_f,
                                                         const int32_t* __restrict__ cu, const int32_t* __restrict__ slots, const int32_t* __restrict__ pos0,
                                                         int heads, int dim, int vdim, float q_scale, float cap)
{
    constexpr int DP = 16 * R, RC_TC = rc_chunk<R>::TC, NPT = RC_TC * DP / 256, NVT = RC_TC * RC_COLS / 256;
    __shared__ __attribute__((aligned(16))) float qs[RC_TC * DP], ks[RC_TC * DP], vs[RC_TC * RC_COLS], sa[RC_TC], sb[RC_TC], se[RC_TC], os[RC_TC * RC_COLS];
    const int b = blockIdx.x, h = blockIdx.y, vt = blockIdx.z;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int kl = lane & 15, cw = w * 4 + (lane >> 4);              // key lane, column inside the workgroup's block
    const int col = vt * RC_COLS + cw;
    const bool col_ok = col < vdim;
    const int first = cu[b], last = cu[b + 1];
    const bool resume = pos0[b] > 0;
    const int64_t sh = (int64_t) slots[b] * heads + h;
    float* st = S_state + (sh * vdim + (col_ok ? col : 0)) * dim;
    float* nst = n_state + sh * dim;
    float S[R], N[R];
    #pragma unroll
    for (int r = 0; r < R; ++r)
    {
        const int c = kl + 16 * r;
        S[r] = (resume && col_ok && c < dim) ? st[c] : 0.f;
        N[r] = (resume && c < dim) ? nst[c] : 0.f;
    }
    float m_run = resume ? m_state[sh] : 0.f;                        // kept current by wave 0
    const float bi = bias_i[h], bfg = bias_f[h];
    T tq[NPT], tk[NPT], tv[NVT], tzi = from_f<T>(0.f), tzf = from_f<T>(0.f);      // held as loaded: a conversion here would wait for the loads before the token loop
    const T zero = from_f<T>(0.f);
    #define ML_FETCH(N0) \
        do { \
            const int f_tc = min(RC_TC, last - (N0)); \
            _Pragma("unroll") \
            for (int e = 0; e < NPT; ++e) \
            { \
                const int idx = threadIdx.x + e * 256, t = idx / DP, c = idx - t * DP; \
                const bool ok = t < f_tc && c < dim; \
                tq[e] = ok ? q[(int64_t) ((N0) + t) * q_ld + (int64_t) h * dim + c] : zero; \
                tk[e] = ok ? k[(int64_t) ((N0) + t) * k_ld + (int64_t) h * dim + c] : zero; \
            } \
            _Pragma("unroll") \
            for (int e = 0; e < NVT; ++e) \
            { \
                const int idx = threadIdx.x + e * 256, t = idx / RC_COLS, c = vt * RC_COLS + (idx - t * RC_COLS); \
                tv[e] = (t < f_tc && c < vdim) ? v[(int64_t) ((N0) + t) * v_ld + (int64_t) h * vdim + c] : zero; \
            } \
            if (w == 0 && lane < f_tc) \
            { \
                tzi = zi[(int64_t) ((N0) + lane) * zi_ld + h]; \
                tzf = zf[(int64_t) ((N0) + lane) * zf_ld + h]; \
            } \
        } while (0)
    if (first < last) ML_FETCH(first);

    for (int n0 = first; n0 < last; n0 += RC_TC)
    {
        const int tc = min(RC_TC, last - n0);
        const int tcp = (tc + 3) & ~3;
        #pragma unroll
        for (int e = 0; e < NPT; ++e)
        {
            const int idx = threadIdx.x + e * 256, t = idx / DP, c = idx - t * DP, at = t * DP + (c & 15) * R + (c >> 4);      // a lane's R channels side by side
            qs[at] = to_f(tq[e]) * q_scale; ks[at] = to_f(tk[e]);
        }
        #pragma unroll
        for (int e = 0; e < NVT; ++e) vs[threadIdx.x + e * 256] = to_f(tv[e]);
        if (w == 0)
        {
            const bool real = lane < tc;
            const float F = real ? log_sigmoid_f(cap * tanhf((to_f(tzf) + bfg) / cap)) : 0.f;
            const float I = real ? cap * tanhf((to_f(tzi) + bi) / cap) : -INFINITY;
            float sF = F, sM = I;                                    // the composition of the chunk's maps up to this lane's token
            #pragma unroll
            for (int off = 1; off < 64; off <<= 1)
            {
                const float pF = __shfl_up(sF, off, 64), pM = __shfl_up(sM, off, 64);
                if (lane >= off) { sM = fmaxf(pM + sF, sM); sF = pF + sF; }
            }
            const float m_t = fmaxf(m_run + sF, sM);
            float m_prev = __shfl_up(m_t, 1, 64);
            if (lane == 0) m_prev = m_run;
            if (lane < RC_TC)
            {
                sa[lane] = real ? expf(F + m_prev - m_t) : 1.0f;
                sb[lane] = real ? expf(I - m_t) : 0.0f;
                se[lane] = expf(-m_t);
            }
            m_run = __shfl(m_t, tc - 1, 64);
        }
        __syncthreads();
        if (n0 + RC_TC < last) ML_FETCH(n0 + RC_TC);                 // in flight during the token loop
        for (int t0 = 0; t0 < tcp; t0 += 4)
        {
            #pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                const int t = t0 + u;
                const float a = sa[t], bb = sb[t];
                const float vv = vs[t * RC_COLS + cw] * bb;
                float po = 0.f, pn = 0.f;
                #pragma unroll
                for (int r = 0; r < R; ++r)
                {
                    const float kk = ks[t * DP + kl * R + r], qq = qs[t * DP + kl * R + r];
                    S[r] = __builtin_fmaf(a, S[r], kk * vv);
                    N[r] = __builtin_fmaf(a, N[r], bb * kk);
                    po = __builtin_fmaf(qq, S[r], po);
                    pn = __builtin_fmaf(qq, N[r], pn);
                }
                po = row16_sum(po);
                pn = row16_sum(pn);
                if (kl == 0) os[t * RC_COLS + cw] = po * __builtin_amdgcn_rcpf(fmaxf(fabsf(pn), se[t]) + 1e-6f);
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < tc * RC_COLS; idx += 256)
        {
            const int t = idx / RC_COLS, c = vt * RC_COLS + (idx - t * RC_COLS);
            if (c < vdim) o[((int64_t) (n0 + t) * heads + h) * vdim + c] = os[idx];
        }
    }
    #undef ML_FETCH
    #pragma unroll
    for (int r = 0; r < R; ++r)
    {
        const int c = kl + 16 * r;
        if (col_ok && c < dim) st[c] = S[r];
        if (vt == 0 && cw == 0 && c < dim) nst[c] = N[r];
    }
    if (vt == 0 && threadIdx.x == 0) m_state[sh] = m_run;
}

// ---------------------------------------------------------------------------------------------------------------------------------------------
// Gated delta rule.  Per head and token, with the decay g and the step size beta:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// (the read-out sees the token's own write).  One pass over the state per token: with the old state, pk = k.S, pq = q.S, then u = beta (v - g pk),
// o = g pq + (q.k) u, S <- g S + k u.  q, k, v, beta, g are float32 (written by delta_prep); query / key heads may be shared by several value heads.
template <int R>
__global__ __launch_bounds__(256) void delta_scan_kernel(float* __restrict__ o, float* __restrict__ S_state, const float* __restrict__ q, const float* __restrict__ k,
                                                         const float* __restrict__ v, const float* __restrict__ beta, const float* __restrict__ decay,
                                                         const int32_t* __restrict__ cu, const int32_t* __restrict__ slots, const int32_t* __restrict__ pos0,
                                                         int heads, int kv_heads, int dim, int vdim)
{
    constexpr int DP = 16 * R, RC_TC = rc_chunk<R>::TC, NPT = RC_TC * DP / 256, NVT = RC_TC * RC_COLS / 256;
    __shared__ __attribute__((aligned(16))) float qs[RC_TC * DP], ks[RC_TC * DP], vs[RC_TC * RC_COLS], gs[RC_TC], bs[RC_TC], os[RC_TC * RC_COLS];
    const int b = blockIdx.x, h = blockIdx.y, vt = blockIdx.z;
    const int g = h / (heads / kv_heads);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int kl = lane & 15, cw = w * 4 + (lane >> 4);
    const int col = vt * RC_COLS + cw;
    const bool col_ok = col < vdim;
    const int first = cu[b], last = cu[b + 1];
    const bool resume = pos0[b] > 0;
    float* st = S_state + (((int64_t) slots[b] * heads + h) * vdim + (col_ok ? col : 0)) * dim;
    const int64_t qk_ld = (int64_t) kv_heads * dim;
    float S[R];
    #pragma unroll
    for (int r = 0; r < R; ++r)
    {
        const int c = kl + 16 * r;
        S[r] = (resume && col_ok && c < dim) ? st[c] : 0.f;
    }
    float tq[NPT], tk[NPT], tv[NVT], tg = 1.0f, tb = 0.0f;
    #define DL_FETCH(N0) \
        do { \
            const int f_tc = min(RC_TC, last - (N0)); \
            _Pragma("unroll") \
            for (int e = 0; e < NPT; ++e) \
            { \
                const int idx = threadIdx.x + e * 256, t = idx / DP, c = idx - t * DP; \
                const int64_t at = (int64_t) ((N0) + t) * qk_ld + (int64_t) g * dim + c; \
                const bool ok = t < f_tc && c < dim; \
                tq[e] = ok ? q[at] : 0.f; \
                tk[e] = ok ? k[at] : 0.f; \
            } \
            _Pragma("unroll") \
            for (int e = 0; e < NVT; ++e) \
            { \
                const int idx = threadIdx.x + e * 256, t = idx / RC_COLS, c = vt * RC_COLS + (idx - t * RC_COLS); \
                tv[e] = (t < f_tc && c < vdim) ? v[((int64_t) ((N0) + t) * heads + h) * vdim + c] : 0.f; \
            } \
            const bool f_real = (int) threadIdx.x < f_tc;            /* padding: g = 1, beta = 0 */ \
            tg = f_real ? decay[(int64_t) ((N0) + threadIdx.x) * heads + h] : 1.0f; \
            tb = f_real ? beta[(int64_t) ((N0) + threadIdx.x) * heads + h] : 0.0f; \
        } while (0)
    if (first < last) DL_FETCH(first);

    for (int n0 = first; n0 < last; n0 += RC_TC)
    {
        const int tc = min(RC_TC, last - n0);
        const int tcp = (tc + 3) & ~3;
        #pragma unroll
        for (int e = 0; e < NPT; ++e)
        {
            const int idx = threadIdx.x + e * 256, t = idx / DP, c = idx - t * DP, at = t * DP + (c & 15) * R + (c >> 4);      // a lane's R channels side by side
            qs[at] = tq[e]; ks[at] = tk[e];
        }
        #pragma unroll
        for (int e = 0; e < NVT; ++e) vs[threadIdx.x + e * 256] = tv[e];
        if (threadIdx.x < RC_TC) { gs[threadIdx.x] = tg; bs[threadIdx.x] = tb; }
        __syncthreads();
        if (n0 + RC_TC < last) DL_FETCH(n0 + RC_TC);                 // in flight during the token loop
        for (int t0 = 0; t0 < tcp; t0 += 4)
        {
            #pragma unroll
            for (int u4 = 0; u4 < 4; ++u4)
            {
                const int t = t0 + u4;
                const float gg = gs[t], bb = bs[t], vv = vs[t * RC_COLS + cw];
                float kk[R];
                float pk = 0.f, pk2 = 0.f, pq = 0.f, qk = 0.f;
                #pragma unroll
                for (int r = 0; r < R; ++r)
                {
                    kk[r] = ks[t * DP + kl * R + r];
                    const float qq = qs[t * DP + kl * R + r];
                    if (r & 1) pk2 = __builtin_fmaf(kk[r], S[r], pk2); else pk = __builtin_fmaf(kk[r], S[r], pk);      // the sum the next state waits for: two chains
                    pq = __builtin_fmaf(qq, S[r], pq);
                    qk = __builtin_fmaf(qq, kk[r], qk);
                }
                pk = row16_sum(pk + pk2);
                const float u = bb * __builtin_fmaf(-gg, pk, vv);
                #pragma unroll
                for (int r = 0; r < R; ++r) S[r] = __builtin_fmaf(kk[r], u, gg * S[r]);
                pq = row16_sum(pq);
                qk = row16_sum(qk);
                if (kl == 0) os[t * RC_COLS + cw] = __builtin_fmaf(qk, u, gg * pq);
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < tc * RC_COLS; idx += 256)
        {
            const int t = idx / RC_COLS, c = vt * RC_COLS + (idx - t * RC_COLS);
            if (c < vdim) o[((int64_t) (n0 + t) * heads + h) * vdim + c] = os[idx];
        }
    }
    #undef DL_FETCH
    #pragma unroll
    for (int r = 0; r < R; ++r)
    {
        const int c = kl + 16 * r;
        if (col_ok && c < dim) st[c] = S[r];
    }
}

// The delta rule's input stage, one workgroup per row.  x [n][C] holds the projections q | k | v side by side (C = 2 G dim + H vdim).  Every channel
// passes a short causal convolution over time (conv_w [taps][C], the last tap is the row's own; predecessors are the step's own rows where the
// sequence has them in the step, the slot's ring of the last taps - 1 rows otherwise, zeros before the sequence's start) and silu.  Then every
// query / key head becomes a unit vector x / sqrt(sum x^2 + 1e-6), queries times q_scale.  beta = sigmoid(zb), decay = exp(-exp(A_log) softplus(za + dt_bias))
// per value head.  Results are float32.  The rows at the last taps - 1 positions of a sequence go into the ring (entry = position mod (taps - 1)).
template <typename T>
__global__ __launch_bounds__(256) void delta_prep_kernel(float* __restrict__ qo, float* __restrict__ ko, float* __restrict__ vo, float* __restrict__ beta, float* __restrict__ decay,
                                                         const T* __restrict__ x, int64_t x_ld, const float* __restrict__ conv_w, int taps, T* __restrict__ ring,
                                                         const T* __restrict__ zb, int64_t zb_ld, const T* __restrict__ za, int64_t za_ld,
                                                         const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                                         const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ slots,
                                                         const int32_t* __restrict__ pos0, const int32_t* __restrict__ len_after,
                                                         int heads, int kv_heads, int dim, int vdim, float q_scale)
{
    extern __shared__ float buf[];                                   // [C]
    const int n = blockIdx.x;
    const int QK = kv_heads * dim, C = 2 * QK + heads * vdim;
    const int b = tok_seq[n], pos = tok_pos[n], keep = taps - 1, start = pos0[b];
    T* rg = ring + (int64_t) slots[b] * (keep > 0 ? keep : 1) * C;
    const bool store = keep > 0 && pos >= len_after[b] - keep;
    for (int c = threadIdx.x; c < C; c += 256)
    {
        const T own = x[(int64_t) n * x_ld + c];
        float acc = conv_w[(int64_t) keep * C + c] * to_f(own);
        for (int j = 0; j < keep; ++j)
        {
            const int back = keep - j, p = pos - back;
            if (p < 0) continue;
            const T pv = p >= start ? x[(int64_t) (n - back) * x_ld + c] : rg[(int64_t) (p % keep) * C + c];
            acc += conv_w[(int64_t) j * C + c] * to_f(pv);
        }
        if (store) rg[(int64_t) (pos % keep) * C + c] = own;         // after this thread's own reads of the channel
        const float y = silu_f(acc);
        buf[c] = y;
        if (c >= 2 * QK) vo[(int64_t) n * heads * vdim + (c - 2 * QK)] = y;
    }
    if (threadIdx.x < heads)
    {
        const int h = threadIdx.x;
        beta[(int64_t) n * heads + h] = sigmoid_f(to_f(zb[(int64_t) n * zb_ld + h]));
        decay[(int64_t) n * heads + h] = expf(-expf(A_log[h]) * softplus_f(to_f(za[(int64_t) n * za_ld + h]) + dt_bias[h]));
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int vec = w; vec < 2 * kv_heads; vec += 4)                  // query heads first, then key heads
    {
        const float* src = buf + (int64_t) vec * dim;
        float ss = 0.f;
        for (int i = lane; i < dim; i += 64) ss += src[i] * src[i];
        ss = wave_sum(ss);
        const float f = (vec < kv_heads ? q_scale : 1.0f) / sqrtf(ss + 1e-6f);
        float* dst = vec < kv_heads ? qo + (int64_t) n * QK + (int64_t) vec * dim : ko + (int64_t) n * QK + (int64_t) (vec - kv_heads) * dim;
        for (int i = lane; i < dim; i += 64) dst[i] = src[i] * f;
    }
}

// out[n][h][i] = o[n][h][i] / sqrt(mean_i(o[n][h]^2) + eps) * w[(per_head ? h vdim : 0) + i] * gate(g[n][h vdim + i]); gate 0: silu, 1: sigmoid
template <typename T>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(T* __restrict__ out, const float* __restrict__ o, const float* __restrict__ w, int per_head, const T* __restrict__ g,
                                                            int64_t g_ld, int gate, float eps, int heads, int vdim)
{
    const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* orow = o + ((int64_t) n * heads + h) * vdim;
    float ss = 0.f;
    for (int i = lane; i < vdim; i += 64) { const float x = orow[i]; ss += x * x; }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float) vdim + eps);
    const T* gr = g + (int64_t) n * g_ld + (int64_t) h * vdim;
    const float* wr = w + (per_head ? (int64_t) h * vdim : 0);
    T* dst = out + ((int64_t) n * heads + h) * vdim;
    for (int i = lane; i < vdim; i += 64)
    {
        const float z = to_f(gr[i]);
        dst[i] = from_f<T>(orow[i] * inv * wr[i] * (gate == 0 ? silu_f(z) : sigmoid_f(z)));
    }
}

// out[n] = scale (a[n] / rms(a[n]) * wa + b[n] / rms(b[n]) * wb): two branches, each RMS-normed over the row with its own plain weight
template <typename T>
__global__ __launch_bounds__(256) void rms_pair_kernel(T* __restrict__ out, const T* __restrict__ a, int64_t a_ld, const float* __restrict__ wa, const T* __restrict__ bq, int64_t b_ld,
                                                       const float* __restrict__ wb, float scale, float eps, int width)
{
    __shared__ float red[4];
    const int n = blockIdx.x;
    const T* ar = a + (int64_t) n * a_ld;
    const T* br = bq + (int64_t) n * b_ld;
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < width; i += 256) { const float x = to_f(ar[i]), y = to_f(br[i]); sa += x * x; sb += y * y; }
    sa = block_sum<4>(sa, red);
    sb = block_sum<4>(sb, red);
    const float ia = 1.0f / sqrtf(sa / (float) width + eps), ib = 1.0f / sqrtf(sb / (float) width + eps);
    for (int i = threadIdx.x; i < width; i += 256)
        out[(int64_t) n * width + i] = from_f<T>(scale * (to_f(ar[i]) * ia * wa[i] + to_f(br[i]) * ib * wb[i]));
}

extern "C" int exl3_mix_mlstm_scan(float* o, float* S_state, float* n_state, float* m_state, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                                   const void* zi, int64_t zi_ld, const void* zf, int64_t zf_ld, const float* bias_i, const float* bias_f,
                                   const int32_t* cu, const int32_t* slots, const int32_t* pos0, int batch, int heads, int dim, int vdim, float q_scale, float cap,
                                   int dtype, void* stream)
{
    MIX_CHECK(o && S_state && n_state && m_state && q && k && v && zi && zf && bias_i && bias_f && cu && slots && pos0, "mix_mlstm_scan: null pointer");
    MIX_CHECK(batch >= 0 && batch <= 65535 * 32 && heads > 0 && heads <= 65535 && dim > 0 && dim <= 256 && vdim > 0 && cap > 0.f, "mix_mlstm_scan: sizes out of range (dim %d <= 256)", dim);
    MIX_CHECK(q_ld >= (int64_t) heads * dim && k_ld >= (int64_t) heads * dim && v_ld >= (int64_t) heads * vdim && zi_ld >= heads && zf_ld >= heads, "mix_mlstm_scan: bad row strides");
    if (batch == 0) return EXL3_MIX_OK;
    const dim3 grid(batch, heads, (vdim + RC_COLS - 1) / RC_COLS);
    const int r = (dim + 15) / 16;
    #define ML_SCAN(RV) hipLaunchKernelGGL((mlstm_scan_kernel<T, RV>), grid, dim3(256), 0, (hipStream_t) stream, o, S_state, n_state, m_state, (const T*) q, q_ld, (const T*) k, k_ld, \
                                           (const T*) v, v_ld, (const T*) zi, zi_ld, (const T*) zf, zf_ld, bias_i, bias_f, cu, slots, pos0, heads, dim, vdim, q_scale, cap)
    MIX_DISPATCH_T(dtype, if (r <= 2) ML_SCAN(2); else if (r <= 4) ML_SCAN(4); else if (r <= 8) ML_SCAN(8); else ML_SCAN(16));
    #undef ML_SCAN
    return mix_check_launch("mix_mlstm_scan");
}

extern "C" int exl3_mix_delta_scan(float* o, float* S_state, const float* q, const float* k, const float* v, const float* beta, const float* decay,
                                   const int32_t* cu, const int32_t* slots, const int32_t* pos0, int batch, int heads, int kv_heads, int dim, int vdim, void* stream)
{
    MIX_CHECK(o && S_state && q && k && v && beta && decay && cu && slots && pos0, "mix_delta_scan: null pointer");
    MIX_CHECK(batch >= 0 && heads > 0 && heads <= 65535 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && dim <= 256 && vdim > 0,
              "mix_delta_scan: sizes out of range (dim %d <= 256, %d heads over %d query/key heads)", dim, heads, kv_heads);
    if (batch == 0) return EXL3_MIX_OK;
    const dim3 grid(batch, heads, (vdim + RC_COLS - 1) / RC_COLS);
    const int r = (dim + 15) / 16;
    #define DL_SCAN(RV) hipLaunchKernelGGL((delta_scan_kernel<RV>), grid, dim3(256), 0, (hipStream_t) stream, o, S_state, q, k, v, beta, decay, cu, slots, pos0, heads, kv_heads, dim, vdim)
    if (r <= 2) DL_SCAN(2); else if (r <= 4) DL_SCAN(4); else if (r <= 8) DL_SCAN(8); else DL_SCAN(16);
    #undef DL_SCAN
    return mix_check_launch("mix_delta_scan");
}

extern "C" int exl3_mix_delta_prep(float* qo, float* ko, float* vo, float* beta, float* decay, const void* x, int64_t x_ld, const float* conv_w, int taps, void* ring,
                                   const void* zb, int64_t zb_ld, const void* za, int64_t za_ld, const float* A_log, const float* dt_bias,
                                   const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* pos0, const int32_t* len_after,
                                   int n, int heads, int kv_heads, int dim, int vdim, float q_scale, int dtype, void* stream)
{
    MIX_CHECK(qo && ko && vo && beta && decay && x && conv_w && ring && zb && za && A_log && dt_bias && tok_seq && tok_pos && slots && pos0 && len_after, "mix_delta_prep: null pointer");
    const int64_t C = 2 * (int64_t) kv_heads * dim + (int64_t) heads * vdim;
    MIX_CHECK(n >= 0 && heads > 0 && heads <= 256 && kv_heads > 0 && dim > 0 && vdim > 0 && taps >= 1 && taps <= 16 && C <= 15360 && x_ld >= C && zb_ld >= heads && za_ld >= heads,
              "mix_delta_prep: sizes out of range (%d heads <= 256, %lld channels <= 15360, 1..16 taps)", heads, (long long) C);
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(delta_prep_kernel<T>, dim3(n), dim3(256), (size_t) C * sizeof(float), (hipStream_t) stream, qo, ko, vo, beta, decay, (const T*) x, x_ld, conv_w, taps,
                                             (T*) ring, (const T*) zb, zb_ld, (const T*) za, za_ld, A_log, dt_bias, tok_seq, tok_pos, slots, pos0, len_after, heads, kv_heads, dim, vdim, q_scale));
    return mix_check_launch("mix_delta_prep");
}

extern "C" int exl3_mix_head_norm_gate(void* out, const float* o, const float* w, int per_head, const void* g, int64_t g_ld, int gate, float eps, int n, int heads, int vdim,
                                       int dtype, void* stream)
{
    MIX_CHECK(out && o && w && g && n >= 0 && heads > 0 && heads <= 65535 && vdim > 0 && g_ld >= (int64_t) heads * vdim && (gate == 0 || gate == 1), "mix_head_norm_gate: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(head_norm_gate_kernel<T>, dim3(n, heads), dim3(64), 0, (hipStream_t) stream, (T*) out, o, w, per_head, (const T*) g, g_ld, gate, eps, heads, vdim));
    return mix_check_launch("mix_head_norm_gate");
}

extern "C" int exl3_mix_rms_pair(void* out, const void* a, int64_t a_ld, const float* wa, const void* b, int64_t b_ld, const float* wb, float scale, float eps, int n, int width,
                                 int dtype, void* stream)
{
    MIX_CHECK(out && a && wa && b && wb && n >= 0 && width > 0 && a_ld >= width && b_ld >= width, "mix_rms_pair: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(rms_pair_kernel<T>, dim3(n), dim3(256), 0, (hipStream_t) stream, (T*) out, (const T*) a, a_ld, wa, (const T*) b, b_ld, wb, scale, eps, width));
    return mix_check_launch("mix_rms_pair");
}
