// Sliding-window attention with a learned sink and a head-wise output gate: cache store (value norm, ring buffers) and the exact
// float32 form of prefill and decode -- one workgroup per (row, query head), keys of the window across lanes and waves, an online softmax
// that starts from the sink.  The matrix-core prefill kernel for bfloat16 lives in mix_attn_mfma.hip; this file is the float32 path and
// the decode path of both element types.
#include "mix_common.cuh"
#include "mix_attn_row.cuh"

template <typename T>
__global__ __launch_bounds__(64) void attn_store_kernel(T* __restrict__ v_norm, T* __restrict__ ring_k, T* __restrict__ ring_v, const T* __restrict__ k, int64_t k_ld,
                                                        const T* __restrict__ v, int64_t v_ld, const int32_t* __restrict__ tok_seq,
                                                        const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ slots,
                                                        const int32_t* __restrict__ len_after, float eps, int kv_heads, int dim, int vdim, int window)
{
    const int n = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
    const T* vr = v + (int64_t) n * v_ld + (int64_t) g * vdim;
    float ss = 0.f;
    for (int i = lane; i < vdim; i += 64) { float x = to_f(vr[i]); ss += x * x; }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float) vdim + eps);
    const int b = tok_seq[n], pos = tok_pos[n];
    const bool keep = pos >= len_after[b] - window;
    const int64_t slot_row = ((int64_t) slots[b] * window + (pos % window)) * kv_heads + g;
    T* vn = v_norm + ((int64_t) n * kv_heads + g) * vdim;
    T* rv = ring_v + slot_row * vdim;
    for (int i = lane; i < vdim; i += 64)
    {
        T o = from_f<T>(to_f(vr[i]) * inv);
        vn[i] = o;
        if (keep) rv[i] = o;
    }
    if (keep)
    {
        const T* kr = k + (int64_t) n * k_ld + (int64_t) g * dim;
        T* rk = ring_k + slot_row * dim;
        for (int i = lane; i < dim; i += 64) rk[i] = kr[i];
    }
}

// `maps` attention maps per head (differential attention: 2): queries are laid out [head][map][dim], keys [kv head][map][dim], every map of a head reads
// the values of the head's key/value head, and the result is [row][head][map][vdim].  mask 0: the last `window` positions; 1: the positions of the row's
// own chunk of `window` positions (a chunk starts where the position is a multiple of `window`).
template <typename T, int MAXV, typename TO, int NW>
__global__ __launch_bounds__(64 * NW) void attn_prefill_kernel(TO* __restrict__ out, const T* __restrict__ q, int64_t q_ld, const T* __restrict__ k, int64_t k_ld,
                                                          const T* __restrict__ v, int64_t v_ld, const T* __restrict__ gate, int64_t gate_ld, const float* __restrict__ sink,
                                                          const int32_t* __restrict__ cu, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                                          int heads, int kv_heads, int maps, int dim, int vdim, float scale, float softcap, int window, int mask)
{
    extern __shared__ float smem[];
    const int n = blockIdx.x, h = blockIdx.y;                 // h counts (head, map)
    const int hh = h / maps, g = hh / (heads / kv_heads), kh = g * maps + (h - hh * maps);
    const int b = tok_seq[n], first = cu[b];
    const int i = n - first;                                  // the row's place in its sequence == its position (the sequence starts in this step)
    const int lo = mask == EXL3_MIX_MASK_CHUNK ? (i / window) * window : max(0, i - window + 1);
    const float gt = gate ? sigmoid_f(to_f(gate[(int64_t) n * gate_ld + h])) : 1.0f;
    const T* kb = k + (int64_t) (first + lo) * k_ld + (int64_t) kh * dim;
    attn_row<T, MAXV, TO, NW>(out + ((int64_t) n * heads * maps + h) * vdim, q + (int64_t) n * q_ld + (int64_t) h * dim, q, dim, kb, k_ld,
                          v + (int64_t) (first + lo) * v_ld + (int64_t) g * vdim, v_ld,
                          i - lo + 1, dim, vdim, scale, sink != nullptr, sink ? sink[h] : 0.f, gt, rows_are_16_byte(kb, k_ld, dim), smem, softcap);
}

// Rings: ring_k [slots][window][kv_heads * maps][dim], ring_v [slots][window][kv_heads][vdim], entry = position % window.  mask 0: the newest
// min(len, window) entries (all of them, in any order); 1: the row's chunk, which is the entries 0 .. (len - 1) % window.
template <typename T, int MAXV, typename TO, int NW>
__global__ __launch_bounds__(64 * NW) void attn_decode_kernel(TO* __restrict__ out, const T* __restrict__ q, int64_t q_ld, const T* __restrict__ ring_k,
                                                         const T* __restrict__ ring_v, const T* __restrict__ gate, int64_t gate_ld, const float* __restrict__ sink,
                                                         const int32_t* __restrict__ slots, const int32_t* __restrict__ len_after,
                                                         int heads, int kv_heads, int maps, int dim, int vdim, float scale, float softcap, int window, int mask)
{
    extern __shared__ float smem[];
    const int n = blockIdx.x, h = blockIdx.y;
    const int hh = h / maps, g = hh / (heads / kv_heads), kh = g * maps + (h - hh * maps), kheads = kv_heads * maps;
    const int len = len_after[n];
    const int count = mask == EXL3_MIX_MASK_CHUNK ? (len - 1) % window + 1 : min(len, window);
    const int64_t row0 = (int64_t) slots[n] * window;
    const float gt = gate ? sigmoid_f(to_f(gate[(int64_t) n * gate_ld + h])) : 1.0f;
    const T* kb = ring_k + (row0 * kheads + kh) * dim;
    attn_row<T, MAXV, TO, NW>(out + ((int64_t) n * heads * maps + h) * vdim, q + (int64_t) n * q_ld + (int64_t) h * dim, q, dim,
                          kb, (int64_t) kheads * dim, ring_v + (row0 * kv_heads + g) * vdim, (int64_t) kv_heads * vdim,
                          count, dim, vdim, scale, sink != nullptr, sink ? sink[h] : 0.f, gt, rows_are_16_byte(kb, (int64_t) kheads * dim, dim), smem, softcap);
}

extern "C" int exl3_mix_attn_store(void* v_norm, void* ring_k, void* ring_v, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                                   const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* len_after,
                                   float eps, int n, int kv_heads, int dim, int vdim, int window, int dtype, void* stream)
{
    MIX_CHECK(v_norm && ring_k && ring_v && k && v && tok_seq && tok_pos && slots && len_after, "mix_attn_store: null pointer");
    MIX_CHECK(n >= 0 && kv_heads > 0 && dim > 0 && vdim > 0 && window > 0 && k_ld >= (int64_t) kv_heads * dim && v_ld >= (int64_t) kv_heads * vdim,
              "mix_attn_store: bad sizes");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(attn_store_kernel<T>, dim3(n, kv_heads), dim3(64), 0, (hipStream_t) stream, (T*) v_norm, (T*) ring_k, (T*) ring_v,
                                             (const T*) k, k_ld, (const T*) v, v_ld, tok_seq, tok_pos, slots, len_after, eps, kv_heads, dim, vdim, window));
    return mix_check_launch("mix_attn_store");
}

#define ATTN_LAUNCH_NW(KERNEL, TO, NWV, ...) \
    do { \
        const size_t sm = (size_t) (dim + NWV * 64 + NWV * (2 + mvt * 64)) * sizeof(float); \
        if (mv == 1)      hipLaunchKernelGGL((KERNEL<T, 1, TO, NWV>), dim3(n, heads * maps), dim3(64 * NWV), sm, (hipStream_t) stream, (TO*) out, __VA_ARGS__); \
        else if (mv == 2) hipLaunchKernelGGL((KERNEL<T, 2, TO, NWV>), dim3(n, heads * maps), dim3(64 * NWV), sm, (hipStream_t) stream, (TO*) out, __VA_ARGS__); \
        else if (mv <= 4) hipLaunchKernelGGL((KERNEL<T, 4, TO, NWV>), dim3(n, heads * maps), dim3(64 * NWV), sm, (hipStream_t) stream, (TO*) out, __VA_ARGS__); \
        else              hipLaunchKernelGGL((KERNEL<T, 8, TO, NWV>), dim3(n, heads * maps), dim3(64 * NWV), sm, (hipStream_t) stream, (TO*) out, __VA_ARGS__); \
    } while (0)
// `wide`: sixteen waves per (row, head) instead of four -- steps of few rows over long caches are bound by the chain of key chunks a wave walks, not by bytes
#define ATTN_LAUNCH_TO(KERNEL, TO, ...) \
    do { if (wide) ATTN_LAUNCH_NW(KERNEL, TO, 16, __VA_ARGS__); else ATTN_LAUNCH_NW(KERNEL, TO, AT_WAVES, __VA_ARGS__); } while (0)
// the result in the activation type, or (out_f32) in float32
#define ATTN_LAUNCH(KERNEL, ...) \
    do { \
        const int mv = (vdim + 63) / 64; \
        const int mvt = mv == 1 ? 1 : (mv == 2 ? 2 : (mv <= 4 ? 4 : 8)); \
        MIX_DISPATCH_T(dtype, if (out_f32) ATTN_LAUNCH_TO(KERNEL, float, __VA_ARGS__); else ATTN_LAUNCH_TO(KERNEL, T, __VA_ARGS__)); \
    } while (0)

static int attn_check(const char* what, int n, int heads, int kv_heads, int maps, int dim, int vdim, int window, int mask, float softcap, const void* gate)
{
    MIX_CHECK(n >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "%s: heads %d must be a multiple of kv_heads %d", what, heads, kv_heads);
    MIX_CHECK(maps >= 1 && heads * maps <= 65535 && (maps == 1 || !gate), "%s: %d maps per head (a gate per head applies to one map only)", what, maps);
    MIX_CHECK((mask == EXL3_MIX_MASK_WINDOW || mask == EXL3_MIX_MASK_CHUNK) && softcap >= 0.f, "%s: unknown mask %d or a negative softcap", what, mask);
    MIX_CHECK(dim > 0 && dim <= 4096 && vdim > 0 && vdim <= 512 && window > 0, "%s: dim %d / vdim %d / window %d out of range", what, dim, vdim, window);
    return EXL3_MIX_OK;
}

extern "C" int exl3_mix_attn_prefill_ex(void* out, int out_f32, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                                        const void* gate, int64_t gate_ld, const float* sink, const int32_t* cu, const int32_t* tok_seq, const int32_t* tok_pos,
                                        int n, int heads, int kv_heads, int maps, int dim, int vdim, float scale, float softcap, int window, int mask, int dtype, void* stream)
{
    MIX_CHECK(out && q && k && v && cu && tok_seq && tok_pos, "mix_attn_prefill: null pointer");
    if (int rc = attn_check("mix_attn_prefill", n, heads, kv_heads, maps, dim, vdim, window, mask, softcap, gate)) return rc;
    MIX_CHECK(q_ld >= (int64_t) heads * maps * dim && k_ld >= (int64_t) kv_heads * maps * dim && v_ld >= (int64_t) kv_heads * vdim && (!gate || gate_ld >= heads),
              "mix_attn_prefill: bad row strides");
    if (n == 0) return EXL3_MIX_OK;
    const bool wide = false;
    ATTN_LAUNCH(attn_prefill_kernel, (const T*) q, q_ld, (const T*) k, k_ld, (const T*) v, v_ld, (const T*) gate, gate_ld, sink, cu, tok_seq, tok_pos,
                heads, kv_heads, maps, dim, vdim, scale, softcap, window, mask);
    return mix_check_launch("mix_attn_prefill");
}

extern "C" int exl3_mix_attn_prefill(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v_norm,
                                     const void* gate, int64_t gate_ld, const float* sink, const int32_t* cu, const int32_t* tok_seq, const int32_t* tok_pos,
                                     int n, int heads, int kv_heads, int dim, int vdim, float scale, int window, int dtype, void* stream)
{
    return exl3_mix_attn_prefill_ex(out, 0, q, q_ld, k, k_ld, v_norm, (int64_t) kv_heads * vdim, gate, gate_ld, sink, cu, tok_seq, tok_pos, n, heads, kv_heads, 1, dim, vdim,
                                    scale, 0.f, window, EXL3_MIX_MASK_WINDOW, dtype, stream);
}

extern "C" int exl3_mix_attn_decode_ex(void* out, int out_f32, const void* q, int64_t q_ld, const void* ring_k, const void* ring_v,
                                       const void* gate, int64_t gate_ld, const float* sink, const int32_t* slots, const int32_t* len_after,
                                       int n, int heads, int kv_heads, int maps, int dim, int vdim, float scale, float softcap, int window, int mask, int dtype, void* stream)
{
    MIX_CHECK(out && q && ring_k && ring_v && slots && len_after, "mix_attn_decode: null pointer");
    if (int rc = attn_check("mix_attn_decode", n, heads, kv_heads, maps, dim, vdim, window, mask, softcap, gate)) return rc;
    MIX_CHECK(q_ld >= (int64_t) heads * maps * dim && (!gate || gate_ld >= heads), "mix_attn_decode: bad row strides");
    if (n == 0) return EXL3_MIX_OK;
    const bool wide = (int64_t) n * heads * maps <= 256 && window > 256 && vdim <= 256;
    ATTN_LAUNCH(attn_decode_kernel, (const T*) q, q_ld, (const T*) ring_k, (const T*) ring_v, (const T*) gate, gate_ld, sink, slots, len_after,
                heads, kv_heads, maps, dim, vdim, scale, softcap, window, mask);
    return mix_check_launch("mix_attn_decode");
}

extern "C" int exl3_mix_attn_decode(void* out, const void* q, int64_t q_ld, const void* ring_k, const void* ring_v,
                                    const void* gate, int64_t gate_ld, const float* sink, const int32_t* slots, const int32_t* len_after,
                                    int n, int heads, int kv_heads, int dim, int vdim, float scale, int window, int dtype, void* stream)
{
    return exl3_mix_attn_decode_ex(out, 0, q, q_ld, ring_k, ring_v, gate, gate_ld, sink, slots, len_after, n, heads, kv_heads, 1, dim, vdim, scale, 0.f, window,
                                   EXL3_MIX_MASK_WINDOW, dtype, stream);
}
