// Kernels of the mixers and arrangements beside the softmax decoder's: layer norm (alone, and fused with
// the scaled residual sum of a post-norm layer), token shift with its per-sequence state, rotation in the
// half layout followed by a unit-RMS norm of q and k with the write into the paged cache, attention whose
// weights are sigmoids of the scores, linear attention with a constant decay per head and a float32 state
// per sequence, the gated RMS norm behind it, and the PolyNorm activation.  Every size is a run-time value.
// Whatever a norm, a score, an attention weight or a recurrent state is made of is float32 here, whatever
// the type of the matrices.
#include "common.h"

struct Pages {
    const void* k;
    const void* v;
    int64_t page_stride;            // elements from one page to the next
    const int* page_table;          // [slots, max_pages]
    int max_pages;
};

__device__ __forceinline__ float sigmoidf(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float siluf(float z) { return z / (1.f + expf(-z)); }

// ---------------------------------------------------------------------------
// Layer norm with a weight and no bias: out = (x - mean) / sqrt(var + eps) * w, var the mean of the
// squared deviations.  `rows` (may be null) picks rows.
// ---------------------------------------------------------------------------
template <class TO>
__global__ void layernorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                 const int* __restrict__ rows, TO* __restrict__ out, int d, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const float* xr = x + (int64_t)(rows ? rows[r] : r) * d;
    TO* o = out + (int64_t)r * d;
    float s = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) s += xr[i];
    const float mean = block_sum(s, scratch) / (float)d;
    float ss = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) { const float v = xr[i] - mean; ss += v * v; }
    const float sd = sqrtf(block_sum(ss, scratch) / (float)d + eps);
    for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = from_f32<TO>((xr[i] - mean) / sd * w[i]);
}

extern "C" int li_layernorm(const float* x, const float* w, const int* rows, void* out, int out_dt, int n_rows,
                            int d, float eps, hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (d <= 0) return LI_BAD_ARG;
    dim3 grid(n_rows), block(d >= 2048 ? 512 : (d >= 256 ? 256 : 64));
    if (out_dt == DT_F32) layernorm_kernel<float><<<grid, block, 0, stream>>>(x, w, rows, (float*)out, d, eps);
    else if (out_dt == DT_F16) layernorm_kernel<f16><<<grid, block, 0, stream>>>(x, w, rows, (f16*)out, d, eps);
    else if (out_dt == DT_BF16) layernorm_kernel<bf16><<<grid, block, 0, stream>>>(x, w, rows, (bf16*)out, d, eps);
    else return LI_BAD_ARG;
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// The residual step of a layer whose norm comes after the sum:
//   x <- LN(alpha * x + (s1 * y1 + s2 * y2)) * w        (y2 may be null)
// in place on the float32 rows of x; `copy` (may be null) receives the new rows in a 16-bit type as well,
// for the product that reads them next.
// ---------------------------------------------------------------------------
template <class TC>
__global__ void add_layernorm_kernel(float* __restrict__ x, float alpha, const float* __restrict__ y1, float s1,
                                     const float* __restrict__ y2, float s2, const float* __restrict__ w, float eps,
                                     TC* __restrict__ copy, int d) {
    __shared__ float scratch[16];
    const int64_t base = (int64_t)blockIdx.x * d;
    float* xr = x + base;
    float s = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        float y = s1 * y1[base + i];
        if (y2) y += s2 * y2[base + i];
        const float v = alpha * xr[i] + y;
        xr[i] = v;                                // read back by the same thread below
        s += v;
    }
    const float mean = block_sum(s, scratch) / (float)d;
    float ss = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) { const float v = xr[i] - mean; ss += v * v; }
    const float sd = sqrtf(block_sum(ss, scratch) / (float)d + eps);
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        const float v = (xr[i] - mean) / sd * w[i];
        xr[i] = v;
        if (copy) copy[base + i] = from_f32<TC>(v);
    }
}

// The same for rows of up to N * blockDim.x elements: a thread keeps its N elements in registers, so the row is
// read once and written once.
template <class TC, int N>
__global__ __launch_bounds__(1024) void add_layernorm_reg_kernel(float* __restrict__ x, float alpha, const float* __restrict__ y1, float s1,
                                         const float* __restrict__ y2, float s2, const float* __restrict__ w, float eps,
                                         TC* __restrict__ copy, int d) {
    __shared__ float scratch[16];
    const int64_t base = (int64_t)blockIdx.x * d;
    float v[N];
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < N; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        v[u] = 0.f;
        if (i < d) {
            float y = s1 * y1[base + i];
            if (y2) y += s2 * y2[base + i];
            v[u] = alpha * x[base + i] + y;
            s += v[u];
        }
    }
    const float mean = block_sum(s, scratch) / (float)d;
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < N; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        if (i < d) { v[u] -= mean; ss += v[u] * v[u]; }
    }
    const float sd = sqrtf(block_sum(ss, scratch) / (float)d + eps);
#pragma unroll
    for (int u = 0; u < N; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        if (i < d) {
            const float r = v[u] / sd * w[i];
            x[base + i] = r;
            if (copy) copy[base + i] = from_f32<TC>(r);
        }
    }
}

// The same with 16-byte loads: N4 pieces of four elements a thread (d a multiple of 4, 16-byte aligned rows).
template <class TC, int N4>
__global__ __launch_bounds__(1024) void add_layernorm_vec_kernel(float* __restrict__ x, float alpha,
                                                                 const float* __restrict__ y1, float s1,
                                                                 const float* __restrict__ y2, float s2,
                                                                 const float* __restrict__ w, float eps,
                                                                 TC* __restrict__ copy, int d) {
    struct alignas(4 * sizeof(TC)) Out4 { TC v[4]; };
    __shared__ float scratch[16];
    const int64_t base = (int64_t)blockIdx.x * d;
    const int n4 = d >> 2;
    f32x4* x4 = (f32x4*)(x + base);
    const f32x4 *a4 = (const f32x4*)(y1 + base), *b4 = y2 ? (const f32x4*)(y2 + base) : nullptr, *w4 = (const f32x4*)w;
    f32x4 v[N4];
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < N4; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        v[u] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (i < n4) {
            const f32x4 xv = x4[i], av = a4[i];
            f32x4 bv = {0.f, 0.f, 0.f, 0.f};
            if (b4) bv = b4[i];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float y = s1 * av[q];
                if (b4) y += s2 * bv[q];
                v[u][q] = alpha * xv[q] + y;
                s += v[u][q];
            }
        }
    }
    const float mean = block_sum(s, scratch) / (float)d;
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < N4; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        if (i < n4) {
#pragma unroll
            for (int q = 0; q < 4; ++q) { v[u][q] -= mean; ss += v[u][q] * v[u][q]; }
        }
    }
    const float sd = sqrtf(block_sum(ss, scratch) / (float)d + eps);
#pragma unroll
    for (int u = 0; u < N4; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        if (i < n4) {
            const f32x4 wv = w4[i];
            f32x4 r;
            Out4 c4;
#pragma unroll
            for (int q = 0; q < 4; ++q) { r[q] = v[u][q] / sd * wv[q]; c4.v[q] = from_f32<TC>(r[q]); }
            x4[i] = r;
            if (copy) ((Out4*)(copy + base))[i] = c4;
        }
    }
}

extern "C" int li_add_layernorm(float* x, float alpha, const float* y1, float s1, const float* y2, float s2,
                                const float* w, float eps, void* copy, int copy_dt, int n_rows, int d,
                                hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (d <= 0 || !y1) return LI_BAD_ARG;
    dim3 grid(n_rows), block(d >= 2048 ? 512 : (d >= 256 ? 256 : 64));
    const bool aligned = d % 4 == 0 && !(((uintptr_t)x | (uintptr_t)y1 | (uintptr_t)y2 | (uintptr_t)w | (uintptr_t)copy) & 15);
    if (aligned && d <= 32 * 1024) {
        const int n4 = d / 4, per = n4 <= 512 ? 1 : (n4 <= 1024 ? 2 : (n4 <= 4096 ? 4 : 8));
        dim3 vb(((n4 + per - 1) / per + 63) / 64 * 64);
#define GO1(TC, N) add_layernorm_vec_kernel<TC, N><<<grid, vb, 0, stream>>>(x, alpha, y1, s1, y2, s2, w, eps, (TC*)copy, d)
#define GO(TC) do { if (per == 1) GO1(TC, 1); else if (per == 2) GO1(TC, 2); else if (per == 4) GO1(TC, 4); else GO1(TC, 8); } while (0)
        if (!copy || copy_dt == DT_F32) GO(float);
        else if (copy_dt == DT_F16) GO(f16);
        else if (copy_dt == DT_BF16) GO(bf16);
        else return LI_BAD_ARG;
#undef GO
#undef GO1
        LI_CHECK_LAUNCH();
        return LI_OK;
    }
    if (d <= 8 * 1024) {
        const int per = d <= 4096 ? 4 : 8;
        dim3 rb(((d + per - 1) / per + 63) / 64 * 64);
#define GO(TC)                                                                                                        \
    do {                                                                                                              \
        if (per == 4) add_layernorm_reg_kernel<TC, 4><<<grid, rb, 0, stream>>>(x, alpha, y1, s1, y2, s2, w, eps, (TC*)copy, d); \
        else add_layernorm_reg_kernel<TC, 8><<<grid, rb, 0, stream>>>(x, alpha, y1, s1, y2, s2, w, eps, (TC*)copy, d);        \
    } while (0)
        if (!copy || copy_dt == DT_F32) GO(float);
        else if (copy_dt == DT_F16) GO(f16);
        else if (copy_dt == DT_BF16) GO(bf16);
        else return LI_BAD_ARG;
#undef GO
        LI_CHECK_LAUNCH();
        return LI_OK;
    }
    if (!copy || copy_dt == DT_F32)
        add_layernorm_kernel<float><<<grid, block, 0, stream>>>(x, alpha, y1, s1, y2, s2, w, eps, (float*)copy, d);
    else if (copy_dt == DT_F16)
        add_layernorm_kernel<f16><<<grid, block, 0, stream>>>(x, alpha, y1, s1, y2, s2, w, eps, (f16*)copy, d);
    else if (copy_dt == DT_BF16)
        add_layernorm_kernel<bf16><<<grid, block, 0, stream>>>(x, alpha, y1, s1, y2, s2, w, eps, (bf16*)copy, d);
    else return LI_BAD_ARG;
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// out = y1 * s1 (+ y2 * s2) added into x: the same sum for an arrangement without the norm behind it.
__global__ void add_scaled_kernel(float* __restrict__ x, const float* __restrict__ y1, float s1,
                                  const float* __restrict__ y2, float s2, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float y = s1 * y1[i];
    if (y2) y += s2 * y2[i];
    x[i] += y;
}

extern "C" int li_add_scaled(float* x, const float* y1, float s1, const float* y2, float s2, int64_t n,
                             hipStream_t stream) {
    if (n <= 0) return LI_OK;
    add_scaled_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, y1, s1, y2, s2, n);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// float32 -> a 16-bit type
template <class TO>
__global__ void cast_kernel(const float* __restrict__ x, TO* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = from_f32<TO>(x[i]);
}

extern "C" int li_cast(const float* x, void* out, int out_dt, int64_t n, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (out_dt == DT_F16) cast_kernel<f16><<<grid, block, 0, stream>>>(x, (f16*)out, n);
    else if (out_dt == DT_BF16) cast_kernel<bf16><<<grid, block, 0, stream>>>(x, (bf16*)out, n);
    else return LI_BAD_ARG;
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// Token shift: out_t = x_t + (x_{t-1} - x_t) * mu, channel by channel, where x_{t-1} is the row of the
// token before in the same sequence: the row above in this step, or, for the first token that a sequence
// brings to this step, the row that the step before left in `state[slot]`; zeros at position 0.  A second
// kernel then leaves each sequence's last row of this step in its state.  The rows of one sequence are
// consecutive and no two sequences share a slot, so a change of tok_slot marks a sequence's edge.
// ---------------------------------------------------------------------------
// `single`: every sequence brings one row (decoding), so each row is its sequence's first and last; the thread
// that has read an element of the state then writes the row's own element there, and no second kernel runs.
template <class TO>
__global__ void token_shift_kernel(const float* __restrict__ x, const float* __restrict__ mu,
                                   float* __restrict__ state, const int* __restrict__ pos,
                                   const int* __restrict__ tok_slot, TO* __restrict__ out, int d, int single) {
    const int t = blockIdx.x;
    const int slot = tok_slot[t];
    const bool first = single || t == 0 || tok_slot[t - 1] != slot;
    float* st = state + (int64_t)slot * d;
    const float* prev = pos[t] == 0 ? nullptr : (first ? st : x + (int64_t)(t - 1) * d);
    const float* xr = x + (int64_t)t * d;
    TO* o = out + (int64_t)t * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        const float h = xr[i], p = prev ? prev[i] : 0.f;
        o[i] = from_f32<TO>(h + (p - h) * mu[i]);
        if (single) st[i] = h;
    }
}

__global__ void token_shift_save_kernel(const float* __restrict__ x, float* __restrict__ state,
                                        const int* __restrict__ tok_slot, int d, int n_tokens) {
    const int t = blockIdx.x;
    const int slot = tok_slot[t];
    if (t + 1 < n_tokens && tok_slot[t + 1] == slot) return;      // not its sequence's last row
    const float* xr = x + (int64_t)t * d;
    float* s = state + (int64_t)slot * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) s[i] = xr[i];
}

extern "C" int li_token_shift(const float* x, const float* mu, float* state, const int* pos, const int* tok_slot,
                              void* out, int out_dt, int n_tokens, int d, int single, hipStream_t stream) {
    if (n_tokens <= 0) return LI_OK;
    if (d <= 0) return LI_BAD_ARG;
    // a few rows (a decode step): as many threads a row as it has elements to four, so that a thread's loads are few
    const int wide = min(1024, (d / 4 + 63) / 64 * 64);
    dim3 grid(n_tokens), block(n_tokens < 256 && wide > 64 ? wide : (d >= 1024 ? 256 : 64));
    if (out_dt == DT_F32) token_shift_kernel<float><<<grid, block, 0, stream>>>(x, mu, state, pos, tok_slot, (float*)out, d, single);
    else if (out_dt == DT_F16) token_shift_kernel<f16><<<grid, block, 0, stream>>>(x, mu, state, pos, tok_slot, (f16*)out, d, single);
    else if (out_dt == DT_BF16) token_shift_kernel<bf16><<<grid, block, 0, stream>>>(x, mu, state, pos, tok_slot, (bf16*)out, d, single);
    else return LI_BAD_ARG;
    LI_CHECK_LAUNCH();
    if (single) return LI_OK;
    token_shift_save_kernel<<<grid, block, 0, stream>>>(x, state, tok_slot, d, n_tokens);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// q, k, v of a step's tokens on their way to an attention over the paged cache.
//   qkv [T, row_stride] float32: H query heads of d, then G key heads of d, then G value heads of dv
// q and k: among the first `rot` dimensions of a head, dimension i is paired with i + rot/2 (half layout)
// or 2j with 2j+1 (adjacent), and the pair (u, v) becomes (u cos a - v sin a, v cos a + u sin a) with
// a = position * inv_freq[pair] (or its cosine and sine from the step's table `cos_sin`, if given); then, if unit_eps >= 0, the head is divided by sqrt(mean square + unit_eps).
// q goes to q_out [T, H, dq] (dq >= d, zeros beyond d), k and v into the token's page in the layout of
// common.h with head sizes dk (>= d, a multiple of 16) and dvp (>= dv, a multiple of 16); what lies beyond
// d and dv is written as zeros, up to the size the page holds.
// One wave a head; a lane keeps up to 4 dimensions (heads of up to 256).
// ---------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(256) void rope_norm_store_kernel(
    const float* __restrict__ qkv, int row_stride, const float* __restrict__ inv_freq,
    const float* __restrict__ cos_sin, int rot, int half_pairing, float unit_eps, const int* __restrict__ pos,
    const int* __restrict__ tok_slot, Pages c, T* __restrict__ q_out, int H, int G, int d, int dv, int dq, int dk,
    int dvp) {
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
    const int p = pos[t];
    const float* row = qkv + (int64_t)t * row_stride;
    int64_t page = 0;
    if (G > 0) page = c.page_table[(int64_t)tok_slot[t] * c.max_pages + p / PAGE];
    const int tp = p % PAGE, half = rot >> 1;
    for (int head = blockIdx.y * n_waves + wave; head < H + 2 * G; head += n_waves * gridDim.y) {
        if (head < H + G) {
            const float* src = row + (int64_t)head * d;
            float val[4];
            float ss = 0.f;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = lane + 64 * u;
                float v = 0.f;
                if (i < d) {
                    v = src[i];
                    if (i < rot) {
                        int pair, other;
                        bool low;
                        if (half_pairing) { low = i < half; pair = low ? i : i - half; other = low ? i + half : i - half; }
                        else { low = !(i & 1); pair = i >> 1; other = i ^ 1; }
                        float sn, cs;
                        if (cos_sin) {           // the step's table [T, rot / 2, 2]: the same two numbers, computed once
                            cs = cos_sin[2 * ((int64_t)t * half + pair)];
                            sn = cos_sin[2 * ((int64_t)t * half + pair) + 1];
                        } else {
                            sincosf((float)p * inv_freq[pair], &sn, &cs);
                        }
                        const float o = src[other];
                        v = low ? v * cs - o * sn : v * cs + o * sn;
                    }
                    ss += v * v;
                }
                val[u] = v;
            }
            if (unit_eps >= 0.f) {
                const float rms = sqrtf(wave_sum(ss) / (float)d + unit_eps);
#pragma unroll
                for (int u = 0; u < 4; ++u) val[u] = val[u] / rms;
            }
            if (head < H) {
                T* q = q_out + ((int64_t)t * H + head) * dq;
#pragma unroll
                for (int u = 0; u < 4; ++u) { const int i = lane + 64 * u; if (i < dq) q[i] = from_f32<T>(val[u]); }
            } else {
                T* kp = (T*)c.k + page * c.page_stride + (int64_t)(head - H) * k_head_elems(dk);
#pragma unroll
                for (int u = 0; u < 4; ++u) { const int i = lane + 64 * u; if (i < dk) kp[k_offset(tp, i, dk)] = from_f32<T>(val[u]); }
            }
        } else {
            const int g = head - H - G;
            const float* src = row + (int64_t)(H + G) * d + (int64_t)g * dv;
            T* vp = (T*)c.v + page * c.page_stride + (int64_t)g * v_head_elems(dvp);
            const int full = round_up(dvp, 32);
            for (int i = lane; i < full; i += 64) vp[v_offset(tp, i, dvp)] = from_f32<T>(i < dv ? src[i] : 0.f);
        }
    }
}

extern "C" int li_rope_norm_store(const float* qkv, int row_stride, const float* inv_freq, const float* cos_sin, int rot,
                                  int half_pairing, float unit_eps, const int* pos, const int* tok_slot, const void* k_pages,
                                  const void* v_pages, int64_t page_stride, const int* page_table, int max_pages,
                                  void* q_out, int dt, int n_tokens, int H, int G, int d, int dv, int dq, int dk,
                                  int dvp, hipStream_t stream) {
    if (n_tokens <= 0) return LI_OK;
    if (H <= 0 || G < 0 || d <= 0 || d > 256 || dq < d || dq > 256 || rot < 0 || rot > d || (rot & 1)) return LI_BAD_ARG;
    if (G > 0 && (dv <= 0 || dk < d || dk > 256 || dk % 16 || dvp < dv || dvp % 16 || !page_table)) return LI_BAD_ARG;
    if (row_stride < (H + G) * d + G * dv || (rot > 0 && !inv_freq)) return LI_BAD_ARG;
    Pages c{k_pages, v_pages, page_stride, page_table, max_pages};
    // few tokens: the heads spread over the grid as well
    dim3 grid(n_tokens, n_tokens >= 512 ? 1 : (H + 2 * G + 3) / 4), block(256);
#define GO(T) rope_norm_store_kernel<T><<<grid, block, 0, stream>>>(qkv, row_stride, inv_freq, cos_sin, rot, half_pairing, \
        unit_eps, pos, tok_slot, c, (T*)q_out, H, G, d, dv, dq, dk, dvp)
    if (dt == DT_F32) GO(float); else if (dt == DT_F16) GO(f16); else if (dt == DT_BF16) GO(bf16); else return LI_BAD_ARG;
#undef GO
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// Sigmoid attention, one workgroup per (token, query head), keys in ascending order:
//   out[t, h, :] = sum over visible j of sigmoid(q_t . k_j * scale + bias[h]) v_j
// (the weights are not normalised over the keys).  q [T, H, dk] and the cache in the type T, scores,
// weights and sums in float32; out [T, H, dv] in the type TO.  This is the float32 path's kernel, and the
// plain form of the 16-bit kernels below.
// ---------------------------------------------------------------------------
template <class T, class TO>
__global__ __launch_bounds__(256) void sigmoid_attn_kernel(
    const T* __restrict__ q, TO* __restrict__ out, Pages c, const int* __restrict__ pos_of,
    const int* __restrict__ tok_slot, const float* __restrict__ bias, int H, int G, int dk, int dv, int dvp,
    float scale, int window) {
    extern __shared__ float lds[];
    float* sq = lds;                 // [dk]
    float* sp = lds + dk;            // [256]
    const int tid = threadIdx.x;
    const int64_t tok = blockIdx.x;
    const int h = blockIdx.y, g = h / (H / G);
    const int pos = pos_of[tok];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int* table = c.page_table + (int64_t)tok_slot[tok] * c.max_pages;
    for (int i = tid; i < dk; i += 256) sq[i] = to_f32(q[(tok * H + h) * dk + i]);
    __syncthreads();
    const float b = bias ? bias[h] : 0.f;
    float acc = 0.f;                 // thread i < dv owns output dimension i
    for (int t0 = lo; t0 <= pos; t0 += 256) {
        const int t = t0 + tid;
        float w = 0.f;
        if (t <= pos) {
            const T* kp = (const T*)c.k + (int64_t)table[t / PAGE] * c.page_stride + (int64_t)g * k_head_elems(dk);
            float dot = 0.f;
            for (int i = 0; i < dk; ++i) dot = fmaf(sq[i], to_f32(kp[k_offset(t % PAGE, i, dk)]), dot);
            w = sigmoidf(dot * scale + b);
        }
        __syncthreads();
        sp[tid] = w;
        __syncthreads();
        const int n = min(256, pos - t0 + 1);
        if (tid < dv) {
            for (int i = 0; i < n; ++i) {
                const int tt = t0 + i;
                const T* vp = (const T*)c.v + (int64_t)table[tt / PAGE] * c.page_stride + (int64_t)g * v_head_elems(dvp);
                acc = fmaf(sp[i], to_f32(vp[v_offset(tt % PAGE, tid, dvp)]), acc);
            }
        }
    }
    if (tid < dv) out[(tok * H + h) * dv + tid] = from_f32<TO>(acc);
}

extern "C" int li_sigmoid_attn(const void* q, void* out, int dt, const void* k_pages, const void* v_pages,
                               int64_t page_stride, const int* page_table, int max_pages, const int* pos,
                               const int* tok_slot, const float* bias, int n_tokens, int H, int G, int dk, int dv,
                               int dvp, float scale, int window, hipStream_t stream) {
    if (n_tokens <= 0) return LI_OK;
    if (H <= 0 || G <= 0 || H % G || dk <= 0 || dk > 256 || dk % 16 || dv <= 0 || dv > 256 || dvp < dv || dvp % 16)
        return LI_BAD_ARG;
    Pages c{k_pages, v_pages, page_stride, page_table, max_pages};
    dim3 grid(n_tokens, H), block(256);
    const size_t lds = (size_t)(dk + 256) * sizeof(float);
#define GO(T) sigmoid_attn_kernel<T, T><<<grid, block, lds, stream>>>((const T*)q, (T*)out, c, pos, tok_slot, bias, \
        H, G, dk, dv, dvp, scale, window)
    if (dt == DT_F32) GO(float); else if (dt == DT_F16) GO(f16); else if (dt == DT_BF16) GO(bf16); else return LI_BAD_ARG;
#undef GO
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// Linear attention with a constant decay per head, token by token:
//   S <- decay[h] * S + k_t v_t^T,   o_t = S^T q_t,        q, k, v = silu of the projections
// One workgroup per (sequence, head).  The state S [d, dv] of the pair is float32; it is read from
// `state[slot, h]` when the workgroup starts and written back when the sequence's tokens of this step are
// done, so a prompt in one step, in portions, or token by token does the same arithmetic in the same order.
// Thread (rg, j) keeps rows rg*ROWS .. rg*ROWS+ROWS-1 of column j in registers; the partial sums of o over the
// row groups are added in ascending order through LDS.
//   proj [T, stride] float32, q at q_off (H heads of d), k at k_off, v at v_off (H heads of dv)
//   seq_qstart / seq_qlen null: one token per sequence, row i of the step belongs to sequence i (decoding)
// TR: q, k and v take this type's values after the silu (float: as they are), so that a 16-bit model's
// decoding multiplies the numbers that its chunked kernel for prompts multiplies.
// ---------------------------------------------------------------------------
template <class T> __device__ __forceinline__ float rounded_to(float v) { return to_f32(from_f32<T>(v)); }
template <> __device__ __forceinline__ float rounded_to<float>(float v) { return v; }

template <int ROWS, class TR>
__global__ void decay_attn_kernel(const float* __restrict__ proj, int stride, int q_off, int k_off, int v_off,
                                  float* __restrict__ state, const float* __restrict__ decay,
                                  const int* __restrict__ seq_slot, const int* __restrict__ seq_qstart,
                                  const int* __restrict__ seq_qlen, float* __restrict__ out, int H, int d, int dv) {
    extern __shared__ float lds[];
    const int RG = blockDim.x / dv;
    float* sq = lds;                    // [d]
    float* sk = sq + d;                 // [d]
    float* sv = sk + d;                 // [dv]
    float* red = sv + dv;               // [RG, dv]
    const int seq = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int j = tid % dv, rg = tid / dv, r0 = rg * ROWS;
    const int q0 = seq_qstart ? seq_qstart[seq] : seq, n = seq_qlen ? seq_qlen[seq] : 1;
    float* S = state + (((int64_t)seq_slot[seq] * H + h) * d) * dv;
    const float lam = decay[h];
    float s[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) s[r] = r0 + r < d ? S[(int64_t)(r0 + r) * dv + j] : 0.f;
    for (int t = 0; t < n; ++t) {
        const float* row = proj + (int64_t)(q0 + t) * stride;
        __syncthreads();
        for (int i = tid; i < d; i += blockDim.x) {
            sq[i] = rounded_to<TR>(siluf(row[q_off + h * d + i]));
            sk[i] = rounded_to<TR>(siluf(row[k_off + h * d + i]));
        }
        for (int i = tid; i < dv; i += blockDim.x) sv[i] = rounded_to<TR>(siluf(row[v_off + h * dv + i]));
        __syncthreads();
        const float vj = sv[j];
        float part = 0.f;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            if (r0 + r < d) {
                s[r] = lam * s[r] + sk[r0 + r] * vj;
                part += s[r] * sq[r0 + r];
            }
        }
        red[rg * dv + j] = part;
        __syncthreads();
        if (rg == 0) {
            float o = 0.f;
            for (int g = 0; g < RG; ++g) o += red[g * dv + j];
            out[(int64_t)(q0 + t) * H * dv + h * dv + j] = o;
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) if (r0 + r < d) S[(int64_t)(r0 + r) * dv + j] = s[r];
}

extern "C" int li_decay_attn(const float* proj, int stride, int q_off, int k_off, int v_off, float* state,
                             const float* decay, const int* seq_slot, const int* seq_qstart, const int* seq_qlen,
                             float* out, int n_seqs, int H, int d, int dv, int round_dt, hipStream_t stream) {
    if (n_seqs <= 0) return LI_OK;
    if (H <= 0 || d <= 0 || dv <= 0 || dv > 256 || d > 256 || round_dt < DT_F32 || round_dt > DT_BF16) return LI_BAD_ARG;
    int rows = 4;
    while (rows < 64 && ((d + rows - 1) / rows) * dv > 512) rows *= 2;
    const int RG = (d + rows - 1) / rows;
    if (RG * dv > 1024) return LI_UNSUPPORTED;
    dim3 grid(n_seqs, H), block(RG * dv);
    const size_t lds = (size_t)(2 * d + dv + RG * dv) * sizeof(float);
#define GO1(R, TR) decay_attn_kernel<R, TR><<<grid, block, lds, stream>>>(proj, stride, q_off, k_off, v_off, state, \
        decay, seq_slot, seq_qstart, seq_qlen, out, H, d, dv)
#define GO(R) do { if (round_dt == DT_F32) GO1(R, float); else if (round_dt == DT_F16) GO1(R, f16); else GO1(R, bf16); } while (0)
    if (rows == 4) GO(4); else if (rows == 8) GO(8); else if (rows == 16) GO(16); else if (rows == 32) GO(32); else GO(64);
#undef GO
#undef GO1
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// The same recurrence for the prompts of a 16-bit model, 32 tokens (a chunk) at a time on the matrix cores.
// With S the state before a chunk of n tokens, t and s tokens of the chunk, and L = decay[h]:
//   o_t  = L^(t+1) S^T q_t + sum over s <= t of L^(t-s) (q_t . k_s) v_s
//   S   <- L^n S + D,   D = sum over s of L^(n-1-s) k_s v_s^T
// q, k, v are silu of the projections rounded to the 16-bit type T; every product accumulates in float32, and
// whatever is float32 on its way into a product (the state, the decayed scores, the decayed keys) enters as the
// sum of two 16-bit numbers, its rounding and the rounding of what is left.  The powers of L are float32.
// Three kernels, of which only the middle one walks a sequence in order.  decay_chunk_kernel, one workgroup per
// (chunk, head), all chunks of the step at once: the sum within the chunk goes to `out`, D to `ds` [chunk, head,
// d, dv], and q in 16 bits to `qa` [T, H, 32 DBLK].  decay_scan_kernel, a thread per element of S: the states
// before every chunk, left where the D were.  decay_carry_kernel, again one workgroup per (chunk, head): adds
// L^(t+1) S^T q_t to `out`.
// Accumulator element r of a lane lies at row 8 (r / 4) + 4 (lane / 32) + r % 4 and column lane % 32; an operand
// whose inner index comes out of an accumulator keeps that order, and the other operand is gathered to match.
// ---------------------------------------------------------------------------
template <class T>
__device__ __forceinline__ void split16(float v, T& hi, T& lo) {
    hi = from_f32<T>(v);
    lo = from_f32<T>(v - to_f32(hi));
}

template <class T, int DBLK, int MAXT>
__global__ __launch_bounds__(MAXT) void decay_chunk_kernel(
    const float* __restrict__ proj, int stride, int q_off, int k_off, int v_off, const float* __restrict__ decay,
    const int* __restrict__ chunk_seq, const int* __restrict__ chunk_t0, const int* __restrict__ seq_qstart,
    const int* __restrict__ seq_qlen, float* __restrict__ out, float* __restrict__ ds, T* __restrict__ qa, int H, int d,
    int dv) {
    typedef typename Vec<T>::v8 v8;
    constexpr int C = 32, DP = 32 * DBLK, LQ = DP + 8;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int nw = blockDim.x >> 6, LV = 32 * nw + 8;
    T* sQ = (T*)smem;
    T* sK = sQ + C * LQ;
    T* sV = sK + C * LQ;
    float* pw = (float*)(sV + C * LV);             // pw[i] = L^i, i = 0 .. 32
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, col = lane & 31;
    const int chunk = blockIdx.x, h = blockIdx.y, seq = chunk_seq[chunk], c0 = chunk_t0[chunk];
    const int q0 = seq_qstart[seq], nc = min(C, seq_qlen[seq] - c0);
    const int j = 32 * wave + col;
    const float lam = decay[h];
    if (nc <= 0) return;                           // a chunk beyond its sequence's tokens (padding)
    for (int idx = tid; idx < C * DP; idx += blockDim.x) {
        const int t = idx / DP, dd = idx - t * DP;
        float qv = 0.f, kv = 0.f;
        if (t < nc && dd < d) {
            const float* row = proj + (int64_t)(q0 + c0 + t) * stride + h * d + dd;
            qv = siluf(row[q_off]);
            kv = siluf(row[k_off]);
        }
        const T q16 = from_f32<T>(qv);
        sQ[t * LQ + dd] = q16;
        sK[t * LQ + dd] = from_f32<T>(kv);
        if (t < nc) qa[((int64_t)(q0 + c0 + t) * H + h) * DP + dd] = q16;
    }
    for (int idx = tid; idx < C * 32 * nw; idx += blockDim.x) {
        const int t = idx / (32 * nw), jj = idx - t * (32 * nw);
        float vv = 0.f;
        if (t < nc && jj < dv) vv = siluf(proj[(int64_t)(q0 + c0 + t) * stride + v_off + h * dv + jj]);
        sV[t * LV + jj] = from_f32<T>(vv);
    }
    if (tid <= C) pw[tid] = powf(lam, (float)tid);
    __syncthreads();
    // 1. x[r] = q_t . k_s for s = row(r), t = col, times L^(t-s) where s <= t
    f32x16 x;
#pragma unroll
    for (int r = 0; r < 16; ++r) x[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 2 * DBLK; ++ks) {
        const v8 a = *(const v8*)(sK + col * LQ + 16 * ks + 8 * half);
        const v8 b = *(const v8*)(sQ + col * LQ + 16 * ks + 8 * half);
        x = mfma32(a, b, x);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int s = 8 * (r >> 2) + 4 * half + (r & 3);
        x[r] = s <= col ? x[r] * pw[col - s] : 0.f;
    }
    // 2. within the chunk: o[t, j] = sum over s of w[t, s] v[s, j]   (t = row(r), j = col)
    f32x16 o;
#pragma unroll
    for (int r = 0; r < 16; ++r) o[r] = 0.f;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        v8 whi, wlo, bv;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            T hi, lo;
            split16<T>(x[8 * u + i], hi, lo);
            whi[i] = hi; wlo[i] = lo;
            bv[i] = sV[(16 * u + 8 * (i >> 2) + 4 * half + (i & 3)) * LV + j];
        }
        o = mfma32(whi, bv, o);
        o = mfma32(wlo, bv, o);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int t = 8 * (r >> 2) + 4 * half + (r & 3);
        if (t < nc && j < dv) out[(int64_t)(q0 + c0 + t) * H * dv + h * dv + j] = o[r];
    }
    // 3. D[dd, j] = sum over s of L^(nc-1-s) k[s, dd] v[s, j]
    float* dst = ds + (((int64_t)chunk * H + h) * d) * dv;
#pragma unroll
    for (int blk = 0; blk < DBLK; ++blk) {
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            v8 khi, klo, bv;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int s = 16 * u + 8 * half + i;
                T hi, lo;
                split16<T>(s < nc ? pw[nc - 1 - s] * to_f32(sK[s * LQ + 32 * blk + col]) : 0.f, hi, lo);
                khi[i] = hi; klo[i] = lo;
                bv[i] = sV[s * LV + j];
            }
            acc = mfma32(khi, bv, acc);
            acc = mfma32(klo, bv, acc);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int dd = 32 * blk + 8 * (r >> 2) + 4 * half + (r & 3);
            if (dd < d && j < dv) dst[(int64_t)dd * dv + j] = acc[r];
        }
    }
}

// The states before every chunk, element by element: thread e of (sequence, head) walks the sequence's chunks
// in order, leaves the state before chunk c where D_c was, and goes on with S <- L^n S + D_c.
__global__ void decay_scan_kernel(float* __restrict__ state, const float* __restrict__ decay,
                                  const int* __restrict__ seq_slot, const int* __restrict__ seq_qlen,
                                  const int* __restrict__ seq_chunk0, float* __restrict__ ds, int H, int d, int dv) {
    constexpr int C = 32;
    const int seq = blockIdx.y, h = blockIdx.z;
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, per = (int64_t)d * dv;
    if (e >= per) return;
    const int n = seq_qlen[seq];
    const float lam = decay[h], full = powf(lam, (float)C);
    float* Sg = state + ((int64_t)seq_slot[seq] * H + h) * per + e;
    float* p = ds + ((int64_t)seq_chunk0[seq] * H + h) * per + e;
    float S = *Sg;
    for (int c0 = 0; c0 < n; c0 += C, p += (int64_t)H * per) {
        const float D = *p;
        *p = S;
        S = (n - c0 >= C ? full : powf(lam, (float)(n - c0))) * S + D;
    }
    *Sg = S;
}

// out[t, j] += L^(t+1) sum over dd of q[t, dd] S[dd, j] for the tokens of one chunk, S the state before the chunk
// (what decay_scan_kernel left in `ds`): one workgroup per (chunk, head), wave w the columns 32w .. 32w+31.  S is
// read in the order in which accumulators hold their rows and q gathered to match.
template <class T, int DBLK, int MAXT>
__global__ __launch_bounds__(MAXT) void decay_carry_kernel(
    const float* __restrict__ decay, const int* __restrict__ chunk_seq, const int* __restrict__ chunk_t0,
    const int* __restrict__ seq_qstart, const int* __restrict__ seq_qlen, float* __restrict__ out,
    const float* __restrict__ ds, const T* __restrict__ qa, int H, int d, int dv) {
    typedef typename Vec<T>::v8 v8;
    typedef typename Vec<T>::v4 v4;
    constexpr int C = 32, DP = 32 * DBLK;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, col = lane & 31;
    const int chunk = blockIdx.x, h = blockIdx.y, seq = chunk_seq[chunk], c0 = chunk_t0[chunk];
    const int q0 = seq_qstart[seq], nc = min(C, seq_qlen[seq] - c0);
    if (nc <= 0) return;
    const int j = 32 * wave + col;
    const float lam = decay[h];
    const float* src = ds + (((int64_t)chunk * H + h) * d) * dv;
    const bool row_ok = col < nc;
    const T* qrow = qa + ((int64_t)(q0 + c0 + (row_ok ? col : 0)) * H + h) * DP + 4 * half;
    f32x16 o2;
#pragma unroll
    for (int r = 0; r < 16; ++r) o2[r] = 0.f;
#pragma unroll
    for (int blk = 0; blk < DBLK; ++blk)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            v8 shi, slo, a;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int dd = 32 * blk + 16 * u + 8 * (i >> 2) + 4 * half + (i & 3);
                T hi, lo;
                split16<T>((dd < d && j < dv) ? src[(int64_t)dd * dv + j] : 0.f, hi, lo);
                shi[i] = hi; slo[i] = lo;
            }
            v4 a0 = {}, a1 = {};
            if (row_ok) { a0 = *(const v4*)(qrow + 32 * blk + 16 * u); a1 = *(const v4*)(qrow + 32 * blk + 16 * u + 8); }
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = a0[i]; a[4 + i] = a1[i]; }
            o2 = mfma32(a, shi, o2);
            o2 = mfma32(a, slo, o2);
        }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int t = 8 * (r >> 2) + 4 * half + (r & 3);
        if (t < nc && j < dv) out[(int64_t)(q0 + c0 + t) * H * dv + h * dv + j] += powf(lam, (float)(t + 1)) * o2[r];
    }
}

// ds: float32 [n_chunks, H, d, dv]; qa: the 16-bit type, [T, H, qa_dim] with qa_dim = 32 DBLK, DBLK the number of
// 32-row blocks the kernels are compiled for (1, 2, 4 or 8: the next of these that holds d)
extern "C" int li_decay_attn_chunked(const float* proj, int stride, int q_off, int k_off, int v_off, float* state,
                                     const float* decay, const int* seq_slot, const int* seq_qstart,
                                     const int* seq_qlen, const int* seq_chunk0, const int* chunk_seq,
                                     const int* chunk_t0, int n_chunks, float* out, float* ds, void* qa, int qa_dim,
                                     int n_seqs, int H, int d, int dv, int dt, hipStream_t stream) {
    if (n_seqs <= 0 || n_chunks <= 0) return LI_OK;
    if (H <= 0 || d <= 0 || dv <= 0 || dv > 256 || d > 256 || !seq_qstart || !seq_qlen || !seq_chunk0 || !chunk_seq ||
        !chunk_t0 || !ds || !qa)
        return LI_BAD_ARG;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    const int nw = (dv + 31) / 32, dblk = d <= 32 ? 1 : (d <= 64 ? 2 : (d <= 128 ? 4 : 8));
    if (qa_dim != 32 * dblk) return LI_BAD_ARG;
    dim3 grid_a(n_chunks, H), block(64 * nw);
    const size_t lds = (size_t)(2 * 32 * (32 * dblk + 8) + 32 * (32 * nw + 8)) * 2 + 36 * sizeof(float);
#define GO2(T, B, M)                                                                                             \
    do {                                                                                                         \
        auto kfn = decay_chunk_kernel<T, B, M>;                                                                  \
        if (lds > 48 * 1024 &&                                                                                   \
            hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
            return LI_HIP_ERROR;                                                                                 \
        kfn<<<grid_a, block, lds, stream>>>(proj, stride, q_off, k_off, v_off, decay, chunk_seq, chunk_t0, seq_qstart, \
                                            seq_qlen, out, ds, (T*)qa, H, d, dv);                                \
        decay_scan_kernel<<<dim3((d * dv + 255) / 256, n_seqs, H), 256, 0, stream>>>(state, decay, seq_slot, seq_qlen, \
                                                                                    seq_chunk0, ds, H, d, dv);    \
        decay_carry_kernel<T, B, M><<<grid_a, block, 0, stream>>>(decay, chunk_seq, chunk_t0, seq_qstart, seq_qlen, out, \
                                                                  ds, (const T*)qa, H, d, dv);                    \
    } while (0)
#define GO1(T, B) do { if (nw <= 4) GO2(T, B, 256); else GO2(T, B, 512); } while (0)
#define GO(T) do { if (dblk == 1) GO1(T, 1); else if (dblk == 2) GO1(T, 2); else if (dblk == 4) GO1(T, 4); else GO1(T, 8); } while (0)
    if (dt == DT_F16) GO(f16); else GO(bf16);
#undef GO
#undef GO1
#undef GO2
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// out = o / sqrt(mean(o^2) + eps) * w * sigmoid(gate): the RMS norm over all heads of a token together, and
// the gate.  o [T, n] float32; gate: float32 rows of `gate_stride` elements.
// ---------------------------------------------------------------------------
template <class TO>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                     const float* __restrict__ gate, int gate_stride, TO* __restrict__ out, int n,
                                     float eps) {
    __shared__ float scratch[16];
    const int64_t t = blockIdx.x;
    const float* orow = o + t * n;
    const float* grow = gate + t * gate_stride;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) { const float v = orow[i]; ss += v * v; }
    const float rms = sqrtf(block_sum(ss, scratch) / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += blockDim.x)
        out[t * n + i] = from_f32<TO>(orow[i] / rms * w[i] * sigmoidf(grow[i]));
}

extern "C" int li_gated_rmsnorm(const float* o, const float* w, const float* gate, int gate_stride, void* out,
                                int out_dt, int n_rows, int n, float eps, hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (n <= 0 || gate_stride < n) return LI_BAD_ARG;
    const int wide = min(1024, (n / 4 + 63) / 64 * 64);
    dim3 grid(n_rows), block(n_rows < 256 && wide > 64 ? wide : (n >= 1024 ? 256 : 64));
    if (out_dt == DT_F32) gated_rmsnorm_kernel<float><<<grid, block, 0, stream>>>(o, w, gate, gate_stride, (float*)out, n, eps);
    else if (out_dt == DT_F16) gated_rmsnorm_kernel<f16><<<grid, block, 0, stream>>>(o, w, gate, gate_stride, (f16*)out, n, eps);
    else if (out_dt == DT_BF16) gated_rmsnorm_kernel<bf16><<<grid, block, 0, stream>>>(o, w, gate, gate_stride, (bf16*)out, n, eps);
    else return LI_BAD_ARG;
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// PolyNorm: out = a N(z) + b N(z^2) + c N(z^3) + e with powers element by element and N the division of a
// row by its root mean square, sqrt(mean square + eps); coef = (a, b, c, e).  z [T, n] float32.
// ---------------------------------------------------------------------------
template <class TO>
__global__ void polynorm_kernel(const float* __restrict__ z, const float* __restrict__ coef, TO* __restrict__ out,
                                int n, float eps) {
    __shared__ float scratch[16];
    const int64_t t = blockIdx.x;
    const float* zr = z + t * n;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = zr[i], v2 = v * v, v3 = v2 * v;
        s1 += v2; s2 += v2 * v2; s3 += v3 * v3;
    }
    const float r1 = sqrtf(block_sum(s1, scratch) / (float)n + eps);
    const float r2 = sqrtf(block_sum(s2, scratch) / (float)n + eps);
    const float r3 = sqrtf(block_sum(s3, scratch) / (float)n + eps);
    const float a = coef[0], b = coef[1], c = coef[2], e = coef[3];
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = zr[i], v2 = v * v, v3 = v2 * v;
        out[t * n + i] = from_f32<TO>(a * (v / r1) + b * (v2 / r2) + c * (v3 / r3) + e);
    }
}

// The same for rows of up to 16 * blockDim.x elements, read once and kept in registers.
template <class TO>
__global__ void polynorm_reg_kernel(const float* __restrict__ z, const float* __restrict__ coef, TO* __restrict__ out,
                                    int n, float eps) {
    __shared__ float scratch[16];
    const int64_t base = (int64_t)blockIdx.x * n;
    float v[16];
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        v[u] = i < n ? z[base + i] : 0.f;
        const float v2 = v[u] * v[u], v3 = v2 * v[u];
        s1 += v2; s2 += v2 * v2; s3 += v3 * v3;
    }
    const float r1 = sqrtf(block_sum(s1, scratch) / (float)n + eps);
    const float r2 = sqrtf(block_sum(s2, scratch) / (float)n + eps);
    const float r3 = sqrtf(block_sum(s3, scratch) / (float)n + eps);
    const float a = coef[0], b = coef[1], c = coef[2], e = coef[3];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        if (i < n) {
            const float v2 = v[u] * v[u], v3 = v2 * v[u];
            out[base + i] = from_f32<TO>(a * (v[u] / r1) + b * (v2 / r2) + c * (v3 / r3) + e);
        }
    }
}

// The same with 16-byte loads: N4 pieces of four elements a thread (n a multiple of 4, 16-byte aligned rows).
template <class TO, int N4>
__global__ __launch_bounds__(1024) void polynorm_vec_kernel(const float* __restrict__ z, const float* __restrict__ coef,
                                                            TO* __restrict__ out, int n, float eps) {
    struct alignas(4 * sizeof(TO)) Out4 { TO v[4]; };
    __shared__ float scratch[16];
    const int64_t base = (int64_t)blockIdx.x * n;
    const int n4 = n >> 2;
    const f32x4* z4 = (const f32x4*)(z + base);
    f32x4 v[N4];
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
    for (int u = 0; u < N4; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        v[u] = i < n4 ? z4[i] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float v2 = v[u][q] * v[u][q], v3 = v2 * v[u][q];
            s1 += v2; s2 += v2 * v2; s3 += v3 * v3;
        }
    }
    const float r1 = sqrtf(block_sum(s1, scratch) / (float)n + eps);
    const float r2 = sqrtf(block_sum(s2, scratch) / (float)n + eps);
    const float r3 = sqrtf(block_sum(s3, scratch) / (float)n + eps);
    // a / r1, b / r2, c / r3 once a row: an element then costs three multiply-adds and no division
    const float a1 = coef[0] / r1, b2 = coef[1] / r2, c3 = coef[2] / r3, e = coef[3];
#pragma unroll
    for (int u = 0; u < N4; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        if (i < n4) {
            Out4 o4;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float x = v[u][q], v2 = x * x, v3 = v2 * x;
                o4.v[q] = from_f32<TO>(a1 * x + b2 * v2 + c3 * v3 + e);
            }
            ((Out4*)(out + base))[i] = o4;
        }
    }
}

extern "C" int li_polynorm(const float* z, const float* coef, void* out, int out_dt, int n_rows, int n, float eps,
                           hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (n <= 0) return LI_BAD_ARG;
    dim3 grid(n_rows), block(n >= 2048 ? 512 : (n >= 256 ? 256 : 64));
    if (n % 4 == 0 && n <= 32 * 1024 && !(((uintptr_t)z | (uintptr_t)out) & 15)) {
        const int n4 = n / 4, per = n4 <= 512 ? 1 : (n4 <= 1024 ? 2 : (n4 <= 4096 ? 4 : 8));
        dim3 vb(((n4 + per - 1) / per + 63) / 64 * 64);
#define GO1(TO, N) polynorm_vec_kernel<TO, N><<<grid, vb, 0, stream>>>(z, coef, (TO*)out, n, eps)
#define GO(TO) do { if (per == 1) GO1(TO, 1); else if (per == 2) GO1(TO, 2); else if (per == 4) GO1(TO, 4); else GO1(TO, 8); } while (0)
        if (out_dt == DT_F32) GO(float); else if (out_dt == DT_F16) GO(f16); else if (out_dt == DT_BF16) GO(bf16);
        else return LI_BAD_ARG;
#undef GO
#undef GO1
        LI_CHECK_LAUNCH();
        return LI_OK;
    }
    if (n <= 16 * 1024) {
        dim3 rb(n <= 1024 ? 64 : (n <= 4096 ? 256 : (n <= 8192 ? 512 : 1024)));
        if (out_dt == DT_F32) polynorm_reg_kernel<float><<<grid, rb, 0, stream>>>(z, coef, (float*)out, n, eps);
        else if (out_dt == DT_F16) polynorm_reg_kernel<f16><<<grid, rb, 0, stream>>>(z, coef, (f16*)out, n, eps);
        else if (out_dt == DT_BF16) polynorm_reg_kernel<bf16><<<grid, rb, 0, stream>>>(z, coef, (bf16*)out, n, eps);
        else return LI_BAD_ARG;
        LI_CHECK_LAUNCH();
        return LI_OK;
    }
    if (out_dt == DT_F32) polynorm_kernel<float><<<grid, block, 0, stream>>>(z, coef, (float*)out, n, eps);
    else if (out_dt == DT_F16) polynorm_kernel<f16><<<grid, block, 0, stream>>>(z, coef, (f16*)out, n, eps);
    else if (out_dt == DT_BF16) polynorm_kernel<bf16><<<grid, block, 0, stream>>>(z, coef, (bf16*)out, n, eps);
    else return LI_BAD_ARG;
    LI_CHECK_LAUNCH();
    return LI_OK;
}
