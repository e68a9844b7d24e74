// Sigmoid attention over the paged cache on the matrix cores, compiled for one pair of head sizes
// (KEY_DIM for queries and keys, VALUE_DIM for values; multiples of 16 up to 256):
//   out[t, h, :] = sum over visible keys j of sigmoid(q_t . k_j * scale + bias[h]) v_j
// Causal (and windowed, if asked), grouped-query; the weights are not normalised over the keys, so there is
// no running maximum and no rescaling: the parts of a context simply add up.
//
// One wave owns 32 rows (query tokens in a prompt, the query heads of a key/value head in decoding).
// S^T = K Q^T and O^T = V^T W^T run on the 32x32x16 matrix instruction with keys and values read from the
// page in operand order (common.h), one contiguous 1 KiB load per fragment.  Scores and weights are float32;
// a weight goes into the second product as the sum of two 16-bit numbers (its rounding and the rounding of
// what is left), so that the product sees 16 bits of it and not 8.
//   prompt : a workgroup is 4 waves = 128 consecutive tokens of one sequence and one query head; a page is
//            fetched once for the four, through two stages of LDS
//   decode : one wave per (sequence, key/value head, split of the context); with more than one split the
//            partial sums are added in ascending order by a second kernel
#include "common.h"

#if !defined(KEY_DIM) || !defined(VALUE_DIM)
#error "compile with -DKEY_DIM=<n> -DVALUE_DIM=<n>"
#endif
static_assert(KEY_DIM % 16 == 0 && KEY_DIM >= 16 && KEY_DIM <= 256, "key size: multiple of 16, at most 256");
static_assert(VALUE_DIM % 16 == 0 && VALUE_DIM >= 16 && VALUE_DIM <= 256, "value size: multiple of 16, at most 256");

constexpr int KD = KEY_DIM, VD = VALUE_DIM;
constexpr int KS = KD / 16;              // steps of the inner index for the scores
constexpr int DB = (VD + 31) / 32;       // 32-row blocks of the output's dimensions
constexpr float LOG2E = 1.4426950408889634f;

struct CachePtrs {
    const void* k;
    const void* v;
    int64_t page_stride;
    const int* page_table;    // [n_slots, max_pages]
    int max_pages;
};

template <class T>
struct WaveSigmoid {
    typedef typename Vec<T>::v8 v8;
    v8 q[KS];
    f32x16 o[DB];

    __device__ __forceinline__ void init(const T* qrow) {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            v8 z = {};
            q[s] = qrow ? *(const v8*)(qrow + 16 * s + 8 * (lane >> 5)) : z;
        }
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[b][r] = 0.f;
    }
    __device__ __forceinline__ void load_k(const T* kpage, v8 (&kf)[2 * KS]) const {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int i = 0; i < 2 * KS; ++i) kf[i] = *(const v8*)(kpage + (i * 64 + lane) * 8);
    }
    __device__ __forceinline__ void load_v(const T* vpage, v8 (&vf)[DB * 4]) const {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int i = 0; i < DB * 4; ++i) vf[i] = *(const v8*)(vpage + (i * 64 + lane) * 8);
    }

    // The weights of the page's 64 keys (the first is key t0) for this wave's rows: this lane's row sees keys
    // lo..hi and adds `bias2` (its head's bias times log2 e) to the score times scale2 (scale times log2 e).
    // sigmoid(z) = 1 / (1 + 2^(-z log2 e)).
    __device__ __forceinline__ void weights(const v8 (&kf)[2 * KS], f32x16 (&s)[2], int t0, int lo, int hi, float scale2,
                                            float bias2, bool masked) {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[b][r] = 0.f;
        // the two blocks of keys in turn, so that no matrix instruction waits for the one before it
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            s[0] = mfma32(kf[ks], q[ks], s[0]);
            s[1] = mfma32(kf[KS + ks], q[ks], s[1]);
        }
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float w = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-fmaf(s[b][r], scale2, bias2)));
                if (masked) {
                    const int t = t0 + 32 * b + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    w = (t >= lo && t <= hi) ? w : 0.f;
                }
                s[b][r] = w;
            }
    }

    // o += V^T W^T with W = hi + lo, both 16-bit
    __device__ __forceinline__ void mix(const v8 (&vf)[DB * 4], const f32x16 (&s)[2]) {
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
            v8 hi, lo;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float w = s[tj >> 1][8 * (tj & 1) + i];
                hi[i] = from_f32<T>(w);
                lo[i] = from_f32<T>(w - to_f32(hi[i]));
            }
#pragma unroll
            for (int b = 0; b < DB; ++b) o[b] = mfma32(vf[b * 4 + tj], hi, o[b]);
#pragma unroll
            for (int b = 0; b < DB; ++b) o[b] = mfma32(vf[b * 4 + tj], lo, o[b]);
        }
    }
};

// ---------------------------------------------------------------------------
// prompts: tile i of the grid is 128 tokens of sequence tile_seq[i] that begin at its token tile_q0[i] of
// this step (a tile that begins beyond its sequence's tokens ends at once); blockIdx.y is the query head.
// ---------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(256) void sigmoid_prefill_kernel(
    const T* __restrict__ q, T* __restrict__ out, CachePtrs c, const int* __restrict__ tile_seq,
    const int* __restrict__ tile_q0, const int* __restrict__ seq_slot, const int* __restrict__ seq_qstart,
    const int* __restrict__ seq_qlen, const int* __restrict__ seq_ctx, const float* __restrict__ bias, int H, int G,
    int dv, float scale, int window) {
    typedef typename WaveSigmoid<T>::v8 v8;
    constexpr int KE = PAGE * KD, VE = PAGE * DB * 32;        // elements of one head's keys and values in a page
    constexpr int KN = KE / 8, KP = (KN + 255) / 256, VP = VE / (256 * 8);   // 16-byte pieces: of the keys, and a thread's
    static_assert(VE % (256 * 8) == 0, "the values of a page divide among the workgroup's threads");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T* smem = (T*)smem_raw;                                   // two stages of [keys | values]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, row = lane & 31;
    // workgroups start in the order of their number: the last tiles of a prompt, which see the most keys, go
    // first and all heads of a tile together, so that the short ones fill the chip's tail
    const int number = blockIdx.x + gridDim.x * blockIdx.y;
    const int tile = gridDim.x - 1 - number / H, h = number % H, g = h / (H / G);
    const int seq = tile_seq[tile];
    const int qlen = seq_qlen[seq], tile0 = tile_q0[tile], q0 = tile0 + 32 * wave;
    if (tile0 >= qlen) return;                                // the whole workgroup: a tile of padding
    const bool active = q0 < qlen;                            // a wave without tokens still helps to fetch
    const int before = seq_ctx[seq] - qlen;                   // the sequence's tokens before this step
    const bool valid = q0 + row < qlen;
    const int64_t tok = (int64_t)seq_qstart[seq] + q0 + row;
    const int pos = before + q0 + row;
    WaveSigmoid<T> a;
    a.init(valid ? q + (tok * H + h) * KD : nullptr);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0, hi = valid ? pos : -1;
    const int pos_min = before + q0, pos_max = before + min(q0 + 31, qlen - 1);
    const int lo_min = window > 0 ? max(0, pos_min - window + 1) : 0, lo_max = window > 0 ? max(0, pos_max - window + 1) : 0;
    const bool all_valid = q0 + 31 < qlen;
    const int p0 = lo_min / PAGE, p1 = active ? pos_max / PAGE + 1 : 0;          // this wave's pages
    // the workgroup's pages: from the first page of its first token to the last page of its last
    const int wg_first = before + tile0, wg_last = before + min(tile0 + 127, qlen - 1);
    const int P0 = (window > 0 ? max(0, wg_first - window + 1) : 0) / PAGE, P1 = wg_last / PAGE + 1;
    const int* table = c.page_table + (int64_t)seq_slot[seq] * c.max_pages;
    const float scale2 = scale * LOG2E, bias2 = (bias ? bias[h] : 0.f) * LOG2E;
    const T* kbase = (const T*)c.k + (int64_t)g * k_head_elems(KD);
    const T* vbase = (const T*)c.v + (int64_t)g * v_head_elems(VD);
    // A page is fetched once for the four waves: every thread brings 16-byte pieces of it into registers while
    // the page before is worked on, and lays them into the other stage of LDS afterwards; one barrier a page.
    v8 rk[KP], rv[VP];
    auto fetch = [&](int p) {
        const T* kp = kbase + (int64_t)table[p] * c.page_stride;
        const T* vp = vbase + (int64_t)table[p] * c.page_stride;
#pragma unroll
        for (int i = 0; i < KP; ++i) if (i * 256 + tid < KN) rk[i] = *(const v8*)(kp + (i * 256 + tid) * 8);
#pragma unroll
        for (int i = 0; i < VP; ++i) rv[i] = *(const v8*)(vp + (i * 256 + tid) * 8);
    };
    auto lay = [&](int stage) {
        T* ks = smem + stage * (KE + VE);
        T* vs = ks + KE;
#pragma unroll
        for (int i = 0; i < KP; ++i) if (i * 256 + tid < KN) *(v8*)(ks + (i * 256 + tid) * 8) = rk[i];
#pragma unroll
        for (int i = 0; i < VP; ++i) *(v8*)(vs + (i * 256 + tid) * 8) = rv[i];
    };
    fetch(P0);
    lay(0);
    __syncthreads();
    f32x16 s[2];
    for (int p = P0; p < P1; ++p) {
        const int stage = (p - P0) & 1;
        if (p + 1 < P1) fetch(p + 1);
        if (p >= p0 && p < p1) {
            const T* ks = smem + stage * (KE + VE);
            const T* vs = ks + KE;
            v8 kf[2 * KS], vf[DB * 4];
            a.load_k(ks, kf);
            a.load_v(vs, vf);
            const bool inside = all_valid && p * PAGE >= lo_max && p * PAGE + PAGE - 1 <= pos_min;
            a.weights(kf, s, p * PAGE, lo, hi, scale2, bias2, !inside);
            a.mix(vf, s);
        }
        if (p + 1 < P1) lay(stage ^ 1);
        __syncthreads();
    }
    if (!valid) return;
    T* orow = out + (tok * H + h) * dv;
#pragma unroll
    for (int blk = 0; blk < DB; ++blk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int d = 32 * blk + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (d < dv) orow[d] = from_f32<T>(a.o[blk][r]);
        }
}

// ---------------------------------------------------------------------------
// decoding: one new token per sequence; the rows of a wave are the query heads of one key/value head (32 at
// a time).  gridDim.z splits of the context; with one split the result is written as it is, else as float32
// partial sums part[seq, head, split, dv] that sigmoid_merge_kernel adds in ascending order.
// ---------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(64) void sigmoid_decode_kernel(
    const T* __restrict__ q, T* __restrict__ out, float* __restrict__ part, CachePtrs c,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_ctx, const float* __restrict__ bias, int H, int G,
    int dv, float scale, int window) {
    const int lane = threadIdx.x & 63;
    const int b = blockIdx.x, group = H / G, gchunks = (group + 31) / 32;
    const int g = blockIdx.y / gchunks, gc = blockIdx.y % gchunks;
    const int S = gridDim.z, split = blockIdx.z;
    const int hg = gc * 32 + (lane & 31);
    const bool live = hg < group;
    const int h = g * group + hg;
    const int pos = seq_ctx[b] - 1;
    WaveSigmoid<T> a;
    a.init(live ? q + ((int64_t)b * H + h) * KD : nullptr);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int p_first = lo / PAGE, p_end = pos / PAGE + 1;
    const int per = (p_end - p_first + S - 1) / S;
    const int p0 = p_first + split * per, p1 = min(p_end, p0 + per);
    const int* table = c.page_table + (int64_t)seq_slot[b] * c.max_pages;
    const float scale2 = scale * LOG2E, bias2 = (bias && live ? bias[h] : 0.f) * LOG2E;
    typename WaveSigmoid<T>::v8 kf[2 * KS], vf[DB * 4];
    f32x16 s[2];
    const T* kbase = (const T*)c.k + (int64_t)g * k_head_elems(KD);
    const T* vbase = (const T*)c.v + (int64_t)g * v_head_elems(VD);
    if (p0 < p1) a.load_k(kbase + (int64_t)table[p0] * c.page_stride, kf);
    for (int p = p0; p < p1; ++p) {
        a.load_v(vbase + (int64_t)table[p] * c.page_stride, vf);
        a.weights(kf, s, p * PAGE, lo, live ? pos : -1, scale2, bias2, p * PAGE < lo || p * PAGE + PAGE - 1 > pos);
        if (p + 1 < p1) a.load_k(kbase + (int64_t)table[p + 1] * c.page_stride, kf);
        a.mix(vf, s);
    }
    if (!live) return;
#pragma unroll
    for (int blk = 0; blk < DB; ++blk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int d = 32 * blk + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (d < dv) {
                if (S == 1) out[((int64_t)b * H + h) * dv + d] = from_f32<T>(a.o[blk][r]);
                else part[(((int64_t)b * H + h) * S + split) * dv + d] = a.o[blk][r];
            }
        }
}

template <class T>
__global__ void sigmoid_merge_kernel(const float* __restrict__ part, T* __restrict__ out, int S, int dv) {
    const int64_t bh = blockIdx.x;
    for (int d = threadIdx.x; d < dv; d += blockDim.x) {
        const float* p = part + bh * S * dv + d;
        float acc = 0.f;
        int s = 0;
        for (; s + 8 <= S; s += 8) {               // eight loads in flight, added in ascending order
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = p[(int64_t)(s + i) * dv];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc += v[i];
        }
        for (; s < S; ++s) acc += p[(int64_t)s * dv];
        out[bh * dv + d] = from_f32<T>(acc);
    }
}

// ---------------------------------------------------------------------------
// C interface
// ---------------------------------------------------------------------------
extern "C" int li_sigattn_key_dim() { return KD; }
extern "C" int li_sigattn_value_dim() { return VD; }

static int check_heads(int H, int G, int dv) { return (H > 0 && G > 0 && H % G == 0 && dv > 0 && dv <= VD) ? LI_OK : LI_BAD_ARG; }

extern "C" int li_sigattn_prefill(const void* q, void* out, int dt, const void* k, const void* v, int64_t page_stride,
                                  const int* page_table, int max_pages, const int* tile_seq, const int* tile_q0,
                                  int n_tiles, const int* seq_slot, const int* seq_qstart, const int* seq_qlen,
                                  const int* seq_ctx, const float* bias, int H, int G, int dv, float scale, int window,
                                  hipStream_t stream) {
    if (check_heads(H, G, dv)) return LI_BAD_ARG;
    if (n_tiles <= 0) return LI_OK;
    CachePtrs c{k, v, page_stride, page_table, max_pages};
    dim3 grid(n_tiles, H), block(256);
    const size_t lds = (size_t)2 * (PAGE * KD + PAGE * DB * 32) * 2;
#define GO(T)                                                                                                        \
    do {                                                                                                             \
        auto kfn = sigmoid_prefill_kernel<T>;                                                                        \
        if (lds > 48 * 1024 &&                                                                                       \
            hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)  \
            return LI_HIP_ERROR;                                                                                     \
        kfn<<<grid, block, lds, stream>>>((const T*)q, (T*)out, c, tile_seq, tile_q0, seq_slot, seq_qstart, seq_qlen,  \
                                          seq_ctx, bias, H, G, dv, scale, window);                                   \
    } while (0)
    if (dt == DT_F16) GO(f16); else if (dt == DT_BF16) GO(bf16); else return LI_BAD_ARG;
#undef GO
    LI_CHECK_LAUNCH();
    return LI_OK;
}

extern "C" int li_sigattn_decode(const void* q, void* out, int dt, const void* k, const void* v, int64_t page_stride,
                                 const int* page_table, int max_pages, const int* seq_slot, const int* seq_ctx,
                                 const float* bias, int n_seqs, int H, int G, int dv, float scale, int window, int splits,
                                 float* part, hipStream_t stream) {
    if (check_heads(H, G, dv) || splits < 1 || splits > 64 || (splits > 1 && !part)) return LI_BAD_ARG;
    if (n_seqs <= 0) return LI_OK;
    CachePtrs c{k, v, page_stride, page_table, max_pages};
    const int group = H / G;
    dim3 grid(n_seqs, G * ((group + 31) / 32), splits), block(64);
#define GO(T)                                                                                                        \
    do {                                                                                                             \
        sigmoid_decode_kernel<T><<<grid, block, 0, stream>>>((const T*)q, (T*)out, part, c, seq_slot, seq_ctx, bias, H, G, \
                                                             dv, scale, window);                                     \
        if (splits > 1) sigmoid_merge_kernel<T><<<n_seqs * H, dv <= 64 ? 64 : (dv <= 128 ? 128 : 256), 0, stream>>>(part, (T*)out, splits, dv); \
    } while (0)
    if (dt == DT_F16) GO(f16); else if (dt == DT_BF16) GO(bf16); else return LI_BAD_ARG;
#undef GO
    LI_CHECK_LAUNCH();
    return LI_OK;
}
