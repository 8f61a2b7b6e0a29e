// Sequence mixers of the hybrid layer stacks.
//
// latent_attn: windowed softmax attention over a paged cache that holds ONE
// row per token (normed latent | rotated key part) shared by all heads —
// the "absorbed" form: queries arrive already multiplied by the key
// up-projection, the output is the probability-weighted sum of latent rows
// (the value up-projection is applied afterwards as a batched GEMM).
// One wave per (token, head): lanes span the row's coordinates, keys are
// walked four at a time with an online softmax; scores, weights and
// accumulators are fp32. The same kernel serves prompt portions and decode
// rows: every row carries its own position and sequence. When a step has
// few rows (decode), the visible keys of each row are split over grid.z so
// the chip is filled, and a second kernel merges the (max, sum, partial)
// triples.
//
// lightning_attn: decayed linear attention S_t = lam_h S_(t-1) + k_t v_t^T,
// o_t = S_t^T q_t with the state in fp32 registers. A workgroup owns a
// 64-column slice of one (sequence, head) state — columns evolve
// independently, which gives Dv/64-way parallelism per head on top of
// sequences x heads — and walks the chunk's tokens in order.
#include "common.h"

namespace {

template <typename T> DEV_INLINE float ldf(const T* p);
template <> DEV_INLINE float ldf<float>(const float* p) { return *p; }
template <> DEV_INLINE float ldf<unsigned short>(const unsigned short* p) {
    return bf2f(*p);
}
template <typename T> DEV_INLINE void stf(T* p, float v);
template <> DEV_INLINE void stf<float>(float* p, float v) { *p = v; }
template <> DEV_INLINE void stf<unsigned short>(unsigned short* p, float v) {
    *p = f2bf(v);
}

constexpr int LA_WAVES = 4;   // heads per workgroup
constexpr int LA_KEYS = 4;    // keys per online-softmax update

template <typename T, int DPL>
__global__ void __launch_bounds__(LA_WAVES * WAVE)
latent_attn_kernel(const T* __restrict__ q_abs,   // [H, Tn, C]
                   const T* __restrict__ q_rot, long qr_tok, long qr_head,
                   const T* __restrict__ gate, long gate_tok,
                   const T* __restrict__ cache,   // [blocks, bs, C + R]
                   const int* __restrict__ block_table, int bt_stride,
                   const int* __restrict__ positions,
                   const int* __restrict__ seq_idx,
                   T* __restrict__ out,           // [H, Tn, C]
                   float* __restrict__ part_acc,  // [splits, H, Tn, C]
                   float* __restrict__ part_ml,   // [splits, H, Tn, 2]
                   int Tn, int H, int C, int R, int bs, int window,
                   float scale) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x % WAVE;
    const int h = blockIdx.y * LA_WAVES + threadIdx.x / WAVE;
    if (h >= H) return;
    const int Dk = C + R;
    const int p = positions[t];
    const int* bt = block_table + (long)seq_idx[t] * bt_stride;
    int lo = max(0, p - window + 1);
    int last = p;
    const int splits = gridDim.z;
    if (splits > 1) {
        // this workgroup's share of the visible keys (whole key groups)
        int per = (p - lo + splits) / splits;
        per = (per + LA_KEYS - 1) / LA_KEYS * LA_KEYS;
        lo += blockIdx.z * per;
        last = min(p, lo + per - 1);
    }

    float qv[DPL], acc[DPL];
    const T* qa = q_abs + ((long)h * Tn + t) * C;
    const T* qr = q_rot + (long)t * qr_tok + (long)h * qr_head;
#pragma unroll
    for (int j = 0; j < DPL; ++j) {
        const int c = lane + WAVE * j;
        float v = 0.f;
        if (c < C) v = ldf(qa + c);
        else if (c < Dk) v = ldf(qr + (c - C));
        qv[j] = v * scale;
        acc[j] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    for (int key = lo; key <= last; key += LA_KEYS) {
        float kv[LA_KEYS][DPL], s[LA_KEYS];
#pragma unroll
        for (int u = 0; u < LA_KEYS; ++u) {
            const int kp = min(key + u, last);  // clamp: stay inside the pages
            const T* row = cache + ((long)bt[kp / bs] * bs + kp % bs) * Dk;
            float d = 0.f;
#pragma unroll
            for (int j = 0; j < DPL; ++j) {
                const int c = lane + WAVE * j;
                kv[u][j] = c < Dk ? ldf(row + c) : 0.f;
                d += qv[j] * kv[u][j];
            }
            s[u] = d;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
#pragma unroll
            for (int u = 0; u < LA_KEYS; ++u) s[u] += __shfl_xor(s[u], off);
        }
        float mn = m;
#pragma unroll
        for (int u = 0; u < LA_KEYS; ++u) {
            if (key + u > last) s[u] = -INFINITY;
            mn = fmaxf(mn, s[u]);
        }
        const float a = expf(m - mn);
        float pu[LA_KEYS], ps = 0.f;
#pragma unroll
        for (int u = 0; u < LA_KEYS; ++u) {
            pu[u] = expf(s[u] - mn);
            ps += pu[u];
        }
        l = l * a + ps;
#pragma unroll
        for (int j = 0; j < DPL; ++j) {
            float v = acc[j] * a;
#pragma unroll
            for (int u = 0; u < LA_KEYS; ++u) v += pu[u] * kv[u][j];
            acc[j] = v;
        }
        m = mn;
    }
    if (splits > 1) {
        // unnormalized partial + (max, sum); an empty share leaves l = 0
        const long row = ((long)blockIdx.z * H + h) * Tn + t;
#pragma unroll
        for (int j = 0; j < DPL; ++j) {
            const int c = lane + WAVE * j;
            if (c < C) part_acc[row * C + c] = acc[j];
        }
        if (lane == 0) {
            part_ml[row * 2] = m;
            part_ml[row * 2 + 1] = l;
        }
        return;
    }
    const float g = 1.f / (1.f + expf(-ldf(gate + (long)t * gate_tok + h)));
    const float r = g / l;
    T* o = out + ((long)h * Tn + t) * C;
#pragma unroll
    for (int j = 0; j < DPL; ++j) {
        const int c = lane + WAVE * j;
        if (c < C) stf(o + c, acc[j] * r);
    }
}

// merge the key-split partials of one (token, head): wave per row
template <typename T>
__global__ void __launch_bounds__(LA_WAVES * WAVE)
latent_attn_combine_kernel(const float* __restrict__ part_acc,
                           const float* __restrict__ part_ml,
                           const T* __restrict__ gate, long gate_tok,
                           T* __restrict__ out, int splits, int Tn, int H,
                           int C) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x % WAVE;
    const int h = blockIdx.y * LA_WAVES + threadIdx.x / WAVE;
    if (h >= H) return;
    float M = -INFINITY;
    for (int z = 0; z < splits; ++z)
        M = fmaxf(M, part_ml[(((long)z * H + h) * Tn + t) * 2]);
    float L = 0.f;
    for (int z = 0; z < splits; ++z) {
        const long row = ((long)z * H + h) * Tn + t;
        const float l = part_ml[row * 2 + 1];
        if (l > 0.f) L += l * expf(part_ml[row * 2] - M);
    }
    const float g = 1.f / (1.f + expf(-ldf(gate + (long)t * gate_tok + h)));
    T* o = out + ((long)h * Tn + t) * C;
    for (int c = lane; c < C; c += WAVE) {
        float a = 0.f;
        for (int z = 0; z < splits; ++z) {
            const long row = ((long)z * H + h) * Tn + t;
            if (part_ml[row * 2 + 1] > 0.f)
                a += part_acc[row * C + c] * expf(part_ml[row * 2] - M);
        }
        stf(o + c, a * g / L);
    }
}

// ------------------------------------------------------------- lightning
constexpr int LI_COLS = 64;    // state columns per workgroup (one per lane)
constexpr int LI_GROUPS = 4;   // row groups = waves; each owns D/4 state rows
constexpr int LI_TB = 8;       // tokens staged per round

DEV_INLINE float silu_f(float x) { return x / (1.f + expf(-x)); }

// Workgroup = (sequence, head, 64-column slice of the state). Thread
// (g, col) keeps rows [g*DPT, (g+1)*DPT) of column col in registers. Per
// round of LI_TB tokens the block stages silu(q), silu(k) (all D rows) and
// silu(v) (its columns) in LDS once — wave g then reads q/k as broadcasts —
// and the four row groups' partial outputs are summed through LDS.
template <typename T, int DPT>
__global__ void __launch_bounds__(LI_COLS * LI_GROUPS)
lightning_kernel(const T* __restrict__ q, const T* __restrict__ k,
                 const T* __restrict__ v, long tok_stride,
                 const float* __restrict__ decay,
                 float* __restrict__ state,        // [slots, H, D, Dv]
                 const int* __restrict__ state_slots,
                 const int* __restrict__ cu,
                 const int* __restrict__ positions,
                 float* __restrict__ out,          // [Tn, H * Dv]
                 int H, int D, int Dv) {
    constexpr int DMAX = DPT * LI_GROUPS;
    __shared__ float qs[LI_TB][DMAX];
    __shared__ float ks[LI_TB][DMAX];
    __shared__ float vs[LI_TB][LI_COLS];
    __shared__ float red[LI_TB][LI_GROUPS][LI_COLS];
    const int b = blockIdx.x, h = blockIdx.y;
    const int lo = cu[b], hi = cu[b + 1];
    if (hi <= lo) return;
    const int nth = LI_COLS * LI_GROUPS;
    const int g = threadIdx.x / LI_COLS, col = threadIdx.x % LI_COLS;
    const int c0 = blockIdx.z * LI_COLS;
    const int dv = c0 + col;
    const bool live = dv < Dv;
    const int d0 = g * DPT;
    const float lam = decay[h];
    float* st = state + (((long)state_slots[b] * H + h) * D) * Dv + dv;
    const bool fresh = positions[lo] == 0;
    float s[DPT];
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
        const int d = d0 + i;
        s[i] = (!fresh && live && d < D) ? st[(long)d * Dv] : 0.f;
    }
    for (int t0 = lo; t0 < hi; t0 += LI_TB) {
        const int n = min(LI_TB, hi - t0);
        for (int idx = threadIdx.x; idx < n * DMAX; idx += nth) {
            const int tt = idx / DMAX, d = idx - tt * DMAX;
            const long base = (long)(t0 + tt) * tok_stride + (long)h * D + d;
            qs[tt][d] = d < D ? silu_f(ldf(q + base)) : 0.f;
            ks[tt][d] = d < D ? silu_f(ldf(k + base)) : 0.f;
        }
        for (int idx = threadIdx.x; idx < n * LI_COLS; idx += nth) {
            const int tt = idx / LI_COLS, c = idx - tt * LI_COLS;
            vs[tt][c] = (c0 + c < Dv)
                ? silu_f(ldf(v + (long)(t0 + tt) * tok_stride + (long)h * Dv + c0 + c))
                : 0.f;
        }
        __syncthreads();
        for (int tt = 0; tt < n; ++tt) {
            const float vv = vs[tt][col];
            float part = 0.f;
#pragma unroll
            for (int i = 0; i < DPT; ++i) {
                s[i] = lam * s[i] + ks[tt][d0 + i] * vv;
                part += s[i] * qs[tt][d0 + i];
            }
            red[tt][g][col] = part;
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < n * LI_COLS; idx += nth) {
            const int tt = idx / LI_COLS, c = idx - tt * LI_COLS;
            float o = 0.f;
#pragma unroll
            for (int gg = 0; gg < LI_GROUPS; ++gg) o += red[tt][gg][c];
            if (c0 + c < Dv)
                out[(long)(t0 + tt) * H * Dv + (long)h * Dv + c0 + c] = o;
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
            const int d = d0 + i;
            if (d < D) st[(long)d * Dv] = s[i];
        }
    }
}

}  // namespace

#define LA_CASE(N)                                                            \
    case N:                                                                   \
        latent_attn_kernel<TT, N><<<grid, LA_WAVES * WAVE, 0, s>>>(           \
            (const TT*)q_abs, (const TT*)q_rot, qr_tok, qr_head,              \
            (const TT*)gate, gate_tok, (const TT*)cache, block_table,         \
            bt_stride, positions, seq_idx, (TT*)out, part_acc, part_ml, Tn,   \
            H, C, R, bs, window, scale);                                      \
        break;

template <typename TT>
static int latent_attn_dispatch(const void* q_abs, const void* q_rot,
                                long qr_tok, long qr_head, const void* gate,
                                long gate_tok, const void* cache,
                                const int* block_table, int bt_stride,
                                const int* positions, const int* seq_idx,
                                void* out, float* part_acc, float* part_ml,
                                int splits, int Tn, int H, int C, int R,
                                int bs, int window, float scale,
                                hipStream_t s) {
    const int need = (C + R + WAVE - 1) / WAVE;
    const int sizes[] = {1, 2, 3, 4, 6, 9, 12, 16};
    int dpl = 0;
    for (int z : sizes)
        if (z >= need) { dpl = z; break; }
    if (!dpl) return 1;
    const dim3 grid(Tn, (H + LA_WAVES - 1) / LA_WAVES, splits);
    switch (dpl) {
        LA_CASE(1) LA_CASE(2) LA_CASE(3) LA_CASE(4) LA_CASE(6) LA_CASE(9)
        LA_CASE(12) LA_CASE(16)
    }
    if (splits > 1) {
        const dim3 g2(Tn, (H + LA_WAVES - 1) / LA_WAVES);
        latent_attn_combine_kernel<TT><<<g2, LA_WAVES * WAVE, 0, s>>>(
            part_acc, part_ml, (const TT*)gate, gate_tok, (TT*)out, splits,
            Tn, H, C);
    }
    return 0;
}

// returns nonzero when the row width (kv_rank + rot_dim) exceeds 1024
extern "C" int launch_latent_attn(const void* q_abs, const void* q_rot,
                                  long qr_tok, long qr_head, const void* gate,
                                  long gate_tok, const void* cache,
                                  const int* block_table, int bt_stride,
                                  const int* positions, const int* seq_idx,
                                  void* out, float* part_acc, float* part_ml,
                                  int splits, int Tn, int H, int C, int R,
                                  int bs, int window, float scale, int f32,
                                  hipStream_t s) {
    if (Tn == 0) return 0;
    if (f32)
        return latent_attn_dispatch<float>(
            q_abs, q_rot, qr_tok, qr_head, gate, gate_tok, cache, block_table,
            bt_stride, positions, seq_idx, out, part_acc, part_ml, splits, Tn,
            H, C, R, bs, window, scale, s);
    return latent_attn_dispatch<unsigned short>(
        q_abs, q_rot, qr_tok, qr_head, gate, gate_tok, cache, block_table,
        bt_stride, positions, seq_idx, out, part_acc, part_ml, splits, Tn, H,
        C, R, bs, window, scale, s);
}

#define LI_CASE(N)                                                            \
    case N:                                                                   \
        lightning_kernel<TT, N><<<grid, LI_COLS * LI_GROUPS, 0, s>>>(         \
            (const TT*)q, (const TT*)k, (const TT*)v, tok_stride, decay,      \
            state, state_slots, cu, positions, out, H, D, Dv);                \
        break;

template <typename TT>
static int lightning_dispatch(const void* q, const void* k, const void* v,
                              long tok_stride, const float* decay,
                              float* state, const int* state_slots,
                              const int* cu, const int* positions, float* out,
                              int B, int H, int D, int Dv, hipStream_t s) {
    const int need = (D + LI_GROUPS - 1) / LI_GROUPS;
    const int sizes[] = {2, 8, 16, 32, 64};
    int dpt = 0;
    for (int z : sizes)
        if (z >= need) { dpt = z; break; }
    if (!dpt) return 1;
    const dim3 grid(B, H, (Dv + LI_COLS - 1) / LI_COLS);
    switch (dpt) { LI_CASE(2) LI_CASE(8) LI_CASE(16) LI_CASE(32) LI_CASE(64) }
    return 0;
}

// returns nonzero when the key dim exceeds 256
extern "C" int launch_lightning(const void* q, const void* k, const void* v,
                                long tok_stride, const float* decay,
                                float* state, const int* state_slots,
                                const int* cu, const int* positions,
                                float* out, int B, int H, int D, int Dv,
                                int f32, hipStream_t s) {
    if (B == 0) return 0;
    if (f32)
        return lightning_dispatch<float>(q, k, v, tok_stride, decay, state,
                                         state_slots, cu, positions, out, B,
                                         H, D, Dv, s);
    return lightning_dispatch<unsigned short>(q, k, v, tok_stride, decay,
                                              state, state_slots, cu,
                                              positions, out, B, H, D, Dv, s);
}
