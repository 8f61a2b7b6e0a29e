// Memory-bound kernels of the hybrid (latent-attention / linear-attention)
// layer stacks: scalar-gain RMS norms fused with the fp32 residual update,
// the causal per-channel input convolution with carried state, the latent
// cache store (norm + rotation), the gated output norm and the clamped GLU.
//
// Every kernel is instantiated for bf16 (ushort bits) and fp32 activations;
// the residual stream, norm statistics and rotation angles are fp32 in both.
// Sequence starts are handled by position: rows whose source position is
// negative read zeros (by select, never by multiply), so reused state slots
// and cache pages need no clearing.
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

// VEC consecutive elements <-> floats. VEC = 4 moves 16 B (fp32) or 8 B
// (bf16) per lane and needs rows whose length is a multiple of 4.
template <typename T, int VEC> DEV_INLINE void ldv(const T* p, float* o);
template <> DEV_INLINE void ldv<float, 1>(const float* p, float* o) { o[0] = *p; }
template <> DEV_INLINE void ldv<unsigned short, 1>(const unsigned short* p, float* o) {
    o[0] = bf2f(*p);
}
template <> DEV_INLINE void ldv<float, 4>(const float* p, float* o) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(p);
    o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
}
template <> DEV_INLINE void ldv<unsigned short, 4>(const unsigned short* p, float* o) {
    typedef __attribute__((ext_vector_type(4))) unsigned short u16x4;
    const u16x4 v = *reinterpret_cast<const u16x4*>(p);
    o[0] = bf2f(v[0]); o[1] = bf2f(v[1]); o[2] = bf2f(v[2]); o[3] = bf2f(v[3]);
}
template <typename T, int VEC> DEV_INLINE void stv(T* p, const float* o);
template <> DEV_INLINE void stv<float, 1>(float* p, const float* o) { *p = o[0]; }
template <> DEV_INLINE void stv<unsigned short, 1>(unsigned short* p, const float* o) {
    *p = f2bf(o[0]);
}
template <> DEV_INLINE void stv<float, 4>(float* p, const float* o) {
    *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
}
template <> DEV_INLINE void stv<unsigned short, 4>(unsigned short* p, const float* o) {
    typedef __attribute__((ext_vector_type(4))) unsigned short u16x4;
    *reinterpret_cast<u16x4*>(p) =
        u16x4{f2bf(o[0]), f2bf(o[1]), f2bf(o[2]), f2bf(o[3])};
}

// sum over the block (<= 1024 threads); every thread gets the total
DEV_INLINE float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    __syncthreads();  // red may still be read from a previous reduction
    if (lane == 0) red[wid] = v;
    __syncthreads();
    const int nw = (blockDim.x + WAVE - 1) / WAVE;
    float total = 0.f;
    for (int i = 0; i < nw; ++i) total += red[i];
    return total;
}

// ------------------------------------------------------ scalar-gain norms
// y = x / sqrt(mean(x^2) + eps) * gain; one workgroup per row, the row is
// held in LDS between the passes.
template <typename OT, int VEC>
__global__ void scalar_rmsnorm_kernel(const float* __restrict__ x,
                                      OT* __restrict__ y, int W, float gain,
                                      float eps) {
    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    float* row = reinterpret_cast<float*>(smem_raw);
    __shared__ float red[16];
    const long t = blockIdx.x;
    const float* xr = x + t * (long)W;
    float ss = 0.f;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float v[VEC];
        ldv<float, VEC>(xr + i, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            row[i + j] = v[j];
            ss += v[j] * v[j];
        }
    }
    const float r = gain / sqrtf(block_sum(ss, red) / (float)W + eps);
    OT* yr = y + t * (long)W;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float v[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = row[i + j] * r;
        stv<OT, VEC>(yr + i, v);
    }
}

// resid += unit(y [+ y2]) * post_gain;  out = unit(resid) * pre_gain
// (out skipped when HAS_OUT is false). One pass over HBM per operand.
template <typename YT, typename OT, bool HAS_OUT, int VEC>
__global__ void add_scalar_rmsnorm_kernel(float* __restrict__ resid,
                                          const YT* __restrict__ y,
                                          const YT* __restrict__ y2,
                                          OT* __restrict__ out, int W,
                                          float post_gain, float pre_gain,
                                          float eps) {
    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    float* row = reinterpret_cast<float*>(smem_raw);
    __shared__ float red[16];
    const long t = blockIdx.x;
    const YT* yr = y + t * (long)W;
    const YT* y2r = y2 ? y2 + t * (long)W : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float v[VEC];
        ldv<YT, VEC>(yr + i, v);
        if (y2r) {
            float u[VEC];
            ldv<YT, VEC>(y2r + i, u);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] += u[j];
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            row[i + j] = v[j];
            ss += v[j] * v[j];
        }
    }
    const float ry = post_gain / sqrtf(block_sum(ss, red) / (float)W + eps);
    float* xr = resid + t * (long)W;
    float sx = 0.f;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float v[VEC];
        ldv<float, VEC>(xr + i, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            v[j] += row[i + j] * ry;
            row[i + j] = v[j];
            sx += v[j] * v[j];
        }
        stv<float, VEC>(xr + i, v);
    }
    if (!HAS_OUT) return;
    const float rx = pre_gain / sqrtf(block_sum(sx, red) / (float)W + eps);
    OT* orow = out + t * (long)W;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float v[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = row[i + j] * rx;
        stv<OT, VEC>(orow + i, v);
    }
}

// y = unit(x) * w * sigmoid(gate): x fp32 [T, N], gate raw with row stride
template <typename T>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ x,
                                     const float* __restrict__ w,
                                     const T* __restrict__ gate,
                                     long gate_stride, T* __restrict__ y,
                                     int N, float eps) {
    __shared__ float red[16];
    const long t = blockIdx.x;
    const float* xr = x + t * (long)N;
    float ss = 0.f;
    for (int i = threadIdx.x; i < N; i += blockDim.x) ss += xr[i] * xr[i];
    const float r = 1.f / sqrtf(block_sum(ss, red) / (float)N + eps);
    const T* gr = gate + t * gate_stride;
    T* yr = y + t * (long)N;
    for (int i = threadIdx.x; i < N; i += blockDim.x) {
        const float g = 1.f / (1.f + expf(-ldf(gr + i)));
        stf(yr + i, xr[i] * r * w[i] * g);
    }
}

// ------------------------------------------------------------ clamped GLU
// [rows, 2I] -> [rows, I]: g = min(gate, L), u = clamp(up, +-L),
// y = g * sigmoid(alpha g) * (u + 1)
template <typename T>
__global__ void clamped_glu_kernel(const T* __restrict__ gu, T* __restrict__ y,
                                   long rows, long I, float limit,
                                   float alpha) {
    const long n = rows * I;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < n;
         idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / I, c = idx - r * I;
        float g = ldf(gu + r * 2 * I + c);
        float u = ldf(gu + r * 2 * I + I + c);
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        stf(y + idx, g / (1.f + expf(-alpha * g)) * (u + 1.f));
    }
}

// ------------------------------------------------------- input convolution
// out[t] = [h[t] +] sum_d w[K-d][c] * h[t-d], d = 0..K (K = taps-1), then
// silu when SILU. RES adds the input itself (the whole-width conv of the
// sandwich layers); the short conv of a delta mixer is plain and activated.
// h may be a column slice of a wider buffer (row stride hs); out is
// contiguous [T, C] of type OT. Rows before the chunk come from the
// sequence's state (its last K inputs), rows before position 0 are zero.
template <typename T, typename OT, int VEC, bool RES, bool SILU>
__global__ void canon_conv_kernel(const T* __restrict__ h, long hs,
                                  const float* __restrict__ w,   // [K+1, C]
                                  const T* __restrict__ state,   // [S, K, C]
                                  const int* __restrict__ state_slots,
                                  const int* __restrict__ cu,
                                  const int* __restrict__ seq_idx,
                                  const int* __restrict__ positions,
                                  OT* __restrict__ out, int C, int K) {
    const long t = blockIdx.x;
    const int c = (blockIdx.y * blockDim.x + threadIdx.x) * VEC;
    if (c >= C) return;
    const int b = seq_idx[t];
    const int local = (int)t - cu[b];
    const int pos = positions[t];
    const long slot = state_slots[b];
    float acc[VEC], v[VEC], wv[VEC];
    ldv<T, VEC>(h + t * hs + c, v);
    ldv<float, VEC>(w + (long)K * C + c, wv);
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        acc[j] = v[j] * (RES ? 1.f + wv[j] : wv[j]);
    for (int d = 1; d <= K; ++d) {
        if (pos - d < 0) break;
        const int src = local - d;
        if (src >= 0)
            ldv<T, VEC>(h + (t - d) * hs + c, v);
        else
            ldv<T, VEC>(state + (slot * K + (K + src)) * C + c, v);
        ldv<float, VEC>(w + (long)(K - d) * C + c, wv);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += wv[j] * v[j];
    }
    if (SILU) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = acc[j] / (1.f + expf(-acc[j]));
    }
    stv<OT, VEC>(out + t * C + c, acc);
}

// state <- the sequence's last K inputs after this chunk (thread per
// channel reads all K old rows before it writes any).
template <typename T>
__global__ void canon_state_kernel(const T* __restrict__ h, long hs,
                                   T* __restrict__ state,
                                   const int* __restrict__ state_slots,
                                   const int* __restrict__ cu, int C, int K) {
    const int b = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int lo = cu[b], L = cu[b + 1] - lo;
    if (L <= 0) return;
    T* st = state + (long)state_slots[b] * K * C + c;
    T keep[8];
    for (int k = 0; k < K; ++k) keep[k] = st[(long)k * C];
    for (int k = 0; k < K; ++k) {
        const int src = L - K + k;
        st[(long)k * C] = src >= 0 ? h[(long)(lo + src) * hs + c]
                                   : keep[K + src];
    }
}

// ----------------------------------------------------- latent cache store
// Per token: cache row = [unit(kv[:C]) * w | rotate(kv[C:])]; q's rotated
// parts are rotated in place. Rotation pairs dim i with i + dims/2 over the
// first `dims` coords of the R-wide part; the rest pass through.
template <typename T>
__global__ void latent_rope_store_kernel(
    T* __restrict__ q_rot, long q_tok_stride, long q_head_stride, int H,
    const T* __restrict__ kv, long kv_stride, const float* __restrict__ w,
    int C, int R, int dims, float eps, const int* __restrict__ positions,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    T* __restrict__ cache, const int* __restrict__ slot_mapping) {
    __shared__ float red[16];
    const long t = blockIdx.x;
    const T* row = kv + t * kv_stride;
    const long slot = slot_mapping[t];
    T* dst = cache + slot * (long)(C + R);
    float ss = 0.f;
    for (int i = threadIdx.x; i < C; i += blockDim.x) {
        const float v = ldf(row + i);
        ss += v * v;
    }
    const float r = 1.f / sqrtf(block_sum(ss, red) / (float)C + eps);
    for (int i = threadIdx.x; i < C; i += blockDim.x)
        stf(dst + i, ldf(row + i) * r * w[i]);
    const int half = dims / 2;
    const int p = positions[t];
    const float* cs = cos_t + (long)p * half;
    const float* sn = sin_t + (long)p * half;
    for (int i = threadIdx.x; i < R; i += blockDim.x) {
        float o;
        if (i < half) {
            o = ldf(row + C + i) * cs[i] - ldf(row + C + i + half) * sn[i];
        } else if (i < dims) {
            const int j = i - half;
            o = ldf(row + C + i) * cs[j] + ldf(row + C + j) * sn[j];
        } else {
            o = ldf(row + C + i);
        }
        stf(dst + C + i, o);
    }
    // q: one thread per (head, pair) reads both coords, then writes both
    T* qt = q_rot + t * q_tok_stride;
    for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
        const int hh = i / half, j = i - hh * half;
        T* qh = qt + hh * q_head_stride;
        const float u = ldf(qh + j), v = ldf(qh + j + half);
        stf(qh + j, u * cs[j] - v * sn[j]);
        stf(qh + j + half, v * cs[j] + u * sn[j]);
    }
}

}  // namespace

// ------------------------------------------- weighted fp32-residual norm
// resid (fp32) += y when y is given; out = unit(resid) * w when out is.
// One workgroup per row, the row held in LDS between the passes.
template <typename YT, typename OT, int VEC>
__global__ void add_rmsnorm_w_kernel(float* __restrict__ resid,
                                     const YT* __restrict__ y,
                                     const float* __restrict__ w,
                                     OT* __restrict__ out, int W, float eps) {
    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    float* row = reinterpret_cast<float*>(smem_raw);
    __shared__ float red[16];
    const long t = blockIdx.x;
    float* rr = resid + t * (long)W;
    const YT* yr = y ? y + t * (long)W : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float v[VEC];
        ldv<float, VEC>(rr + i, v);
        if (yr) {
            float a[VEC];
            ldv<YT, VEC>(yr + i, a);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] += a[j];
            stv<float, VEC>(rr + i, v);
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            row[i + j] = v[j];
            ss += v[j] * v[j];
        }
    }
    if (!out) return;
    const float r = 1.f / sqrtf(block_sum(ss, red) / (float)W + eps);
    OT* orow = out + t * (long)W;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
        float v[VEC], wv[VEC];
        ldv<float, VEC>(w + i, wv);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = row[i + j] * r * wv[j];
        stv<OT, VEC>(orow + i, v);
    }
}

// --------------------------------------------------------------- relu^2
// out[r, c] = max(x[r, c], 0)^2 over column slices (row strides xs, os)
template <typename T, int VEC>
__global__ void relu2_kernel(const T* __restrict__ x, long xs,
                             T* __restrict__ out, long os, long rows, int n) {
    const int per = n / VEC;
    const long total = rows * per;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / per;
        const int c = (int)(idx - r * per) * VEC;
        float v[VEC];
        ldv<T, VEC>(x + r * xs + c, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const float z = fmaxf(v[j], 0.f);
            v[j] = z * z;
        }
        stv<T, VEC>(out + r * os + c, v);
    }
}

// ------------------------------------------------- per-head gated norm
// Wave per (token, head): y = unit(o_head) [* w] * act(gate) * out_scale,
// act = silu or sigmoid. o fp32 [T, H, Dv]; gate and out are column slices.
template <typename T>
__global__ void head_gated_norm_kernel(const float* __restrict__ o,
                                       const float* __restrict__ w,
                                       const T* __restrict__ gate, long gs,
                                       T* __restrict__ out, long os, long rows,
                                       int H, int Dv, float eps, int sigmoid,
                                       float out_scale) {
    const long row = (long)blockIdx.x * (blockDim.x / WAVE) +
                     threadIdx.x / WAVE;       // (token, head)
    if (row >= rows) return;
    const int lane = threadIdx.x % WAVE;
    const long t = row / H;
    const int h = (int)(row - t * H);
    const float* orow = o + row * Dv;
    float ss = 0.f;
    for (int i = lane; i < Dv; i += WAVE) ss += orow[i] * orow[i];
    const float r = out_scale / sqrtf(wave_sum(ss) / (float)Dv + eps);
    const T* gr = gate + t * gs + (long)h * Dv;
    T* yr = out + t * os + (long)h * Dv;
    for (int i = lane; i < Dv; i += WAVE) {
        const float g = ldf(gr + i);
        const float sg = 1.f / (1.f + expf(-g));
        float v = orow[i] * r * (sigmoid ? sg : g * sg);
        if (w) v *= w[i];
        stf(yr + i, v);
    }
}

// ------------------------------------------------ delta-rule gate inputs
// Workgroup per token. (1) the 2*NQ q/k heads of the fp32 conv output are
// made unit vectors in place, x / sqrt(sum x^2 + 1e-6), q also times
// D^-1/2; (2) beta = sigmoid(b); (3) decay g = exp(-rate_h *
// softplus(a + dt_bias)), one per head or one per head and key channel.
template <typename T>
__global__ void delta_gates_kernel(float* __restrict__ qk, long qs, int NQ,
                                   int D, const T* __restrict__ b, long bs,
                                   const T* __restrict__ a, long as,
                                   const float* __restrict__ dt_bias,
                                   const float* __restrict__ rate,
                                   float* __restrict__ beta,
                                   float* __restrict__ g, int H, int per_head) {
    const long t = blockIdx.x;
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int nw = blockDim.x / WAVE;
    float* row = qk + t * qs;
    const float qmul = 1.f / sqrtf((float)D);
    for (int hh = wid; hh < 2 * NQ; hh += nw) {
        float* v = row + (long)hh * D;
        float ss = 0.f;
        for (int i = lane; i < D; i += WAVE) ss += v[i] * v[i];
        const float r = (hh < NQ ? qmul : 1.f) / sqrtf(wave_sum(ss) + 1e-6f);
        for (int i = lane; i < D; i += WAVE) v[i] *= r;
    }
    for (int h = threadIdx.x; h < H; h += blockDim.x)
        beta[t * H + h] = 1.f / (1.f + expf(-ldf(b + t * bs + h)));
    const int n = H * per_head;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float z = ldf(a + t * as + i) + dt_bias[i];
        const float sp = z > 20.f ? z : log1pf(expf(z));
        g[t * n + i] = expf(-rate[i / per_head] * sp);
    }
}

// ------------------------------------- query/key norm, rotation, page store
// Workgroup per token, a wave per head in turn (H query heads, then G key
// heads). Query head: q <- rotate(unit(q) * wq) * q_mult[h] in place. Key
// head: rotate(unit(k) * wk) -> k_cache, k as projected -> v_cache (pages
// [n_blocks, G, bs, D]). Rotation pairs dim i with i + dims/2 over the
// first `dims` coordinates; cos/sin fp32 tables [max_pos, dims/2].
constexpr int QKN_MAXD = 512;
template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_store_kernel(T* __restrict__ q, long q_tok, int H,
                          const T* __restrict__ k, long k_tok, int G, int D,
                          const float* __restrict__ wq,
                          const float* __restrict__ wk, float eps, int dims,
                          const int* __restrict__ positions,
                          const float* __restrict__ cos_t,
                          const float* __restrict__ sin_t,
                          const float* __restrict__ q_mult,
                          T* __restrict__ k_cache, T* __restrict__ v_cache,
                          int bs, const int* __restrict__ slot_mapping) {
    __shared__ float buf[4][QKN_MAXD];
    const long t = blockIdx.x;
    const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int pos = positions[t];
    const int half = dims / 2;
    const int slot = slot_mapping[t];
    const long blk = slot / bs, off = slot % bs;
    float* nb = buf[wid];
    for (int hh = wid; hh < H + G; hh += 4) {
        const bool is_q = hh < H;
        const int g = hh - H;
        const T* src = is_q ? q + t * q_tok + (long)hh * D
                            : k + t * k_tok + (long)g * D;
        const float* w = is_q ? wq : wk;
        float ss = 0.f;
        for (int i = lane; i < D; i += WAVE) {
            const float x = ldf(src + i);
            nb[i] = x;
            ss += x * x;
        }
        const float r = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
        const float mul = is_q ? q_mult[hh] : 1.f;
        T* dst = is_q ? q + t * q_tok + (long)hh * D
                      : k_cache + ((blk * G + g) * bs + off) * D;
        T* vdst = is_q ? nullptr : v_cache + ((blk * G + g) * bs + off) * D;
        // every lane has written its nb entries before any lane reads a
        // partner's: the wave_sum above is a full-wave exchange, and the
        // LDS writes of a wave complete in order before its later reads
        WAVE_LDS_SYNC();
        for (int i = lane; i < D; i += WAVE) {
            const float x = nb[i];
            float y = x * r * w[i];
            if (i < dims) {
                const int j = i < half ? i : i - half;
                const int pi = i < half ? i + half : i - half;
                const float yp = nb[pi] * r * w[pi];
                const float c = cos_t[(long)pos * half + j];
                const float s = sin_t[(long)pos * half + j];
                y = i < half ? y * c - yp * s : y * c + yp * s;
            }
            stf(dst + i, y * mul);
            if (vdst) stf(vdst + i, x);
        }
        WAVE_LDS_SYNC();
    }
}

// ------------------------------------------------------------- launchers
// dtype codes: 0 = bf16 (ushort bits), 1 = fp32

static inline int row_threads(int W) {
    int th = 64;
    while (th < W && th < 1024) th <<= 1;
    return th > 256 && W < 2048 ? 256 : th;
}

extern "C" void launch_scalar_rmsnorm(const float* x, void* y, long T, int W,
                                      float gain, float eps, int out_f32,
                                      hipStream_t s) {
    if (T == 0) return;
    const size_t sh = (size_t)W * sizeof(float);
    if (W % 4 == 0) {
        const int th = row_threads(W / 4);
        if (out_f32)
            scalar_rmsnorm_kernel<float, 4><<<T, th, sh, s>>>(
                x, (float*)y, W, gain, eps);
        else
            scalar_rmsnorm_kernel<unsigned short, 4><<<T, th, sh, s>>>(
                x, (unsigned short*)y, W, gain, eps);
        return;
    }
    const int th = row_threads(W);
    if (out_f32)
        scalar_rmsnorm_kernel<float, 1><<<T, th, sh, s>>>(
            x, (float*)y, W, gain, eps);
    else
        scalar_rmsnorm_kernel<unsigned short, 1><<<T, th, sh, s>>>(
            x, (unsigned short*)y, W, gain, eps);
}

template <typename YT, typename OT>
static void add_norm_dispatch(float* resid, const void* y, const void* y2,
                              void* out, long T, int W, float post, float pre,
                              float eps, hipStream_t s) {
    const size_t sh = (size_t)W * sizeof(float);
    if (W % 4 == 0) {
        const int th = row_threads(W / 4);
        if (out)
            add_scalar_rmsnorm_kernel<YT, OT, true, 4><<<T, th, sh, s>>>(
                resid, (const YT*)y, (const YT*)y2, (OT*)out, W, post, pre, eps);
        else
            add_scalar_rmsnorm_kernel<YT, OT, false, 4><<<T, th, sh, s>>>(
                resid, (const YT*)y, (const YT*)y2, (OT*)nullptr, W, post, pre,
                eps);
        return;
    }
    const int th = row_threads(W);
    if (out)
        add_scalar_rmsnorm_kernel<YT, OT, true, 1><<<T, th, sh, s>>>(
            resid, (const YT*)y, (const YT*)y2, (OT*)out, W, post, pre, eps);
    else
        add_scalar_rmsnorm_kernel<YT, OT, false, 1><<<T, th, sh, s>>>(
            resid, (const YT*)y, (const YT*)y2, (OT*)nullptr, W, post, pre, eps);
}

extern "C" void launch_add_scalar_rmsnorm(float* resid, const void* y,
                                          const void* y2, void* out, long T,
                                          int W, float post, float pre,
                                          float eps, int y_f32, int out_f32,
                                          hipStream_t s) {
    if (T == 0) return;
    if (y_f32 && out_f32)
        add_norm_dispatch<float, float>(resid, y, y2, out, T, W, post, pre, eps, s);
    else if (y_f32)
        add_norm_dispatch<float, unsigned short>(resid, y, y2, out, T, W, post, pre, eps, s);
    else if (out_f32)
        add_norm_dispatch<unsigned short, float>(resid, y, y2, out, T, W, post, pre, eps, s);
    else
        add_norm_dispatch<unsigned short, unsigned short>(resid, y, y2, out, T, W, post, pre, eps, s);
}

extern "C" void launch_gated_rmsnorm(const float* x, const float* w,
                                     const void* gate, long gate_stride,
                                     void* y, long T, int N, float eps,
                                     int f32, hipStream_t s) {
    if (T == 0) return;
    const int th = row_threads(N);
    if (f32)
        gated_rmsnorm_kernel<float><<<T, th, 0, s>>>(
            x, w, (const float*)gate, gate_stride, (float*)y, N, eps);
    else
        gated_rmsnorm_kernel<unsigned short><<<T, th, 0, s>>>(
            x, w, (const unsigned short*)gate, gate_stride,
            (unsigned short*)y, N, eps);
}

extern "C" void launch_clamped_glu(const void* gu, void* y, long rows, long I,
                                   float limit, float alpha, int f32,
                                   hipStream_t s) {
    const long n = rows * I;
    if (n == 0) return;
    const int th = 256;
    long blocks = (n + th - 1) / th;
    if (blocks > 65536) blocks = 65536;
    if (f32)
        clamped_glu_kernel<float><<<(int)blocks, th, 0, s>>>(
            (const float*)gu, (float*)y, rows, I, limit, alpha);
    else
        clamped_glu_kernel<unsigned short><<<(int)blocks, th, 0, s>>>(
            (const unsigned short*)gu, (unsigned short*)y, rows, I, limit, alpha);
}

template <typename T, typename OT, bool RES, bool SILU>
static void conv_dispatch(const void* h, long hs, const float* w, void* state,
                          const int* state_slots, const int* cu,
                          const int* seq_idx, const int* positions, void* out,
                          long T_, int B, int C, int K, bool vec4,
                          hipStream_t s) {
    const int th = C >= 256 ? 256 : 64;
    const int vec = vec4 ? 4 : 1;
    const int lanes = (C + vec - 1) / vec;
    const dim3 g1((unsigned)T_, (lanes + th - 1) / th), g2(B, (C + th - 1) / th);
    if (vec4)
        canon_conv_kernel<T, OT, 4, RES, SILU><<<g1, th, 0, s>>>(
            (const T*)h, hs, w, (const T*)state, state_slots, cu, seq_idx,
            positions, (OT*)out, C, K);
    else
        canon_conv_kernel<T, OT, 1, RES, SILU><<<g1, th, 0, s>>>(
            (const T*)h, hs, w, (const T*)state, state_slots, cu, seq_idx,
            positions, (OT*)out, C, K);
    if (K > 0)
        canon_state_kernel<T><<<g2, th, 0, s>>>(
            (const T*)h, hs, (T*)state, state_slots, cu, C, K);
}

// h + conv(h), same dtype out (the sandwich layers' whole-width conv)
extern "C" void launch_canon_conv(const void* h, const float* w, void* state,
                                  const int* state_slots, const int* cu,
                                  const int* seq_idx, const int* positions,
                                  void* out, long T, int B, int C, int K,
                                  int f32, hipStream_t s) {
    if (T == 0) return;
    const bool v4 = C % 4 == 0;
    if (f32)
        conv_dispatch<float, float, true, false>(
            h, C, w, state, state_slots, cu, seq_idx, positions, out, T, B, C,
            K, v4, s);
    else
        conv_dispatch<unsigned short, unsigned short, true, false>(
            h, C, w, state, state_slots, cu, seq_idx, positions, out, T, B, C,
            K, v4, s);
}

// conv(h) [silu] -> fp32, h a column slice with row stride hs
extern "C" void launch_short_conv(const void* h, long hs, const float* w,
                                  void* state, const int* state_slots,
                                  const int* cu, const int* seq_idx,
                                  const int* positions, float* out, long T,
                                  int B, int C, int K, int silu, int vec4,
                                  int f32, hipStream_t s) {
    if (T == 0) return;
#define SC_CALL(TT, SI)                                                       \
    conv_dispatch<TT, float, false, SI>(h, hs, w, state, state_slots, cu,     \
                                        seq_idx, positions, out, T, B, C, K,  \
                                        vec4 != 0, s)
    if (f32) { if (silu) SC_CALL(float, true); else SC_CALL(float, false); }
    else if (silu) SC_CALL(unsigned short, true);
    else SC_CALL(unsigned short, false);
#undef SC_CALL
}

extern "C" void launch_add_rmsnorm_w(float* resid, const void* y,
                                     const float* w, void* out, long T, int W,
                                     float eps, int y_f32, int out_f32,
                                     hipStream_t s) {
    if (T == 0) return;
    const size_t sh = (size_t)W * sizeof(float);
#define ARW(YT, OT)                                                           \
    do {                                                                      \
        if (W % 4 == 0)                                                       \
            add_rmsnorm_w_kernel<YT, OT, 4><<<T, row_threads(W / 4), sh, s>>>(\
                resid, (const YT*)y, w, (OT*)out, W, eps);                    \
        else                                                                  \
            add_rmsnorm_w_kernel<YT, OT, 1><<<T, row_threads(W), sh, s>>>(    \
                resid, (const YT*)y, w, (OT*)out, W, eps);                    \
    } while (0)
    if (y_f32 && out_f32) ARW(float, float);
    else if (y_f32) ARW(float, unsigned short);
    else if (out_f32) ARW(unsigned short, float);
    else ARW(unsigned short, unsigned short);
#undef ARW
}

extern "C" void launch_relu2(const void* x, long xs, void* out, long os,
                             long rows, int n, int vec4, int f32,
                             hipStream_t s) {
    if (rows == 0 || n == 0) return;
    const int th = 256;
    long blocks = (rows * (long)(vec4 ? n / 4 : n) + th - 1) / th;
    if (blocks > 65536) blocks = 65536;
#define R2(TT, V)                                                             \
    relu2_kernel<TT, V><<<(int)blocks, th, 0, s>>>((const TT*)x, xs,          \
                                                   (TT*)out, os, rows, n)
    if (f32) { if (vec4) R2(float, 4); else R2(float, 1); }
    else if (vec4) R2(unsigned short, 4);
    else R2(unsigned short, 1);
#undef R2
}

extern "C" void launch_head_gated_norm(const float* o, const float* w,
                                       const void* gate, long gs, void* out,
                                       long os, long T, int H, int Dv,
                                       float eps, int sigmoid,
                                       float out_scale, int f32,
                                       hipStream_t s) {
    const long rows = T * H;
    if (rows == 0) return;
    const int wpb = 4;
    const unsigned blocks = (unsigned)((rows + wpb - 1) / wpb);
    if (f32)
        head_gated_norm_kernel<float><<<blocks, wpb * WAVE, 0, s>>>(
            o, w, (const float*)gate, gs, (float*)out, os, rows, H, Dv, eps,
            sigmoid, out_scale);
    else
        head_gated_norm_kernel<unsigned short><<<blocks, wpb * WAVE, 0, s>>>(
            o, w, (const unsigned short*)gate, gs, (unsigned short*)out, os,
            rows, H, Dv, eps, sigmoid, out_scale);
}

extern "C" void launch_delta_gates(float* qk, long qs, int NQ, int D,
                                   const void* b, long bs, const void* a,
                                   long as, const float* dt_bias,
                                   const float* rate, float* beta, float* g,
                                   long T, int H, int per_head, int f32,
                                   hipStream_t s) {
    if (T == 0) return;
    if (f32)
        delta_gates_kernel<float><<<T, 256, 0, s>>>(
            qk, qs, NQ, D, (const float*)b, bs, (const float*)a, as, dt_bias,
            rate, beta, g, H, per_head);
    else
        delta_gates_kernel<unsigned short><<<T, 256, 0, s>>>(
            qk, qs, NQ, D, (const unsigned short*)b, bs,
            (const unsigned short*)a, as, dt_bias, rate, beta, g, H, per_head);
}

// returns nonzero when the head dim exceeds 512
extern "C" int launch_qk_norm_rope_store(
    void* q, long q_tok, int H, const void* k, long k_tok, int G, int D,
    const float* wq, const float* wk, float eps, int dims,
    const int* positions, const float* cos_t, const float* sin_t,
    const float* q_mult, void* k_cache, void* v_cache, int bs,
    const int* slot_mapping, long T, int f32, hipStream_t s) {
    if (D > QKN_MAXD) return 1;
    if (T == 0) return 0;
    if (f32)
        qk_norm_rope_store_kernel<float><<<T, 256, 0, s>>>(
            (float*)q, q_tok, H, (const float*)k, k_tok, G, D, wq, wk, eps,
            dims, positions, cos_t, sin_t, q_mult, (float*)k_cache,
            (float*)v_cache, bs, slot_mapping);
    else
        qk_norm_rope_store_kernel<unsigned short><<<T, 256, 0, s>>>(
            (unsigned short*)q, q_tok, H, (const unsigned short*)k, k_tok, G,
            D, wq, wk, eps, dims, positions, cos_t, sin_t, q_mult,
            (unsigned short*)k_cache, (unsigned short*)v_cache, bs,
            slot_mapping);
    return 0;
}

extern "C" void launch_latent_rope_store(
    void* q_rot, long q_tok_stride, long q_head_stride, int H, const void* kv,
    long kv_stride, const float* w, int C, int R, int dims, float eps,
    const int* positions, const float* cos_t, const float* sin_t, void* cache,
    const int* slot_mapping, long T, int f32, hipStream_t s) {
    if (T == 0) return;
    const int th = 256;
    if (f32)
        latent_rope_store_kernel<float><<<T, th, 0, s>>>(
            (float*)q_rot, q_tok_stride, q_head_stride, H, (const float*)kv,
            kv_stride, w, C, R, dims, eps, positions, cos_t, sin_t,
            (float*)cache, slot_mapping);
    else
        latent_rope_store_kernel<unsigned short><<<T, th, 0, s>>>(
            (unsigned short*)q_rot, q_tok_stride, q_head_stride, H,
            (const unsigned short*)kv, kv_stride, w, C, R, dims, eps,
            positions, cos_t, sin_t, (unsigned short*)cache, slot_mapping);
}
