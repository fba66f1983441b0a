// Kernels of hyper-connected pre-norm decoders for MI355X (gfx950): the write
// of a sublayer into several residual streams fused with the read and layer
// norm of the next one, rotation of projection rows into float32 (what enters
// a recurrence), the combine / head norm / gate step after a mixer's
// read-out, and ungated routed experts for few tokens.
//
// Same conventions as mixers.hip: a FLAT multi-sequence batch (cu, past,
// seq_of), activations bf16 (dt = 0) or float32 (dt = 1), float32 for norm
// weights and statistics, angles and the residual streams. All sizes are
// run-time values.

#include "mixer_util.h"

#define HC_MAXS 8    // residual streams at most
#define HC_NR 16     // channels of the normed read a thread keeps in registers

__device__ __forceinline__ void hc_ld4(const float* p, int64_t i, float* o) {
    const float4 a = *reinterpret_cast<const float4*>(p + i);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
}
__device__ __forceinline__ void hc_ld4(const bf16s* p, int64_t i, float* o) {
    const uint2 a = *reinterpret_cast<const uint2*>(p + i);
    o[0] = bf16_lo(a.x); o[1] = bf16_hi(a.x); o[2] = bf16_lo(a.y); o[3] = bf16_hi(a.y);
}
__device__ __forceinline__ void hc_st4(float* p, int64_t i, const float* v) {
    *reinterpret_cast<float4*>(p + i) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void hc_st4(bf16s* p, int64_t i, const float* v) {
    uint2 a;
    a.x = pack_bf16x2(v[0], v[1]);
    a.y = pack_bf16x2(v[2], v[3]);
    *reinterpret_cast<uint2*>(p + i) = a;
}

// ---------------------------------------------------------------------------
// streams [T, S, C] float32. One block per token.
//   yy    = y + sigmoid(g2) * y2                      (y2, g2 optional)
//   new_t = sum_s mix[s, t] old_s + write[t] * yy     (if y; all t from the OLD streams)
//   u     = sum_s read[s] new_s                       (if read)
//   out   = (u - mean(u)) / sqrt(mean((u - mean(u))^2) + eps) * w + b
// The sums over streams run in stream order, so a token's result is the same
// in every batch. The first 256 * HC_NR channels of u stay in registers
// between the passes; wider rows rebuild u from the (just written) streams.
template <typename TC, bool VEC, int NSTR>
__global__ __launch_bounds__(256) void hyper_norm_kernel(
    float* __restrict__ streams, int S_rt, const TC* __restrict__ y, int64_t ys,
    const TC* __restrict__ y2, int64_t y2s, const float* __restrict__ g2, int64_t g2s,
    const float* __restrict__ mix, const float* __restrict__ write,
    const float* __restrict__ read, const float* __restrict__ w, const float* __restrict__ b,
    TC* __restrict__ out, int C, float eps) {
    __shared__ float red_a[16], red_b[16];
    __shared__ float smix[NSTR * NSTR], swr[NSTR], srd[NSTR];
    constexpr int W = VEC ? 4 : 1;
    constexpr int NS = HC_NR / W;
    // NSTR < HC_MAXS: exactly NSTR streams (loops fold); NSTR == HC_MAXS: any count up to it
    const int S = NSTR == HC_MAXS ? S_rt : NSTR;
    const int t = blockIdx.x, tid = threadIdx.x;
    if (tid < NSTR * NSTR) {
        const int s = tid / NSTR, k = tid % NSTR;
        smix[tid] = (mix && s < S && k < S) ? mix[s * S + k] : 0.0f;
    }
    if (tid < NSTR) {
        swr[tid] = (write && tid < S) ? write[tid] : 0.0f;
        srd[tid] = (read && tid < S) ? read[tid] : 0.0f;
    }
    __syncthreads();
    float* xs = streams + (int64_t)t * S * C;
    const TC* yr = y ? y + (int64_t)t * ys : nullptr;
    const TC* y2r = y2 ? y2 + (int64_t)t * y2s : nullptr;
    const float gate = (y2 && g2) ? sigmoidf_(g2[(int64_t)t * g2s]) : 1.0f;
    // channels c .. c+W-1: update the streams, return u
    auto step = [&](int c, float* u) {
        float x[NSTR][W];
#pragma unroll
        for (int s = 0; s < NSTR; ++s) {
            if (s < S) {
                if (VEC) hc_ld4(xs + (int64_t)s * C, c, x[s]);
                else x[s][0] = xs[(int64_t)s * C + c];
            }
        }
        if (yr) {
            float yy[W], a[W];
            if (VEC) hc_ld4(yr, c, yy);
            else yy[0] = ldf(yr, c);
            if (y2r) {
                if (VEC) hc_ld4(y2r, c, a);
                else a[0] = ldf(y2r, c);
#pragma unroll
                for (int e = 0; e < W; ++e) yy[e] += gate * a[e];
            }
            float nx[NSTR][W];
#pragma unroll
            for (int k = 0; k < NSTR; ++k) {
                if (k < S) {
#pragma unroll
                    for (int e = 0; e < W; ++e) {
                        float acc = 0.0f;
#pragma unroll
                        for (int s = 0; s < NSTR; ++s)
                            if (s < S) acc = fmaf(smix[s * NSTR + k], x[s][e], acc);
                        nx[k][e] = fmaf(swr[k], yy[e], acc);
                    }
                    if (VEC) hc_st4(xs + (int64_t)k * C, c, nx[k]);
                    else xs[(int64_t)k * C + c] = nx[k][0];
                }
            }
#pragma unroll
            for (int k = 0; k < NSTR; ++k)
                if (k < S) {
#pragma unroll
                    for (int e = 0; e < W; ++e) x[k][e] = nx[k][e];
                }
        }
#pragma unroll
        for (int e = 0; e < W; ++e) {
            float acc = 0.0f;
#pragma unroll
            for (int s = 0; s < NSTR; ++s)
                if (s < S) acc = fmaf(srd[s], x[s][e], acc);
            u[e] = acc;
        }
    };
    // u again from the streams as they are now (rows wider than the registers hold)
    auto reread = [&](int c, float* u) {
#pragma unroll
        for (int e = 0; e < W; ++e) {
            float acc = 0.0f;
            for (int s = 0; s < S; ++s) acc = fmaf(srd[s], xs[(int64_t)s * C + c + e], acc);
            u[e] = acc;
        }
    };
    float vals[HC_NR];
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int c = (tid + 256 * j) * W;
#pragma unroll
        for (int e = 0; e < W; ++e) vals[j * W + e] = 0.0f;
        if (c < C) step(c, vals + j * W);
#pragma unroll
        for (int e = 0; e < W; ++e) sum += vals[j * W + e];
    }
    for (int c = (tid + 256 * NS) * W; c < C; c += 256 * W) {
        float u[W];
        step(c, u);
#pragma unroll
        for (int e = 0; e < W; ++e) sum += u[e];
    }
    if (!read) return;
    const float mean = block_reduce_sum<4>(sum, red_a) / (float)C;
    float sq = 0.0f;
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int c = (tid + 256 * j) * W;
        if (c < C) {
#pragma unroll
            for (int e = 0; e < W; ++e) {
                const float d = vals[j * W + e] - mean;
                sq += d * d;
            }
        }
    }
    for (int c = (tid + 256 * NS) * W; c < C; c += 256 * W) {
        float u[W];
        reread(c, u);
#pragma unroll
        for (int e = 0; e < W; ++e) {
            const float d = u[e] - mean;
            sq += d * d;
        }
    }
    const float var = block_reduce_sum<4>(sq, red_b) / (float)C;
    const float rs = 1.0f / sqrtf(var + eps);
    TC* o = out + (int64_t)t * C;
    auto emit = [&](int c, const float* u) {
        float x[W];
#pragma unroll
        for (int e = 0; e < W; ++e) {
            x[e] = (u[e] - mean) * rs * w[c + e];
            if (b) x[e] += b[c + e];
        }
        if (VEC) hc_st4(o, c, x);
        else stf(o, c, x[0]);
    };
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int c = (tid + 256 * j) * W;
        if (c < C) emit(c, vals + j * W);
    }
    for (int c = (tid + 256 * NS) * W; c < C; c += 256 * W) {
        float u[W];
        reread(c, u);
        emit(c, u);
    }
}

// y, y2 and out share the activation type.
extern "C" int oa_hyper_norm(void* stream, void* streams, int S, const void* y, int64_t ys, int y_dt,
                             const void* y2, int64_t y2s, int y2_dt, const void* g2, int64_t g2s,
                             const void* mix, const void* write, const void* read, const void* w,
                             const void* b, void* out, int out_dt, int T, int C, float eps) {
    if (T <= 0 || C <= 0) return 0;
    if (S < 1 || S > HC_MAXS || !streams) return -100;
    if (y && (!mix || !write)) return -101;
    if (y2 && !y) return -101;
    if (read && (!w || !out)) return -101;
    int dt = -1;
    if (y) dt = y_dt;
    if (y2) {
        if (y2_dt != dt) return -102;
    }
    if (read) {
        if (dt >= 0 && out_dt != dt) return -102;
        dt = out_dt;
    }
    if (dt < 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int esz = dt == 1 ? 4 : 2;
    auto al = [&](const void* p, int64_t stride) {
        return !p || ((uintptr_t)p % (4 * esz) == 0 && stride % 4 == 0);
    };
    const bool vec = C % 4 == 0 && (uintptr_t)streams % 16 == 0 && al(y, ys) && al(y2, y2s) &&
                     al(out, 0);
#define HC_LAUNCH_N(TC, V, N)                                                                     \
    hipLaunchKernelGGL((hyper_norm_kernel<TC, V, N>), dim3(T), dim3(256), 0, s, (float*)streams,  \
                       S, (const TC*)y, ys, (const TC*)y2, y2s, (const float*)g2, g2s,             \
                       (const float*)mix, (const float*)write, (const float*)read,                \
                       (const float*)w, (const float*)b, (TC*)out, C, eps)
    // one to four streams have kernels of their own size; more share the widest
#define HC_LAUNCH(TC, V)                              \
    do {                                              \
        if (S == 1) HC_LAUNCH_N(TC, V, 1);            \
        else if (S == 2) HC_LAUNCH_N(TC, V, 2);       \
        else if (S == 3) HC_LAUNCH_N(TC, V, 3);       \
        else if (S == 4) HC_LAUNCH_N(TC, V, 4);       \
        else HC_LAUNCH_N(TC, V, HC_MAXS);             \
    } while (0)
    if (dt == 1) {
        if (vec) HC_LAUNCH(float, true);
        else HC_LAUNCH(float, false);
    } else {
        if (vec) HC_LAUNCH(bf16s, true);
        else HC_LAUNCH(bf16s, false);
    }
#undef HC_LAUNCH
#undef HC_LAUNCH_N
    HIP_CHECK_LAUNCH();
    return 0;
}

// ---------------------------------------------------------------------------
// Rotation of projection rows into float32. x [T, n] with row stride xs: the
// first n_rot * D columns are heads of D channels (D even) whose pairs
// (2i, 2i+1), i < nfreq, turn by position * inv_freq[i]; every other column is
// copied. out [T, n] float32. grid = (tokens, column blocks); the token's
// cos/sin table is built once per block in LDS.
template <typename TC>
__global__ __launch_bounds__(256) void rope_rows_kernel(
    const TC* __restrict__ x, int64_t xs, float* __restrict__ out, int n, int n_rot, int D,
    const float* __restrict__ inv_freq, int nfreq, const int* __restrict__ seq_of,
    const int* __restrict__ cu, const int* __restrict__ past, int B) {
    extern __shared__ float lds[];
    float* cs = lds;
    float* sn = lds + nfreq;
    const int t = blockIdx.x;
    if (t >= cu[B]) return;      // padding row of a fixed-size (captured) launch
    const int b = seq_of[t];
    const float pos = (float)(past[b] + t - cu[b]);
    for (int i = threadIdx.x; i < nfreq; i += blockDim.x) {
        float s_, c_;
        sincosf(pos * inv_freq[i], &s_, &c_);
        cs[i] = c_;
        sn[i] = s_;
    }
    __syncthreads();
    const TC* row = x + (int64_t)t * xs;
    float* o = out + (int64_t)t * n;
    const int nr = n_rot * D;
    const int tid = blockIdx.y * blockDim.x + threadIdx.x, nth = gridDim.y * blockDim.x;
    for (int p = tid; 2 * p < nr; p += nth) {
        const int c = 2 * p, i = (c % D) >> 1;
        const float u = ldf(row, c), v = ldf(row, c + 1);
        if (i < nfreq) {
            o[c] = u * cs[i] - v * sn[i];
            o[c + 1] = v * cs[i] + u * sn[i];
        } else {
            o[c] = u;
            o[c + 1] = v;
        }
    }
    for (int c = nr + tid; c < n; c += nth) o[c] = ldf(row, c);
}

extern "C" int oa_rope_rows(void* stream, const void* x, int64_t xs, int dt, void* out, int n,
                            int n_rot, int D, const void* inv_freq, int nfreq, const void* seq_of,
                            const void* cu, const void* past, int B, int T) {
    if (T <= 0 || n <= 0) return 0;
    if (n_rot < 0 || D < 1 || (int64_t)n_rot * D > n || 2 * nfreq > D ||
        (n_rot > 0 && nfreq > 0 && D % 2 != 0))
        return -100;
    hipStream_t s = (hipStream_t)stream;
    const int ny = std::max(1, std::min(CEIL_DIV(n, 512), std::max(1, 2048 / T)));
    const size_t lds = (size_t)2 * std::max(nfreq, 1) * sizeof(float);
    if (dt == 1)
        hipLaunchKernelGGL((rope_rows_kernel<float>), dim3(T, ny), dim3(256), lds, s, (const float*)x,
                           xs, (float*)out, n, n_rot, D, (const float*)inv_freq, nfreq,
                           (const int*)seq_of, (const int*)cu, (const int*)past, B);
    else
        hipLaunchKernelGGL((rope_rows_kernel<bf16s>), dim3(T, ny), dim3(256), lds, s, (const bf16s*)x,
                           xs, (float*)out, n, n_rot, D, (const float*)inv_freq, nfreq,
                           (const int*)seq_of, (const int*)cu, (const int*)past, B);
    HIP_CHECK_LAUNCH();
    return 0;
}

// ---------------------------------------------------------------------------
// After a mixer's read-out: o = a - lam * a2 (a2 optional); with `norm` each
// head's Dv values are divided by sqrt(mean(o^2) + eps) and multiplied by
// post_scale; then o * gate_fn(gate) (gate optional; 0 sigmoid, 1 silu).
// a, a2 [T, H*Dv] of type TA with their row strides, gate and out of type TO.
// grid = (tokens, head groups): a wave per head, four heads per block. A lane
// keeps CN_NR of its channels in registers, the rest is read again.
#define CN_NR 4
template <typename TA, typename TO>
__global__ __launch_bounds__(256) void combine_norm_gate_kernel(
    const TA* __restrict__ a, int64_t as_, const TA* __restrict__ a2, int64_t a2s, float lam,
    const TO* __restrict__ gate, int64_t gs, int gate_act, TO* __restrict__ out, int H, int Dv,
    int norm, float eps, float post_scale) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = blockIdx.y * 4 + wave;
    if (h >= H) return;
    const TA* ar = a + (int64_t)t * as_ + (int64_t)h * Dv;
    const TA* a2r = a2 ? a2 + (int64_t)t * a2s + (int64_t)h * Dv : nullptr;
    auto value = [&](int i) {
        float v = ldf(ar, i);
        if (a2r) v -= lam * ldf(a2r, i);
        return v;
    };
    float vals[CN_NR];
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < CN_NR; ++j) {
        const int i = lane + 64 * j;
        vals[j] = i < Dv ? value(i) : 0.0f;
        ss += vals[j] * vals[j];
    }
    for (int i = lane + 64 * CN_NR; i < Dv; i += 64) {
        const float v = value(i);
        ss += v * v;
    }
    float r = 1.0f;
    if (norm) {
        ss = wave_reduce_sum(ss);
        r = post_scale / sqrtf(ss / (float)Dv + eps);
    }
    const TO* gr = gate ? gate + (int64_t)t * gs + (int64_t)h * Dv : nullptr;
    TO* o = out + ((int64_t)t * H + h) * Dv;
    auto emit = [&](int i, float v) {
        v *= r;
        if (gr) {
            const float g = ldf(gr, i);
            v *= gate_act ? g / (1.0f + expf(-g)) : sigmoidf_(g);
        }
        stf(o, i, v);
    };
#pragma unroll
    for (int j = 0; j < CN_NR; ++j) {
        const int i = lane + 64 * j;
        if (i < Dv) emit(i, vals[j]);
    }
    for (int i = lane + 64 * CN_NR; i < Dv; i += 64) emit(i, value(i));
}

extern "C" int oa_combine_norm_gate(void* stream, const void* a, int64_t as_, int a_dt,
                                    const void* a2, int64_t a2s, float lam, const void* gate,
                                    int64_t gs, int gate_act, void* out, int out_dt, int T, int H,
                                    int Dv, int norm, float eps, float post_scale) {
    if (T <= 0) return 0;
    if (H < 1 || Dv < 1 || !a || !out) return -100;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(T, CEIL_DIV(H, 4));
#define CN_LAUNCH(TA, TO)                                                                        \
    hipLaunchKernelGGL((combine_norm_gate_kernel<TA, TO>), grid, dim3(256), 0, s, (const TA*)a,   \
                       as_, (const TA*)a2, a2s, lam, (const TO*)gate, gs, gate_act, (TO*)out, H,  \
                       Dv, norm, eps, post_scale)
    if (a_dt == 1 && out_dt == 1) CN_LAUNCH(float, float);
    else if (a_dt == 1) CN_LAUNCH(float, bf16s);
    else if (out_dt == 0) CN_LAUNCH(bf16s, bf16s);
    else return -102;
#undef CN_LAUNCH
    HIP_CHECK_LAUNCH();
    return 0;
}

// ---------------------------------------------------------------------------
// Elementwise activation of an ungated feed-forward. act 0 silu, 1 gelu (tanh
// form), 3 relu squared; float32 inside.
__device__ __forceinline__ float plain_act_f(float z, int act) {
    if (act == 3) {
        const float r = fmaxf(z, 0.0f);
        return r * r;
    }
    if (act == 1) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    return z / (1.0f + expf(-z));
}

template <typename TC, bool VEC>
__global__ __launch_bounds__(256) void act_rows_kernel(const TC* __restrict__ x, TC* __restrict__ out,
                                                       int64_t n, int act) {
    if (VEC) {
        const int64_t nv = n / 8;
        for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nv;
             i += (int64_t)gridDim.x * blockDim.x) {
            float v[8];
            ld8(x, i * 8, v);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = plain_act_f(v[e], act);
            st8(out, i * 8, v);
        }
    } else {
        for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
             i += (int64_t)gridDim.x * blockDim.x)
            stf(out, i, plain_act_f(ldf(x, i), act));
    }
}

extern "C" int oa_act_rows(void* stream, const void* x, void* out, int64_t n, int dt, int act) {
    if (n <= 0) return 0;
    if (act != 0 && act != 1 && act != 3) return -100;
    hipStream_t s = (hipStream_t)stream;
    const bool vec = n % 8 == 0 && (uintptr_t)x % 32 == 0 && (uintptr_t)out % 32 == 0;
#define AR_LAUNCH(TC, V)                                                                     \
    hipLaunchKernelGGL((act_rows_kernel<TC, V>), dim3(grid_for(V ? n / 8 : n)), dim3(256), 0, s, \
                       (const TC*)x, (TC*)out, n, act)
    if (dt == 1) {
        if (vec) AR_LAUNCH(float, true);
        else AR_LAUNCH(float, false);
    } else {
        if (vec) AR_LAUNCH(bf16s, true);
        else AR_LAUNCH(bf16s, false);
    }
#undef AR_LAUNCH
    HIP_CHECK_LAUNCH();
    return 0;
}

// ---------------------------------------------------------------------------
// Up-projection of ungated routed experts for few (token, expert) pairs:
// mid[p, r] = act(W1[e_p][r, :] . x[t_p]). grid = (pairs, row groups): a wave
// per weight row, 16 bytes per lane where the sizes allow. w1 [E, I, K].
template <typename TC>
__global__ __launch_bounds__(256) void moe_pairs_up_kernel(
    const TC* __restrict__ x, const TC* __restrict__ w1, const int* __restrict__ idx,
    TC* __restrict__ mid, int top, int E, int I, int K, int act, int vec) {
    const int p = blockIdx.x, t = p / top;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int e = min(max(idx[p], 0), E - 1);
    const TC* we = w1 + (int64_t)e * I * K;
    const TC* xr = x + (int64_t)t * K;
    for (int r = blockIdx.y * 4 + wave; r < I; r += gridDim.y * 4) {
        const TC* wr = we + (int64_t)r * K;
        float a = 0.0f;
        if (vec) {
            for (int i = lane * 8; i < K; i += 64 * 8) {
                float xv[8], wv[8];
                ld8(xr, i, xv);
                ld8(wr, i, wv);
#pragma unroll
                for (int q = 0; q < 8; ++q) a = fmaf(wv[q], xv[q], a);
            }
        } else {
            for (int i = lane; i < K; i += 64) a = fmaf(ldf(wr, i), ldf(xr, i), a);
        }
        a = wave_reduce_sum(a);
        if (lane == 0) stf(mid, (int64_t)p * I + r, plain_act_f(a, act));
    }
}

extern "C" int oa_moe_pairs_up(void* stream, const void* x, const void* w1, const void* idx,
                               void* mid, int T, int top, int E, int I, int K, int dt, int act) {
    if (T <= 0) return 0;
    if (top < 1 || E < 1 || I < 1 || K < 1 || (act != 0 && act != 1 && act != 3)) return -100;
    const int vec = (K % 8 == 0 && (uintptr_t)x % 32 == 0 && (uintptr_t)w1 % 32 == 0) ? 1 : 0;
    dim3 grid(T * top, std::min(CEIL_DIV(I, 4), 512));
    hipStream_t s = (hipStream_t)stream;
    if (dt == 1)
        hipLaunchKernelGGL((moe_pairs_up_kernel<float>), grid, dim3(256), 0, s, (const float*)x,
                           (const float*)w1, (const int*)idx, (float*)mid, top, E, I, K, act, vec);
    else
        hipLaunchKernelGGL((moe_pairs_up_kernel<bf16s>), grid, dim3(256), 0, s, (const bf16s*)x,
                           (const bf16s*)w1, (const int*)idx, (bf16s*)mid, top, E, I, K, act, vec);
    HIP_CHECK_LAUNCH();
    return 0;
}
