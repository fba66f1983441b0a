// Decoder-block kernels for MI355X (gfx950) beside the sequence mixers:
// dynamic-tanh norm fused with the residual add, per-head query/key norm with
// rotary positions and the scatter into the paged cache, gated activations,
// expert routing (sigmoid or softmax scores, choice correction, group-limited
// top-k) and routed experts for few (token, expert) pairs.
//
// Same conventions as mixers.hip: a FLAT multi-sequence batch (cu, past,
// seq_of), activations and weights bf16 (dt = 0) or float32 (dt = 1), and
// float32 for everything that is a norm, an angle, a router score or the
// residual. All sizes are run-time values.

#include "mixer_util.h"

// ---------------------------------------------------------------------------
// Dynamic-tanh norm dyt(x; w, b, a) = tanh(a x) w + b (a is one scalar read
// from device memory). One launch does the add after a sublayer and the norm
// before the next:
//   y given:   r = residual + dyt(y; post);  residual = r
//   out given: out = dyt(r; next)
// VEC: 4 channels per thread (C % 4 == 0, rows 16-byte aligned).
//
// tanh in float32 without the library's slow path (two tanh per element made
// the kernel VALU-bound): below 1/8 the odd series x (1 - x^2/3 + 2x^4/15 -
// 17x^6/315), whose next term is under 2e-9 relative there; above it
// 1 - 2/(e^(2|x|) + 1) with the hardware exponential and reciprocal, where the
// subtraction loses nothing that matters (the result is at least 0.124 and
// the error stays near 1e-7 absolute).
__device__ __forceinline__ float tanh_f32(float x) {
    const float ax = fabsf(x), x2 = x * x;
    const float small = x * fmaf(x2, fmaf(x2, fmaf(x2, -17.0f / 315.0f, 2.0f / 15.0f), -1.0f / 3.0f), 1.0f);
    const float e = __expf(2.0f * ax);
    const float big = copysignf(1.0f - __fdividef(2.0f, e + 1.0f), x);
    return ax < 0.125f ? small : big;
}

template <typename TY, typename TO, int VEC>
__global__ __launch_bounds__(256) void dyt_norm_kernel(
    const TY* __restrict__ y, int64_t ys, const float* __restrict__ pw,
    const float* __restrict__ pb, const float* __restrict__ pa, float* __restrict__ residual,
    const float* __restrict__ nw, const float* __restrict__ nb, const float* __restrict__ na,
    TO* __restrict__ out, int T, int C) {
    const float a_post = y ? pa[0] : 0.0f, a_next = out ? na[0] : 0.0f;
    const int cv = C / VEC;
    const int64_t total = (int64_t)T * cv;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int t = (int)(i / cv), c = (int)(i % cv) * VEC;
        float r[VEC];
        if (VEC == 4) {
            const float4 rv = *reinterpret_cast<const float4*>(residual + (int64_t)t * C + c);
            r[0] = rv.x; r[1] = rv.y; r[2] = rv.z; r[3] = rv.w;
        } else {
            r[0] = residual[(int64_t)t * C + c];
        }
        if (y) {
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                r[e] += tanh_f32(a_post * ldf(y, (int64_t)t * ys + c + e)) * pw[c + e] + pb[c + e];
            if (VEC == 4)
                *reinterpret_cast<float4*>(residual + (int64_t)t * C + c) =
                    make_float4(r[0], r[1], r[2], r[3]);
            else
                residual[(int64_t)t * C + c] = r[0];
        }
        if (out) {
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                stf(out, (int64_t)t * C + c + e, tanh_f32(a_next * r[e]) * nw[c + e] + nb[c + e]);
        }
    }
}

extern "C" int oa_dyt_norm(void* stream, const void* y, int64_t ys, int y_dt, const void* pw,
                           const void* pb, const void* pa, void* residual, const void* nw,
                           const void* nb, const void* na, void* out, int out_dt, int T, int C) {
    if (T <= 0 || C <= 0) return 0;
    if (!residual || (y && (!pw || !pb || !pa)) || (out && (!nw || !nb || !na))) return -100;
    hipStream_t s = (hipStream_t)stream;
    const bool vec = C % 4 == 0 && (!y || ys % 4 == 0) && (uintptr_t)residual % 16 == 0;
    const int grid = grid_for((int64_t)T * (vec ? C / 4 : C));
#define DY_ARGS(TY, TO)                                                                          \
    (const TY*)y, ys, (const float*)pw, (const float*)pb, (const float*)pa, (float*)residual,   \
        (const float*)nw, (const float*)nb, (const float*)na, (TO*)out, T, C
#define DY(TY, TO)                                                                               \
    do {                                                                                         \
        if (vec) hipLaunchKernelGGL((dyt_norm_kernel<TY, TO, 4>), dim3(grid), dim3(256), 0, s,  \
                                    DY_ARGS(TY, TO));                                            \
        else hipLaunchKernelGGL((dyt_norm_kernel<TY, TO, 1>), dim3(grid), dim3(256), 0, s,      \
                                DY_ARGS(TY, TO));                                                \
    } while (0)
    if (y_dt == 1 && out_dt == 1) DY(float, float);
    else if (y_dt == 1) DY(float, bf16s);
    else if (out_dt == 1) DY(bf16s, float);
    else DY(bf16s, bf16s);
#undef DY
#undef DY_ARGS
    HIP_CHECK_LAUNCH();
    return 0;
}

// ---------------------------------------------------------------------------
// Attention input preparation with rotary positions. grid = (tokens, head
// groups): a block takes every gridDim.y-th group of 16 heads of one token, a
// wave four heads at a time. Query and key heads: RMS norm over the head's D
// channels (x / sqrt(mean(x^2) + eps)) times a float32 weight [D] shared by
// the heads, then the channel pairs (2i, 2i+1), i < nfreq, are rotated by the
// angle th = position * inv_freq[i], as a plane rotation
//   [x0'; x1'] = [cos th, -sin th; sin th, cos th] [x0; x1];
// channels from 2*nfreq on pass unrotated (qw and kw null: no norm, rotation
// only). q goes to q_out [T, H, D], k and the unchanged v (Gv value heads of
// Dv channels after the G key heads) to their cache slot. The position of token t of sequence b is past[b] + t - cu[b].
// Everything between load and store is float32. A lane keeps its pairs in
// registers (RP_NP pairs: D <= 128 * RP_NP), so every element is read once;
// the token's cos/sin table is computed once per block into LDS.
// PAIRED: D, the row stride and the head offsets are even, pairs are loaded
// and stored as one 4-byte (bf16) or 8-byte (float32) access.
#define RP_NP 4
__device__ __forceinline__ void ld2(const float* p, int64_t i, float& u, float& v) {
    const float2 t = *reinterpret_cast<const float2*>(p + i);
    u = t.x; v = t.y;
}
__device__ __forceinline__ void ld2(const bf16s* p, int64_t i, float& u, float& v) {
    const uint32_t t = *reinterpret_cast<const uint32_t*>(p + i);
    u = bf16_lo(t); v = bf16_hi(t);
}
__device__ __forceinline__ void st2(float* p, int64_t i, float u, float v) {
    *reinterpret_cast<float2*>(p + i) = make_float2(u, v);
}
__device__ __forceinline__ void st2(bf16s* p, int64_t i, float u, float v) {
    *reinterpret_cast<uint32_t*>(p + i) = pack_bf16x2(u, v);
}

#define RP_HU 4   // heads a wave has in flight at once
template <typename TC, bool PAIRED>
__global__ __launch_bounds__(256) void attn_rope_prepare_kernel(
    const TC* __restrict__ qkv, int64_t qs, const float* __restrict__ qw,
    const float* __restrict__ kw, const float* __restrict__ inv_freq, int nfreq,
    TC* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int* __restrict__ slot_mapping, const int* __restrict__ seq_of,
    const int* __restrict__ cu, const int* __restrict__ past, int B, int H, int G, int Gv, int D,
    int Dv, float eps) {
    const int t = blockIdx.x;
    if (t >= cu[B]) return;  // padding row of a fixed-size (captured) launch
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int b = seq_of[t];
    const float pos = (float)(past[b] + t - cu[b]);
    const TC* row = qkv + (int64_t)t * qs;
    const int64_t slot = slot_mapping[t];
    const int npair = (D + 1) / 2;
    // the token's cos/sin table, once per block (cos 1, sin 0 past the rotated pairs)
    extern __shared__ float lds[];
    float* cs = lds;            // [npair]
    float* sn = lds + npair;    // [npair]
    for (int i = threadIdx.x; i < npair; i += blockDim.x) {
        float s_ = 0.0f, c_ = 1.0f;
        if (i < nfreq) sincosf(pos * inv_freq[i], &s_, &c_);
        cs[i] = c_;
        sn[i] = s_;
    }
    __syncthreads();
    // query and key heads, RP_HU per wave at a time: all loads are issued
    // before the first reduction waits for one
    const int nh = H + G, stride = gridDim.y * 4 * RP_HU;
    for (int h0 = (blockIdx.y * 4 + wave) * RP_HU; h0 < nh; h0 += stride) {
        float u[RP_HU][RP_NP], v[RP_HU][RP_NP];
#pragma unroll
        for (int k = 0; k < RP_HU; ++k) {
            const int hd = h0 + k;
            const TC* src = row + (int64_t)hd * D;     // q heads, then k heads: one run of columns
#pragma unroll
            for (int j = 0; j < RP_NP; ++j) {
                const int i = lane + 64 * j;
                u[k][j] = v[k][j] = 0.0f;
                if (hd < nh && i < npair) {
                    if (PAIRED) {
                        ld2(src, 2 * i, u[k][j], v[k][j]);
                    } else {
                        u[k][j] = ldf(src, 2 * i);
                        if (2 * i + 1 < D) v[k][j] = ldf(src, 2 * i + 1);
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < RP_HU; ++k) {
            const int hd = h0 + k;
            if (hd >= nh) continue;                // uniform over the wave
            float ss = 0.0f;
#pragma unroll
            for (int j = 0; j < RP_NP; ++j) ss += u[k][j] * u[k][j] + v[k][j] * v[k][j];
            ss = wave_reduce_sum(ss);
            const float rn = qw ? 1.0f / sqrtf(ss / (float)D + eps) : 1.0f;
            const bool is_q = hd < H;
            TC* dst = is_q ? q_out + ((int64_t)t * H + hd) * D
                           : k_cache + (slot * G + (hd - H)) * D;
#pragma unroll
            for (int j = 0; j < RP_NP; ++j) {
                const int i = lane + 64 * j;
                if (i >= npair) continue;
                const float* w = is_q ? qw : kw;
                const float a = w ? u[k][j] * rn * w[2 * i] : u[k][j];
                const float c = (2 * i + 1 < D) ? (w ? v[k][j] * rn * w[2 * i + 1] : v[k][j]) : 0.0f;
                const float ra = a * cs[i] - c * sn[i];
                const float rc = c * cs[i] + a * sn[i];
                if (PAIRED) {
                    st2(dst, 2 * i, ra, rc);
                } else {
                    stf(dst, 2 * i, ra);
                    if (2 * i + 1 < D) stf(dst, 2 * i + 1, rc);
                }
            }
        }
    }
    // values: a plain copy of Gv*Dv contiguous columns to the token's slot
    const TC* vsrc = row + (int64_t)nh * D;
    TC* vdst = v_cache + slot * (int64_t)(Gv * Dv);
    const int nv = Gv * Dv, tid = blockIdx.y * blockDim.x + threadIdx.x, nt = gridDim.y * blockDim.x;
    if (PAIRED) {
        for (int i = tid; 2 * i < nv; i += nt) {
            float a, c;
            ld2(vsrc, 2 * i, a, c);
            st2(vdst, 2 * i, a, c);
        }
    } else {
        for (int i = tid; i < nv; i += nt) vdst[i] = vsrc[i];
    }
}

// The same for the common shapes, 16 bytes per lane: D/8 a power of two up to
// 64 lanes (D = 8 .. 512), Dv and the row stride multiples of 8, 16-byte
// aligned buffers. A lane holds 8 consecutive channels (4 rotation pairs) of
// one head, LPH = D/8 lanes make a head, a wave load covers 64/LPH heads;
// the head's sum of squares is a shuffle reduction inside its lane group.
// RV_IT wave loads are in flight before the first one is consumed.
#define RV_IT 3
template <typename TC>
__global__ __launch_bounds__(256) void attn_rope_prepare_vec_kernel(
    const TC* __restrict__ qkv, int64_t qs, const float* __restrict__ qw,
    const float* __restrict__ kw, const float* __restrict__ inv_freq, int nfreq,
    TC* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int* __restrict__ slot_mapping, const int* __restrict__ seq_of,
    const int* __restrict__ cu, const int* __restrict__ past, int B, int H, int G, int Gv, int D,
    int Dv, float eps) {
    extern __shared__ float lds[];
    const int npair = D / 2;
    float* cs = lds;            // [npair]
    float* sn = lds + npair;    // [npair]
    const int t = blockIdx.x;
    if (t >= cu[B]) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int b = seq_of[t];
    const float pos = (float)(past[b] + t - cu[b]);
    for (int i = threadIdx.x; i < npair; i += blockDim.x) {
        float s_ = 0.0f, c_ = 1.0f;
        if (i < nfreq) sincosf(pos * inv_freq[i], &s_, &c_);
        cs[i] = c_;
        sn[i] = s_;
    }
    __syncthreads();
    const TC* row = qkv + (int64_t)t * qs;
    const int64_t slot = slot_mapping[t];
    const int lph = D / 8, hpw = 64 / lph;           // lanes per head, heads per wave load
    const int sub = lane / lph, ch = (lane % lph) * 8;
    const int nh = H + G;
    float wq[8], wk[8];
    if (qw) {
        ld8(qw, ch, wq);
        ld8(kw, ch, wk);
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) wq[e] = wk[e] = 1.0f;
    }
    const int step = gridDim.y * 4 * hpw;
    for (int h0 = (blockIdx.y * 4 + wave) * hpw + sub; h0 < nh + step * RV_IT; h0 += step * RV_IT) {
        if (h0 - sub >= nh) break;                   // uniform over the wave
        float x[RV_IT][8];
#pragma unroll
        for (int k = 0; k < RV_IT; ++k) {
            const int hd = h0 + k * step;
            if (hd < nh) ld8(row, (int64_t)hd * D + ch, x[k]);
            else {
#pragma unroll
                for (int e = 0; e < 8; ++e) x[k][e] = 0.0f;
            }
        }
#pragma unroll
        for (int k = 0; k < RV_IT; ++k) {
            const int hd = h0 + k * step;
            float ss = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += x[k][e] * x[k][e];
            for (int off = lph >> 1; off > 0; off >>= 1) ss += __shfl_xor(ss, off, WAVE);
            if (hd >= nh) continue;
            const float rn = qw ? 1.0f / sqrtf(ss / (float)D + eps) : 1.0f;
            const bool is_q = hd < H;
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const float a = x[k][e] * rn * (is_q ? wq[e] : wk[e]);
                const float c = x[k][e + 1] * rn * (is_q ? wq[e + 1] : wk[e + 1]);
                const float cc = cs[(ch + e) >> 1], sv = sn[(ch + e) >> 1];
                o[e] = a * cc - c * sv;
                o[e + 1] = c * cc + a * sv;
            }
            if (is_q) st8(q_out, ((int64_t)t * H + hd) * D + ch, o);
            else st8(k_cache, (slot * G + (hd - H)) * D + ch, o);
        }
    }
    const TC* vsrc = row + (int64_t)nh * D;
    TC* vdst = v_cache + slot * (int64_t)(Gv * Dv);
    const int nv = Gv * Dv;
    for (int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8; i < nv; i += gridDim.y * blockDim.x * 8) {
        float tmp[8];
        ld8(vsrc, i, tmp);
        st8(vdst, i, tmp);
    }
}

extern "C" int oa_attn_rope_prepare(void* stream, const void* qkv, int64_t qs, const void* qw,
                                    const void* kw, const void* inv_freq, int nfreq,
                                    void* q_out, void* k_cache, void* v_cache,
                                    const void* slot_mapping, const void* seq_of, const void* cu,
                                    const void* past, int B, int T, int H, int G, int Gv, int D,
                                    int Dv, float eps, int dt) {
    // qw, kw both null: no norm, rotation only. Gv value heads follow the key heads.
    if (T <= 0) return 0;
    if (2 * nfreq > D || H < 1 || G < 1 || Gv < 1 || D > 128 * RP_NP || (qw == nullptr) != (kw == nullptr))
        return -100;
    hipStream_t s = (hipStream_t)stream;
    const int esz = dt == 1 ? 4 : 2;
    const bool paired = D % 2 == 0 && Dv % 2 == 0 && qs % 2 == 0 && (uintptr_t)qkv % (2 * esz) == 0 &&
                        (uintptr_t)q_out % (2 * esz) == 0 && (uintptr_t)k_cache % (2 * esz) == 0 &&
                        (uintptr_t)v_cache % (2 * esz) == 0;
    // few tokens: spread a token's heads over blocks; many: one block a token
    const int groups = CEIL_DIV(H + G, 4 * RP_HU);
    const int ny = std::max(1, std::min(groups, 1024 / T));
    const size_t lds = (size_t)2 * ((D + 1) / 2) * sizeof(float);
#define RP_ARGS(TC)                                                                            \
    (const TC*)qkv, qs, (const float*)qw, (const float*)kw, (const float*)inv_freq, nfreq,     \
        (TC*)q_out, (TC*)k_cache, (TC*)v_cache, (const int*)slot_mapping, (const int*)seq_of,  \
        (const int*)cu, (const int*)past, B, H, G, Gv, D, Dv, eps
#define RP(TC)                                                                                 \
    do {                                                                                       \
        if (paired) hipLaunchKernelGGL((attn_rope_prepare_kernel<TC, true>), dim3(T, ny),      \
                                       dim3(256), lds, s, RP_ARGS(TC));                        \
        else hipLaunchKernelGGL((attn_rope_prepare_kernel<TC, false>), dim3(T, ny), dim3(256), \
                                lds, s, RP_ARGS(TC));                                          \
    } while (0)
    const int lph = D / 8;
    const int al = dt == 1 ? 32 : 16;
    const bool vec8 = D % 8 == 0 && lph >= 1 && lph <= 64 && (lph & (lph - 1)) == 0 && Dv % 8 == 0 &&
                      qs % 8 == 0 && (uintptr_t)qkv % al == 0 && (uintptr_t)q_out % al == 0 &&
                      (uintptr_t)k_cache % al == 0 && (uintptr_t)v_cache % al == 0 &&
                      (uintptr_t)qw % 16 == 0 && (uintptr_t)kw % 16 == 0;
    if (vec8) {
        const int hpw = 64 / lph;
        const int vy = std::max(1, std::min(CEIL_DIV(H + G, 4 * hpw), 1024 / T));
        const size_t vlds = (size_t)D * sizeof(float);
        if (dt == 1)
            hipLaunchKernelGGL((attn_rope_prepare_vec_kernel<float>), dim3(T, vy), dim3(256), vlds, s,
                               RP_ARGS(float));
        else
            hipLaunchKernelGGL((attn_rope_prepare_vec_kernel<bf16s>), dim3(T, vy), dim3(256), vlds, s,
                               RP_ARGS(bf16s));
        HIP_CHECK_LAUNCH();
        return 0;
    }
    if (dt == 1) RP(float);
    else RP(bf16s);
#undef RP
#undef RP_ARGS
    HIP_CHECK_LAUNCH();
    return 0;
}

// ---------------------------------------------------------------------------
// Gated activation over rows of [gate | up]: out = act(gate) * up.
// act 0: silu g * sigmoid(g); act 1: gelu in its tanh approximation,
// g/2 * (1 + tanh(k (g + 0.044715 g^3))), k = sqrt(2/pi); act 2: the clamped
// form g' = min(g, limit), u' = clamp(u, -limit, limit),
// out = g' sigmoid(alpha g') (u' + 1). Evaluated in float32.
__device__ __forceinline__ float gate_act_f(float z, int act) {
    if (act == 1) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    return z / (1.0f + expf(-z));
}
__device__ __forceinline__ float gated_act_f(float g, float u, int act, float limit, float alpha) {
    if (act == 2) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
    }
    return gate_act_f(g, act) * u;
}

template <typename TC>
__global__ __launch_bounds__(256) void act_mul_rows_kernel(const TC* __restrict__ gu,
                                                           TC* __restrict__ out, int64_t M,
                                                           int I, int act, float limit,
                                                           float alpha) {
    const int64_t total = M * I;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t m = i / I;
        const int c = (int)(i % I);
        stf(out, i, gated_act_f(ldf(gu, m * 2 * I + c), ldf(gu, m * 2 * I + I + c), act, limit, alpha));
    }
}

// 8 channels per thread (I % 8 == 0)
template <typename TC>
__global__ __launch_bounds__(256) void act_mul_rows_vec_kernel(const TC* __restrict__ gu,
                                                               TC* __restrict__ out, int64_t M,
                                                               int I, int act, float limit,
                                                               float alpha) {
    const int iv = I / 8;
    const int64_t total = M * iv;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t m = i / iv;
        const int c = (int)(i % iv) * 8;
        float g[8], u[8];
        ld8(gu, m * 2 * I + c, g);
        ld8(gu, m * 2 * I + I + c, u);
#pragma unroll
        for (int e = 0; e < 8; ++e) g[e] = gated_act_f(g[e], u[e], act, limit, alpha);
        st8(out, m * I + c, g);
    }
}

extern "C" int oa_act_mul_rows(void* stream, const void* gu, void* out, int64_t M, int I, int dt,
                               int act, float limit, float alpha) {
    if (M <= 0 || I <= 0) return 0;
    if (act < 0 || act > 2) return -100;
    hipStream_t s = (hipStream_t)stream;
    const bool vec = I % 8 == 0 && (uintptr_t)gu % 32 == 0 && (uintptr_t)out % 32 == 0;
    if (vec) {
        const int grid = grid_for(M * (I / 8));
        if (dt == 1)
            hipLaunchKernelGGL((act_mul_rows_vec_kernel<float>), dim3(grid), dim3(256), 0, s,
                               (const float*)gu, (float*)out, M, I, act, limit, alpha);
        else
            hipLaunchKernelGGL((act_mul_rows_vec_kernel<bf16s>), dim3(grid), dim3(256), 0, s,
                               (const bf16s*)gu, (bf16s*)out, M, I, act, limit, alpha);
    } else {
        const int grid = grid_for(M * I);
        if (dt == 1)
            hipLaunchKernelGGL((act_mul_rows_kernel<float>), dim3(grid), dim3(256), 0, s,
                               (const float*)gu, (float*)out, M, I, act, limit, alpha);
        else
            hipLaunchKernelGGL((act_mul_rows_kernel<bf16s>), dim3(grid), dim3(256), 0, s,
                               (const bf16s*)gu, (bf16s*)out, M, I, act, limit, alpha);
    }
    HIP_CHECK_LAUNCH();
    return 0;
}

// ---------------------------------------------------------------------------
// Expert choice, one wave per token, all float32.
//   s_e = sigmoid(z_e) (score 0) or softmax(z)_e (score 1)
//   c_e = s_e + correction_e          (the CHOICE score; correction may be null)
//   groups > 1: runs of E/groups neighbouring experts; a run is rated
//     max1(c) + max2(c) (just max1 for runs of one) and only the `keep`
//     top-rated runs may be picked from: c of every other expert is set to
//     -inf (a zero would outrank negative c)
//   the `top` largest eligible c are chosen (ties: the lower index)
//   weight = s_chosen / (sum of the chosen s + 1e-20) * scale
// LDS per block: S[E], Cc[E], Gs[groups].
struct ArgMax {
    float v;
    int i;
};
__device__ __forceinline__ ArgMax wave_argmax(ArgMax a) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(a.v, off, WAVE);
        const int oi = __shfl_xor(a.i, off, WAVE);
        if (ov > a.v || (ov == a.v && oi < a.i)) {
            a.v = ov;
            a.i = oi;
        }
    }
    return a;
}

__global__ __launch_bounds__(64) void route_topk_kernel(
    const float* __restrict__ logits, const float* __restrict__ correction,
    int* __restrict__ idx_out, float* __restrict__ w_out, int E, int top, int groups, int keep,
    float scale, int score, int64_t ls, int rating, int renorm) {
    extern __shared__ float lds[];
    float* S = lds;
    float* Cc = S + E;
    float* Gs = Cc + E;
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (int64_t)t * ls;
    if (score == 1) {
        float mx = -INFINITY;
        for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
        mx = wave_reduce_max(mx);
        float sum = 0.0f;
        for (int e = lane; e < E; e += 64) sum += expf(z[e] - mx);
        sum = wave_reduce_sum(sum);
        for (int e = lane; e < E; e += 64) S[e] = expf(z[e] - mx) / sum;
    } else {
        for (int e = lane; e < E; e += 64) S[e] = 1.0f / (1.0f + expf(-z[e]));
    }
    for (int e = lane; e < E; e += 64) Cc[e] = S[e] + (correction ? correction[e] : 0.0f);
    __syncthreads();
    if (groups > 1) {
        const int per = E / groups;
        for (int g = lane; g < groups; g += 64) {
            float a = -INFINITY, b2 = -INFINITY;      // largest, second largest
            for (int j = 0; j < per; ++j) {
                const float c = Cc[g * per + j];
                if (c > a) {
                    b2 = a;
                    a = c;
                } else if (c > b2) {
                    b2 = c;
                }
            }
            Gs[g] = (per > 1 && rating == 0) ? a + b2 : a;
        }
        __syncthreads();
        // mark the keep best groups by lifting them to +inf, one per round
        for (int r = 0; r < keep; ++r) {
            ArgMax m{-INFINITY, 0x7fffffff};
            for (int g = lane; g < groups; g += 64) {
                const float v = Gs[g];
                if (v != INFINITY && (v > m.v || (v == m.v && g < m.i))) {
                    m.v = v;
                    m.i = g;
                }
            }
            m = wave_argmax(m);
            __syncthreads();
            if (lane == 0 && m.i != 0x7fffffff) Gs[m.i] = INFINITY;
            __syncthreads();
        }
        for (int e = lane; e < E; e += 64)
            if (Gs[e / per] != INFINITY) Cc[e] = -INFINITY;
        __syncthreads();
    }
    float wsum = 0.0f;  // lane 0 only
    for (int r = 0; r < top; ++r) {
        ArgMax m{-INFINITY, 0x7fffffff};
        for (int e = lane; e < E; e += 64) {
            const float v = Cc[e];
            if (v > m.v || (v == m.v && e < m.i)) {
                m.v = v;
                m.i = e;
            }
        }
        m = wave_argmax(m);
        const int e = m.i == 0x7fffffff ? 0 : m.i;
        __syncthreads();
        if (lane == 0) {
            idx_out[(int64_t)t * top + r] = e;
            w_out[(int64_t)t * top + r] = S[e];
            wsum += S[e];
            Cc[e] = -INFINITY;
        }
        __syncthreads();
    }
    if (lane == 0) {
        const float inv = renorm ? scale / (wsum + 1e-20f) : scale;
        for (int r = 0; r < top; ++r) w_out[(int64_t)t * top + r] *= inv;
    }
}

extern "C" int oa_route_topk(void* stream, const void* logits, int64_t ls, const void* correction,
                             void* idx, void* w, int T, int E, int top, int groups, int keep,
                             float scale, int score, int rating, int renorm) {
    if (T <= 0) return 0;
    if (E < 1 || top < 1 || top > E || groups < 1 || E % groups != 0 || keep < 1 ||
        keep > groups || (int64_t)keep * (E / groups) < top)
        return -100;
    const size_t lds = (size_t)(2 * E + groups) * sizeof(float);
    if (lds > 60 * 1024) return -101;
    hipLaunchKernelGGL(route_topk_kernel, dim3(T), dim3(64), lds, (hipStream_t)stream,
                       (const float*)logits, (const float*)correction, (int*)idx, (float*)w, E, top,
                       groups, keep, scale, score, ls, rating, renorm);
    HIP_CHECK_LAUNCH();
    return 0;
}

// ---------------------------------------------------------------------------
// Routed experts for few (token, expert) pairs: two launches, no host sync,
// no atomics. Pair p = t * top + j uses expert idx[p].
//   gate-up: mid[p, r] = act(Wg[e][r] . x_t) * (Wu[e][r] . x_t),  w13 [E, 2I, K]
//   down:    out[t, c] = sum_j wts[t, j] * (W2[e_tj][c] . mid[t*top + j]),  w2 [E, C, I]
// A wave owns an output row; its lanes stride the reduction (8 elements at a
// time where the sizes allow). A token's result depends on no other token.
template <typename TC>
__device__ __forceinline__ void dot2_rows(const TC* __restrict__ wa, const TC* __restrict__ wb,
                                          const TC* __restrict__ x, int K, int lane, bool vec,
                                          float& ra, float& rb) {
    float a = 0.0f, b = 0.0f;
    if (vec) {
        for (int i = lane * 8; i < K; i += 64 * 8) {
            float xv[8], av[8], bv[8];
            ld8(x, i, xv);
            ld8(wa, i, av);
            ld8(wb, i, bv);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                a = fmaf(av[e], xv[e], a);
                b = fmaf(bv[e], xv[e], b);
            }
        }
    } else {
        for (int i = lane; i < K; i += 64) {
            const float xv = ldf(x, i);
            a = fmaf(ldf(wa, i), xv, a);
            b = fmaf(ldf(wb, i), xv, b);
        }
    }
    ra = wave_reduce_sum(a);
    rb = wave_reduce_sum(b);
}

template <typename TC>
__global__ __launch_bounds__(256) void moe_pairs_gateup_kernel(
    const TC* __restrict__ x, const TC* __restrict__ w13, const int* __restrict__ idx,
    TC* __restrict__ mid, int top, int E, int I, int K, int act, int vec, float limit,
    float alpha) {
    const int p = blockIdx.x, t = p / top;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int e = min(max(idx[p], 0), E - 1);
    const TC* we = w13 + (int64_t)e * 2 * I * K;
    const TC* xr = x + (int64_t)t * K;
    for (int r = blockIdx.y * 4 + wave; r < I; r += gridDim.y * 4) {
        float g, u;
        dot2_rows(we + (int64_t)r * K, we + (int64_t)(I + r) * K, xr, K, lane, vec != 0, g, u);
        if (lane == 0) stf(mid, (int64_t)p * I + r, gated_act_f(g, u, act, limit, alpha));
    }
}

template <typename TC>
__global__ __launch_bounds__(256) void moe_pairs_down_kernel(
    const TC* __restrict__ mid, const TC* __restrict__ w2, const int* __restrict__ idx,
    const float* __restrict__ wts, TC* __restrict__ out, int top, int E, int C, int I, int vec) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int c = blockIdx.y * 4 + wave; c < C; c += gridDim.y * 4) {
        float acc = 0.0f;
        for (int j = 0; j < top; ++j) {
            const int p = t * top + j;
            const int e = min(max(idx[p], 0), E - 1);
            const TC* wr = w2 + ((int64_t)e * C + c) * I;
            const TC* mr = mid + (int64_t)p * I;
            float a = 0.0f;
            if (vec) {
                for (int i = lane * 8; i < I; i += 64 * 8) {
                    float wv[8], mv[8];
                    ld8(wr, i, wv);
                    ld8(mr, i, mv);
#pragma unroll
                    for (int q = 0; q < 8; ++q) a = fmaf(wv[q], mv[q], a);
                }
            } else {
                for (int i = lane; i < I; i += 64) a = fmaf(ldf(wr, i), ldf(mr, i), a);
            }
            acc += wts[p] * wave_reduce_sum(a);
        }
        if (lane == 0) stf(out, (int64_t)t * C + c, acc);
    }
}

extern "C" int oa_moe_pairs_gateup(void* stream, const void* x, const void* w13, const void* idx,
                                   void* mid, int T, int top, int E, int I, int K, int dt,
                                   int act, float limit, float alpha) {
    if (T <= 0) return 0;
    if (top < 1 || E < 1 || I < 1 || K < 1 || act < 0 || act > 2) return -100;
    const int vec = (K % 8 == 0 && (uintptr_t)x % 32 == 0 && (uintptr_t)w13 % 32 == 0) ? 1 : 0;
    dim3 grid(T * top, std::min(CEIL_DIV(I, 4), 64));
    hipStream_t s = (hipStream_t)stream;
    if (dt == 1)
        hipLaunchKernelGGL((moe_pairs_gateup_kernel<float>), grid, dim3(256), 0, s, (const float*)x,
                           (const float*)w13, (const int*)idx, (float*)mid, top, E, I, K, act, vec, limit, alpha);
    else
        hipLaunchKernelGGL((moe_pairs_gateup_kernel<bf16s>), grid, dim3(256), 0, s, (const bf16s*)x,
                           (const bf16s*)w13, (const int*)idx, (bf16s*)mid, top, E, I, K, act, vec, limit, alpha);
    HIP_CHECK_LAUNCH();
    return 0;
}

extern "C" int oa_moe_pairs_down(void* stream, const void* mid, const void* w2, const void* idx,
                                 const void* wts, void* out, int T, int top, int E, int C, int I,
                                 int dt) {
    if (T <= 0) return 0;
    if (top < 1 || E < 1 || I < 1 || C < 1) return -100;
    const int vec = (I % 8 == 0 && (uintptr_t)mid % 32 == 0 && (uintptr_t)w2 % 32 == 0) ? 1 : 0;
    dim3 grid(T, std::min(CEIL_DIV(C, 4), 64));
    hipStream_t s = (hipStream_t)stream;
    if (dt == 1)
        hipLaunchKernelGGL((moe_pairs_down_kernel<float>), grid, dim3(256), 0, s, (const float*)mid,
                           (const float*)w2, (const int*)idx, (const float*)wts, (float*)out, top, E,
                           C, I, vec);
    else
        hipLaunchKernelGGL((moe_pairs_down_kernel<bf16s>), grid, dim3(256), 0, s, (const bf16s*)mid,
                           (const bf16s*)w2, (const int*)idx, (const float*)wts, (bf16s*)out, top, E,
                           C, I, vec);
    HIP_CHECK_LAUNCH();
    return 0;
}
