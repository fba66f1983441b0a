// Kernels of pre-norm decoder blocks with latent attention for MI355X
// (gfx950): the residual add fused with the layer norm that follows it, and
// the two preparation steps of latent attention (cache rows, queries).
//
// Same conventions as mixers.hip: a FLAT multi-sequence batch (cu, past,
// seq_of), activations bf16 (dt = 0) or float32 (dt = 1), float32 for norm
// weights and statistics, angles and the residual. All sizes are run-time
// values.

#include "mixer_util.h"

// ---------------------------------------------------------------------------
// One launch for the add after a sublayer and the layer norm before the next:
//   r = residual + y + sigmoid(g2) * y2      (y, y2, g2 each optional; g2 is
//                                              one float32 logit per token)
//   residual = r                              (if anything was added)
//   out = (r - mean(r)) / sqrt(mean((r - mean(r))^2) + eps) * w   (if w)
// One block per token, 16 bytes per lane and access where the row allows.
// The first 256 * LN_NR channels of the row stay in registers between the
// passes; wider rows re-read the (just written)
// residual for the rest. The variance is the mean of squared deviations
// from the already known mean: two passes, no cancellation.
#define LN_NR 16

__device__ __forceinline__ void ld4(const float* p, int64_t i, float* o) {
    const float4 a = *reinterpret_cast<const float4*>(p + i);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
}
__device__ __forceinline__ void ld4(const bf16s* p, int64_t i, float* o) {
    const uint2 a = *reinterpret_cast<const uint2*>(p + i);
    o[0] = bf16_lo(a.x); o[1] = bf16_hi(a.x); o[2] = bf16_lo(a.y); o[3] = bf16_hi(a.y);
}
__device__ __forceinline__ void st4(float* p, int64_t i, const float* v) {
    *reinterpret_cast<float4*>(p + i) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void st4(bf16s* p, int64_t i, const float* v) {
    uint2 a;
    a.x = pack_bf16x2(v[0], v[1]);
    a.y = pack_bf16x2(v[2], v[3]);
    *reinterpret_cast<uint2*>(p + i) = a;
}

// VEC: a thread takes 4 consecutive channels at a time (C % 4 == 0, rows and
// bases aligned to 4 elements); otherwise one channel at a time.
template <typename TC, bool VEC>
__global__ __launch_bounds__(256) void add_layer_norm_kernel(
    float* __restrict__ residual, const TC* __restrict__ y, int64_t ys,
    const TC* __restrict__ y2, int64_t y2s, const float* __restrict__ g2, int64_t g2s,
    const float* __restrict__ w, TC* __restrict__ out, int C, float eps) {
    __shared__ float red_a[16], red_b[16];
    constexpr int W = VEC ? 4 : 1;            // channels per step
    constexpr int NS = LN_NR / W;             // steps kept in registers
    const int t = blockIdx.x, tid = threadIdx.x;
    float* r = residual + (int64_t)t * C;
    const TC* yr = y ? y + (int64_t)t * ys : nullptr;
    const TC* y2r = y2 ? y2 + (int64_t)t * y2s : nullptr;
    const float gate = (y2 && g2) ? sigmoidf_(g2[(int64_t)t * g2s]) : 1.0f;
    const bool adds = y || y2;
    // channel of step j, element e: (tid + 256 j) * W + e
    auto load = [&](int c, float* x) {
        if (VEC) {
            ld4(r, c, x);
            float a[4];
            if (yr) {
                ld4(yr, c, a);
#pragma unroll
                for (int e = 0; e < 4; ++e) x[e] += a[e];
            }
            if (y2r) {
                ld4(y2r, c, a);
#pragma unroll
                for (int e = 0; e < 4; ++e) x[e] += gate * a[e];
            }
            if (adds) st4(r, c, x);
        } else {
            x[0] = r[c];
            if (yr) x[0] += ldf(yr, c);
            if (y2r) x[0] += gate * ldf(y2r, c);
            if (adds) r[c] = x[0];
        }
    };
    float vals[LN_NR];
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int c = (tid + 256 * j) * W;
#pragma unroll
        for (int e = 0; e < W; ++e) vals[j * W + e] = 0.0f;
        if (c < C) load(c, vals + j * W);
#pragma unroll
        for (int e = 0; e < W; ++e) sum += vals[j * W + e];
    }
    for (int c = (tid + 256 * NS) * W; c < C; c += 256 * W) {
        float x[W];
        load(c, x);
#pragma unroll
        for (int e = 0; e < W; ++e) sum += x[e];
    }
    if (!w) return;
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
#pragma unroll
        for (int e = 0; e < W; ++e) {
            const float d = r[c + e] - mean;
            sq += d * d;
        }
    }
    const float var = block_reduce_sum<4>(sq, red_b) / (float)C;
    const float rs = 1.0f / sqrtf(var + eps);
    TC* o = out + (int64_t)t * C;
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int c = (tid + 256 * j) * W;
        if (c < C) {
            float x[W];
#pragma unroll
            for (int e = 0; e < W; ++e) x[e] = (vals[j * W + e] - mean) * rs * w[c + e];
            if (VEC) st4(o, c, x);
            else stf(o, c, x[0]);
        }
    }
    for (int c = (tid + 256 * NS) * W; c < C; c += 256 * W) {
        float x[W];
#pragma unroll
        for (int e = 0; e < W; ++e) x[e] = (r[c + e] - mean) * rs * w[c + e];
        if (VEC) st4(o, c, x);
        else stf(o, c, x[0]);
    }
}

// y, y2 and out share the activation type dt.
extern "C" int oa_add_layer_norm(void* stream, void* residual, const void* y, int64_t ys, int y_dt,
                                 const void* y2, int64_t y2s, int y2_dt, const void* g2,
                                 int64_t g2s, const void* w, void* out, int out_dt, int T, int C,
                                 float eps) {
    if (T <= 0 || C <= 0) return 0;
    int dt = -1;
    if (y) dt = y_dt;
    if (y2) {
        if (dt >= 0 && y2_dt != dt) return -100;
        dt = y2_dt;
    }
    if (w) {
        if (!out) return -101;
        if (dt >= 0 && out_dt != dt) return -100;
        dt = out_dt;
    }
    if (dt < 0) return 0;   // nothing to add, nothing to norm
    hipStream_t s = (hipStream_t)stream;
    const int esz = dt == 1 ? 4 : 2;
    auto al = [&](const void* p, int64_t stride) {
        return !p || ((uintptr_t)p % (4 * esz) == 0 && stride % 4 == 0);
    };
    const bool vec = C % 4 == 0 && (uintptr_t)residual % 16 == 0 && al(y, ys) && al(y2, y2s) &&
                     al(out, 0) && (!w || (uintptr_t)w % 16 == 0);
#define LN_LAUNCH(TC, V)                                                                         \
    hipLaunchKernelGGL((add_layer_norm_kernel<TC, V>), dim3(T), dim3(256), 0, s, (float*)residual, \
                       (const TC*)y, ys, (const TC*)y2, y2s, (const float*)g2, g2s,               \
                       (const float*)w, (TC*)out, C, eps)
    if (dt == 1) {
        if (vec) LN_LAUNCH(float, true);
        else LN_LAUNCH(float, false);
    } else {
        if (vec) LN_LAUNCH(bf16s, true);
        else LN_LAUNCH(bf16s, false);
    }
#undef LN_LAUNCH
    HIP_CHECK_LAUNCH();
    return 0;
}

// ---------------------------------------------------------------------------
// Cache rows of latent attention. Per token, from dkv [rank + rot]:
//   row[0 .. rank)          = dkv[i] / sqrt(mean_i(dkv[i]^2) + eps) * nw[i]
//   row[rank .. rank + rot) = the pairs (2i, 2i+1), i < nfreq, rotated by
//                             position * inv_freq[i]; the rest unchanged
// written to k_cache[slot] (rows of rank + rot). One wave per token, four
// tokens per block. The position of token t of sequence b is
// past[b] + t - cu[b]. Everything between load and store is float32.
template <typename TC>
__global__ __launch_bounds__(256) void latent_kv_prepare_kernel(
    const TC* __restrict__ dkv, int64_t ds, const float* __restrict__ nw,
    const float* __restrict__ inv_freq, int nfreq, TC* __restrict__ k_cache,
    const int* __restrict__ slot_mapping, const int* __restrict__ seq_of,
    const int* __restrict__ cu, const int* __restrict__ past, int B, int T, int rank, int rot,
    float eps) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x * 4 + wave;
    if (t >= T || t >= cu[B]) return;       // also the padding rows of a captured launch
    const int b = seq_of[t];
    const float pos = (float)(past[b] + t - cu[b]);
    const TC* row = dkv + (int64_t)t * ds;
    TC* dst = k_cache + (int64_t)slot_mapping[t] * (rank + rot);
    float ss = 0.0f;
    for (int i = lane; i < rank; i += 64) {
        const float x = ldf(row, i);
        ss += x * x;
    }
    ss = wave_reduce_sum(ss);
    const float rn = 1.0f / sqrtf(ss / (float)rank + eps);
    for (int i = lane; i < rank; i += 64) stf(dst, i, ldf(row, i) * rn * nw[i]);
    const int npair = rot / 2;
    for (int i = lane; i < npair; i += 64) {
        const float u = ldf(row, rank + 2 * i), v = ldf(row, rank + 2 * i + 1);
        float s_ = 0.0f, c_ = 1.0f;
        if (i < nfreq) sincosf(pos * inv_freq[i], &s_, &c_);
        stf(dst, rank + 2 * i, u * c_ - v * s_);
        stf(dst, rank + 2 * i + 1, v * c_ + u * s_);
    }
    if ((rot & 1) && lane == 0) stf(dst, rank + rot - 1, ldf(row, rank + rot - 1));
}

extern "C" int oa_latent_kv_prepare(void* stream, const void* dkv, int64_t ds, const void* nw,
                                    const void* inv_freq, int nfreq, void* k_cache,
                                    const void* slot_mapping, const void* seq_of, const void* cu,
                                    const void* past, int B, int T, int rank, int rot, float eps,
                                    int dt) {
    if (T <= 0) return 0;
    if (rank < 1 || rot < 0 || 2 * nfreq > rot) return -100;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(CEIL_DIV(T, 4));
    if (dt == 1)
        hipLaunchKernelGGL((latent_kv_prepare_kernel<float>), grid, dim3(256), 0, s, (const float*)dkv,
                           ds, (const float*)nw, (const float*)inv_freq, nfreq, (float*)k_cache,
                           (const int*)slot_mapping, (const int*)seq_of, (const int*)cu,
                           (const int*)past, B, T, rank, rot, eps);
    else
        hipLaunchKernelGGL((latent_kv_prepare_kernel<bf16s>), grid, dim3(256), 0, s, (const bf16s*)dkv,
                           ds, (const float*)nw, (const float*)inv_freq, nfreq, (bf16s*)k_cache,
                           (const int*)slot_mapping, (const int*)seq_of, (const int*)cu,
                           (const int*)past, B, T, rank, rot, eps);
    HIP_CHECK_LAUNCH();
    return 0;
}

// ---------------------------------------------------------------------------
// Queries of latent attention against the cached rows. q [T, H * (D + rot)]
// holds per head D unrotated and rot rotated channels; q_lat [H, T, rank] is
// the unrotated part already taken through the key up-projection (null: the
// caller's batched GEMM has written it into out already). out
// [T, H, rank + rot] = q_lat beside the part rotated by position. One wave
// per (token, head).
template <typename TC>
__global__ __launch_bounds__(256) void latent_q_assemble_kernel(
    const TC* __restrict__ q, int64_t qs, const TC* __restrict__ q_lat,
    const float* __restrict__ inv_freq, int nfreq, TC* __restrict__ out,
    const int* __restrict__ seq_of, const int* __restrict__ cu, const int* __restrict__ past,
    int B, int T, int H, int D, int rot, int rank) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x;
    if (t >= cu[B]) return;
    const int b = seq_of[t];
    const float pos = (float)(past[b] + t - cu[b]);
    const int npair = rot / 2;
    for (int h = blockIdx.y * 4 + wave; h < H; h += gridDim.y * 4) {
        const TC* src = q_lat + ((int64_t)h * T + t) * rank;
        TC* dst = out + ((int64_t)t * H + h) * (rank + rot);
        if (q_lat)
            for (int i = lane; i < rank; i += 64) dst[i] = src[i];
        const TC* qr = q + (int64_t)t * qs + (int64_t)h * (D + rot) + D;
        for (int i = lane; i < npair; i += 64) {
            const float u = ldf(qr, 2 * i), v = ldf(qr, 2 * i + 1);
            float s_ = 0.0f, c_ = 1.0f;
            if (i < nfreq) sincosf(pos * inv_freq[i], &s_, &c_);
            stf(dst, rank + 2 * i, u * c_ - v * s_);
            stf(dst, rank + 2 * i + 1, v * c_ + u * s_);
        }
        if ((rot & 1) && lane == 0) dst[rank + rot - 1] = qr[rot - 1];
    }
}

extern "C" int oa_latent_q_assemble(void* stream, const void* q, int64_t qs, const void* q_lat,
                                    const void* inv_freq, int nfreq, void* out, const void* seq_of,
                                    const void* cu, const void* past, int B, int T, int H, int D,
                                    int rot, int rank, int dt) {
    if (T <= 0) return 0;
    if (H < 1 || rank < 1 || rot < 0 || 2 * nfreq > rot) return -100;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(T, std::min(CEIL_DIV(H, 4), 8));
    if (dt == 1)
        hipLaunchKernelGGL((latent_q_assemble_kernel<float>), grid, dim3(256), 0, s, (const float*)q, qs,
                           (const float*)q_lat, (const float*)inv_freq, nfreq, (float*)out,
                           (const int*)seq_of, (const int*)cu, (const int*)past, B, T, H, D, rot, rank);
    else
        hipLaunchKernelGGL((latent_q_assemble_kernel<bf16s>), grid, dim3(256), 0, s, (const bf16s*)q, qs,
                           (const bf16s*)q_lat, (const float*)inv_freq, nfreq, (bf16s*)out, (const int*)seq_of, (const int*)cu, (const int*)past,
                           B, T, H, D, rot, rank);
    HIP_CHECK_LAUNCH();
    return 0;
}
