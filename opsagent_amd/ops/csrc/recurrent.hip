// Linear attention with decay for MI355X (gfx950): the recurrence
//   S_t = diag(a_t) S_{t-1} + k_t v_t^T,   o_t = S_t^T q_t
// per sequence and head over a float32 state, and the gated RMS norm of its
// read-out.
//
// Same conventions as mixers.hip: a FLAT multi-sequence batch (cu, past,
// slots), activations bf16 (dt = 0) or float32 (dt = 1); decays, their
// logarithms, the state and the read-out are float32. All sizes are run-time
// values.

#include "mixer_util.h"

__device__ __forceinline__ float row16_total(float x) {
    // all-reduce over the 16 lanes of a DPP row: quad swaps, then mirrors
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xF, 0xF, true));
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xF, 0xF, true));
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xF, 0xF, true));
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xF, 0xF, true));
    return x;
}

// ---------------------------------------------------------------------------
// grid = (sequences, heads, column splits). Lane = (row group, column): the
// 16 lanes of a DPP row split the D key rows of one value column (RPL
// consecutive rows each), a wave holds 4 columns per pass and P passes, a
// block Dv / gridDim.z columns of the head. S stays in registers over the
// whole portion; between steps it lives in the state slot as [H, Dv, D] (a
// column's rows contiguous). A sequence that starts at position 0 starts
// from zero whatever the slot holds.
// Decay: head_decay given: a = head_decay[h] for every row; else per row
//   a = sigmoid(z + z_bias)^inv_tau = exp(-softplus(-(z + z_bias)) * inv_tau).
// act = 1 applies silu to q, k and v as they are staged; q is then scaled.
// Per chunk of TCK tokens the block stages q, k, a and its v columns in LDS
// as float32 (rows past D as zero), runs the recurrence (the column sum of
// the read-out is a DPP add inside a 16-lane row), and stores the read-out
// [T, H*Dv] float32.
template <int RPL, int P, typename TC>
__global__ void decay_scan_kernel(
    const TC* __restrict__ q, int64_t qs, const TC* __restrict__ k, int64_t ks,
    const TC* __restrict__ v, int64_t vs, const TC* __restrict__ z, int64_t zs,
    const float* __restrict__ z_bias, float inv_tau, const float* __restrict__ head_decay,
    float* __restrict__ state, float* __restrict__ o_raw, const int* __restrict__ cu,
    const int* __restrict__ past, const int* __restrict__ slots, int H, int D, int Dv, int TCK,
    int act, float q_scale) {
    constexpr int DP = RPL * 16;  // padded key size
    extern __shared__ float lds[];
    const int cpb = Dv / gridDim.z, cb = blockIdx.z * cpb, cend = cb + cpb;
    float* sq = lds;
    float* sk = sq + TCK * DP;
    float* sv = sk + TCK * DP;
    float* so = sv + TCK * cpb;
    float* sg = so + TCK * cpb;       // only with per-row decays
    const int b = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, nth = blockDim.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int rg = lane & 15, cs = lane >> 4;
    const int lo = cu[b], n = cu[b + 1] - lo;
    if (n <= 0) return;
    float* st = state + (((int64_t)slots[b] * H + h) * Dv) * D;
    const bool per_row = head_decay == nullptr;
    const float hd = per_row ? 1.0f : head_decay[h];
    float S[P][RPL];
    int col[P];
    const bool fresh = past[b] == 0;
    const bool vec4 = (D & 3) == 0;   // a lane's rows of a column are 16-byte pieces
#pragma unroll
    for (int p = 0; p < P; ++p) {
        col[p] = cb + (wave * P + p) * 4 + cs;
        if (col[p] >= cend) col[p] = Dv;              // past this block's share: idle
        const bool live = !fresh && col[p] < Dv;
#pragma unroll
        for (int i4 = 0; i4 < RPL / 4; ++i4) {
            const int r = rg * RPL + 4 * i4;
            float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
            if (live && vec4 && r < D) {
                x = *reinterpret_cast<const float4*>(st + (int64_t)col[p] * D + r);
            } else if (live) {
                if (r < D) x.x = st[(int64_t)col[p] * D + r];
                if (r + 1 < D) x.y = st[(int64_t)col[p] * D + r + 1];
                if (r + 2 < D) x.z = st[(int64_t)col[p] * D + r + 2];
                if (r + 3 < D) x.w = st[(int64_t)col[p] * D + r + 3];
            }
            S[p][4 * i4] = x.x;
            S[p][4 * i4 + 1] = x.y;
            S[p][4 * i4 + 2] = x.z;
            S[p][4 * i4 + 3] = x.w;
        }
    }
    for (int c0 = 0; c0 < n; c0 += TCK) {
        const int nc = min(TCK, n - c0);
        const int tb = lo + c0;
        for (int i = tid; i < nc * DP; i += nth) {
            const int tt = i / DP, r = i % DP;
            const int64_t t = tb + tt;
            float qv = 0.0f, kv = 0.0f, gv = 0.0f;
            if (r < D) {
                qv = ldf(q, t * qs + h * D + r);
                kv = ldf(k, t * ks + h * D + r);
                if (act) {
                    qv = qv / (1.0f + expf(-qv));
                    kv = kv / (1.0f + expf(-kv));
                }
                qv *= q_scale;
                if (per_row) {
                    const float zz = ldf(z, t * zs + h * D + r) + z_bias[h * D + r];
                    gv = expf(-softplusf_(-zz) * inv_tau);
                }
            }
            sq[i] = qv;
            sk[i] = kv;
            if (per_row) sg[i] = gv;
        }
        // only this block's share of the value columns is read
        for (int i = tid; i < nc * cpb; i += nth) {
            const int tt = i / cpb, c = i % cpb;
            float x = ldf(v, (int64_t)(tb + tt) * vs + h * Dv + cb + c);
            if (act) x = x / (1.0f + expf(-x));
            sv[i] = x;
        }
        __syncthreads();
        for (int tt = 0; tt < nc; ++tt) {
            float kr[RPL], gr[RPL], qr[RPL];
#pragma unroll
            for (int i = 0; i < RPL; ++i) {
                kr[i] = sk[tt * DP + rg * RPL + i];
                qr[i] = sq[tt * DP + rg * RPL + i];
                gr[i] = per_row ? sg[tt * DP + rg * RPL + i] : hd;
            }
            float o[P];
#pragma unroll
            for (int p = 0; p < P; ++p) {
                const float vv = col[p] < Dv ? sv[tt * cpb + col[p] - cb] : 0.0f;
                o[p] = 0.0f;
#pragma unroll
                for (int i = 0; i < RPL; ++i) {
                    S[p][i] = fmaf(S[p][i], gr[i], kr[i] * vv);
                    o[p] = fmaf(S[p][i], qr[i], o[p]);
                }
            }
#pragma unroll
            for (int p = 0; p < P; ++p) {
                o[p] = row16_total(o[p]);
                if (rg == 0 && col[p] < Dv) so[tt * cpb + col[p] - cb] = o[p];
            }
        }
        __syncthreads();
        for (int i = tid; i < nc * cpb; i += nth) {
            const int tt = i / cpb, c = i % cpb;
            o_raw[((int64_t)(tb + tt) * H + h) * Dv + cb + c] = so[i];
        }
        // the next chunk's staging does not touch `so`; its recurrence, which
        // does, comes after the barrier that follows the staging
    }
#pragma unroll
    for (int p = 0; p < P; ++p) {
        if (col[p] >= Dv) continue;
#pragma unroll
        for (int i4 = 0; i4 < RPL / 4; ++i4) {
            const int r = rg * RPL + 4 * i4;
            float* dst = st + (int64_t)col[p] * D + r;
            if (vec4 && r < D) {
                *reinterpret_cast<float4*>(dst) =
                    make_float4(S[p][4 * i4], S[p][4 * i4 + 1], S[p][4 * i4 + 2], S[p][4 * i4 + 3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (r + e < D) dst[e] = S[p][4 * i4 + e];
            }
        }
    }
}

template <int RPL, int P>
static int launch_decay_scan(hipStream_t s, const void* q, int64_t qs, const void* k, int64_t ks,
                             const void* v, int64_t vs, const void* z, int64_t zs,
                             const void* z_bias, float inv_tau, const void* head_decay,
                             void* state, void* o_raw, const void* cu, const void* past,
                             const void* slots, int B, int H, int D, int Dv, int act,
                             float q_scale, int dt, int csplit) {
    const int cpb = Dv / csplit;
    const int nw = CEIL_DIV(cpb, 4 * P);
    if (nw > 16) return -106;
    const int nstage = head_decay ? 2 : 3;
    int tck = 16;
    auto bytes = [&](int t) { return (size_t)(nstage * t * RPL * 16 + 2 * t * cpb) * 4; };
    while (tck > 2 && bytes(tck) > 60 * 1024) tck >>= 1;
    dim3 grid(B, H, csplit), blk(64 * nw);
#define SARGS(TC)                                                                            \
    (const TC*)q, qs, (const TC*)k, ks, (const TC*)v, vs, (const TC*)z, zs,                   \
        (const float*)z_bias, inv_tau, (const float*)head_decay, (float*)state, (float*)o_raw, \
        (const int*)cu, (const int*)past, (const int*)slots, H, D, Dv, tck, act, q_scale
    if (dt == 1)
        hipLaunchKernelGGL((decay_scan_kernel<RPL, P, float>), grid, blk, bytes(tck), s, SARGS(float));
    else
        hipLaunchKernelGGL((decay_scan_kernel<RPL, P, bf16s>), grid, blk, bytes(tck), s, SARGS(bf16s));
#undef SARGS
    HIP_CHECK_LAUNCH();
    return 0;
}

// q, k, z [T, H*D], v [T, H*Dv]: rows with the given strides; o_raw [T, H*Dv]
// float32 contiguous; state [slots, H, Dv, D] float32. Exactly one of
// head_decay (float32 [H]) and z (with z_bias float32 [H*D]) is given.
// csplit splits each head's value columns over that many blocks (Dv must
// divide by csplit).
extern "C" int oa_decay_scan(void* stream, const void* q, int64_t qs, const void* k, int64_t ks,
                             const void* v, int64_t vs, const void* z, int64_t zs,
                             const void* z_bias, float inv_tau, const void* head_decay,
                             void* state, void* o_raw, const void* cu, const void* past,
                             const void* slots, int T, int B, int H, int D, int Dv, int act,
                             float q_scale, int dt, int csplit) {
    if (T <= 0 || B <= 0) return 0;
    if (H < 1 || D < 1 || Dv < 1) return -100;
    if (D > 256) return -105;
    if ((head_decay == nullptr) == (z == nullptr) || (z && !z_bias)) return -101;
    if (csplit < 1 || Dv % csplit != 0) return -107;
    hipStream_t s = (hipStream_t)stream;
#define SL(R, PP)                                                                                  \
    launch_decay_scan<R, PP>(s, q, qs, k, ks, v, vs, z, zs, z_bias, inv_tau, head_decay, state,     \
                             o_raw, cu, past, slots, B, H, D, Dv, act, q_scale, dt, csplit)
    const int r = D <= 64 ? 4 : (D <= 128 ? 8 : 16);
    const int cpb = Dv / csplit;
    // passes per wave: 64 columns per pass at 16 waves
    const int p = cpb <= 64 ? 1 : (cpb <= 128 ? 2 : (cpb <= 256 ? 4 : 0));
    if (p == 0) return -105;
    int rc;
    if (r == 4) rc = p == 1 ? SL(4, 1) : (p == 2 ? SL(4, 2) : SL(4, 4));
    else if (r == 8) rc = p == 1 ? SL(8, 1) : (p == 2 ? SL(8, 2) : SL(8, 4));
    else rc = p == 1 ? SL(16, 1) : (p == 2 ? SL(16, 2) : SL(16, 4));
#undef SL
    return rc;
}

// ---------------------------------------------------------------------------
// Gated RMS norm of a float32 read-out o [T, N]: the row is cut into `groups`
// equal parts, each divided by sqrt(mean(part^2) + eps), times the float32
// weight (wlen = N: one per channel; wlen = N / groups: shared by the parts),
// times gate_act(gate): 0 sigmoid, 1 silu. grid = (tokens, part groups): one
// part, the whole block reduces the row; several, a wave per part and four
// parts per block. A lane keeps its channels in registers between the sum
// and the scaling (GN_NR per lane, the rest is read again).
#define GN_NR 16

__device__ __forceinline__ float gate_fn(float g, int gate_act) {
    return gate_act ? g / (1.0f + expf(-g)) : sigmoidf_(g);
}
__device__ __forceinline__ void gn_ld4(const float* p, int64_t i, float* o) {
    const float4 a = *reinterpret_cast<const float4*>(p + i);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
}
__device__ __forceinline__ void gn_ld4(const bf16s* p, int64_t i, float* o) {
    const uint2 a = *reinterpret_cast<const uint2*>(p + i);
    o[0] = bf16_lo(a.x); o[1] = bf16_hi(a.x); o[2] = bf16_lo(a.y); o[3] = bf16_hi(a.y);
}
__device__ __forceinline__ void gn_st4(float* p, int64_t i, const float* v) {
    *reinterpret_cast<float4*>(p + i) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void gn_st4(bf16s* p, int64_t i, const float* v) {
    uint2 a;
    a.x = pack_bf16x2(v[0], v[1]);
    a.y = pack_bf16x2(v[2], v[3]);
    *reinterpret_cast<uint2*>(p + i) = a;
}

// VEC: 4 consecutive channels per lane and access (part size % 4 == 0, rows
// and bases aligned to 4 elements).
template <typename TG, typename TO, bool VEC>
__global__ __launch_bounds__(256) void gated_rms_norm_kernel(
    const float* __restrict__ o, const float* __restrict__ w, int wlen,
    const TG* __restrict__ gate, int64_t gs, int gate_act, TO* __restrict__ out, int N,
    int groups, float eps) {
    __shared__ float red[16];
    constexpr int W = VEC ? 4 : 1;
    constexpr int NS = GN_NR / W;
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* src = o + (int64_t)t * N;
    const TG* gr = gate + (int64_t)t * gs;
    TO* dst = out + (int64_t)t * N;
    const int per = N / groups;
    // one part: the block's 256 threads stride it; several: a wave per part
    const int nth = groups == 1 ? 256 : 64;
    const int me = groups == 1 ? threadIdx.x : lane;
    const int gi = groups == 1 ? 0 : blockIdx.y * 4 + wave;
    if (gi >= groups) return;
    const int base = gi * per;
    float vals[GN_NR];
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int i = (me + nth * j) * W;
#pragma unroll
        for (int e = 0; e < W; ++e) vals[j * W + e] = 0.0f;
        if (i < per) {
            if (VEC) gn_ld4(src, base + i, vals + j * W);
            else vals[j] = src[base + i];
        }
#pragma unroll
        for (int e = 0; e < W; ++e) ss += vals[j * W + e] * vals[j * W + e];
    }
    for (int i = (me + nth * NS) * W; i < per; i += nth * W)
#pragma unroll
        for (int e = 0; e < W; ++e) ss += src[base + i + e] * src[base + i + e];
    ss = groups == 1 ? block_reduce_sum<4>(ss, red) : wave_reduce_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)per + eps);
    auto emit = [&](int i, const float* x) {
        const int c = base + i;
        float g[W], y[W];
        if (VEC) gn_ld4(gr, c, g);
        else g[0] = ldf(gr, c);
#pragma unroll
        for (int e = 0; e < W; ++e)
            y[e] = x[e] * r * w[(wlen == N ? c : i) + e] * gate_fn(g[e], gate_act);
        if (VEC) gn_st4(dst, c, y);
        else stf(dst, c, y[0]);
    };
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int i = (me + nth * j) * W;
        if (i < per) emit(i, vals + j * W);
    }
    for (int i = (me + nth * NS) * W; i < per; i += nth * W) {
        float x[W];
#pragma unroll
        for (int e = 0; e < W; ++e) x[e] = src[base + i + e];
        emit(i, x);
    }
}

extern "C" int oa_gated_rms_norm(void* stream, const void* o, const void* w, int wlen,
                                 const void* gate, int64_t gs, int gate_dt, int gate_act,
                                 void* out, int out_dt, int T, int N, int groups, float eps) {
    if (T <= 0 || N <= 0) return 0;
    if (groups < 1 || N % groups != 0 || (wlen != N && wlen != N / groups)) return -100;
    if (gate_dt != out_dt) return -101;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(T, groups == 1 ? 1 : CEIL_DIV(groups, 4));
    const int esz = out_dt == 1 ? 4 : 2;
    const bool vec = (N / groups) % 4 == 0 && (uintptr_t)o % 16 == 0 && (uintptr_t)w % 16 == 0 &&
                     (uintptr_t)gate % (4 * esz) == 0 && gs % 4 == 0 &&
                     (uintptr_t)out % (4 * esz) == 0;
#define GN_LAUNCH(TG, V)                                                                       \
    hipLaunchKernelGGL((gated_rms_norm_kernel<TG, TG, V>), grid, dim3(256), 0, s,               \
                       (const float*)o, (const float*)w, wlen, (const TG*)gate, gs, gate_act,   \
                       (TG*)out, N, groups, eps)
    if (out_dt == 1) {
        if (vec) GN_LAUNCH(float, true);
        else GN_LAUNCH(float, false);
    } else {
        if (vec) GN_LAUNCH(bf16s, true);
        else GN_LAUNCH(bf16s, false);
    }
#undef GN_LAUNCH
    HIP_CHECK_LAUNCH();
    return 0;
}
