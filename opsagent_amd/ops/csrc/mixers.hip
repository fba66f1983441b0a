// Sequence-mixer kernels for hybrid decoders on MI355X (gfx950): grouped RMS
// norm onto a float32 residual, causal short convolutions with carried
// inputs, softmax attention with a per-head linear distance penalty over
// the paged cache (separate key and value sizes, per-head output gate), and
// the gated delta rule with one decay per head and key channel.
//
// Every kernel works on a FLAT multi-sequence batch: T new tokens of B
// sequences laid end to end. cu[b]..cu[b+1] are sequence b's tokens, which
// continue it from position past[b]; slots[b] is its row in the state
// tensors; seq_of[t] is the sequence of token t. A prompt portion and a
// single decoded token are the same case with different counts.
//
// Precision: norms, softmax scores and weights, decays, gates, the
// recurrent state and the residual are float32 whatever the activation
// type is. Activations/weights are bf16 (dt = 0) or float32 (dt = 1).
//
// All sizes are run-time values; nothing assumes a multiple of 64.

#include "mixer_util.h"

// ---------------------------------------------------------------------------
// Causal convolution over time, per channel, continued from carried inputs.
//   y_t = sum_j w[c, j] * x_(t - taps + 1 + j)   (+ x_t) (-> silu)
// Inputs at positions < 0 are zero. state[slot, i, c] (float32) holds the
// input at position past - (taps-1) + i.
template <typename TI, typename TW, typename TO>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    const TI* __restrict__ x, int64_t xs, const TW* __restrict__ w,
    const float* __restrict__ state, TO* __restrict__ out, int64_t os,
    const int* __restrict__ seq_of, const int* __restrict__ cu,
    const int* __restrict__ past, const int* __restrict__ slots, int T, int C,
    int taps, int add_input, int act_silu) {
    const int64_t total = (int64_t)T * C;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int t = (int)(idx / C), c = (int)(idx % C);
        const int b = seq_of[t];
        const int lo = cu[b];
        const int local = t - lo;
        const int pos = past[b] + local;
        const float* st = state + (int64_t)slots[b] * (taps - 1) * C;
        float acc = 0.0f;
        for (int j = 0; j < taps; ++j) {
            const int d = j - (taps - 1);  // <= 0
            if (pos + d < 0) continue;
            const int s = local + d;
            float xv = (s >= 0) ? ldf(x, (int64_t)(lo + s) * xs + c)
                                : st[(int64_t)(taps - 1 + s) * C + c];
            acc += ldf(w, (int64_t)c * taps + j) * xv;
        }
        if (add_input) acc += ldf(x, (int64_t)t * xs + c);
        if (act_silu) acc = acc * sigmoidf_(acc);
        stf(out, (int64_t)t * os + c, acc);
    }
}

// The same with 8 channels per thread (C, row strides multiples of 8).
template <int TAPS, typename TI, typename TW, typename TO>
__global__ __launch_bounds__(256) void causal_conv_vec_kernel(
    const TI* __restrict__ x, int64_t xs, const TW* __restrict__ w,
    const float* __restrict__ state, TO* __restrict__ out, int64_t os,
    const int* __restrict__ seq_of, const int* __restrict__ cu,
    const int* __restrict__ past, const int* __restrict__ slots, int T, int C,
    int taps_rt, int add_input, int act_silu) {
    constexpr int taps = TAPS;
    const int C8 = C / 8;
    const int64_t total = (int64_t)T * C8;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int t = (int)(idx / C8), c = (int)(idx % C8) * 8;
        const int b = seq_of[t];
        const int lo = cu[b];
        const int local = t - lo;
        const int pos = past[b] + local;
        const float* st = state + (int64_t)slots[b] * (taps - 1) * C;
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        float xv[8];
        float wv[TAPS][8];   // the 8 channels' weights: 8*TAPS consecutive values
#pragma unroll
        for (int j = 0; j < TAPS; ++j) ld8(w, (int64_t)c * taps + 8 * j, wv[j]);
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {
            const int d = j - (taps - 1);
            if (pos + d < 0) continue;
            const int s = local + d;
            if (s >= 0) ld8(x, (int64_t)(lo + s) * xs + c, xv);
            else ld8(st, (int64_t)(taps - 1 + s) * C + c, xv);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += wv[(e * TAPS + j) / 8][(e * TAPS + j) % 8] * xv[e];
        }
        if (add_input) {
            ld8(x, (int64_t)t * xs + c, xv);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += xv[e];
        }
        if (act_silu) {
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = acc[e] * sigmoidf_(acc[e]);
        }
        st8(out, (int64_t)t * os + c, acc);
    }
}

// After the convolution: carry the last taps-1 inputs of every sequence.
// One thread per (sequence, channel) walks the entries in ascending order,
// so a shifted old entry is read before it is overwritten.
template <typename TI>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    const TI* __restrict__ x, int64_t xs, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ past,
    const int* __restrict__ slots, int B, int C, int taps) {
    const int64_t total = (int64_t)B * C;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int b = (int)(idx / C), c = (int)(idx % C);
        const int lo = cu[b], n = cu[b + 1] - lo;
        if (n <= 0) continue;
        const int p = past[b];
        float* st = state + (int64_t)slots[b] * (taps - 1) * C;
        for (int i = 0; i < taps - 1; ++i) {
            const int local = n - (taps - 1) + i;
            float v;
            if (local >= 0) v = ldf(x, (int64_t)(lo + local) * xs + c);
            else v = (p + local < 0) ? 0.0f : st[(int64_t)(i + n) * C + c];
            st[(int64_t)i * C + c] = v;
        }
    }
}

// Convolution and carry in ONE launch for steps whose portions are a few
// tokens (decoding): one thread per (sequence, channel) walks its tokens in
// order and then rewrites its own column of the carried inputs, so no other
// thread reads what it overwrites.
template <typename TI, typename TW, typename TO>
__global__ __launch_bounds__(256) void causal_conv_small_kernel(
    const TI* __restrict__ x, int64_t xs, const TW* __restrict__ w,
    float* __restrict__ state, TO* __restrict__ out, int64_t os,
    const int* __restrict__ cu, const int* __restrict__ past,
    const int* __restrict__ slots, int B, int C, int taps, int add_input,
    int act_silu) {
    const int64_t total = (int64_t)B * C;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int b = (int)(idx / C), c = (int)(idx % C);
        const int lo = cu[b], n = cu[b + 1] - lo;
        if (n <= 0) continue;
        const int p = past[b];
        float* st = state + (int64_t)slots[b] * (taps - 1) * C;
        for (int i = 0; i < n; ++i) {
            float acc = 0.0f;
            for (int j = 0; j < taps; ++j) {
                const int s = i + j - (taps - 1);
                if (p + s < 0) continue;
                const float xv = (s >= 0) ? ldf(x, (int64_t)(lo + s) * xs + c)
                                          : st[(int64_t)(taps - 1 + s) * C + c];
                acc += ldf(w, (int64_t)c * taps + j) * xv;
            }
            if (add_input) acc += ldf(x, (int64_t)(lo + i) * xs + c);
            if (act_silu) acc = acc * sigmoidf_(acc);
            stf(out, (int64_t)(lo + i) * os + c, acc);
        }
        for (int i = 0; i < taps - 1; ++i) {
            const int local = n - (taps - 1) + i;
            float v;
            if (local >= 0) v = ldf(x, (int64_t)(lo + local) * xs + c);
            else v = (p + local < 0) ? 0.0f : st[(int64_t)(i + n) * C + c];
            st[(int64_t)i * C + c] = v;
        }
    }
}

// ---------------------------------------------------------------------------
// RMS norm in `groups` consecutive parts, times w; one block per token, one
// wave per part. residual (float32, may be null) is updated in place:
// residual += norm(y) * w; `copy` (may be null) gets the result in the
// activation type.
template <typename TY, typename TW, typename TO>
__global__ __launch_bounds__(256) void group_rmsnorm_kernel(
    const TY* __restrict__ y, int64_t ys, const TW* __restrict__ w,
    float* __restrict__ residual, TO* __restrict__ copy, int C, int groups,
    float eps) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int gs = C / groups;
    for (int g = wave; g < groups; g += nw) {
        const int64_t base = (int64_t)t * ys + (int64_t)g * gs;
        float ss = 0.0f;
        for (int i = lane; i < gs; i += 64) {
            float v = ldf(y, base + i);
            ss += v * v;
        }
        ss = wave_reduce_sum(ss);
        const float r = 1.0f / sqrtf(ss / (float)gs + eps);
        for (int i = lane; i < gs; i += 64) {
            const int c = g * gs + i;
            float v = ldf(y, base + i) * r * ldf(w, c);
            if (residual) {
                v += residual[(int64_t)t * C + c];
                residual[(int64_t)t * C + c] = v;
            }
            if (copy) stf(copy, (int64_t)t * C + c, v);
        }
    }
}

// The same with 8 elements per lane and the part held in registers between
// the two passes (part size a multiple of 8, at most 64*8*GN_IT).
#define GN_IT 4
template <typename TY, typename TW, typename TO>
__global__ __launch_bounds__(256) void group_rmsnorm_vec_kernel(
    const TY* __restrict__ y, int64_t ys, const TW* __restrict__ w,
    float* __restrict__ residual, TO* __restrict__ copy, int C, int groups,
    float eps) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int gs = C / groups;
    for (int g = wave; g < groups; g += nw) {
        const int64_t base = (int64_t)t * ys + (int64_t)g * gs;
        float v[GN_IT][8];
        float ss = 0.0f;
#pragma unroll
        for (int it = 0; it < GN_IT; ++it) {
            const int i = (it * 64 + lane) * 8;
            if (i < gs) {
                ld8(y, base + i, v[it]);
#pragma unroll
                for (int e = 0; e < 8; ++e) ss += v[it][e] * v[it][e];
            }
        }
        ss = wave_reduce_sum(ss);
        const float r = 1.0f / sqrtf(ss / (float)gs + eps);
#pragma unroll
        for (int it = 0; it < GN_IT; ++it) {
            const int i = (it * 64 + lane) * 8;
            if (i < gs) {
                const int c = g * gs + i;
                float wv[8], rv[8];
                ld8(w, c, wv);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[it][e] = v[it][e] * r * wv[e];
                if (residual) {
                    ld8(residual, (int64_t)t * C + c, rv);
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[it][e] += rv[e];
                    st8(residual, (int64_t)t * C + c, v[it]);
                }
                if (copy) st8(copy, (int64_t)t * C + c, v[it]);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Attention input preparation, one block per token: the projection biases
// are added (bias over q | k | v columns, may be null), then weighted RMS
// norm over the WHOLE q projection and over the whole k projection and an
// unweighted RMS norm of each value head; q goes to q_out, k and v to their
// cache slot.
template <typename TC>
__global__ __launch_bounds__(256) void attn_prepare_kernel(
    const TC* __restrict__ qkv, int64_t qs, const TC* __restrict__ bias,
    const TC* __restrict__ qw, const TC* __restrict__ kw, TC* __restrict__ q_out,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int* __restrict__ slot_mapping, const int* __restrict__ cu, int B, int H,
    int G, int D, int Dv, float eps) {
    __shared__ float red[8];
    const int t = blockIdx.x;
    if (t >= cu[B]) return;  // padding row of a fixed-size (captured) launch
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const TC* row = qkv + (int64_t)t * qs;
    const int nq = H * D, nk = G * D;
    const int64_t slot = slot_mapping[t];
    auto val = [&](int i) { return ldf(row, i) + (bias ? ldf(bias, i) : 0.0f); };
    float sq = 0.0f, sk = 0.0f;
    for (int i = threadIdx.x; i < nq; i += blockDim.x) {
        float v = val(i);
        sq += v * v;
    }
    for (int i = threadIdx.x; i < nk; i += blockDim.x) {
        float v = val(nq + i);
        sk += v * v;
    }
    sq = wave_reduce_sum(sq);
    sk = wave_reduce_sum(sk);
    if (lane == 0) {
        red[wave] = sq;
        red[4 + wave] = sk;
    }
    __syncthreads();
    sq = 0.0f;
    sk = 0.0f;
    for (int i = 0; i < nw; ++i) {
        sq += red[i];
        sk += red[4 + i];
    }
    const float rq = 1.0f / sqrtf(sq / (float)nq + eps);
    const float rk = 1.0f / sqrtf(sk / (float)nk + eps);
    for (int i = threadIdx.x; i < nq; i += blockDim.x)
        stf(q_out, (int64_t)t * nq + i, val(i) * rq * ldf(qw, i));
    for (int i = threadIdx.x; i < nk; i += blockDim.x)
        stf(k_cache, slot * nk + i, val(nq + i) * rk * ldf(kw, i));
    for (int g = wave; g < G; g += nw) {
        const int off = nq + nk + g * Dv;
        float sv = 0.0f;
        for (int i = lane; i < Dv; i += 64) {
            float v = val(off + i);
            sv += v * v;
        }
        sv = wave_reduce_sum(sv);
        const float rv = 1.0f / sqrtf(sv / (float)Dv + eps);
        for (int i = lane; i < Dv; i += 64)
            stf(v_cache, slot * (int64_t)(G * Dv) + g * Dv + i, val(off + i) * rv);
    }
}

// The same with 8 elements per thread (all sizes and strides multiples of 8).
template <typename TC>
__global__ __launch_bounds__(256) void attn_prepare_vec_kernel(
    const TC* __restrict__ qkv, int64_t qs, const TC* __restrict__ bias,
    const TC* __restrict__ qw, const TC* __restrict__ kw, TC* __restrict__ q_out,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int* __restrict__ slot_mapping, const int* __restrict__ cu, int B, int H,
    int G, int D, int Dv, float eps) {
    __shared__ float red[8];
    const int t = blockIdx.x;
    if (t >= cu[B]) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const TC* row = qkv + (int64_t)t * qs;
    const int nq = H * D, nk = G * D;
    const int64_t slot = slot_mapping[t];
    auto val8 = [&](int i, float* o) {
        ld8(row, i, o);
        if (bias) {
            float bv[8];
            ld8(bias, i, bv);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] += bv[e];
        }
    };
    float sq = 0.0f, sk = 0.0f, x[8], wv[8];
    for (int i = threadIdx.x * 8; i < nq; i += blockDim.x * 8) {
        val8(i, x);
#pragma unroll
        for (int e = 0; e < 8; ++e) sq += x[e] * x[e];
    }
    for (int i = threadIdx.x * 8; i < nk; i += blockDim.x * 8) {
        val8(nq + i, x);
#pragma unroll
        for (int e = 0; e < 8; ++e) sk += x[e] * x[e];
    }
    sq = wave_reduce_sum(sq);
    sk = wave_reduce_sum(sk);
    if (lane == 0) {
        red[wave] = sq;
        red[4 + wave] = sk;
    }
    __syncthreads();
    sq = 0.0f;
    sk = 0.0f;
    for (int i = 0; i < nw; ++i) {
        sq += red[i];
        sk += red[4 + i];
    }
    const float rq = 1.0f / sqrtf(sq / (float)nq + eps);
    const float rk = 1.0f / sqrtf(sk / (float)nk + eps);
    for (int i = threadIdx.x * 8; i < nq; i += blockDim.x * 8) {
        val8(i, x);
        ld8(qw, i, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] *= rq * wv[e];
        st8(q_out, (int64_t)t * nq + i, x);
    }
    for (int i = threadIdx.x * 8; i < nk; i += blockDim.x * 8) {
        val8(nq + i, x);
        ld8(kw, i, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] *= rk * wv[e];
        st8(k_cache, slot * nk + i, x);
    }
    // value heads: 8 lanes... a 16-lane group per head pass keeps it simple:
    // each wave takes heads wave, wave+nw, ...; lanes take 8 channels each
    for (int g = wave; g < G; g += nw) {
        const int off = nq + nk + g * Dv;
        float sv = 0.0f;
        for (int i = lane * 8; i < Dv; i += 64 * 8) {
            val8(off + i, x);
#pragma unroll
            for (int e = 0; e < 8; ++e) sv += x[e] * x[e];
        }
        sv = wave_reduce_sum(sv);
        const float rv = 1.0f / sqrtf(sv / (float)Dv + eps);
        for (int i = lane * 8; i < Dv; i += 64 * 8) {
            val8(off + i, x);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] *= rv;
            st8(v_cache, slot * (int64_t)(G * Dv) + g * Dv + i, x);
        }
    }
}

// ---------------------------------------------------------------------------
// Softmax attention over the paged cache with optional parts, each switched
// by its argument:
//   score(i, j) = q_i . k_j * scale - slope_h * (i - j),  j <= i
//                 (slopes null: no distance penalty)
//   window > 0: only keys j > i - window are visible (the last `window`
//                 positions up to the query); key tiles that end before
//                 that range are never visited
//   softcap > 0: q_i . k_j * scale is replaced by softcap * tanh(that / softcap)
//   Gv value heads (Gv divides G): key head g reads value head g mod Gv
//   sinks given: Z_i,h = sum_j exp(score(i, j)) + exp(sink_h): the sink
//                 enlarges the normaliser only, contributes no value
//                 vector, and `scale` is not applied to it
//   out_i,h = (sigmoid(gate_i,h)) * sum_j softmax_j(score) v_j  (gate null: 1)
// grid = (query tiles, kv heads, key splits). A tile is up to TQ
// consecutive new tokens of ONE sequence with all R = H/G query heads of
// the kv head: ROWS = TQ*R rows share every staged key/value tile. Each of
// the 4 waves owns rows wave, wave+4, ...; in the score phase a lane is a
// key, in the value phase a lane is a value channel. Keys KT at a time go
// through LDS (K padded to an odd word stride).
// With nsplit > 1 a block covers every nsplit-th key tile and writes
// unnormalised partials (acc, m, l) that attn_combine_kernel merges.
#define ATT_MAXR 4   // rows per wave
#define ATT_MAXV 4   // value channels per lane (Dv <= 256)

template <typename TC>
__global__ __launch_bounds__(256) void attn_bias_paged_kernel(
    const TC* __restrict__ q, const TC* __restrict__ gate, int64_t gs,
    const TC* __restrict__ k_cache, const TC* __restrict__ v_cache,
    TC* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const int* __restrict__ cu, const int* __restrict__ past,
    const int* __restrict__ block_table, int max_blocks, int block_size,
    const float* __restrict__ slopes, const float* __restrict__ sinks, int B, int H, int G,
    int D, int Dv, int TQ, int KT, int kstride, float scale, int nsplit, int RB, int window,
    int64_t vrow, int Gv, float softcap) {
    extern __shared__ float lds[];
    // a block takes up to RB of the H/G query heads of one kv head
    const int hgroups = (H / G + RB - 1) / RB;
    const int g = blockIdx.y / hgroups;
    const int h0 = g * (H / G) + (blockIdx.y % hgroups) * RB;
    const int R = min(RB, (g + 1) * (H / G) - h0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int split = blockIdx.z;
    // locate this block's tile: walk the sequences
    int tile = blockIdx.x, b = 0, lo = 0, n = 0;
    for (; b < B; ++b) {
        lo = cu[b];
        n = cu[b + 1] - lo;
        const int nt = (n + TQ - 1) / TQ;
        if (tile < nt) break;
        tile -= nt;
    }
    if (b >= B) return;
    const int t0 = tile * TQ;                       // local offset in the portion
    const int nq_tok = min(TQ, n - t0);
    const int rows = nq_tok * R;
    const int p0 = past[b] + t0;                    // position of the first query
    const int last_pos = p0 + nq_tok - 1;
    const int* bt = block_table + (int64_t)b * max_blocks;

    float* Qs = lds;                                // [TQ*RB][D]
    float* Ps = Qs + (size_t)TQ * RB * D;           // [4][KT]
    TC* Ks = (TC*)(Ps + 4 * KT);                    // [KT][kstride]
    TC* Vs = Ks + (size_t)KT * kstride;             // [KT][Dv]

    for (int i = threadIdx.x; i < rows * D; i += blockDim.x) {
        const int r = i / D, d = i % D;
        const int tok = lo + t0 + r / R, h = h0 + r % R;
        Qs[i] = ldf(q, ((int64_t)tok * H + h) * D + d) * scale;
    }
    float m[ATT_MAXR], l[ATT_MAXR], acc[ATT_MAXR][ATT_MAXV];
#pragma unroll
    for (int i = 0; i < ATT_MAXR; ++i) {
        m[i] = -INFINITY;
        l[i] = 0.0f;
#pragma unroll
        for (int c = 0; c < ATT_MAXV; ++c) acc[i][c] = 0.0f;
    }
    const int nkt = last_pos / KT + 1;
    // the first key any query of the tile sees
    const int kt_first = window > 0 ? max(0, p0 - window + 1) / KT : 0;
    for (int kt = kt_first + split; kt < nkt; kt += nsplit) {
        const int k0 = kt * KT;
        const int nk = min(KT, last_pos + 1 - k0);
        __syncthreads();
        for (int i = threadIdx.x; i < nk * D; i += blockDim.x) {
            const int j = i / D, d = i % D;
            const int key = k0 + j;
            const int64_t slot = (int64_t)bt[key / block_size] * block_size + key % block_size;
            Ks[j * kstride + d] = k_cache[(slot * G + g) * D + d];
        }
        for (int i = threadIdx.x; i < nk * Dv; i += blockDim.x) {
            const int j = i / Dv, d = i % Dv;
            const int key = k0 + j;
            const int64_t slot = (int64_t)bt[key / block_size] * block_size + key % block_size;
            Vs[j * Dv + d] = v_cache[slot * vrow + (g % Gv) * Dv + d];
        }
        __syncthreads();
#pragma unroll
        for (int ri = 0; ri < ATT_MAXR; ++ri) {
            const int r = wave + 4 * ri;
            if (r >= rows) break;
            const int pos = p0 + r / R;
            const int kmin = window > 0 ? pos - window + 1 : 0;   // first key seen
            if (k0 > pos || k0 + nk <= kmin) continue;
            const float slope = slopes ? slopes[h0 + r % R] : 0.0f;
            float s = -INFINITY;
            if (lane < nk && k0 + lane <= pos && k0 + lane >= kmin) {
                const float* qr = Qs + r * D;
                const TC* kr = Ks + lane * kstride;
                float a = 0.0f;
                for (int d = 0; d < D; ++d) a += qr[d] * ldf(kr, d);
                if (softcap > 0.0f) a = softcap * tanhf(a / softcap);
                s = a - slope * (float)(pos - (k0 + lane));
            }
            const float mx = fmaxf(m[ri], wave_reduce_max(s));
            const float p = (s == -INFINITY) ? 0.0f : expf(s - mx);
            const float corr = (m[ri] == -INFINITY) ? 0.0f : expf(m[ri] - mx);
            l[ri] = l[ri] * corr + wave_reduce_sum(p);
            m[ri] = mx;
            if (lane < KT) Ps[wave * KT + lane] = p;
            // a wave's lanes run in lockstep; LDS writes of this wave are
            // visible to it after the wait below
            __builtin_amdgcn_s_waitcnt(0xc07f);
            __builtin_amdgcn_wave_barrier();
            const int jmax = min(nk, pos - k0 + 1);
#pragma unroll
            for (int c = 0; c < ATT_MAXV; ++c) {
                const int ch = lane + 64 * c;
                float a = acc[ri][c] * corr;
                if (ch < Dv)
                    for (int j = 0; j < jmax; ++j) a += Ps[wave * KT + j] * ldf(Vs, j * Dv + ch);
                acc[ri][c] = a;
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
#pragma unroll
    for (int ri = 0; ri < ATT_MAXR; ++ri) {
        const int r = wave + 4 * ri;
        if (r >= rows) break;
        const int tok = lo + t0 + r / R, h = h0 + r % R;
        if (nsplit == 1) {
            const float gt = gate ? sigmoidf_(ldf(gate, (int64_t)tok * gs + h)) : 1.0f;
            const float lt = sinks ? l[ri] + expf(sinks[h] - m[ri]) : l[ri];
            const float inv = gt / lt;
#pragma unroll
            for (int c = 0; c < ATT_MAXV; ++c) {
                const int ch = lane + 64 * c;
                if (ch < Dv) stf(out, ((int64_t)tok * H + h) * Dv + ch, acc[ri][c] * inv);
            }
        } else {
            const int64_t pr = ((int64_t)tok * H + h) * nsplit + split;
#pragma unroll
            for (int c = 0; c < ATT_MAXV; ++c) {
                const int ch = lane + 64 * c;
                if (ch < Dv) part_o[pr * Dv + ch] = acc[ri][c];
            }
            if (lane == 0) {
                part_ml[pr * 2] = m[ri];
                part_ml[pr * 2 + 1] = l[ri];
            }
        }
    }
}

// ---------------------------------------------------------------------------
// The same attention on the matrix cores (bf16 activations, key and value
// sizes multiples of 16). Each wave owns 16 consecutive new tokens of one
// query head; the 4 waves of a block are HB heads of one kv head times 4/HB
// token sub-tiles, and share the staged key/value tiles.
//
// Swapped products keep everything in registers: S^T = K Q^T puts a token in
// a lane's column (lane & 15), so the online-softmax statistics are per-lane
// scalars, and S^T's accumulator layout IS the B-operand layout of
// O^T = V^T P^T. v_mfma_f32_16x16x16_bf16: A[i][k]: lane holds i = lane&15,
// k = 4*(lane>>4)..+3; B[k][j]: j = lane&15, same k; C[i][j]: j = lane&15,
// i = 4*(lane>>4)..+3.
// Scores, the distance penalty, softmax statistics and weights are float32;
// a weight enters the value product as a bf16 pair hi + lo (two MFMAs), so
// it keeps 16 bits of mantissa.
// LDS: K tile [64][D+8], V tile transposed [Dv][64+4] (bf16).
// Where the key size divides by 32 (QK32) and always for the value product,
// the gfx950 form v_mfma_f32_16x16x32_bf16 is used: same i/j mapping, a lane
// holds k = 8*(lane>>4)..+7. The value product feeds it the weights a lane
// already holds (keys 16*mt + 4*(lane>>4) + r of two adjacent 16-key tiles)
// and reads V^T at the same keys, so no lane exchange is needed: the sum
// over k does not care about the order of the keys.
typedef short s4_t __attribute__((ext_vector_type(4)));
typedef short s8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
#define MF_KT 64
#define MF_KPAD 8

template <int MAXD, int MAXDV, bool QK32, int NT>
__global__ __launch_bounds__(256) void attn_bias_mfma_kernel(
    const bf16s* __restrict__ q, const bf16s* __restrict__ gate, int64_t gs,
    const bf16s* __restrict__ k_cache, const bf16s* __restrict__ v_cache,
    bf16s* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const int* __restrict__ cu, const int* __restrict__ past,
    const int* __restrict__ block_table, int max_blocks, int block_size,
    const float* __restrict__ slopes, const float* __restrict__ sinks, int B, int H, int G,
    int D, int Dv, int HB, float scale, int nsplit, int window, int vrow, int hrows, int Gv,
    float softcap) {
    // hrows (decode steps of many query heads per kv head): a step brings one
    // token per sequence, so the 16 columns of a wave's tile are 16 HEADS at
    // that token's position instead of 16 tokens of one head; a block covers
    // 64 heads of one kv head and every staged key/value tile serves them
    // all. The head (and with it slope, sink, gate and output row) is then a
    // per-lane value.
    // NT: 16-token sub-tiles per wave. Every K and V fragment read from LDS
    // feeds NT MFMAs, and a staged tile serves NT times the query rows.
    extern __shared__ float lds[];
    bf16s* Ks = (bf16s*)lds;                        // [64][D+8]
    const int kst = D + MF_KPAD;
    bf16s* Vt = Ks + (size_t)MF_KT * kst;           // [Dv][68]
    const int vst = MF_KT + 4;
    const int R = H / G;
    const int TT = 4 / HB, TQ = 16 * TT * NT;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lc = lane & 15, lg = lane >> 4;
    const int hgroups = hrows ? (R + 63) / 64 : R / HB;
    const int g = blockIdx.y / hgroups;
    const int hoff = (blockIdx.y % hgroups) * 64 + wave * 16;      // hrows: the wave's first head
    const int h = hrows ? g * R + min(hoff + lc, R - 1)
                        : g * R + (blockIdx.y % hgroups) * HB + wave % HB;
    const int hvalid = max(0, min(16, R - hoff));                  // hrows: heads in this wave
    const int split = blockIdx.z;
    int tile = blockIdx.x, b = 0, lo = 0, n = 0;
    for (; b < B; ++b) {
        lo = cu[b];
        n = cu[b + 1] - lo;
        const int nt = (n + TQ - 1) / TQ;
        if (tile < nt) break;
        tile -= nt;
    }
    if (b >= B) return;
    const int pb = past[b];
    const int t0 = hrows ? 0 : tile * TQ + (wave / HB) * 16 * NT;   // this wave's first local token
    int ntok[NT], pos[NT];
#pragma unroll
    for (int u = 0; u < NT; ++u) {
        ntok[u] = max(0, min(16, n - (t0 + 16 * u)));
        pos[u] = pb + t0 + 16 * u + lc;                  // this lane's token position
        if (hrows) {
            ntok[u] = (u == 0 && n > 0) ? hvalid : 0;    // valid columns = valid heads
            pos[u] = pb;
        }
    }
    const int wave_ntok = hrows ? ((n > 0 && hvalid > 0) ? 1 : 0) : max(0, min(16 * NT, n - t0));
    const int wave_last = pb + t0 + wave_ntok - 1;
    const int block_last = pb + min(n, tile * TQ + TQ) - 1;
    const int* bt = block_table + (int64_t)b * max_blocks;
    // softmax in the exp2 domain: log2(e) folded into the scale and the slope
    const float LOG2E = 1.4426950408889634f;
    const float slope = slopes ? slopes[h] * LOG2E : 0.0f;
    const float scale2 = scale * LOG2E;
    // soft cap: cap * tanh(s / cap) = cap - 2 cap / (exp(2 s / cap) + 1), here
    // with s = raw * scale and the result in the exp2 domain
    const float cap_in = softcap > 0.0f ? 2.0f * scale * LOG2E / softcap : 0.0f;
    const float cap_out = softcap * LOG2E;
    // window as a bound that no position reaches when there is none
    const int wlim = window > 0 ? window : 0x7fffffff;

    s4_t qf[NT][QK32 ? 1 : MAXD];
    s8_t qf8[NT][QK32 ? MAXD / 2 : 1];
#pragma unroll
    for (int u = 0; u < NT; ++u) {
        const int tk = hrows ? lo : lo + t0 + 16 * u + min(lc, max(ntok[u] - 1, 0));
        const bf16s* qr = q + ((int64_t)min(tk, lo + n - 1) * H + h) * D;
        if (QK32) {
#pragma unroll
            for (int ks = 0; ks < MAXD / 2; ++ks) {
                if (32 * ks < D && ntok[u] > 0)
                    qf8[u][ks] = *reinterpret_cast<const s8_t*>(qr + 32 * ks + 8 * lg);
                else qf8[u][ks] = s8_t{0, 0, 0, 0, 0, 0, 0, 0};
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < MAXD; ++ks) {
                if (16 * ks < D && ntok[u] > 0)
                    qf[u][ks] = *reinterpret_cast<const s4_t*>(qr + 16 * ks + 4 * lg);
                else qf[u][ks] = s4_t{0, 0, 0, 0};
            }
        }
    }
    float kbias[4][4];                       // slope * (16*mt + r), exp2 domain
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) kbias[mt][r] = slope * (float)(16 * mt + r);
    f4_t o[NT][MAXDV];
    float m[NT], l[NT];
#pragma unroll
    for (int u = 0; u < NT; ++u) {
        m[u] = -INFINITY;
        l[u] = 0.0f;
#pragma unroll
        for (int i = 0; i < MAXDV; ++i) o[u][i] = f4_t{0.f, 0.f, 0.f, 0.f};
    }

    const int nkt = block_last / MF_KT + 1;
    const int dch = D / 8, vch = Dv / 8;
    // pages are a power of two: shifts, not divisions
    const int bsh = 31 - __clz(block_size), bmask = block_size - 1;
    // Staging map: a thread owns ONE key per tile for K (key tid/4, every 4th
    // 16-byte piece of its row) and one for V (key tid%64, every 4th piece),
    // so a tile costs it two page lookups. The next tile's pieces are loaded
    // into registers while the current tile is computed.
    constexpr int KC = MAXD / 2, VC = MAXDV / 2;
    const int kj = threadIdx.x >> 2, kc0 = threadIdx.x & 3;
    const int vj = threadIdx.x & 63, vc0 = threadIdx.x >> 6;
    uint4 kreg[KC], vreg[VC];
    auto fetch = [&](int kt) {
        const int k0 = kt * MF_KT;
        const int nk = min(MF_KT, block_last + 1 - k0);
        const int keyk = k0 + kj, keyv = k0 + vj;
        const bool okk = kj < nk, okv = vj < nk;
        const int64_t sk_ = okk ? ((int64_t)bt[keyk >> bsh] << bsh) + (keyk & bmask) : 0;
        const int64_t sv_ = okv ? ((int64_t)bt[keyv >> bsh] << bsh) + (keyv & bmask) : 0;
        const bf16s* kp = k_cache + (sk_ * G + g) * D;
        const bf16s* vp = v_cache + (sv_ * vrow + (g % Gv) * Dv);
#pragma unroll
        for (int u = 0; u < KC; ++u) {
            const int c = kc0 + 4 * u;
            kreg[u] = (okk && c < dch) ? *reinterpret_cast<const uint4*>(kp + 8 * c)
                                       : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < VC; ++u) {
            const int c = vc0 + 4 * u;
            vreg[u] = (okv && c < vch) ? *reinterpret_cast<const uint4*>(vp + 8 * c)
                                       : make_uint4(0, 0, 0, 0);
        }
    };
    // key tiles before the window of the block's first query are skipped
    const int kt_first = window > 0 ? max(0, pb + tile * TQ - window + 1) / MF_KT : 0;
    if (kt_first + split < nkt) fetch(kt_first + split);
    for (int kt = kt_first + split; kt < nkt; kt += nsplit) {
        const int k0 = kt * MF_KT;
        __syncthreads();
#pragma unroll
        for (int u = 0; u < KC; ++u) {
            const int c = kc0 + 4 * u;
            if (c < dch) *reinterpret_cast<uint4*>(Ks + kj * kst + 8 * c) = kreg[u];
        }
#pragma unroll
        for (int u = 0; u < VC; ++u) {
            const int c = vc0 + 4 * u;
            if (c < vch) {
                const uint32_t w[4] = {vreg[u].x, vreg[u].y, vreg[u].z, vreg[u].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    Vt[(8 * c + 2 * e) * vst + vj] = (bf16s)(w[e] & 0xffffu);
                    Vt[(8 * c + 2 * e + 1) * vst + vj] = (bf16s)(w[e] >> 16);
                }
            }
        }
        __syncthreads();
        if (kt + nsplit < nkt) fetch(kt + nsplit);
        if (wave_ntok <= 0 || k0 > wave_last || k0 + MF_KT - 1 <= pb + t0 - wlim) continue;
        // S^T tiles: keys k0 + 16*mt + 4*lg + r, token lc of sub-tile u
        f4_t sc[NT][4];
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
            for (int u = 0; u < NT; ++u) sc[u][mt] = f4_t{0.f, 0.f, 0.f, 0.f};
            const bf16s* kr = Ks + (16 * mt + lc) * kst;
            if (QK32) {
#pragma unroll
                for (int ks = 0; ks < MAXD / 2; ++ks)
                    if (32 * ks < D) {
                        const s8_t kf = *reinterpret_cast<const s8_t*>(kr + 32 * ks + 8 * lg);
#pragma unroll
                        for (int u = 0; u < NT; ++u)
                            sc[u][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf8[u][ks],
                                                                               sc[u][mt], 0, 0, 0);
                    }
            } else {
#pragma unroll
                for (int ks = 0; ks < MAXD; ++ks)
                    if (16 * ks < D) {
                        const s4_t kf = *reinterpret_cast<const s4_t*>(kr + 16 * ks + 4 * lg);
#pragma unroll
                        for (int u = 0; u < NT; ++u)
                            sc[u][mt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kf, qf[u][ks],
                                                                                 sc[u][mt], 0, 0, 0);
                    }
            }
        }
        s4_t phi[NT][4], plo[NT][4];
        float corr[NT];
#pragma unroll
        for (int u = 0; u < NT; ++u) {
            // score = s*scale2 - slope*(pos - key), key = k0 + 16*mt + 4*lg + r:
            // the key part is a per-lane constant table, the rest one value
            // per tile, so an element costs one add and one fma
            const float base = slope * (float)(pos[u] - k0 - 4 * lg);
            float mloc = -INFINITY;
            // only tiles that reach past some token of the wave need the mask
            // (past the diagonal, or short of the window of the sub-tile's last token)
            const bool diag = k0 + MF_KT - 1 > pb + t0 + 16 * u ||
                              k0 <= pb + t0 + 16 * u + 15 - wlim;
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v;
                    if (softcap > 0.0f) {
                        const float e2 = __builtin_amdgcn_exp2f(sc[u][mt][r] * cap_in);
                        v = cap_out - 2.0f * cap_out * __builtin_amdgcn_rcpf(e2 + 1.0f)
                            + (kbias[mt][r] - base);
                    } else {
                        v = fmaf(sc[u][mt][r], scale2, kbias[mt][r] - base);
                    }
                    if (diag) {
                        const int key = k0 + 16 * mt + 4 * lg + r;
                        v = (key <= pos[u] && key > pos[u] - wlim) ? v : -INFINITY;
                    }
                    sc[u][mt][r] = v;
                    mloc = fmaxf(mloc, v);
                }
            mloc = fmaxf(mloc, __shfl_xor(mloc, 16, WAVE));
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32, WAVE));
            const float mnew = fmaxf(m[u], mloc);
            // v_exp_f32 gives 0 for -inf, so masked keys need no select; only a
            // row that has seen no key yet (m = mnew = -inf) must be kept off NaN
            const float msub = (mnew == -INFINITY) ? 0.0f : mnew;
            corr[u] = __builtin_amdgcn_exp2f(m[u] - msub);
            float lsum = 0.0f;
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = __builtin_amdgcn_exp2f(sc[u][mt][r] - msub);
                    lsum += p;
                    // p = hi + lo + (less than 2^-16 p): both halves by
                    // truncation, so the first remainder is exact
                    const uint32_t pu = __float_as_uint(p);
                    phi[u][mt][r] = (short)(pu >> 16);
                    const float rem = p - __uint_as_float(pu & 0xffff0000u);
                    plo[u][mt][r] = (short)(__float_as_uint(rem) >> 16);
                }
            lsum += __shfl_xor(lsum, 16, WAVE);
            lsum += __shfl_xor(lsum, 32, WAVE);
            l[u] = l[u] * corr[u] + lsum;
            m[u] = mnew;
        }
#pragma unroll
        for (int dt = 0; dt < MAXDV; ++dt) {
            if (16 * dt < Dv) {
#pragma unroll
                for (int u = 0; u < NT; ++u) o[u][dt] *= corr[u];
                const bf16s* vr = Vt + (16 * dt + lc) * vst + 4 * lg;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    const s4_t a0 = *reinterpret_cast<const s4_t*>(vr + 32 * kb);
                    const s4_t a1 = *reinterpret_cast<const s4_t*>(vr + 32 * kb + 16);
                    const s8_t a = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                    for (int u = 0; u < NT; ++u) {
                        const s8_t bh = __builtin_shufflevector(phi[u][2 * kb], phi[u][2 * kb + 1],
                                                                0, 1, 2, 3, 4, 5, 6, 7);
                        const s8_t bl = __builtin_shufflevector(plo[u][2 * kb], plo[u][2 * kb + 1],
                                                                0, 1, 2, 3, 4, 5, 6, 7);
                        o[u][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bh, o[u][dt], 0, 0, 0);
                        o[u][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bl, o[u][dt], 0, 0, 0);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int u = 0; u < NT; ++u) {
        if (lc >= ntok[u]) continue;
        const int tok = hrows ? lo : lo + t0 + 16 * u + lc;
        if (nsplit == 1) {
            const float lt = sinks ? l[u] + __builtin_amdgcn_exp2f(sinks[h] * LOG2E - m[u]) : l[u];
            const float gt = (gate ? sigmoidf_(ldf(gate, (int64_t)tok * gs + h)) : 1.0f) / lt;
            bf16s* orow = out + ((int64_t)tok * H + h) * Dv + 4 * lg;
#pragma unroll
            for (int dt = 0; dt < MAXDV; ++dt)
                if (16 * dt < Dv) {
                    uint2 w;
                    w.x = pack_bf16x2(o[u][dt][0] * gt, o[u][dt][1] * gt);
                    w.y = pack_bf16x2(o[u][dt][2] * gt, o[u][dt][3] * gt);
                    *reinterpret_cast<uint2*>(orow + 16 * dt) = w;
                }
        } else {
            const int64_t pr = ((int64_t)tok * H + h) * nsplit + split;
#pragma unroll
            for (int dt = 0; dt < MAXDV; ++dt)
                if (16 * dt < Dv)
                    *reinterpret_cast<f4_t*>(part_o + pr * Dv + 16 * dt + 4 * lg) = o[u][dt];
            if (lg == 0) {
                part_ml[pr * 2] = m[u] * 0.6931471805599453f;   // back to the natural-log domain
                part_ml[pr * 2 + 1] = l[u];
            }
        }
    }
}

// merge key-split partials: one wave per (token, head); lanes first take
// one split each for the statistics, then one value channel each
template <typename TC>
__global__ __launch_bounds__(64) void attn_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const TC* __restrict__ gate, int64_t gs, const float* __restrict__ sinks,
    TC* __restrict__ out, int H, int Dv, int nsplit) {
    __shared__ float wsh[64];
    const int64_t row = blockIdx.x;  // tok * H + h
    const int tok = (int)(row / H), h = (int)(row % H);
    const int lane = threadIdx.x;
    float mx = -INFINITY, lsum = 0.0f;
    for (int s0 = 0; s0 < nsplit; s0 += 64) {          // running merge over groups of 64 splits
        const int s = s0 + lane;
        const float ms = s < nsplit ? part_ml[(row * nsplit + s) * 2] : -INFINITY;
        const float ls = s < nsplit ? part_ml[(row * nsplit + s) * 2 + 1] : 0.0f;
        const float gmx = fmaxf(mx, wave_reduce_max(ms));
        const float wgt = (ms == -INFINITY) ? 0.0f : expf(ms - gmx);
        lsum = lsum * ((mx == -INFINITY) ? 0.0f : expf(mx - gmx)) + wave_reduce_sum(ls * wgt);
        mx = gmx;
    }
    if (sinks) lsum += expf(sinks[h] - mx);
    const float gt = (gate ? sigmoidf_(ldf(gate, (int64_t)tok * gs + h)) : 1.0f) / lsum;
    float acc[ATT_MAXV];
#pragma unroll
    for (int c = 0; c < ATT_MAXV; ++c) acc[c] = 0.0f;
    for (int s0 = 0; s0 < nsplit; s0 += 64) {
        const int s = s0 + lane;
        const float ms = s < nsplit ? part_ml[(row * nsplit + s) * 2] : -INFINITY;
        __syncthreads();
        wsh[lane] = (ms == -INFINITY) ? 0.0f : expf(ms - mx);
        __syncthreads();
        const int ns = min(64, nsplit - s0);
#pragma unroll 4
        for (int j = 0; j < ns; ++j) {
            const float wj = wsh[j];
            const float* po = part_o + (row * nsplit + s0 + j) * Dv;
#pragma unroll
            for (int c = 0; c < ATT_MAXV; ++c) {
                const int ch = lane + 64 * c;
                if (ch < Dv) acc[c] += po[ch] * wj;
            }
        }
    }
#pragma unroll
    for (int c = 0; c < ATT_MAXV; ++c) {
        const int ch = lane + 64 * c;
        if (ch < Dv) stf(out, row * Dv + ch, acc[c] * gt);
    }
}

// ---------------------------------------------------------------------------
// Gated delta rule with one decay per head and key channel, fused from the
// convolved q/k/v to the gated, normed read-out. grid = (sequences, heads).
// Lane = (row group, column): the 16 lanes of a DPP row split the D key rows
// of one value column (RPL consecutive rows each), a wave holds 4 columns
// per pass and P passes, a block all Dv columns of the head. S stays in
// registers over the whole portion; between steps it lives in float32 in
// the state slot as [H, Dv, D] (a column's rows contiguous). A sequence that
// starts at position 0 starts from zero whatever the slot holds.
// Per chunk of TCK tokens the block
//   1. stages q, k (raw), decay = exp(-exp(A_log) softplus(a + dt_bias)),
//      v and beta = sigmoid(b) in LDS as float32 (rows past D as zero),
//   2. makes q and k unit vectors (q also times D^-1/2), a wave per token,
//   3. runs the recurrence, every wave on its own columns:
//        S <- decay * S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//      (the two column sums are DPP adds inside a 16-lane row),
//   4. RMS-norms o over the head's value columns, times w, times
//      sigmoid(gate), a wave per token, and stores it.
__device__ __forceinline__ float row16_sum(float x) {
    // all-reduce over the 16 lanes of a DPP row: quad swaps, then mirrors
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xF, 0xF, true));
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xF, 0xF, true));
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xF, 0xF, true));
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xF, 0xF, true));
    return x;
}

template <int RPL, int P, typename TC>
__global__ void delta_fused_kernel(
    const TC* __restrict__ q, int64_t qs, const TC* __restrict__ k, int64_t ks,
    const TC* __restrict__ v, int64_t vs, const TC* __restrict__ bl, int64_t bs,
    const TC* __restrict__ a, int64_t as, const TC* __restrict__ dt_bias,
    const TC* __restrict__ a_log, const TC* __restrict__ norm_w,
    const TC* __restrict__ gate, int64_t gs, float* __restrict__ state,
    TC* __restrict__ out, float* __restrict__ o_raw, const int* __restrict__ cu,
    const int* __restrict__ past, const int* __restrict__ slots, int H, int G, int D,
    int Dv, int TCK, float eps) {
    constexpr int DP = RPL * 16;  // padded key size
    extern __shared__ float lds[];
    float* sq = lds;
    float* sk = sq + TCK * DP;
    float* sg = sk + TCK * DP;
    float* sv = sg + TCK * DP;
    float* so = sv + TCK * Dv;
    float* sb = so + TCK * Dv;
    const int b = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, nth = blockDim.x;
    const int lane = tid & 63, wave = tid >> 6, nw = nth >> 6;
    const int rg = lane & 15, cs = lane >> 4;
    const int lo = cu[b], n = cu[b + 1] - lo;
    if (n <= 0) return;
    const int kvh = h / (H / G);
    float* st = state + (((int64_t)slots[b] * H + h) * Dv) * D;
    const float A = expf(ldf(a_log, h));
    const float qscale = 1.0f / sqrtf((float)D);
    float S[P][RPL];
    int col[P];
    const bool fresh = past[b] == 0;
    const bool vec4 = (D & 3) == 0;   // a lane's rows of a column are 16-byte pieces
    // gridDim.z > 1: the head's value columns are split over blocks (few
    // (sequence, head) pairs, long portions); the read-out then goes to
    // o_raw and the head norm runs as its own launch
    const int cpb = Dv / gridDim.z, cb = blockIdx.z * cpb, cend = cb + cpb;
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
        // four pieces per thread and pass: all loads are issued before any
        // of the softplus/exp chains, so their latencies overlap
        for (int i0 = tid; i0 < nc * DP; i0 += 4 * nth) {
            float qv[4], kv[4], zv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = i0 + u * nth;
                const int tt = i / DP, r = i % DP;
                const int64_t t = tb + tt;
                qv[u] = kv[u] = zv[u] = 0.0f;
                if (i < nc * DP && r < D) {
                    qv[u] = ldf(q, t * qs + kvh * D + r);
                    kv[u] = ldf(k, t * ks + kvh * D + r);
                    zv[u] = ldf(a, t * as + h * D + r) + ldf(dt_bias, h * D + r);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = i0 + u * nth;
                if (i < nc * DP) {
                    sq[i] = qv[u];
                    sk[i] = kv[u];
                    sg[i] = (i % DP < D) ? expf(-A * softplusf_(zv[u])) : 0.0f;
                }
            }
        }
        // only this block's share of the value columns is read
        for (int i = tid; i < nc * cpb; i += nth) {
            const int tt = i / cpb, c = cb + i % cpb;
            sv[tt * Dv + c] = ldf(v, (int64_t)(tb + tt) * vs + h * Dv + c);
        }
        for (int tt = tid; tt < nc; tt += nth)
            sb[tt] = sigmoidf_(ldf(bl, (int64_t)(tb + tt) * bs + h));
        __syncthreads();
        for (int tt = wave; tt < nc; tt += nw) {
            float ssq = 0.0f, ssk = 0.0f;
            for (int i = lane; i < DP; i += 64) {
                const float x = sq[tt * DP + i], y = sk[tt * DP + i];
                ssq += x * x;
                ssk += y * y;
            }
            ssq = wave_reduce_sum(ssq);
            ssk = wave_reduce_sum(ssk);
            const float rq = qscale / sqrtf(ssq + 1e-6f), rk = 1.0f / sqrtf(ssk + 1e-6f);
            for (int i = lane; i < DP; i += 64) {
                sq[tt * DP + i] *= rq;
                sk[tt * DP + i] *= rk;
            }
        }
        __syncthreads();
        for (int tt = 0; tt < nc; ++tt) {
            const float bt = sb[tt];
            float kr[RPL], gr[RPL], qr[RPL];
#pragma unroll
            for (int i = 0; i < RPL; ++i) {
                kr[i] = sk[tt * DP + rg * RPL + i];
                gr[i] = sg[tt * DP + rg * RPL + i];
                qr[i] = sq[tt * DP + rg * RPL + i];
            }
            float dot[P], o[P];
#pragma unroll
            for (int p = 0; p < P; ++p) {
                dot[p] = 0.0f;
#pragma unroll
                for (int i = 0; i < RPL; ++i) {
                    S[p][i] *= gr[i];
                    dot[p] += S[p][i] * kr[i];
                }
            }
#pragma unroll
            for (int p = 0; p < P; ++p) dot[p] = row16_sum(dot[p]);
#pragma unroll
            for (int p = 0; p < P; ++p) {
                const float vv = col[p] < Dv ? sv[tt * Dv + col[p]] : 0.0f;
                const float u = bt * (vv - dot[p]);
                o[p] = 0.0f;
#pragma unroll
                for (int i = 0; i < RPL; ++i) {
                    S[p][i] += kr[i] * u;
                    o[p] += S[p][i] * qr[i];
                }
            }
#pragma unroll
            for (int p = 0; p < P; ++p) {
                o[p] = row16_sum(o[p]);
                if (rg == 0 && col[p] < Dv) so[tt * Dv + col[p]] = o[p];
            }
        }
        __syncthreads();
        if (gridDim.z > 1) {
            for (int i = tid; i < nc * cpb; i += nth) {
                const int tt = i / cpb, c = cb + i % cpb;
                o_raw[((int64_t)(tb + tt) * H + h) * Dv + c] = so[tt * Dv + c];
            }
            __syncthreads();   // `so` is rewritten by the next chunk's recurrence
            continue;
        }
        for (int tt = wave; tt < nc; tt += nw) {
            float ss = 0.0f;
            for (int c = lane; c < Dv; c += 64) ss += so[tt * Dv + c] * so[tt * Dv + c];
            ss = wave_reduce_sum(ss);
            const float r = 1.0f / sqrtf(ss / (float)Dv + eps);
            const int64_t t = tb + tt;
            for (int c = lane; c < Dv; c += 64) {
                const float gt = sigmoidf_(ldf(gate, t * gs + h * Dv + c));
                stf(out, (t * H + h) * Dv + c, so[tt * Dv + c] * r * ldf(norm_w, c) * gt);
            }
        }
        // the next chunk's staging does not touch `so`, and its recurrence
        // (which does) comes two barriers later
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

// per-head RMS norm of a float32 read-out, times w[Dv], times sigmoid(gate):
// one block per token, one wave per head (used when the delta rule's columns
// were split over blocks)
template <typename TC>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(
    const float* __restrict__ o, const TC* __restrict__ w,
    const TC* __restrict__ gate, int64_t gs, TC* __restrict__ out, int H, int Dv,
    float eps) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    for (int h = wave; h < H; h += nw) {
        const float* src = o + ((int64_t)t * H + h) * Dv;
        float ss = 0.0f;
        for (int i = lane; i < Dv; i += 64) ss += src[i] * src[i];
        ss = wave_reduce_sum(ss);
        const float r = 1.0f / sqrtf(ss / (float)Dv + eps);
        for (int i = lane; i < Dv; i += 64) {
            const float gt = sigmoidf_(ldf(gate, (int64_t)t * gs + h * Dv + i));
            stf(out, ((int64_t)t * H + h) * Dv + i, src[i] * r * ldf(w, i) * gt);
        }
    }
}

// ---------------------------------------------------------------------------
// logits -> cap * tanh(logits / cap), float32 out
template <typename TC>
__global__ __launch_bounds__(256) void softcap_kernel(const TC* __restrict__ x,
                                                      float* __restrict__ out,
                                                      int64_t n, float cap) {
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x)
        out[i] = cap * tanhf(ldf(x, i) / cap);
}

// silu(gate) * up over rows of a [M, 2I] gate|up buffer (any float type)
template <typename TC>
__global__ __launch_bounds__(256) void silu_mul_rows_kernel(const TC* __restrict__ gu,
                                                            TC* __restrict__ out,
                                                            int64_t M, int I) {
    const int64_t total = M * I;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t m = idx / I;
        const int i = (int)(idx % I);
        const float g = ldf(gu, m * 2 * I + i), u = ldf(gu, m * 2 * I + I + i);
        stf(out, idx, g * sigmoidf_(g) * u);
    }
}

// float32 rows -> activation type (embedding rows gathered into the residual)
template <typename TC>
__global__ __launch_bounds__(256) void embed_rows_kernel(const TC* __restrict__ table,
                                                         const int64_t* __restrict__ ids,
                                                         float* __restrict__ out, int T,
                                                         int C, float scale) {
    const int64_t total = (int64_t)T * C;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int t = (int)(idx / C), c = (int)(idx % C);
        out[idx] = ldf(table, ids[t] * (int64_t)C + c) * scale;
    }
}

// ===========================================================================
// C entry points. dt: 0 = bf16 activations/weights, 1 = float32.

// x_dt: type of x (0 bf16, 1 f32); dt: type of w and out
extern "C" int oa_causal_conv_seq(void* stream, const void* x, int64_t xs, int x_dt,
                                  const void* w, void* state, void* out, int64_t os,
                                  const void* seq_of, const void* cu, const void* past,
                                  const void* slots, int T, int B, int C, int taps,
                                  int add_input, int act_silu, int dt, int max_chunk) {
    if (T <= 0) return 0;
    if (taps < 1) return -100;
    hipStream_t s = (hipStream_t)stream;
    dim3 g1(grid_for((int64_t)T * C)), g2(grid_for((int64_t)B * C)), blk(256);
    if (max_chunk >= 1 && max_chunk <= 4) {
#define CS_ARGS(TI, TW)                                                                      \
    (const TI*)x, xs, (const TW*)w, (float*)state, (TW*)out, os, (const int*)cu,             \
        (const int*)past, (const int*)slots, B, C, taps, add_input, act_silu
        if (x_dt == 1 && dt == 1)
            hipLaunchKernelGGL((causal_conv_small_kernel<float, float, float>), g2, blk, 0, s, CS_ARGS(float, float));
        else if (x_dt == 1 && dt == 0)
            hipLaunchKernelGGL((causal_conv_small_kernel<float, bf16s, bf16s>), g2, blk, 0, s, CS_ARGS(float, bf16s));
        else if (x_dt == 0 && dt == 0)
            hipLaunchKernelGGL((causal_conv_small_kernel<bf16s, bf16s, bf16s>), g2, blk, 0, s, CS_ARGS(bf16s, bf16s));
        else
            return -101;
#undef CS_ARGS
        HIP_CHECK_LAUNCH();
        return 0;
    }
#define CONV_ARGS(TI, TW)                                                          \
    (const TI*)x, xs, (const TW*)w, (const float*)state, (TW*)out, os,             \
        (const int*)seq_of, (const int*)cu, (const int*)past, (const int*)slots, T, \
        C, taps, add_input, act_silu
    const bool vec = C % 8 == 0 && xs % 8 == 0 && os % 8 == 0 && taps >= 2 && taps <= 4 &&
                     ((uintptr_t)x % 32 == 0) && ((uintptr_t)out % 16 == 0) &&
                     ((uintptr_t)w % 32 == 0);
    if (vec) {
        dim3 gv(grid_for((int64_t)T * (C / 8)));
#define CV(TP)                                                                                        \
    do {                                                                                              \
        if (x_dt == 1 && dt == 1)                                                                     \
            hipLaunchKernelGGL((causal_conv_vec_kernel<TP, float, float, float>), gv, blk, 0, s,      \
                               CONV_ARGS(float, float));                                              \
        else if (x_dt == 1 && dt == 0)                                                                \
            hipLaunchKernelGGL((causal_conv_vec_kernel<TP, float, bf16s, bf16s>), gv, blk, 0, s,      \
                               CONV_ARGS(float, bf16s));                                              \
        else if (x_dt == 0 && dt == 0)                                                                \
            hipLaunchKernelGGL((causal_conv_vec_kernel<TP, bf16s, bf16s, bf16s>), gv, blk, 0, s,      \
                               CONV_ARGS(bf16s, bf16s));                                              \
        else                                                                                          \
            return -101;                                                                              \
    } while (0)
        if (taps == 2) CV(2);
        else if (taps == 3) CV(3);
        else CV(4);
#undef CV
    } else if (x_dt == 1 && dt == 1)
        hipLaunchKernelGGL((causal_conv_kernel<float, float, float>), g1, blk, 0, s, CONV_ARGS(float, float));
    else if (x_dt == 1 && dt == 0)
        hipLaunchKernelGGL((causal_conv_kernel<float, bf16s, bf16s>), g1, blk, 0, s, CONV_ARGS(float, bf16s));
    else if (x_dt == 0 && dt == 0)
        hipLaunchKernelGGL((causal_conv_kernel<bf16s, bf16s, bf16s>), g1, blk, 0, s, CONV_ARGS(bf16s, bf16s));
    else
        return -101;
#undef CONV_ARGS
    HIP_CHECK_LAUNCH();
    if (taps > 1) {
        if (x_dt == 1)
            hipLaunchKernelGGL((conv_state_update_kernel<float>), g2, blk, 0, s, (const float*)x, xs,
                               (float*)state, (const int*)cu, (const int*)past, (const int*)slots, B, C, taps);
        else
            hipLaunchKernelGGL((conv_state_update_kernel<bf16s>), g2, blk, 0, s, (const bf16s*)x, xs,
                               (float*)state, (const int*)cu, (const int*)past, (const int*)slots, B, C, taps);
        HIP_CHECK_LAUNCH();
    }
    return 0;
}

// y_dt: type of y; dt: type of w and copy. residual/copy may be null (not both).
extern "C" int oa_group_rmsnorm(void* stream, const void* y, int64_t ys, int y_dt,
                                const void* w, void* residual, void* copy, int T, int C,
                                int groups, float eps, int dt) {
    if (T <= 0) return 0;
    if (groups < 1 || C % groups != 0 || (!residual && !copy)) return -100;
    hipStream_t s = (hipStream_t)stream;
    dim3 g(T), blk(256);
#define GN_ARGS(TY, TW) (const TY*)y, ys, (const TW*)w, (float*)residual, (TW*)copy, C, groups, eps
    const int gsz = C / groups;
    if (gsz % 8 == 0 && gsz <= 64 * 8 * GN_IT && ys % 8 == 0 && (uintptr_t)y % 32 == 0) {
        if (y_dt == 1 && dt == 1)
            hipLaunchKernelGGL((group_rmsnorm_vec_kernel<float, float, float>), g, blk, 0, s, GN_ARGS(float, float));
        else if (y_dt == 1 && dt == 0)
            hipLaunchKernelGGL((group_rmsnorm_vec_kernel<float, bf16s, bf16s>), g, blk, 0, s, GN_ARGS(float, bf16s));
        else if (y_dt == 0 && dt == 0)
            hipLaunchKernelGGL((group_rmsnorm_vec_kernel<bf16s, bf16s, bf16s>), g, blk, 0, s, GN_ARGS(bf16s, bf16s));
        else
            return -101;
    } else if (y_dt == 1 && dt == 1)
        hipLaunchKernelGGL((group_rmsnorm_kernel<float, float, float>), g, blk, 0, s, GN_ARGS(float, float));
    else if (y_dt == 1 && dt == 0)
        hipLaunchKernelGGL((group_rmsnorm_kernel<float, bf16s, bf16s>), g, blk, 0, s, GN_ARGS(float, bf16s));
    else if (y_dt == 0 && dt == 0)
        hipLaunchKernelGGL((group_rmsnorm_kernel<bf16s, bf16s, bf16s>), g, blk, 0, s, GN_ARGS(bf16s, bf16s));
    else
        return -101;
#undef GN_ARGS
    HIP_CHECK_LAUNCH();
    return 0;
}

extern "C" int oa_attn_prepare(void* stream, const void* qkv, int64_t qs, const void* bias, const void* qw,
                               const void* kw, void* q_out, void* k_cache, void* v_cache,
                               const void* slot_mapping, const void* cu, int B, int T, int H,
                               int G, int D, int Dv, float eps, int dt) {
    if (T <= 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (D % 8 == 0 && Dv % 8 == 0 && qs % 8 == 0 && (uintptr_t)qkv % 32 == 0 &&
        (!bias || (uintptr_t)bias % 32 == 0)) {
        if (dt == 1)
            hipLaunchKernelGGL((attn_prepare_vec_kernel<float>), dim3(T), dim3(256), 0, s, (const float*)qkv,
                               qs, (const float*)bias, (const float*)qw, (const float*)kw, (float*)q_out,
                               (float*)k_cache, (float*)v_cache, (const int*)slot_mapping, (const int*)cu,
                               B, H, G, D, Dv, eps);
        else
            hipLaunchKernelGGL((attn_prepare_vec_kernel<bf16s>), dim3(T), dim3(256), 0, s, (const bf16s*)qkv,
                               qs, (const bf16s*)bias, (const bf16s*)qw, (const bf16s*)kw, (bf16s*)q_out,
                               (bf16s*)k_cache, (bf16s*)v_cache, (const int*)slot_mapping, (const int*)cu,
                               B, H, G, D, Dv, eps);
        HIP_CHECK_LAUNCH();
        return 0;
    }
    if (dt == 1)
        hipLaunchKernelGGL((attn_prepare_kernel<float>), dim3(T), dim3(256), 0, s, (const float*)qkv, qs,
                           (const float*)bias, (const float*)qw, (const float*)kw, (float*)q_out, (float*)k_cache,
                           (float*)v_cache, (const int*)slot_mapping, (const int*)cu, B, H, G, D, Dv, eps);
    else
        hipLaunchKernelGGL((attn_prepare_kernel<bf16s>), dim3(T), dim3(256), 0, s, (const bf16s*)qkv, qs,
                           (const bf16s*)bias, (const bf16s*)qw, (const bf16s*)kw, (bf16s*)q_out, (bf16s*)k_cache,
                           (bf16s*)v_cache, (const int*)slot_mapping, (const int*)cu, B, H, G, D, Dv, eps);
    HIP_CHECK_LAUNCH();
    return 0;
}

// Which kernel serves a shape, and the geometry the host must agree with:
// query tokens per tile (TQ), keys per staged tile (KT), K row stride, LDS
// bytes. path 1 = matrix cores (bf16, sizes multiples of 16), 0 = VALU.
static int attn_path(int H, int G, int D, int Dv, int dt) {
    if (std::getenv("OPSAGENT_ATTN_VALU")) return 0;
    // key sizes above 128 take the matrix-core kernel only in steps of 32:
    // the 16-wide K step would hold twice the query fragments and spill
    return (dt == 0 && D % 16 == 0 && Dv % 16 == 0 && D <= 256 && Dv <= 256 &&
            (D <= 128 || D % 32 == 0)) ? 1 : 0;
}
static int attn_hb(int R) { return R % 4 == 0 ? 4 : (R % 2 == 0 ? 2 : 1); }

// token sub-tiles per wave of the matrix-core kernel. Two sub-tiles halve
// the LDS fragment reads and the staging per query row, but at 128-wide
// heads they need ~300 registers per lane (one wave per SIMD) and measured
// no faster than one sub-tile at three waves per SIMD; one is used.
static int attn_nt(int D, int Dv, int max_chunk) {
    (void)D; (void)Dv; (void)max_chunk;
    return 1;
}

extern "C" int oa_attn_bias_geometry(int H, int G, int D, int Dv, int dt, int max_chunk, int* TQ,
                                     int* KT, int* kstride, int* lds_bytes) {
    if (G < 1 || H % G != 0 || Dv > 64 * ATT_MAXV) return -100;
    const int R = H / G;
    if (attn_path(H, G, D, Dv, dt)) {
        *TQ = 16 * (4 / attn_hb(R)) * attn_nt(D, Dv, max_chunk);
        *KT = MF_KT;
        *kstride = D + MF_KPAD;
        *lds_bytes = (MF_KT * (D + MF_KPAD) + Dv * (MF_KT + 4)) * 2;
        return 0;
    }
    const int rb = std::min(R, 4 * ATT_MAXR);        // query heads per block
    int tq = std::max(1, (4 * ATT_MAXR) / rb);
    const int esz = dt == 1 ? 4 : 2;
    int ks = D;
    if (dt == 1) ks = (D % 2 == 0) ? D + 1 : D;
    else ks = ((D / 2) % 2 == 0) ? D + 2 : D + (D % 2);
    for (int kt = 64; kt >= 8; kt >>= 1) {
        size_t bytes = ((size_t)tq * rb * D + 4 * kt) * 4 + ((size_t)kt * ks + (size_t)kt * Dv) * esz;
        if (bytes <= 64 * 1024) {
            *TQ = tq; *KT = kt; *kstride = ks; *lds_bytes = (int)bytes;
            return 0;
        }
    }
    return -103;
}

template <int MAXD, int MAXDV, bool QK32, int NT>
static void launch_attn_mfma(hipStream_t s, dim3 grid, int lds_bytes, const void* q, const void* gate,
                             int64_t gs, const void* k_cache, const void* v_cache, void* out,
                             void* part_o, void* part_ml, const void* cu, const void* past,
                             const void* block_table, int max_blocks, int block_size,
                             const void* slopes, const void* sinks, int B, int H, int G, int D,
                             int Dv, int HB, float scale, int nsplit, int window, int64_t vrow,
                             int hrows, int Gv, float softcap) {
    if (lds_bytes > 48 * 1024)
        (void)hipFuncSetAttribute((const void*)attn_bias_mfma_kernel<MAXD, MAXDV, QK32, NT>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    hipLaunchKernelGGL((attn_bias_mfma_kernel<MAXD, MAXDV, QK32, NT>), grid, dim3(256), lds_bytes, s,
                       (const bf16s*)q, (const bf16s*)gate, gs, (const bf16s*)k_cache,
                       (const bf16s*)v_cache, (bf16s*)out, (float*)part_o, (float*)part_ml,
                       (const int*)cu, (const int*)past, (const int*)block_table, max_blocks,
                       block_size, (const float*)slopes, (const float*)sinks, B, H, G, D, Dv, HB,
                       scale, nsplit, window, (int)vrow, hrows, Gv, softcap);
}

// ntiles = sum_b ceil(n_b / TQ) (host-computed). part_* may be null when nsplit == 1.
extern "C" int oa_attn_bias_paged(void* stream, const void* q, const void* gate, int64_t gs,
                                  const void* k_cache, const void* v_cache, void* out,
                                  void* part_o, void* part_ml, const void* cu, const void* past,
                                  const void* block_table, int max_blocks, int block_size,
                                  const void* slopes, const void* sinks, int T, int B, int ntiles,
                                  int H, int G, int D, int Dv, float scale, int nsplit, int dt,
                                  int max_chunk, int window, int64_t vrow, int Gv, float softcap) {
    // vrow: elements between the value rows of consecutive cache slots
    // (Gv * Dv for a cache of its own; more when the values are the leading
    // channels of wider rows). Gv value heads: key head g reads value head
    // g mod Gv. softcap > 0: score <- softcap * tanh(score / softcap).
    if (T <= 0 || ntiles <= 0) return 0;
    if (window < 0) return -105;
    if (Gv < 1 || G % Gv != 0 || vrow < (int64_t)Gv * Dv) return -106;
    int TQ, KT, ks, lds_bytes;
    int rc = oa_attn_bias_geometry(H, G, D, Dv, dt, max_chunk, &TQ, &KT, &ks, &lds_bytes);
    if (rc) return rc;
    if (nsplit < 1 || (nsplit > 1 && (!part_o || !part_ml))) return -104;
    hipStream_t s = (hipStream_t)stream;
    if (attn_path(H, G, D, Dv, dt)) {
        if (vrow % 8 != 0) return -107;   // 16-byte value loads
        const int R = H / G, HB = attn_hb(R);
        // decode steps of 16 or more query heads per kv head put the heads
        // in the tile's columns
        const int hrows = (max_chunk == 1 && R >= 16) ? 1 : 0;
        dim3 grid(ntiles, hrows ? G * CEIL_DIV(R, 64) : G * (R / HB), nsplit);
#define MF_ARGS                                                                                   \
    s, grid, lds_bytes, q, gate, gs, k_cache, v_cache, out, part_o, part_ml, cu, past, block_table, \
        max_blocks, block_size, slopes, sinks, B, H, G, D, Dv, HB, scale, nsplit, window, vrow, hrows, \
        Gv, softcap
#define MF(A, Bv)                                                               \
    do {                                                                        \
        if (D % 32 == 0) launch_attn_mfma<A, Bv, true, 1>(MF_ARGS);             \
        else launch_attn_mfma<A, Bv, false, 1>(MF_ARGS);                        \
    } while (0)
        const int a = D <= 64 ? 4 : (D <= 128 ? 8 : 16), bv = Dv <= 64 ? 4 : (Dv <= 128 ? 8 : 16);
        if (a == 4 && bv == 4) MF(4, 4);
        else if (a == 4 && bv == 8) MF(4, 8);
        else if (a == 4) MF(4, 16);
        else if (a == 8 && bv == 4) MF(8, 4);
        else if (a == 8 && bv == 8) MF(8, 8);
        else if (a == 8) MF(8, 16);
        else if (bv == 4) launch_attn_mfma<16, 4, true, 1>(MF_ARGS);
        else if (bv == 8) launch_attn_mfma<16, 8, true, 1>(MF_ARGS);
        else launch_attn_mfma<16, 16, true, 1>(MF_ARGS);
#undef MF
#undef MF_ARGS
        HIP_CHECK_LAUNCH();
    } else {
        const int rb = std::min(H / G, 4 * ATT_MAXR);
        dim3 grid(ntiles, G * CEIL_DIV(H / G, rb), nsplit), blk(256);
#define AT_ARGS(TC)                                                                      \
    (const TC*)q, (const TC*)gate, gs, (const TC*)k_cache, (const TC*)v_cache, (TC*)out,  \
        (float*)part_o, (float*)part_ml, (const int*)cu, (const int*)past,                \
        (const int*)block_table, max_blocks, block_size, (const float*)slopes,            \
        (const float*)sinks, B, H, G, D, Dv, TQ, KT, ks, scale, nsplit, rb, window, vrow, Gv,  \
        softcap
        if (dt == 1)
            hipLaunchKernelGGL((attn_bias_paged_kernel<float>), grid, blk, lds_bytes, s, AT_ARGS(float));
        else
            hipLaunchKernelGGL((attn_bias_paged_kernel<bf16s>), grid, blk, lds_bytes, s, AT_ARGS(bf16s));
#undef AT_ARGS
        HIP_CHECK_LAUNCH();
    }
    if (nsplit > 1) {
        if (dt == 1)
            hipLaunchKernelGGL((attn_combine_kernel<float>), dim3((unsigned)((int64_t)T * H)), dim3(64), 0, s,
                               (const float*)part_o, (const float*)part_ml, (const float*)gate, gs,
                               (const float*)sinks, (float*)out, H, Dv, nsplit);
        else
            hipLaunchKernelGGL((attn_combine_kernel<bf16s>), dim3((unsigned)((int64_t)T * H)), dim3(64), 0, s,
                               (const float*)part_o, (const float*)part_ml, (const bf16s*)gate, gs,
                               (const float*)sinks, (bf16s*)out, H, Dv, nsplit);
        HIP_CHECK_LAUNCH();
    }
    return 0;
}

template <int RPL, int P>
static int launch_delta(hipStream_t s, const void* q, int64_t qs, const void* k, int64_t ks,
                        const void* v, int64_t vs, const void* bl, int64_t bs, const void* a,
                        int64_t as, const void* dt_bias, const void* a_log, const void* norm_w,
                        const void* gate, int64_t gs, void* state, void* out, void* o_raw,
                        const void* cu, const void* past, const void* slots, int B, int H, int G,
                        int D, int Dv, float eps, int dt, int csplit) {
    const int nw = CEIL_DIV(Dv / csplit, 4 * P);
    if (nw > 16) return -106;
    int tck = 16;
    auto bytes = [&](int t) { return (size_t)(3 * t * RPL * 16 + 2 * t * Dv + t) * 4; };
    while (tck > 2 && bytes(tck) > 60 * 1024) tck >>= 1;
    dim3 grid(B, H, csplit), blk(64 * nw);
#define DARGS(TC)                                                                              \
    (const TC*)q, qs, (const TC*)k, ks, (const TC*)v, vs, (const TC*)bl, bs, (const TC*)a, as,  \
        (const TC*)dt_bias, (const TC*)a_log, (const TC*)norm_w, (const TC*)gate, gs,           \
        (float*)state, (TC*)out, (float*)o_raw, (const int*)cu, (const int*)past,               \
        (const int*)slots, H, G, D, Dv, tck, eps
    if (dt == 1)
        hipLaunchKernelGGL((delta_fused_kernel<RPL, P, float>), grid, blk, bytes(tck), s, DARGS(float));
    else
        hipLaunchKernelGGL((delta_fused_kernel<RPL, P, bf16s>), grid, blk, bytes(tck), s, DARGS(bf16s));
#undef DARGS
    HIP_CHECK_LAUNCH();
    return 0;
}

// q, k [T, G*D], v [T, H*Dv], bl [T, H], a [T, H*D], gate [T, H*Dv]: rows with
// the given strides; out [T, H*Dv] contiguous; state [slots, H, Dv, D].
// csplit > 1 splits each head's value columns over that many blocks (Dv must
// divide by 4*csplit) and needs o_raw, float32 [T, H*Dv].
extern "C" int oa_delta_rule_fused(void* stream, const void* q, int64_t qs, const void* k,
                                   int64_t ks, const void* v, int64_t vs, const void* bl,
                                   int64_t bs, const void* a, int64_t as, const void* dt_bias,
                                   const void* a_log, const void* norm_w, const void* gate,
                                   int64_t gs, void* state, void* out, void* o_raw,
                                   const void* cu, const void* past, const void* slots, int T,
                                   int B, int H, int G, int D, int Dv, float eps, int dt,
                                   int csplit) {
    if (T <= 0 || B <= 0) return 0;
    if (G < 1 || H % G != 0) return -100;
    if (D > 256 || Dv > 256) return -105;
    if (csplit < 1 || Dv % (4 * csplit) != 0 || (csplit > 1 && !o_raw)) return -107;
    hipStream_t s = (hipStream_t)stream;
#define DL(R, PP)                                                                                     \
    launch_delta<R, PP>(s, q, qs, k, ks, v, vs, bl, bs, a, as, dt_bias, a_log, norm_w, gate, gs, state, \
                        out, o_raw, cu, past, slots, B, H, G, D, Dv, eps, dt, csplit)
    const int r = D <= 64 ? 4 : (D <= 128 ? 8 : 16);
    const int cpb = Dv / csplit;
    const int p = cpb <= 64 ? 1 : (cpb <= 128 ? 2 : 4);
    int rc;
    if (r == 4) rc = p == 1 ? DL(4, 1) : (p == 2 ? DL(4, 2) : DL(4, 4));
    else if (r == 8) rc = p == 1 ? DL(8, 1) : (p == 2 ? DL(8, 2) : DL(8, 4));
    else rc = p == 1 ? DL(16, 1) : (p == 2 ? DL(16, 2) : DL(16, 4));
#undef DL
    if (rc || csplit == 1) return rc;
    if (dt == 1)
        hipLaunchKernelGGL((gated_head_norm_kernel<float>), dim3(T), dim3(256), 0, s, (const float*)o_raw,
                           (const float*)norm_w, (const float*)gate, gs, (float*)out, H, Dv, eps);
    else
        hipLaunchKernelGGL((gated_head_norm_kernel<bf16s>), dim3(T), dim3(256), 0, s, (const float*)o_raw,
                           (const bf16s*)norm_w, (const bf16s*)gate, gs, (bf16s*)out, H, Dv, eps);
    HIP_CHECK_LAUNCH();
    return 0;
}

extern "C" int oa_softcap(void* stream, const void* x, void* out, int64_t n, float cap, int dt) {
    if (n <= 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (dt == 1)
        hipLaunchKernelGGL((softcap_kernel<float>), dim3(grid_for(n)), dim3(256), 0, s, (const float*)x,
                           (float*)out, n, cap);
    else
        hipLaunchKernelGGL((softcap_kernel<bf16s>), dim3(grid_for(n)), dim3(256), 0, s, (const bf16s*)x,
                           (float*)out, n, cap);
    HIP_CHECK_LAUNCH();
    return 0;
}

extern "C" int oa_silu_mul_rows(void* stream, const void* gu, void* out, int64_t M, int I, int dt) {
    if (M <= 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (dt == 1)
        hipLaunchKernelGGL((silu_mul_rows_kernel<float>), dim3(grid_for(M * I)), dim3(256), 0, s,
                           (const float*)gu, (float*)out, M, I);
    else
        hipLaunchKernelGGL((silu_mul_rows_kernel<bf16s>), dim3(grid_for(M * I)), dim3(256), 0, s,
                           (const bf16s*)gu, (bf16s*)out, M, I);
    HIP_CHECK_LAUNCH();
    return 0;
}

extern "C" int oa_embed_rows(void* stream, const void* table, const void* ids, void* out, int T,
                             int C, int dt, float scale) {
    if (T <= 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (dt == 1)
        hipLaunchKernelGGL((embed_rows_kernel<float>), dim3(grid_for((int64_t)T * C)), dim3(256), 0, s,
                           (const float*)table, (const int64_t*)ids, (float*)out, T, C, scale);
    else
        hipLaunchKernelGGL((embed_rows_kernel<bf16s>), dim3(grid_for((int64_t)T * C)), dim3(256), 0, s,
                           (const bf16s*)table, (const int64_t*)ids, (float*)out, T, C, scale);
    HIP_CHECK_LAUNCH();
    return 0;
}
