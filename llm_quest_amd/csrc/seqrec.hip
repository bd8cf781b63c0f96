// Row operations and recurrences of hybrid decoders with PARALLEL sublayers, served in ragged batches (gfx950 only): the residual sum with up to two
// RMS norms in groups of the row, short causal convolutions over time with a carried state, query / key / value rows of grouped-query attention
// (bias, per-head RMS norm, rotary, per-head query scale) written into a slot cache, the gated delta rule with carried fp32 state, and gated
// feed-forward activations.
//
// Conventions as in seqmix.hip: operands come as bf16 or fp32 (a MI355_DT_* code each); the residual stream, norm statistics, rotary angles, decays,
// gates of a recurrence and recurrent state are fp32 in both modes.  A "row" is a token of the packed batch; sequences are described by int32 device arrays.
#include "common.h"
#include "lane_sums.h"

#define ST(s) ((hipStream_t)(s))

__device__ __forceinline__ float ldr_dt(const void* p, int dt, int64_t i) { return dt == MI355_DT_F32 ? ((const float*)p)[i] : bf2f(((const bf16_t*)p)[i]); }
__device__ __forceinline__ void str_dt(void* p, int dt, int64_t i, float v) {
    if (dt == MI355_DT_F32) ((float*)p)[i] = v;
    else ((bf16_t*)p)[i] = f2bf(v);
}
static inline int rec_rows_grid(int64_t rows, int per_block) {
    int64_t g = (rows + per_block - 1) / per_block;
    return (int)(g < 1 ? 1 : (g > 65535 * 16 ? 65535 * 16 : g));
}
static inline bool rec_dt_ok(int dt) { return dt == MI355_DT_BF16 || dt == MI355_DT_F32; }
// four consecutive elements (the caller vouches for 16-byte alignment of fp32 rows, 8-byte of bf16 rows)
__device__ __forceinline__ f32x4 ld4_dt(const void* p, int dt, int64_t i) {
    if (dt == MI355_DT_F32) return *(const f32x4*)((const float*)p + i);
    const u32x2 r = *(const u32x2*)((const bf16_t*)p + i);
    return f32x4{__uint_as_float(r[0] << 16), __uint_as_float(r[0] & 0xffff0000u), __uint_as_float(r[1] << 16), __uint_as_float(r[1] & 0xffff0000u)};
}
__device__ __forceinline__ void st4_dt(void* p, int dt, int64_t i, f32x4 v) {
    if (dt == MI355_DT_F32) *(f32x4*)((float*)p + i) = v;
    else *(u32x2*)((bf16_t*)p + i) = u32x2{pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3])};
}
static inline bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// ------------------------------------------------------------------------------------------- residual sum + RMS norms in groups
// v = x + y1[t] + sum_{p < parts} y2[t * parts + p]  (fp32; either summand may be absent); x_out (optional, may be x) receives v.
// For each of up to two weights w_n: out_n[t, i] = v[i] / sqrt(mean over i's group of v^2 + eps) * w_n[i], the row cut into `groups` equal consecutive
// groups; out_n in dtype dt_n, and a second fp32 copy out32_n if asked for.  One wave per row; a lane holds elements lane + 64 j.
struct GroupNormArgs {
    const float* x;
    const void* y1;
    const void* y2;
    float* x_out;
    const float* w[2];
    void* out[2];
    float* out32[2];
    int64_t ldy1, ldy2;
    int y1_dt, y2_dt, parts, groups, out_dt[2];
    float eps;
};

template <int EPL>
__global__ __launch_bounds__(256) void group_rmsnorm_sum_kernel(int64_t T, int width, GroupNormArgs p) {
    const int lane = threadIdx.x & 63;
    const int gs = width / p.groups;
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += (int64_t)gridDim.x * 4) {
        float v[EPL], r[EPL];
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int i = lane + 64 * j;
            float a = 0.f;
            if (i < width) {
                a = p.x[t * width + i];
                float ys = 0.f;
                if (p.y1) ys = ldr_dt(p.y1, p.y1_dt, t * p.ldy1 + i);
                if (p.y2) {
                    float y2s = 0.f;
                    for (int q = 0; q < p.parts; ++q) y2s += ldr_dt(p.y2, p.y2_dt, (t * p.parts + q) * p.ldy2 + i);
                    ys += y2s;
                }
                a += ys;
                if (p.x_out) p.x_out[t * width + i] = a;
            }
            v[j] = a;
            r[j] = 0.f;
        }
        if (!p.w[0] && !p.w[1]) continue;
        for (int g = 0; g < p.groups; ++g) {
            const int lo = g * gs, hi = lo + gs;
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                const int i = lane + 64 * j;
                if (i >= lo && i < hi) s += v[j] * v[j];
            }
            const float rg = 1.0f / sqrtf(wave_sum(s) / (float)gs + p.eps);
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                const int i = lane + 64 * j;
                if (i >= lo && i < hi) r[j] = rg;
            }
        }
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            if (!p.w[n]) continue;
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                const int i = lane + 64 * j;
                if (i < width) {
                    const float o = v[j] * r[j] * p.w[n][i];
                    if (p.out[n]) str_dt(p.out[n], p.out_dt[n], t * width + i, o);
                    if (p.out32[n]) p.out32[n][t * width + i] = o;
                }
            }
        }
    }
}

// The same for wide rows: one workgroup per row, 16-byte accesses; thread t owns elements 4 (t + 256 j) .. + 4 (a group's size is a multiple of 4, so
// the four lie in one group).  A wave sums its share of every group, the four waves' shares meet in LDS in a fixed order.
#define GN_MAXG 64
template <int V4>
__global__ __launch_bounds__(256) void group_rmsnorm_sum_wide_kernel(int64_t T, int width, GroupNormArgs p) {
    __shared__ float red[4][GN_MAXG];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gs = width / p.groups;
    for (int64_t t = blockIdx.x; t < T; t += gridDim.x) {
        f32x4 v[V4];
        int grp[V4];
#pragma unroll
        for (int j = 0; j < V4; ++j) {
            const int i = 4 * (tid + 256 * j);
            f32x4 a = {0.f, 0.f, 0.f, 0.f};
            grp[j] = -1;
            if (i < width) {
                grp[j] = i / gs;
                a = *(const f32x4*)(p.x + t * width + i);
                f32x4 ys = {0.f, 0.f, 0.f, 0.f};
                if (p.y1) ys = ld4_dt(p.y1, p.y1_dt, t * p.ldy1 + i);
                if (p.y2) {
                    f32x4 y2s = {0.f, 0.f, 0.f, 0.f};
                    for (int q = 0; q < p.parts; ++q) y2s += ld4_dt(p.y2, p.y2_dt, (t * p.parts + q) * p.ldy2 + i);
                    ys += y2s;
                }
                a += ys;
                if (p.x_out) *(f32x4*)(p.x_out + t * width + i) = a;
            }
            v[j] = a;
        }
        if (!p.w[0] && !p.w[1]) continue;
        for (int g = 0; g < p.groups; ++g) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < V4; ++j)
                if (grp[j] == g) s += (v[j][0] * v[j][0] + v[j][1] * v[j][1]) + (v[j][2] * v[j][2] + v[j][3] * v[j][3]);
            s = wave_sum(s);
            if (lane == 0) red[wave][g] = s;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < V4; ++j) {
            const int i = 4 * (tid + 256 * j);
            if (i >= width) continue;
            const int g = grp[j];
            const float r = 1.0f / sqrtf(((red[0][g] + red[1][g]) + (red[2][g] + red[3][g])) / (float)gs + p.eps);
#pragma unroll
            for (int n = 0; n < 2; ++n) {
                if (!p.w[n]) continue;
                const f32x4 o = v[j] * r * *(const f32x4*)(p.w[n] + i);
                if (p.out[n]) st4_dt(p.out[n], p.out_dt[n], t * width + i, o);
                if (p.out32[n]) *(f32x4*)(p.out32[n] + t * width + i) = o;
            }
        }
        __syncthreads();  // red[] is reused by the next row
    }
}

extern "C" int mi355_group_rmsnorm_sum(int64_t tokens, int width, const float* x, const void* y1, int y1_dt, int64_t ldy1, const void* y2, int y2_dt, int64_t ldy2,
                                       int parts, float* x_out, int groups, float eps, const float* w_a, void* out_a, int out_a_dt, float* out_a32, const float* w_b,
                                       void* out_b, int out_b_dt, float* out_b32, void* stream) {
    MI355_REQUIRE(tokens > 0 && width > 0 && width <= 8192 && x && groups >= 1 && width % groups == 0, "group_rmsnorm_sum: bad arguments (width <= 8192, a multiple of the groups)");
    MI355_REQUIRE(!y1 || (rec_dt_ok(y1_dt) && ldy1 >= width), "group_rmsnorm_sum: bad first summand");
    MI355_REQUIRE(!y2 || (rec_dt_ok(y2_dt) && ldy2 >= width && parts >= 1), "group_rmsnorm_sum: bad second summand");
    MI355_REQUIRE((!w_a || out_a || out_a32) && (!w_b || out_b || out_b32) && (!out_a || rec_dt_ok(out_a_dt)) && (!out_b || rec_dt_ok(out_b_dt)), "group_rmsnorm_sum: a norm needs an output");
    MI355_REQUIRE(x_out || w_a || w_b, "group_rmsnorm_sum: nothing to write");
    GroupNormArgs p;
    p.x = x, p.y1 = y1, p.y2 = y2, p.x_out = x_out;
    p.w[0] = w_a, p.w[1] = w_b, p.out[0] = out_a, p.out[1] = out_b, p.out32[0] = out_a32, p.out32[1] = out_b32;
    p.ldy1 = ldy1, p.ldy2 = ldy2, p.y1_dt = y1_dt, p.y2_dt = y2_dt, p.parts = parts, p.groups = groups, p.out_dt[0] = out_a_dt, p.out_dt[1] = out_b_dt;
    p.eps = eps;
    const bool wide = width > 256 && width % 4 == 0 && (width / groups) % 4 == 0 && groups <= GN_MAXG && al16(x) && (!y1 || (al16(y1) && ldy1 % 4 == 0)) &&
                      (!y2 || (al16(y2) && ldy2 % 4 == 0)) && al16(x_out) && al16(w_a) && al16(w_b) && al16(out_a) && al16(out_b) && al16(out_a32) && al16(out_b32);
    if (wide) {
        const int g = (int)(tokens < 65535 * 8 ? tokens : 65535 * 8);
#define GNW_CASE(V)                                                                         \
    if (width <= 1024 * V) {                                                                \
        group_rmsnorm_sum_wide_kernel<V><<<g, 256, 0, ST(stream)>>>(tokens, width, p);      \
        MI355_LAUNCH_CHECK("group_rmsnorm_sum");                                            \
        return 0;                                                                           \
    }
        GNW_CASE(1) GNW_CASE(2) GNW_CASE(4) GNW_CASE(8)
#undef GNW_CASE
    }
    const int grid = rec_rows_grid(tokens, 4);
#define GN_CASE(E)                                                                      \
    if (width <= 64 * E) {                                                              \
        group_rmsnorm_sum_kernel<E><<<grid, 256, 0, ST(stream)>>>(tokens, width, p);    \
        MI355_LAUNCH_CHECK("group_rmsnorm_sum");                                        \
        return 0;                                                                       \
    }
    GN_CASE(2) GN_CASE(4) GN_CASE(8) GN_CASE(16) GN_CASE(32) GN_CASE(64) GN_CASE(128)
#undef GN_CASE
    return 1;
}

// ------------------------------------------------------------------------------------------- short causal convolution over time, ragged, carried state
// y[t, c] = (residual ? x[t, c] : 0) + act( sum_{j < taps} w[c, j] * in(t - taps + 1 + j, c) ): in(.) is the same sequence's row of this step, or -- before
// the step's first row -- the carried state: state[slot, i, c] (fp32 [slots, taps - 1, C]) holds the input taps - 1 - i tokens before the step's first
// one (zeros before the sequence's start).  act: 0 none, 1 silu.  bias (fp32 [C], may be null) is added to the convolution before the activation.
// Afterwards the state takes the step's last taps - 1 inputs.
#define CONV_MAX_TAPS 16
__global__ __launch_bounds__(256) void ragged_conv_kernel(int64_t T, int C, int taps, const void* __restrict__ x, int x_dt, int64_t ldx, const float* __restrict__ w,
                                                          const int* __restrict__ row_seq, const int* __restrict__ seq_off, const int* __restrict__ slot,
                                                          const float* __restrict__ state, int act, int residual, void* __restrict__ y, int y_dt, int64_t ldy,
                                                          const float* __restrict__ bias) {
    const int64_t total = T * C;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = e / C;
        const int c = (int)(e % C);
        const int s = row_seq[t];
        const int start = seq_off[s];
        const int local = (int)(t - start);
        const float* st = state + (int64_t)slot[s] * (taps - 1) * C;
        float acc = bias ? bias[c] : 0.f;
        for (int j = 0; j < taps; ++j) {
            const int sl = local - (taps - 1) + j;
            const float in = sl >= 0 ? ldr_dt(x, x_dt, (int64_t)(start + sl) * ldx + c) : st[(int64_t)(taps - 1 + sl) * C + c];
            acc = fmaf(w[c * taps + j], in, acc);
        }
        if (act == 1) acc = acc / (1.0f + expf(-acc));
        if (residual) acc += ldr_dt(x, x_dt, t * ldx + c);
        str_dt(y, y_dt, t * ldy + c, acc);
    }
}

// Four channels per thread, one token per blockIdx.x (C % 4 == 0, 16-byte aligned rows).  TAPS > 0: the thread's 4 x TAPS weights are TAPS consecutive
// 16-byte words (w is [C, TAPS] and the channel a multiple of 4), fetched as such; TAPS == 0: any number of taps, one weight at a time.
template <int TAPS>
__global__ __launch_bounds__(256) void ragged_conv_vec_kernel(int C, int taps, const void* __restrict__ x, int x_dt, int64_t ldx, const float* __restrict__ w,
                                                              const int* __restrict__ row_seq, const int* __restrict__ seq_off, const int* __restrict__ slot,
                                                              const float* __restrict__ state, int act, int residual, void* __restrict__ y, int y_dt, int64_t ldy,
                                                              const float* __restrict__ bias) {
    const int64_t t = blockIdx.x;
    const int c = 4 * (blockIdx.y * 256 + threadIdx.x);
    if (c >= C) return;
    const int s = row_seq[t];
    const int start = seq_off[s];
    const int local = (int)(t - start);
    const float* st = state + (int64_t)slot[s] * (taps - 1) * C;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f}, cur = {0.f, 0.f, 0.f, 0.f};
    if (bias) acc = *(const f32x4*)(bias + c);
    if constexpr (TAPS > 0) {
        float wf[4 * TAPS];
#pragma unroll
        for (int i = 0; i < TAPS; ++i) {
            const f32x4 wv = *(const f32x4*)(w + (int64_t)c * TAPS + 4 * i);
#pragma unroll
            for (int e = 0; e < 4; ++e) wf[4 * i + e] = wv[e];
        }
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {
            const int sl = local - (TAPS - 1) + j;
            const f32x4 in = sl >= 0 ? ld4_dt(x, x_dt, (int64_t)(start + sl) * ldx + c) : *(const f32x4*)(st + (int64_t)(TAPS - 1 + sl) * C + c);
            if (j == TAPS - 1) cur = in;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = fmaf(wf[e * TAPS + j], in[e], acc[e]);
        }
    } else {
        for (int j = 0; j < taps; ++j) {
            const int sl = local - (taps - 1) + j;
            const f32x4 in = sl >= 0 ? ld4_dt(x, x_dt, (int64_t)(start + sl) * ldx + c) : *(const f32x4*)(st + (int64_t)(taps - 1 + sl) * C + c);
            if (j == taps - 1) cur = in;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = fmaf(w[(c + e) * taps + j], in[e], acc[e]);
        }
    }
    if (act == 1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = acc[e] / (1.0f + expf(-acc[e]));
    }
    if (residual) acc += cur;
    st4_dt(y, y_dt, t * ldy + c, acc);
}

__global__ __launch_bounds__(256) void ragged_conv_state_kernel(int n_seq, int C, int taps, const void* __restrict__ x, int x_dt, int64_t ldx, const int* __restrict__ seq_off,
                                                                const int* __restrict__ slot, float* __restrict__ state) {
    const int64_t total = (int64_t)n_seq * C;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int s = (int)(e / C), c = (int)(e % C);
        const int start = seq_off[s], n = seq_off[s + 1] - start;
        float* st = state + (int64_t)slot[s] * (taps - 1) * C;
        float keep[CONV_MAX_TAPS];
#pragma unroll
        for (int i = 0; i < CONV_MAX_TAPS; ++i) {
            keep[i] = 0.f;
            if (i < taps - 1) {
                const int sl = n - (taps - 1) + i;  // the step's row that becomes state entry i, or an older input that stays
                keep[i] = sl >= 0 ? ldr_dt(x, x_dt, (int64_t)(start + sl) * ldx + c) : st[(int64_t)(taps - 1 + sl) * C + c];
            }
        }
#pragma unroll
        for (int i = 0; i < CONV_MAX_TAPS; ++i)
            if (i < taps - 1) st[(int64_t)i * C + c] = keep[i];
    }
}

extern "C" int mi355_ragged_conv(int64_t tokens, int n_seq, int C, int taps, const void* x, int x_dt, int64_t ldx, const float* w, const int* row_seq, const int* seq_off,
                                 const int* slot, float* state, int act, int residual, void* y, int y_dt, int64_t ldy, const float* bias, void* stream) {
    MI355_REQUIRE(tokens > 0 && n_seq > 0 && C > 0 && taps >= 1 && taps <= CONV_MAX_TAPS && x && w && row_seq && seq_off && slot && y && (taps == 1 || state),
                  "ragged_conv: bad arguments (taps <= 16)");
    MI355_REQUIRE(rec_dt_ok(x_dt) && rec_dt_ok(y_dt) && ldx >= C && ldy >= C && (act == 0 || act == 1), "ragged_conv: bad operands");
    const int64_t total = tokens * C;
    if (C % 4 == 0 && ldx % 4 == 0 && ldy % 4 == 0 && al16(x) && al16(y) && al16(state) && al16(bias) && tokens < ((int64_t)1 << 31)) {
        const dim3 grid((unsigned)tokens, (C / 4 + 255) / 256);
#define CONV_CASE(TP)                                                                                                                                          \
    case TP:                                                                                                                                                   \
        ragged_conv_vec_kernel<TP><<<grid, 256, 0, ST(stream)>>>(C, taps, x, x_dt, ldx, w, row_seq, seq_off, slot, state, act, residual, y, y_dt, ldy, bias);      \
        break;
        switch (al16(w) ? taps : 0) {
            CONV_CASE(2) CONV_CASE(3) CONV_CASE(4) CONV_CASE(5) CONV_CASE(6) CONV_CASE(7) CONV_CASE(8)
            default:
                ragged_conv_vec_kernel<0><<<grid, 256, 0, ST(stream)>>>(C, taps, x, x_dt, ldx, w, row_seq, seq_off, slot, state, act, residual, y, y_dt, ldy, bias);
        }
#undef CONV_CASE
    } else {
        const int g = (int)((total + 255) / 256 > 65535 * 8 ? 65535 * 8 : (total + 255) / 256);
        ragged_conv_kernel<<<g, 256, 0, ST(stream)>>>(tokens, C, taps, x, x_dt, ldx, w, row_seq, seq_off, slot, state, act, residual, y, y_dt, ldy, bias);
    }
    MI355_LAUNCH_CHECK("ragged_conv");
    if (taps > 1) {
        const int64_t tot2 = (int64_t)n_seq * C;
        ragged_conv_state_kernel<<<(int)((tot2 + 255) / 256), 256, 0, ST(stream)>>>(n_seq, C, taps, x, x_dt, ldx, seq_off, slot, state);
        MI355_LAUNCH_CHECK("ragged_conv(state)");
    }
    return 0;
}

// ------------------------------------------------------------------------------------------- query / key / value rows of grouped-query attention
// src[t] = [H query heads x d | G key heads x d | G value heads x dv] (+ bias).  Query and key heads: RMS norm over d with a weight shared by the heads
// (absent: none), rotary on the first `dims` entries (layout 0: pairs (2i, 2i+1); 1: pairs (i, i + dims/2)), angle = pos * freq[i]; a query head is then
// multiplied by qscale[h] and written as fp32 to q_out[t, h * d + .]; key and value heads go to cache row dst_row[t]: [G x d | G x dv] in dtype c_dt.
// Query temperature (qt_every > 0): the query at position p is also multiplied by 1 + qt_coef * ln(floor((p + 1) / qt_every) + 1).  Value mixing
// (vmix given): v <- (1 - lam) v + lam * vmix[t] before it is cached, vmix fp32 rows [G x dv] (another layer's values of the same tokens).
struct QkvRowsArgs {
    const float* vmix;
    int64_t ldvm;
    float lam, qt_coef;
    int qt_every;
    const void* src;
    const float* bias;
    const float *qw, *kw, *qscale, *freq;
    const int *pos, *dst_row;
    float* q_out;
    void* cache;
    int64_t lds_, ldq, ldc;
    int src_dt, c_dt, H, G, d, dv, dims, layout;
    float eps;
};

__global__ __launch_bounds__(256) void qkv_rows_kernel(int64_t T, QkvRowsArgs p) {
    const int lane = threadIdx.x & 63;
    const int HT = p.H + 2 * p.G;
    const int64_t items = T * HT;
    for (int64_t it = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); it < items; it += (int64_t)gridDim.x * 4) {
        const int64_t t = it / HT;
        const int hh = (int)(it % HT);
        const bool is_q = hh < p.H, is_k = !is_q && hh < p.H + p.G;
        const int n = (is_q || is_k) ? p.d : p.dv;
        const int col0 = is_q ? hh * p.d : (is_k ? p.H * p.d + (hh - p.H) * p.d : (p.H + p.G) * p.d + (hh - p.H - p.G) * p.dv);
        const int64_t so = t * p.lds_ + col0;
        auto val = [&](int i) { return ldr_dt(p.src, p.src_dt, so + i) + (p.bias ? p.bias[col0 + i] : 0.f); };
        if (!is_q && !is_k) {
            const int64_t d0 = (int64_t)p.dst_row[t] * p.ldc + p.G * p.d + (hh - p.H - p.G) * p.dv;
            if (p.vmix) {
                const int64_t m0 = t * p.ldvm + (hh - p.H - p.G) * p.dv;
                for (int i = lane; i < n; i += 64) str_dt(p.cache, p.c_dt, d0 + i, (1.0f - p.lam) * val(i) + p.lam * p.vmix[m0 + i]);
            } else {
                for (int i = lane; i < n; i += 64) str_dt(p.cache, p.c_dt, d0 + i, val(i));
            }
            continue;
        }
        const float* w = is_q ? p.qw : p.kw;
        float r = 1.0f;
        if (w) {
            float s = 0.f;
            for (int i = lane; i < n; i += 64) {
                const float a = val(i);
                s += a * a;
            }
            r = 1.0f / sqrtf(wave_sum(s) / (float)n + p.eps);
        }
        float sc = is_q ? (p.qscale ? p.qscale[hh] : 1.0f) : 1.0f;
        if (is_q && p.qt_every > 0) sc *= 1.0f + p.qt_coef * logf((float)((p.pos[t] + 1) / p.qt_every + 1));
        const float ps = (float)p.pos[t];
        const int64_t qo = t * p.ldq + (int64_t)hh * p.d, ko = (int64_t)p.dst_row[t] * p.ldc + (int64_t)(hh - p.H) * p.d;
        auto put = [&](int i, float v) {
            if (is_q) p.q_out[qo + i] = v * sc;
            else str_dt(p.cache, p.c_dt, ko + i, v);
        };
        for (int i = p.dims + lane; i < n; i += 64) put(i, val(i) * r * (w ? w[i] : 1.0f));
        const int half = p.dims / 2;
        for (int i = lane; i < half; i += 64) {
            const int a = p.layout ? i : 2 * i, b = p.layout ? i + half : 2 * i + 1;
            const float u = val(a) * r * (w ? w[a] : 1.0f), v = val(b) * r * (w ? w[b] : 1.0f);
            const float ang = ps * p.freq[i];
            const float c = cosf(ang), s = sinf(ang);
            put(a, u * c - v * s);
            put(b, v * c + u * s);
        }
    }
}

extern "C" int mi355_qkv_rows_append(int64_t tokens, int H, int G, int d, int dv, const void* src, int src_dt, int64_t ld_src, const float* bias, const float* qw,
                                     const float* kw, float eps, const float* qscale, int dims, int layout, const float* freq, const int* pos, const int* dst_row,
                                     float* q_out, int64_t ldq, void* cache, int c_dt, int64_t ldc, float qt_coef, int qt_every, const float* vmix, int64_t ldvm,
                                     float lam, void* stream) {
    MI355_REQUIRE(qt_every >= 0 && (!vmix || ldvm >= (int64_t)G * dv), "qkv_rows_append: bad query temperature or value-mix rows");
    MI355_REQUIRE(tokens > 0 && H > 0 && G > 0 && d > 0 && dv > 0 && src && pos && dst_row && q_out && cache && rec_dt_ok(src_dt) && rec_dt_ok(c_dt), "qkv_rows_append: bad arguments");
    MI355_REQUIRE(dims >= 0 && dims % 2 == 0 && dims <= d && (dims == 0 || freq) && (layout == 0 || layout == 1), "qkv_rows_append: the rotated range must lie inside a head");
    MI355_REQUIRE(ld_src >= (int64_t)(H + G) * d + (int64_t)G * dv && ldq >= (int64_t)H * d && ldc >= (int64_t)G * (d + dv), "qkv_rows_append: rows too short");
    QkvRowsArgs p;
    p.src = src, p.bias = bias, p.qw = qw, p.kw = kw, p.qscale = qscale, p.freq = freq, p.pos = pos, p.dst_row = dst_row, p.q_out = q_out, p.cache = cache;
    p.lds_ = ld_src, p.ldq = ldq, p.ldc = ldc, p.src_dt = src_dt, p.c_dt = c_dt, p.H = H, p.G = G, p.d = d, p.dv = dv, p.dims = dims, p.layout = layout, p.eps = eps;
    p.vmix = vmix, p.ldvm = ldvm, p.lam = lam, p.qt_coef = qt_coef, p.qt_every = qt_every;
    qkv_rows_kernel<<<rec_rows_grid(tokens * (H + 2 * G), 4), 256, 0, ST(stream)>>>(tokens, p);
    MI355_LAUNCH_CHECK("qkv_rows_append");
    return 0;
}

// ------------------------------------------------------------------------------------------- gated delta rule, ragged, carried state
// Per value head h a state S [dk, dv] (fp32, carried per sequence slot); its query / key head is h / (H / G).  Per token:
//   k^ = k / sqrt(sum k^2 + 1e-6), q^ = q / sqrt(sum q^2 + 1e-6) * qscale   (unit vectors; raw q / k rows come in)
//   beta = sigmoid(b), g = exp(-exp(A_log[h]) * softplus(a + dt_bias[h]))
//   S <- g S;  u = beta (v - S^T k^);  S <- S + k^ u^T;  o = S^T q^
// Column c of S obeys its own recurrence, so columns are spread over lanes and the time loop stays inside: DR_LPR lanes share a column (CPL key
// channels each, in registers), the two dot products of a step close with lane sums -- no LDS, no barrier.  The per-token scalars (g, beta and the two
// unit-vector factors, which multiply the dot products instead of the rows) are prepared once per (token, head) by delta_prep_kernel; the operands of
// step t + 1 are requested before step t's arithmetic.
#define DR_LPR 8
struct DeltaArgs {
    const int *seq_off, *slot;
    const void *q, *k, *v, *b, *a;
    const float *A_log, *dt_bias;
    float *state, *o;
    f32x4* ws;  // [tokens, H]: g, beta, key factor, query factor * qscale
    int64_t ldq, ldk, ldv, ldb, lda;
    int H, G, dk, dv, qk_dt, v_dt, ba_dt;
    float qscale;
};

__global__ __launch_bounds__(256) void delta_prep_kernel(int64_t T, DeltaArgs p) {
    const int lane = threadIdx.x & 63;
    const int64_t items = T * p.H;
    for (int64_t it = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); it < items; it += (int64_t)gridDim.x * 4) {
        const int64_t t = it / p.H;
        const int h = (int)(it % p.H), hq = h / (p.H / p.G);
        float sq = 0.f, sk = 0.f;
        for (int i = lane; i < p.dk; i += 64) {
            const float qv = ldr_dt(p.q, p.qk_dt, t * p.ldq + (int64_t)hq * p.dk + i), kv = ldr_dt(p.k, p.qk_dt, t * p.ldk + (int64_t)hq * p.dk + i);
            sq += qv * qv;
            sk += kv * kv;
        }
        sq = wave_sum(sq);
        sk = wave_sum(sk);
        if (lane == 0) {
            const float bb = ldr_dt(p.b, p.ba_dt, t * p.ldb + h), aa = ldr_dt(p.a, p.ba_dt, t * p.lda + h) + p.dt_bias[h];
            const float sp = aa > 20.f ? aa : log1pf(expf(aa));
            p.ws[it] = f32x4{expf(-expf(p.A_log[h]) * sp), 1.0f / (1.0f + expf(-bb)), 1.0f / sqrtf(sk + 1e-6f), p.qscale / sqrtf(sq + 1e-6f)};
        }
    }
}

template <int CPL, bool VEC>
__global__ __launch_bounds__(256) void delta_rule_kernel(DeltaArgs p) {
    constexpr int RPW = 64 / DR_LPR;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int s = blockIdx.z, h = blockIdx.y;
    const int col0 = (blockIdx.x * 4 + wave) * RPW;
    if (col0 >= p.dv) return;  // whole wave out of range; no block-level synchronisation below
    const int col = col0 + lane / DR_LPR, cg = lane % DR_LPR, ch0 = cg * CPL;
    const bool col_ok = col < p.dv;
    const int hq = h / (p.H / p.G), dk = p.dk;
    const int t0 = p.seq_off[s], t1 = p.seq_off[s + 1];
    float* S = p.state + (((int64_t)p.slot[s] * p.H + h) * dk) * p.dv;
    float st[CPL];
#pragma unroll
    for (int i = 0; i < CPL; ++i) st[i] = (col_ok && ch0 + i < dk) ? S[(int64_t)(ch0 + i) * p.dv + col] : 0.f;
    struct In {
        float k[CPL], q[CPL];
        f32x4 sc;
        float v;
    };
    auto load_in = [&](In& in, int t) {
        const int64_t ko = (int64_t)t * p.ldk + (int64_t)hq * dk + ch0, qo = (int64_t)t * p.ldq + (int64_t)hq * dk + ch0;
        if (VEC) {
#pragma unroll
            for (int i = 0; i < CPL; i += 4) {
                f32x4 kv = {0.f, 0.f, 0.f, 0.f}, qv = {0.f, 0.f, 0.f, 0.f};
                if (ch0 + i < dk) {
                    kv = *(const f32x4*)((const float*)p.k + ko + i);
                    qv = *(const f32x4*)((const float*)p.q + qo + i);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) in.k[i + e] = kv[e], in.q[i + e] = qv[e];
            }
        } else {
#pragma unroll
            for (int i = 0; i < CPL; ++i) {
                const bool ok = ch0 + i < dk;
                in.k[i] = ok ? ldr_dt(p.k, p.qk_dt, ko + i) : 0.f;
                in.q[i] = ok ? ldr_dt(p.q, p.qk_dt, qo + i) : 0.f;
            }
        }
        in.sc = p.ws[(int64_t)t * p.H + h];
        in.v = col_ok ? ldr_dt(p.v, p.v_dt, (int64_t)t * p.ldv + (int64_t)h * p.dv + col) : 0.f;
    };
    auto step = [&](const In& in, int t) {
        const float a = in.sc[0], b = in.sc[1], kn = in.sc[2], qn = in.sc[3];
        float u0 = 0.f, u1 = 0.f;
#pragma unroll
        for (int i = 0; i < CPL; i += 2) {
            st[i] *= a;
            st[i + 1] *= a;
            u0 = fmaf(st[i], in.k[i], u0);
            u1 = fmaf(st[i + 1], in.k[i + 1], u1);
        }
        const float u = lanes_sum<DR_LPR>(u0 + u1) * kn;
        const float c = b * (in.v - u) * kn;
        float o0 = 0.f, o1 = 0.f;
#pragma unroll
        for (int i = 0; i < CPL; i += 2) {
            st[i] = fmaf(c, in.k[i], st[i]);
            st[i + 1] = fmaf(c, in.k[i + 1], st[i + 1]);
            o0 = fmaf(st[i], in.q[i], o0);
            o1 = fmaf(st[i + 1], in.q[i + 1], o1);
        }
        const float oo = lanes_sum<DR_LPR>(o0 + o1) * qn;
        if (cg == 0 && col_ok) p.o[(int64_t)t * p.H * p.dv + (int64_t)h * p.dv + col] = oo;
    };
    In inA, inB;
    if (t0 < t1) load_in(inA, t0);
    for (int t = t0; t < t1; t += 2) {
        if (t + 1 < t1) load_in(inB, t + 1);
        step(inA, t);
        if (t + 1 < t1) {
            if (t + 2 < t1) load_in(inA, t + 2);
            step(inB, t + 1);
        }
    }
#pragma unroll
    for (int i = 0; i < CPL; ++i)
        if (col_ok && ch0 + i < dk) S[(int64_t)(ch0 + i) * p.dv + col] = st[i];
}

template <int CPL>
static void launch_delta(const DeltaArgs& p, dim3 grid, bool vec, hipStream_t st) {
    if (vec) delta_rule_kernel<CPL, true><<<grid, 256, 0, st>>>(p);
    else delta_rule_kernel<CPL, false><<<grid, 256, 0, st>>>(p);
}

extern "C" int mi355_delta_rule_ragged(int64_t tokens, int n_seq, const int* seq_off, const int* slot, int H, int G, int dk, int dv, const void* q, const void* k, int qk_dt,
                                       int64_t ldq, int64_t ldk, const void* v, int v_dt, int64_t ldv, const void* b, const void* a, int ba_dt, int64_t ldb, int64_t lda,
                                       const float* A_log, const float* dt_bias, float qscale, float* state, float* o, float* ws, void* stream) {
    MI355_REQUIRE(tokens > 0 && n_seq > 0 && n_seq <= 65535 && seq_off && slot && H > 0 && H <= 65535 && G > 0 && H % G == 0 && dk > 0 && dk <= 32 * DR_LPR && dv > 0 && q && k && v &&
                      b && a && A_log && dt_bias && state && o && ws,
                  "delta_rule_ragged: bad arguments (key channels per head <= 256, value heads a multiple of the query / key heads, workspace of 4 floats per token and head)");
    MI355_REQUIRE(rec_dt_ok(qk_dt) && rec_dt_ok(v_dt) && rec_dt_ok(ba_dt) && ldq >= (int64_t)G * dk && ldk >= (int64_t)G * dk && ldv >= (int64_t)H * dv && ldb >= H && lda >= H,
                  "delta_rule_ragged: rows too short");
    MI355_REQUIRE(((uintptr_t)ws & 15) == 0, "delta_rule_ragged: the workspace must be 16-byte aligned");
    DeltaArgs p;
    p.seq_off = seq_off, p.slot = slot, p.q = q, p.k = k, p.v = v, p.b = b, p.a = a, p.A_log = A_log, p.dt_bias = dt_bias, p.state = state, p.o = o, p.ws = (f32x4*)ws;
    p.ldq = ldq, p.ldk = ldk, p.ldv = ldv, p.ldb = ldb, p.lda = lda, p.H = H, p.G = G, p.dk = dk, p.dv = dv, p.qk_dt = qk_dt, p.v_dt = v_dt, p.ba_dt = ba_dt, p.qscale = qscale;
    delta_prep_kernel<<<rec_rows_grid(tokens * H, 4), 256, 0, ST(stream)>>>(tokens, p);
    MI355_LAUNCH_CHECK("delta_rule_ragged(prep)");
    const bool vec = qk_dt == MI355_DT_F32 && dk % 4 == 0 && ldq % 4 == 0 && ldk % 4 == 0 && ((uintptr_t)q & 15) == 0 && ((uintptr_t)k & 15) == 0;
    const dim3 grid((dv + 31) / 32, H, n_seq);
    if (dk <= 4 * DR_LPR) launch_delta<4>(p, grid, vec, ST(stream));
    else if (dk <= 8 * DR_LPR) launch_delta<8>(p, grid, vec, ST(stream));
    else if (dk <= 16 * DR_LPR) launch_delta<16>(p, grid, vec, ST(stream));
    else launch_delta<32>(p, grid, vec, ST(stream));
    MI355_LAUNCH_CHECK("delta_rule_ragged");
    return 0;
}

// ------------------------------------------------------------------------------------------- gated feed-forward activations
// in[r] = [gate (F) | up (F)] -> out[r, i] (F wide).  kind 0: gelu_tanh(gate) * up.  kind 1: g = min(gate, limit), u = clamp(up, -limit, limit),
// out = g * sigmoid(1.702 g) * (u + 1).  kind 2: silu(gate) * up.
__global__ __launch_bounds__(256) void glu_rows_kernel(int64_t R, int F, const void* __restrict__ in, int in_dt, int64_t ldi, int kind, float limit, void* __restrict__ out,
                                                       int out_dt, int64_t ldo) {
    const int64_t total = R * F;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = e / F;
        const int i = (int)(e % F);
        float g = ldr_dt(in, in_dt, r * ldi + i), u = ldr_dt(in, in_dt, r * ldi + F + i), o;
        if (kind == 0) {
            o = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
        } else if (kind == 2) {
            o = g / (1.0f + expf(-g)) * u;
        } else {
            g = fminf(g, limit);
            u = fminf(fmaxf(u, -limit), limit);
            o = g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
        }
        str_dt(out, out_dt, r * ldo + i, o);
    }
}

__global__ __launch_bounds__(256) void glu_rows_vec_kernel(int64_t R, int F, const void* __restrict__ in, int in_dt, int64_t ldi, int kind, float limit, void* __restrict__ out,
                                                           int out_dt, int64_t ldo) {
    const int F4 = F / 4;
    const int64_t total = R * F4;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = e / F4;
        const int i = 4 * (int)(e % F4);
        const f32x4 g4 = ld4_dt(in, in_dt, r * ldi + i), u4 = ld4_dt(in, in_dt, r * ldi + F + i);
        f32x4 o;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float g = g4[q], u = u4[q];
            if (kind == 0) {
                o[q] = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
            } else if (kind == 2) {
                o[q] = g / (1.0f + expf(-g)) * u;
            } else {
                g = fminf(g, limit);
                u = fminf(fmaxf(u, -limit), limit);
                o[q] = g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
            }
        }
        st4_dt(out, out_dt, r * ldo + i, o);
    }
}

extern "C" int mi355_glu_rows(int64_t rows, int F, const void* in, int in_dt, int64_t ld_in, int kind, float limit, void* out, int out_dt, int64_t ld_out, void* stream) {
    MI355_REQUIRE(rows > 0 && F > 0 && in && out && rec_dt_ok(in_dt) && rec_dt_ok(out_dt) && ld_in >= 2 * (int64_t)F && ld_out >= F && kind >= 0 && kind <= 2, "glu_rows: bad arguments");
    if (F % 4 == 0 && ld_in % 4 == 0 && ld_out % 4 == 0 && al16(in) && al16(out)) {
        const int64_t total4 = rows * (F / 4);
        const int g4 = (int)((total4 + 255) / 256 > 65535 * 8 ? 65535 * 8 : (total4 + 255) / 256);
        glu_rows_vec_kernel<<<g4, 256, 0, ST(stream)>>>(rows, F, in, in_dt, ld_in, kind, limit, out, out_dt, ld_out);
        MI355_LAUNCH_CHECK("glu_rows");
        return 0;
    }
    const int64_t total = rows * F;
    const int g = (int)((total + 255) / 256 > 65535 * 8 ? 65535 * 8 : (total + 255) / 256);
    glu_rows_kernel<<<g, 256, 0, ST(stream)>>>(rows, F, in, in_dt, ld_in, kind, limit, out, out_dt, ld_out);
    MI355_LAUNCH_CHECK("glu_rows");
    return 0;
}
