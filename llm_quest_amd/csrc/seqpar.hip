// Row operations and recurrences of hybrid decoders whose mixers run two branches SIDE BY SIDE and whose norms take no statistics, served in ragged
// batches (gfx950 only):
//   * the residual sum with a per-channel layer scale, the join of two branch outputs (each optionally RMS-normed with its own weight, each with its own
//     factor) and of routed expert rows, and the Dynamic-Tanh norm tanh(alpha v) w + b of the sum for the next sublayer -- one kernel;
//   * token shift: several learned blends of a row with the previous token's row, the last row carried per sequence;
//   * a linear recurrence over a matrix state per head in two flavours -- read-then-update with a bonus for the current token and a decay per key channel
//     (time mixing with data-dependent decay), update-then-read with one decay per head and token, a step size on the value and a skip term (state-space duality);
//   * the real-gated linear recurrent unit: a diagonal recurrence per channel with input and recurrence gates;
//   * RMS norm in groups of a row with a full-length weight and a SiLU gate before or after it;
//   * small row-wise activations: squared ReLU, tanh, one sigmoid gate per head.
//
// Conventions as in seqmix.hip / seqrec.hip: operands come as bf16 or fp32 (a MI355_DT_* code each); the residual stream, norm statistics, decays, gates
// of a recurrence and recurrent state are fp32 in both modes.  A "row" is a token of the packed batch; sequences are described by int32 device arrays.
#include "common.h"
#include "lane_sums.h"

#define ST(s) ((hipStream_t)(s))

__device__ __forceinline__ float ldp_dt(const void* p, int dt, int64_t i) { return dt == MI355_DT_F32 ? ((const float*)p)[i] : bf2f(((const bf16_t*)p)[i]); }
__device__ __forceinline__ void stp_dt(void* p, int dt, int64_t i, float v) {
    if (dt == MI355_DT_F32) ((float*)p)[i] = v;
    else ((bf16_t*)p)[i] = f2bf(v);
}
static inline bool par_dt_ok(int dt) { return dt == MI355_DT_BF16 || dt == MI355_DT_F32; }
static inline bool par_al16(const void* p) { return ((uintptr_t)p & 15) == 0; }
static inline int par_grid(int64_t items, int per_block, int cap) {
    int64_t g = (items + per_block - 1) / per_block;
    return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}
__device__ __forceinline__ f32x4 ldp4_dt(const void* p, int dt, int64_t i) {
    if (dt == MI355_DT_F32) return *(const f32x4*)((const float*)p + i);
    const u32x2 r = *(const u32x2*)((const bf16_t*)p + i);
    return f32x4{__uint_as_float(r[0] << 16), __uint_as_float(r[0] & 0xffff0000u), __uint_as_float(r[1] << 16), __uint_as_float(r[1] & 0xffff0000u)};
}
__device__ __forceinline__ void stp4_dt(void* p, int dt, int64_t i, f32x4 v) {
    if (dt == MI355_DT_F32) *(f32x4*)((float*)p + i) = v;
    else *(u32x2*)((bf16_t*)p + i) = u32x2{pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3])};
}
__device__ __forceinline__ float softplus_p(float a) { return a > 20.f ? a : log1pf(expf(a)); }
__device__ __forceinline__ float silu_p(float g) { return g / (1.0f + expf(-g)); }

// ------------------------------------------------------------------------------------------- residual sum, branch join, Dynamic-Tanh norm
// y = ca * N_a(ya[t]) + cb * N_b(yb[t]) + sum_{p < parts} y2[t * parts + p];  N(y) = y / sqrt(mean(y^2) + eps) * w_n if the branch has a norm weight, else y.
// v = x[t] + ls * y (ls fp32 [width] or absent: 1);  x_out <- v;  out <- tanh(alpha * v) * w + b (dtype out_dt), out32 <- the same in fp32.
// One wave per row.
struct DytArgs {
    const float* x;
    float* x_out;
    const void *ya, *yb, *y2;
    int64_t ldya, ldyb, ldy2;
    int ya_dt, yb_dt, y2_dt, parts;
    const float *wa, *wb, *ls, *w, *b;
    float ca, cb, eps, alpha;
    void* out;
    float* out32;
    int out_dt;
};

// Rows of fp32 / bf16 words that are 16-byte aligned, NIT trips of 256 entries per wave (width <= 256 NIT): the branch rows stay in registers between the
// pass that sums their squares and the pass that joins them, and the vectors (layer scale, weights, bias) come as 16-byte words.  NIT == 0: any width, the
// branch rows are read twice.
template <int NIT>
__global__ __launch_bounds__(256) void dyt_sum_vec_kernel(int64_t T, int width, DytArgs p) {
    const int lane = threadIdx.x & 63;
    constexpr int NR = NIT > 0 ? NIT : 1;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    auto ssq = [](f32x4 a) { return a[0] * a[0] + a[1] * a[1] + a[2] * a[2] + a[3] * a[3]; };
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += (int64_t)gridDim.x * 4) {
        f32x4 ka[NR], kb[NR];
        float ra = 1.f, rb = 1.f, sa = 0.f, sb = 0.f;
        if constexpr (NIT > 0) {
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                const int i = (it * 64 + lane) * 4;
                ka[it] = (p.ya && i < width) ? ldp4_dt(p.ya, p.ya_dt, t * p.ldya + i) : zero;
                kb[it] = (p.yb && i < width) ? ldp4_dt(p.yb, p.yb_dt, t * p.ldyb + i) : zero;
                sa += ssq(ka[it]), sb += ssq(kb[it]);
            }
        } else {
            for (int i = lane * 4; i < width; i += 256) {
                if (p.ya && p.wa) sa += ssq(ldp4_dt(p.ya, p.ya_dt, t * p.ldya + i));
                if (p.yb && p.wb) sb += ssq(ldp4_dt(p.yb, p.yb_dt, t * p.ldyb + i));
            }
        }
        if (p.ya && p.wa) ra = 1.0f / sqrtf(wave_sum(sa) / (float)width + p.eps);
        if (p.yb && p.wb) rb = 1.0f / sqrtf(wave_sum(sb) / (float)width + p.eps);
        const bool any = p.ya || p.yb || p.y2;
        auto finish = [&](int i, f32x4 a, f32x4 bq) {
            f32x4 v = *(const f32x4*)(p.x + t * width + i), y = zero;
            if (p.ya) {
                if (p.wa) a = a * ra * *(const f32x4*)(p.wa + i);
                y += p.ca * a;
            }
            if (p.yb) {
                if (p.wb) bq = bq * rb * *(const f32x4*)(p.wb + i);
                y += p.cb * bq;
            }
            if (p.y2)
                for (int q = 0; q < p.parts; ++q) y += ldp4_dt(p.y2, p.y2_dt, (t * p.parts + q) * p.ldy2 + i);
            if (any) v += p.ls ? *(const f32x4*)(p.ls + i) * y : y;
            if (p.x_out) *(f32x4*)(p.x_out + t * width + i) = v;
            if (p.w) {
                const f32x4 w4 = *(const f32x4*)(p.w + i), b4 = *(const f32x4*)(p.b + i);
                f32x4 h;
#pragma unroll
                for (int e = 0; e < 4; ++e) h[e] = tanhf(p.alpha * v[e]) * w4[e] + b4[e];
                if (p.out) stp4_dt(p.out, p.out_dt, t * width + i, h);
                if (p.out32) *(f32x4*)(p.out32 + t * width + i) = h;
            }
        };
        if constexpr (NIT > 0) {
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                const int i = (it * 64 + lane) * 4;
                if (i < width) finish(i, ka[it], kb[it]);
            }
        } else {
            for (int i = lane * 4; i < width; i += 256)
                finish(i, p.ya ? ldp4_dt(p.ya, p.ya_dt, t * p.ldya + i) : zero, p.yb ? ldp4_dt(p.yb, p.yb_dt, t * p.ldyb + i) : zero);
        }
    }
}

// Any alignment, one entry per lane and trip.
__global__ __launch_bounds__(256) void dyt_sum_kernel(int64_t T, int width, DytArgs p) {
    const int lane = threadIdx.x & 63;
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += (int64_t)gridDim.x * 4) {
        float ra = 1.f, rb = 1.f;
        if (p.ya && p.wa) {
            float s = 0.f;
            for (int i = lane; i < width; i += 64) {
                const float a = ldp_dt(p.ya, p.ya_dt, t * p.ldya + i);
                s += a * a;
            }
            ra = 1.0f / sqrtf(wave_sum(s) / (float)width + p.eps);
        }
        if (p.yb && p.wb) {
            float s = 0.f;
            for (int i = lane; i < width; i += 64) {
                const float a = ldp_dt(p.yb, p.yb_dt, t * p.ldyb + i);
                s += a * a;
            }
            rb = 1.0f / sqrtf(wave_sum(s) / (float)width + p.eps);
        }
        for (int i = lane; i < width; i += 64) {
            float v = p.x[t * width + i], y = 0.f;
            if (p.ya) {
                const float a = ldp_dt(p.ya, p.ya_dt, t * p.ldya + i);
                y += p.ca * (p.wa ? a * ra * p.wa[i] : a);
            }
            if (p.yb) {
                const float a = ldp_dt(p.yb, p.yb_dt, t * p.ldyb + i);
                y += p.cb * (p.wb ? a * rb * p.wb[i] : a);
            }
            if (p.y2)
                for (int q = 0; q < p.parts; ++q) y += ldp_dt(p.y2, p.y2_dt, (t * p.parts + q) * p.ldy2 + i);
            if (p.ya || p.yb || p.y2) v += p.ls ? p.ls[i] * y : y;
            if (p.x_out) p.x_out[t * width + i] = v;
            if (p.w) {
                const float h = tanhf(p.alpha * v) * p.w[i] + p.b[i];
                if (p.out) stp_dt(p.out, p.out_dt, t * width + i, h);
                if (p.out32) p.out32[t * width + i] = h;
            }
        }
    }
}

extern "C" int mi355_dyt_sum(int64_t tokens, int width, const float* x, const void* ya, int ya_dt, int64_t ldya, const float* wa, float ca, const void* yb, int yb_dt,
                             int64_t ldyb, const float* wb, float cb, const void* y2, int y2_dt, int64_t ldy2, int parts, const float* ls, float eps, float* x_out, float alpha,
                             const float* w, const float* b, void* out, int out_dt, float* out32, void* stream) {
    MI355_REQUIRE(tokens > 0 && width > 0 && x, "dyt_sum: bad arguments");
    MI355_REQUIRE((!ya || (par_dt_ok(ya_dt) && ldya >= width)) && (!yb || (par_dt_ok(yb_dt) && ldyb >= width)) && (!y2 || (par_dt_ok(y2_dt) && ldy2 >= width && parts >= 1)),
                  "dyt_sum: bad summands");
    MI355_REQUIRE((w != nullptr) == (b != nullptr) && (!w || out || out32) && (!out || par_dt_ok(out_dt)), "dyt_sum: the norm takes a weight, a bias and an output");
    DytArgs p;
    p.x = x, p.x_out = x_out, p.ya = ya, p.yb = yb, p.y2 = y2, p.ldya = ldya, p.ldyb = ldyb, p.ldy2 = ldy2;
    p.ya_dt = ya_dt, p.yb_dt = yb_dt, p.y2_dt = y2_dt, p.parts = parts;
    p.wa = wa, p.wb = wb, p.ls = ls, p.w = w, p.b = b, p.ca = ca, p.cb = cb, p.eps = eps, p.alpha = alpha;
    p.out = out, p.out32 = out32, p.out_dt = out_dt;
    const bool vec = width % 4 == 0 && par_al16(x) && par_al16(x_out) && par_al16(ya) && par_al16(yb) && par_al16(y2) && par_al16(out) && par_al16(out32) && ldya % 4 == 0 &&
                     ldyb % 4 == 0 && ldy2 % 4 == 0 && par_al16(wa) && par_al16(wb) && par_al16(ls) && par_al16(w) && par_al16(b);
    const int grid = par_grid(tokens, 4, 65535 * 16);
    if (!vec) dyt_sum_kernel<<<grid, 256, 0, ST(stream)>>>(tokens, width, p);
    else if (width <= 256) dyt_sum_vec_kernel<1><<<grid, 256, 0, ST(stream)>>>(tokens, width, p);
    else if (width <= 512) dyt_sum_vec_kernel<2><<<grid, 256, 0, ST(stream)>>>(tokens, width, p);
    else if (width <= 1024) dyt_sum_vec_kernel<4><<<grid, 256, 0, ST(stream)>>>(tokens, width, p);
    else if (width <= 2048) dyt_sum_vec_kernel<8><<<grid, 256, 0, ST(stream)>>>(tokens, width, p);
    else dyt_sum_vec_kernel<0><<<grid, 256, 0, ST(stream)>>>(tokens, width, p);
    MI355_LAUNCH_CHECK("dyt_sum");
    return 0;
}

// ------------------------------------------------------------------------------------------- token shift
// out[t, s * C + c] = h[t, c] + (h'[t, c] - h[t, c]) * mu[s * C + c] for s < n_mix, h' the previous token's row of the same sequence: this step's, or -- for
// the step's first row -- state[slot, c] (fp32 [slots, C], zeros before the sequence's start).  Afterwards the state takes the step's last row.
__global__ __launch_bounds__(256) void token_shift_kernel(int64_t T, int C, int n_mix, const float* __restrict__ h, int64_t ldh, const float* __restrict__ mu,
                                                          const int* __restrict__ row_seq, const int* __restrict__ seq_off, const int* __restrict__ slot,
                                                          const float* __restrict__ state, void* __restrict__ out, int out_dt, int64_t ldo) {
    const int64_t total = T * C;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = e / C;
        const int c = (int)(e % C);
        const int s = row_seq[t];
        const float cur = h[t * ldh + c];
        const float prev = t > seq_off[s] ? h[(t - 1) * ldh + c] : state[(int64_t)slot[s] * C + c];
        const float d = prev - cur;
        for (int m = 0; m < n_mix; ++m) stp_dt(out, out_dt, t * ldo + (int64_t)m * C + c, cur + d * mu[(int64_t)m * C + c]);
    }
}
__global__ __launch_bounds__(256) void token_shift_state_kernel(int n_seq, int C, const float* __restrict__ h, int64_t ldh, const int* __restrict__ seq_off,
                                                                const int* __restrict__ slot, float* __restrict__ state) {
    const int64_t total = (int64_t)n_seq * C;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int s = (int)(e / C), c = (int)(e % C);
        state[(int64_t)slot[s] * C + c] = h[(int64_t)(seq_off[s + 1] - 1) * ldh + c];
    }
}

extern "C" int mi355_token_shift(int64_t tokens, int n_seq, int C, int n_mix, const float* h, int64_t ldh, const float* mu, const int* row_seq, const int* seq_off,
                                 const int* slot, float* state, void* out, int out_dt, int64_t ldo, void* stream) {
    MI355_REQUIRE(tokens > 0 && n_seq > 0 && C > 0 && n_mix > 0 && h && mu && row_seq && seq_off && slot && state && out && par_dt_ok(out_dt) && ldh >= C &&
                      ldo >= (int64_t)n_mix * C,
                  "token_shift: bad arguments");
    token_shift_kernel<<<par_grid(tokens * C, 256, 65535 * 8), 256, 0, ST(stream)>>>(tokens, C, n_mix, h, ldh, mu, row_seq, seq_off, slot, state, out, out_dt, ldo);
    MI355_LAUNCH_CHECK("token_shift");
    token_shift_state_kernel<<<par_grid((int64_t)n_seq * C, 256, 65535 * 8), 256, 0, ST(stream)>>>(n_seq, C, h, ldh, seq_off, slot, state);
    MI355_LAUNCH_CHECK("token_shift(state)");
    return 0;
}

// ------------------------------------------------------------------------------------------- linear recurrence over a matrix state per head
// Per head a state S [dk, dv] (fp32, carried per sequence slot).  Query / key head of value head h: h / qk_rep.
//   POST == false (read, then update; bonus):  o_t = S^T q_t + (sum_i q_i u_i k_i) v_t;  S <- diag(a_t) S + k_t v_t^T,  a_t[i] = exp(-exp(z[t, h, i]))
//   POST == true  (update, then read; skip):   dt = softplus(z[t, h] + dt_bias[h]);  S <- exp(-exp(A_log[h]) dt) S + k_t (dt v_t)^T;  o_t = S^T q_t + D[h] v_t
// Block: 64 value columns x RC row chunks of LR_R (8 or 16) key channels; a thread keeps LR_R state entries of one column in registers.  Tokens go through in
// groups of LR_TB: the group's q / k / decay rows are staged in LDS once (the next group's travel from memory meanwhile), partial sums of the row
// chunks meet in LDS.
#define LR_TB 8
struct LinRecArgs {
    const int *seq_off, *slot;
    int H, dk, dv, qk_rep;
    const void *q, *k, *v;
    const float* z;
    int q_dt, v_dt;
    int64_t ldq, ldk, ldv, ldz;
    const float *u, *dt_bias, *A_log, *D;
    float* state;
    float* o;
};

template <bool POST, int LR_R>
__global__ void linrec_kernel(LinRecArgs p) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int RC = blockDim.x >> 6, dk = p.dk, dv = p.dv, H = p.H;
    float* sq = smem;                    // [TB][dk]
    float* sk = sq + LR_TB * dk;         // [TB][dk]
    float* sa = sk + LR_TB * dk;         // [TB][dk]
    float* sv = sa + LR_TB * dk;         // [TB][64]
    float* sp = sv + LR_TB * 64;         // [TB][RC][64]
    float* sb = sp + LR_TB * RC * 64;    // [TB]: the bonus sum (read-then-update) or the step size (update-then-read)
    const int s = blockIdx.x, h = blockIdx.y, col = blockIdx.z * 64 + (threadIdx.x & 63), chunk = threadIdx.x >> 6;
    const int hq = h / p.qk_rep;
    const int t0 = p.seq_off[s], t1 = p.seq_off[s + 1];
    const bool col_ok = col < dv;
    float* S = p.state + (((int64_t)p.slot[s] * H + h) * dk) * dv;
    float st[LR_R];
#pragma unroll
    for (int r = 0; r < LR_R; ++r) {
        const int i = chunk * LR_R + r;
        st[r] = (col_ok && i < dk) ? S[(int64_t)i * dv + col] : 0.f;
    }
    const float negA = POST ? -expf(p.A_log[h]) : 0.f, dtb = POST ? p.dt_bias[h] : 0.f, skip = POST ? p.D[h] : 0.f;
    float rq[2], rk[2], rz[2], rv[8], rdt = 0.f;
    auto fetch = [&](int tb) {
        const int nt = min(LR_TB, t1 - tb);
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            const int e = threadIdx.x + w * blockDim.x;
            rq[w] = rk[w] = rz[w] = 0.f;
            if (e < nt * dk) {
                const int j = e / dk, i = e % dk;
                const int64_t t = tb + j;
                rq[w] = ldp_dt(p.q, p.q_dt, t * p.ldq + (int64_t)hq * dk + i);
                rk[w] = ldp_dt(p.k, p.q_dt, t * p.ldk + (int64_t)hq * dk + i);
                if (!POST) rz[w] = p.z[t * p.ldz + (int64_t)h * dk + i];
            }
        }
        if (POST && threadIdx.x < nt) rdt = p.z[(int64_t)(tb + threadIdx.x) * p.ldz + h];
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            const int e = threadIdx.x + w * blockDim.x;
            rv[w] = 0.f;
            if (e < nt * 64) {
                const int j = e >> 6, c = blockIdx.z * 64 + (e & 63);
                if (c < dv) rv[w] = ldp_dt(p.v, p.v_dt, (int64_t)(tb + j) * p.ldv + (int64_t)h * dv + c);
            }
        }
    };
    if (t0 < t1) fetch(t0);
    for (int tb = t0; tb < t1; tb += LR_TB) {
        const int nt = min(LR_TB, t1 - tb);
        __syncthreads();  // the previous group's rows and partial sums are consumed
        if (POST && threadIdx.x < nt) sb[threadIdx.x] = softplus_p(rdt + dtb);
        if (POST) __syncthreads();
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            const int e = threadIdx.x + w * blockDim.x;
            if (e < nt * dk) {
                sq[e] = rq[w];
                sk[e] = rk[w];
                sa[e] = POST ? expf(negA * sb[e / dk]) : expf(-expf(rz[w]));
            }
        }
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            const int e = threadIdx.x + w * blockDim.x;
            if (e < nt * 64) sv[e] = rv[w];
        }
        __syncthreads();
        if (tb + LR_TB < t1) fetch(tb + LR_TB);
        if (!POST && threadIdx.x < 64) {  // the bonus sums of the group's tokens: 8 lanes per token
            const int j = threadIdx.x >> 3, part = threadIdx.x & 7;
            float b = 0.f;
            if (j < nt)
                for (int i = part; i < dk; i += 8) b += sq[j * dk + i] * sk[j * dk + i] * p.u[(int64_t)h * dk + i];
            b = lanes_sum<8>(b);
            if (part == 0 && j < nt) sb[j] = b;
        }
        const bool full = chunk * LR_R + LR_R <= dk && dk % 4 == 0;
        for (int j = 0; j < nt; ++j) {
            const float vraw = sv[j * 64 + (threadIdx.x & 63)];
            const float vv = POST ? vraw * sb[j] : vraw;
            const float* qa = sq + j * dk + chunk * LR_R;
            const float* ka = sk + j * dk + chunk * LR_R;
            const float* aa = sa + j * dk + chunk * LR_R;
            const float a1 = POST ? sa[j * dk] : 0.f;  // update-then-read: one decay for all key channels of the head
            float acc = 0.f;
            if (full) {
#pragma unroll
                for (int r4 = 0; r4 < LR_R / 4; ++r4) {
                    const f32x4 q4 = *(const f32x4*)(qa + 4 * r4), k4 = *(const f32x4*)(ka + 4 * r4);
                    if constexpr (POST) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            st[4 * r4 + i] = a1 * st[4 * r4 + i] + k4[i] * vv;
                            acc += st[4 * r4 + i] * q4[i];
                        }
                    } else {
                        const f32x4 a4 = *(const f32x4*)(aa + 4 * r4);
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            acc += st[4 * r4 + i] * q4[i];
                            st[4 * r4 + i] = a4[i] * st[4 * r4 + i] + k4[i] * vv;
                        }
                    }
                }
            } else {
#pragma unroll
                for (int r = 0; r < LR_R; ++r) {
                    if (chunk * LR_R + r < dk) {
                        if (POST) {
                            st[r] = aa[r] * st[r] + ka[r] * vv;
                            acc += st[r] * qa[r];
                        } else {
                            acc += st[r] * qa[r];
                            st[r] = aa[r] * st[r] + ka[r] * vv;
                        }
                    }
                }
            }
            sp[(j * RC + chunk) * 64 + (threadIdx.x & 63)] = acc;
        }
        __syncthreads();
        for (int e = threadIdx.x; e < nt * 64; e += blockDim.x) {
            const int j = e >> 6, c = blockIdx.z * 64 + (e & 63);
            if (c < dv) {
                float acc = 0.f;
                for (int rc = 0; rc < RC; ++rc) acc += sp[(j * RC + rc) * 64 + (e & 63)];
                acc += (POST ? skip : sb[j]) * sv[e];
                p.o[(int64_t)(tb + j) * H * dv + (int64_t)h * dv + c] = acc;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < LR_R; ++r) {
        const int i = chunk * LR_R + r;
        if (col_ok && i < dk) S[(int64_t)i * dv + col] = st[r];
    }
}

extern "C" int mi355_linrec_ragged(int n_seq, const int* seq_off, const int* slot, int H, int qk_rep, int dk, int dv, const void* q, const void* k, int q_dt, int64_t ldq,
                                   int64_t ldk, const void* v, int v_dt, int64_t ldv, const float* z, int64_t ldz, int post, const float* u, const float* dt_bias,
                                   const float* A_log, const float* D, float* state, float* o, void* stream) {
    MI355_REQUIRE(n_seq > 0 && n_seq <= 65535 && seq_off && slot && H > 0 && H <= 65535 && qk_rep >= 1 && H % qk_rep == 0 && dk > 0 && dk <= 256 && dv > 0 && q && k &&
                      v && z && state && o && par_dt_ok(q_dt) && par_dt_ok(v_dt),
                  "linrec_ragged: bad arguments (key channels per head <= 256)");
    MI355_REQUIRE(post ? (dt_bias && A_log && D && ldz >= H) : (u && ldz >= (int64_t)H * dk), "linrec_ragged: the update-then-read form takes dt_bias, A_log and D, the other one the bonus");
    MI355_REQUIRE(ldq >= (int64_t)(H / qk_rep) * dk && ldk >= (int64_t)(H / qk_rep) * dk && ldv >= (int64_t)H * dv, "linrec_ragged: rows too short");
    // few key channels per head: eight per thread instead of sixteen, twice the waves to hide the chain's latencies behind
    const int R = dk <= 64 ? 8 : 16;
    const int RC = (dk + R - 1) / R;
    const size_t lds_bytes = sizeof(float) * ((size_t)3 * LR_TB * dk + (size_t)LR_TB * 64 + (size_t)LR_TB * RC * 64 + LR_TB);
    MI355_REQUIRE(lds_bytes <= 64 * 1024, "linrec_ragged: LDS budget exceeded");
    LinRecArgs p;
    p.seq_off = seq_off, p.slot = slot, p.H = H, p.dk = dk, p.dv = dv, p.qk_rep = qk_rep, p.q = q, p.k = k, p.v = v, p.z = z, p.q_dt = q_dt, p.v_dt = v_dt;
    p.ldq = ldq, p.ldk = ldk, p.ldv = ldv, p.ldz = ldz, p.u = u, p.dt_bias = dt_bias, p.A_log = A_log, p.D = D, p.state = state, p.o = o;
    const dim3 grid(n_seq, H, (dv + 63) / 64);
    if (post && R == 8) linrec_kernel<true, 8><<<grid, 64 * RC, lds_bytes, ST(stream)>>>(p);
    else if (post) linrec_kernel<true, 16><<<grid, 64 * RC, lds_bytes, ST(stream)>>>(p);
    else if (R == 8) linrec_kernel<false, 8><<<grid, 64 * RC, lds_bytes, ST(stream)>>>(p);
    else linrec_kernel<false, 16><<<grid, 64 * RC, lds_bytes, ST(stream)>>>(p);
    MI355_LAUNCH_CHECK("linrec_ragged");
    return 0;
}

// ------------------------------------------------------------------------------------------- real-gated linear recurrent unit
// Per channel c (block b = c / n of n = C / blocks channels, j = c % n): r = sigmoid(gates[t, b * 2n + j] + gbias[b * 2n + j]), i = sigmoid(gates[t, b * 2n + n + j]
// + gbias[b * 2n + n + j]) (gbias fp32 [2 C] in the gates' layout, may be null);
// log a = -decay_c * r * softplus(lam[c]);  S <- a S + sqrt(1 - a^2) * (i * u[t, c]);  out[t, c] = S * gelu_tanh(y[t, c]).  1 - a^2 = -expm1(2 log a).
// state fp32 [slots, C].
#define RG_TB 8  // tokens per wave and tile
#define RG_W 8   // waves of a workgroup: a tile is RG_W * RG_TB consecutive tokens of one sequence
// Workgroup = 64 channels (lanes) x RG_W waves.  The recurrence S <- a S + b is linear in S, so wave w scans its RG_TB tokens of the tile from zero
// (local values L_q and the running products P_q of the decays), the waves exchange (P, L) of their last token through LDS, every wave folds what
// lies before it onto the state the tile came in with, and S_q = L_q + P_q * S_in.  The next tile's rows are requested before the current tile's arithmetic.
__global__ __launch_bounds__(64 * RG_W) void rglru_kernel(int n_seq, int C, int n, float decay_c, const float* __restrict__ u, int64_t ldu, const float* __restrict__ gates,
                                                          int64_t ldg, const float* __restrict__ gbias, const float* __restrict__ lam, const void* __restrict__ y, int y_dt,
                                                          int64_t ldy, const int* __restrict__ seq_off, const int* __restrict__ slot, float* __restrict__ state,
                                                          void* __restrict__ out, int out_dt, int64_t ldo) {
    __shared__ float sP[RG_W][64], sL[RG_W][64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int ctiles = (C + 63) / 64;
    const int s = blockIdx.x / ctiles, c = (blockIdx.x % ctiles) * 64 + lane;
    const bool ok = c < C;
    const int cc = ok ? c : 0;
    const int b = cc / n, j = cc % n;
    const int64_t gr = (int64_t)b * 2 * n + j, gi = gr + n;
    const float sp = decay_c * softplus_p(lam[cc]);
    const float br = gbias ? gbias[gr] : 0.f, bi = gbias ? gbias[gi] : 0.f;
    float S = state[(int64_t)slot[s] * C + cc];  // the state the tile comes in with (every wave keeps its own copy)
    const int t0 = seq_off[s], t1 = seq_off[s + 1];
    float nu[RG_TB], nr[RG_TB], ni[RG_TB], ny[RG_TB];
    auto fetch = [&](int tb) {
#pragma unroll
        for (int q = 0; q < RG_TB; ++q) {
            const int64_t t = min(tb + q, t1 - 1);
            nu[q] = u[t * ldu + cc], nr[q] = gates[t * ldg + gr], ni[q] = gates[t * ldg + gi], ny[q] = ldp_dt(y, y_dt, t * ldy + cc);
        }
    };
    if (t0 + w * RG_TB < t1) fetch(t0 + w * RG_TB);
    for (int tile = t0; tile < t1; tile += RG_W * RG_TB) {
        const int tb = tile + w * RG_TB;  // this wave's first token
        float P[RG_TB], L[RG_TB], gv[RG_TB];
        float pa = 1.f, ls = 0.f;
#pragma unroll
        for (int q = 0; q < RG_TB; ++q) {
            if (tb + q < t1) {
                const float r = 1.0f / (1.0f + expf(-(nr[q] + br))), g = 1.0f / (1.0f + expf(-(ni[q] + bi)));
                const float la = -sp * r, av = expf(la);
                ls = av * ls + sqrtf(-expm1f(2.0f * la)) * (g * nu[q]);
                pa *= av;
                gv[q] = gelu_val<1>(ny[q]);
            }
            P[q] = pa, L[q] = ls;
        }
        if (tb + RG_W * RG_TB < t1) fetch(tb + RG_W * RG_TB);
        sP[w][lane] = pa, sL[w][lane] = ls;  // a wave whose tokens lie past the sequence's end leaves (1, 0): the identity
        __syncthreads();
        float sin = S, send = S;
#pragma unroll
        for (int v = 0; v < RG_W; ++v) {
            send = sP[v][lane] * send + sL[v][lane];
            if (v + 1 == w) sin = send;
        }
#pragma unroll
        for (int q = 0; q < RG_TB; ++q)
            if (ok && tb + q < t1) stp_dt(out, out_dt, (int64_t)(tb + q) * ldo + c, (L[q] + P[q] * sin) * gv[q]);
        S = send;
        __syncthreads();
    }
    if (ok && w == 0) state[(int64_t)slot[s] * C + c] = S;
}

extern "C" int mi355_rglru_ragged(int n_seq, int C, int blocks, float decay_c, const float* u, int64_t ldu, const float* gates, int64_t ldg, const float* gbias, const float* lam,
                                  const void* y, int y_dt, int64_t ldy, const int* seq_off, const int* slot, float* state, void* out, int out_dt, int64_t ldo, void* stream) {
    MI355_REQUIRE(n_seq > 0 && C > 0 && blocks > 0 && C % blocks == 0 && u && gates && lam && y && seq_off && slot && state && out && par_dt_ok(y_dt) && par_dt_ok(out_dt) &&
                      ldu >= C && ldg >= 2 * (int64_t)C && ldy >= C && ldo >= C && (int64_t)n_seq * ((C + 63) / 64) < ((int64_t)1 << 31),
                  "rglru_ragged: bad arguments");
    rglru_kernel<<<(unsigned)((int64_t)n_seq * ((C + 63) / 64)), 64 * RG_W, 0, ST(stream)>>>(n_seq, C, C / blocks, decay_c, u, ldu, gates, ldg, gbias, lam, y, y_dt, ldy, seq_off, slot, state,
                                                                                       out, out_dt, ldo);
    MI355_LAUNCH_CHECK("rglru_ragged");
    return 0;
}

// ------------------------------------------------------------------------------------------- RMS norm in groups with a SiLU gate
// o fp32 [T, n] cut into `groups` equal consecutive groups; w fp32 [n].  gate_first 0: out = o / rms_group(o) * w * silu(gate);
// gate_first 1: g = o * silu(gate), out = g / rms_group(g) * w.  One wave per (row, group).
__global__ __launch_bounds__(256) void gated_groupnorm_kernel(int64_t T, int n, int groups, const float* __restrict__ o, int64_t ldo_in, const float* __restrict__ w,
                                                              const void* __restrict__ gate, int g_dt, int64_t ldg, int gate_first, float eps, void* __restrict__ out,
                                                              int out_dt, int64_t ldo) {
    const int lane = threadIdx.x & 63, gs = n / groups;
    const int64_t items = T * groups;
    for (int64_t it = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); it < items; it += (int64_t)gridDim.x * 4) {
        const int64_t t = it / groups;
        const int c0 = (int)(it % groups) * gs;
        float s = 0.f;
        for (int i = lane; i < gs; i += 64) {
            float a = o[t * ldo_in + c0 + i];
            if (gate_first) a *= silu_p(ldp_dt(gate, g_dt, t * ldg + c0 + i));
            s += a * a;
        }
        const float r = 1.0f / sqrtf(wave_sum(s) / (float)gs + eps);
        for (int i = lane; i < gs; i += 64) {
            const float sg = silu_p(ldp_dt(gate, g_dt, t * ldg + c0 + i));
            stp_dt(out, out_dt, t * ldo + c0 + i, o[t * ldo_in + c0 + i] * sg * r * w[c0 + i]);
        }
    }
}

extern "C" int mi355_gated_groupnorm(int64_t tokens, int n, int groups, const float* o, int64_t ldo_in, const float* w, const void* gate, int g_dt, int64_t ldg, int gate_first,
                                     float eps, void* out, int out_dt, int64_t ldo, void* stream) {
    MI355_REQUIRE(tokens > 0 && n > 0 && groups > 0 && n % groups == 0 && o && w && gate && out && par_dt_ok(g_dt) && par_dt_ok(out_dt) && ldo_in >= n && ldg >= n && ldo >= n,
                  "gated_groupnorm: bad arguments");
    gated_groupnorm_kernel<<<par_grid(tokens * groups, 4, 65535 * 16), 256, 0, ST(stream)>>>(tokens, n, groups, o, ldo_in, w, gate, g_dt, ldg, gate_first, eps, out, out_dt, ldo);
    MI355_LAUNCH_CHECK("gated_groupnorm");
    return 0;
}

// ------------------------------------------------------------------------------------------- small row-wise activations
// kind 0: relu(x)^2.  kind 1: tanh(x).  kind 2: x[r, i] * sigmoid(gate[r, i / group]) -- one gate per run of `group` entries (a head).
__global__ __launch_bounds__(256) void unary_rows_kernel(int64_t R, int n, const void* __restrict__ x, int x_dt, int64_t ldx, int kind, const void* __restrict__ gate, int g_dt,
                                                         int64_t ldg, int group, void* __restrict__ out, int out_dt, int64_t ldo) {
    const int64_t total = R * n;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = e / n;
        const int i = (int)(e % n);
        const float a = ldp_dt(x, x_dt, r * ldx + i);
        float v;
        if (kind == 0) v = a > 0.f ? a * a : 0.f;
        else if (kind == 1) v = tanhf(a);
        else v = a / (1.0f + expf(-ldp_dt(gate, g_dt, r * ldg + i / group)));
        stp_dt(out, out_dt, r * ldo + i, v);
    }
}
template <int KIND>
__global__ __launch_bounds__(256) void unary_rows_vec_kernel(int64_t R, int n, const void* __restrict__ x, int x_dt, int64_t ldx, const void* __restrict__ gate, int g_dt,
                                                             int64_t ldg, int group, void* __restrict__ out, int out_dt, int64_t ldo) {
    const int n4 = n / 4;
    const int64_t total = R * n4;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = e / n4;
        const int i = 4 * (int)(e % n4);
        f32x4 a = ldp4_dt(x, x_dt, r * ldx + i);
        if constexpr (KIND == 2) {  // four neighbours share a gate (group is a multiple of 4)
            const float sg = 1.0f / (1.0f + expf(-ldp_dt(gate, g_dt, r * ldg + i / group)));
            a = a * sg;
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) a[q] = KIND == 0 ? (a[q] > 0.f ? a[q] * a[q] : 0.f) : tanhf(a[q]);
        }
        stp4_dt(out, out_dt, r * ldo + i, a);
    }
}

extern "C" int mi355_unary_rows(int64_t rows, int n, const void* x, int x_dt, int64_t ldx, int kind, const void* gate, int g_dt, int64_t ldg, int group, void* out,
                                int out_dt, int64_t ldo, void* stream) {
    MI355_REQUIRE(rows > 0 && n > 0 && x && out && par_dt_ok(x_dt) && par_dt_ok(out_dt) && ldx >= n && ldo >= n && kind >= 0 && kind <= 2, "unary_rows: bad arguments");
    MI355_REQUIRE(kind != 2 || (gate && par_dt_ok(g_dt) && group >= 1 && ldg >= (n + group - 1) / group), "unary_rows: a head gate needs its rows and the head size");
    if ((kind < 2 || group % 4 == 0) && n % 4 == 0 && ldx % 4 == 0 && ldo % 4 == 0 && par_al16(x) && par_al16(out)) {
        const int g4 = par_grid(rows * (n / 4), 256, 65535 * 8);
        if (kind == 0) unary_rows_vec_kernel<0><<<g4, 256, 0, ST(stream)>>>(rows, n, x, x_dt, ldx, gate, g_dt, ldg, group, out, out_dt, ldo);
        else if (kind == 1) unary_rows_vec_kernel<1><<<g4, 256, 0, ST(stream)>>>(rows, n, x, x_dt, ldx, gate, g_dt, ldg, group, out, out_dt, ldo);
        else unary_rows_vec_kernel<2><<<g4, 256, 0, ST(stream)>>>(rows, n, x, x_dt, ldx, gate, g_dt, ldg, group, out, out_dt, ldo);
        MI355_LAUNCH_CHECK("unary_rows");
        return 0;
    }
    unary_rows_kernel<<<par_grid(rows * n, 256, 65535 * 8), 256, 0, ST(stream)>>>(rows, n, x, x_dt, ldx, kind, gate, g_dt, ldg, group, out, out_dt, ldo);
    MI355_LAUNCH_CHECK("unary_rows");
    return 0;
}
