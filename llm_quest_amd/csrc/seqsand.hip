// Row operations of decoders with SANDWICH norms (a norm before and after every sublayer), served in ragged batches (gfx950 only): the residual sum
// that first norms the sublayer's output and then norms the new residual row for the next sublayer, the pooled (mean) key / value rows of attention
// that sees old tokens only block-wise, and un-gated activations / output gates on rows.
//
// Conventions as in seqmix.hip / seqrec.hip: operands come as bf16 or fp32 (a MI355_DT_* code each); the residual stream and every norm statistic are
// fp32 in both modes.  A "row" is a token of the packed batch; sequences are described by int32 device arrays.
#include "common.h"
#include "lane_sums.h"

#define ST(s) ((hipStream_t)(s))

__device__ __forceinline__ float lds_dt(const void* p, int dt, int64_t i) { return dt == MI355_DT_F32 ? ((const float*)p)[i] : bf2f(((const bf16_t*)p)[i]); }
__device__ __forceinline__ void sts_dt(void* p, int dt, int64_t i, float v) {
    if (dt == MI355_DT_F32) ((float*)p)[i] = v;
    else ((bf16_t*)p)[i] = f2bf(v);
}
__device__ __forceinline__ f32x4 lds4_dt(const void* p, int dt, int64_t i) {
    if (dt == MI355_DT_F32) return *(const f32x4*)((const float*)p + i);
    const u32x2 r = *(const u32x2*)((const bf16_t*)p + i);
    return f32x4{__uint_as_float(r[0] << 16), __uint_as_float(r[0] & 0xffff0000u), __uint_as_float(r[1] << 16), __uint_as_float(r[1] & 0xffff0000u)};
}
__device__ __forceinline__ void sts4_dt(void* p, int dt, int64_t i, f32x4 v) {
    if (dt == MI355_DT_F32) *(f32x4*)((float*)p + i) = v;
    else *(u32x2*)((bf16_t*)p + i) = u32x2{pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3])};
}
static inline bool sand_dt_ok(int dt) { return dt == MI355_DT_BF16 || dt == MI355_DT_F32; }
static inline bool sand_al16(const void* p) { return ((uintptr_t)p & 15) == 0; }
static inline int sand_grid(int64_t items, int per_block, int64_t cap) {
    int64_t g = (items + per_block - 1) / per_block;
    return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

// ------------------------------------------------------------------------------------------- residual sum between two norms
// v = x + (y ? y / sqrt(mean(y^2) + eps) * w_post : 0);  x_out (optional, may be x) <- v;  out (optional) <- v / sqrt(mean(v^2) + eps) * w_next.
// The sublayer's output is normed, joins the stream, and the stream is normed for the next sublayer, in one pass over the row.
struct SandwichArgs {
    const float* x;
    const void* y;
    const float *w_post, *w_next;
    float* x_out;
    void* out;
    int64_t ldy;
    int y_dt, out_dt;
    float eps;
};

// one wave per row; a lane holds elements lane + 64 j
template <int EPL>
__global__ __launch_bounds__(256) void sandwich_rmsnorm_kernel(int64_t T, int width, SandwichArgs p) {
    const int lane = threadIdx.x & 63;
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += (int64_t)gridDim.x * 4) {
        float v[EPL];
        float sy = 0.f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int i = lane + 64 * j;
            v[j] = (p.y && i < width) ? lds_dt(p.y, p.y_dt, t * p.ldy + i) : 0.f;
            sy += v[j] * v[j];
        }
        const float ry = p.y ? 1.0f / sqrtf(wave_sum(sy) / (float)width + p.eps) : 0.f;
        float sv = 0.f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int i = lane + 64 * j;
            float a = 0.f;
            if (i < width) {
                a = p.x[t * width + i];
                if (p.y) a += v[j] * ry * p.w_post[i];
                if (p.x_out) p.x_out[t * width + i] = a;
            }
            v[j] = a;
            sv += a * a;
        }
        if (!p.out) continue;
        const float rv = 1.0f / sqrtf(wave_sum(sv) / (float)width + p.eps);
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int i = lane + 64 * j;
            if (i < width) sts_dt(p.out, p.out_dt, t * width + i, v[j] * rv * p.w_next[i]);
        }
    }
}

// wide rows: one workgroup per row, 16-byte accesses; thread t owns elements 4 (t + 256 j) .. + 4; the four waves' sums meet in LDS in a fixed order
template <int V4>
__global__ __launch_bounds__(256) void sandwich_rmsnorm_wide_kernel(int64_t T, int width, SandwichArgs p) {
    __shared__ float red[2][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int64_t t = blockIdx.x; t < T; t += gridDim.x) {
        f32x4 v[V4];
        float sy = 0.f;
#pragma unroll
        for (int j = 0; j < V4; ++j) {
            const int i = 4 * (tid + 256 * j);
            v[j] = (p.y && i < width) ? lds4_dt(p.y, p.y_dt, t * p.ldy + i) : f32x4{0.f, 0.f, 0.f, 0.f};
            sy += v[j][0] * v[j][0] + v[j][1] * v[j][1] + v[j][2] * v[j][2] + v[j][3] * v[j][3];
        }
        float ry = 0.f;
        __syncthreads();  // the previous row's sums have been read by every thread
        if (p.y) {
            sy = wave_sum(sy);
            if (lane == 0) red[0][wave] = sy;
            __syncthreads();
            ry = 1.0f / sqrtf((red[0][0] + red[0][1] + red[0][2] + red[0][3]) / (float)width + p.eps);
        }
        float sv = 0.f;
#pragma unroll
        for (int j = 0; j < V4; ++j) {
            const int i = 4 * (tid + 256 * j);
            f32x4 a = {0.f, 0.f, 0.f, 0.f};
            if (i < width) {
                a = *(const f32x4*)(p.x + t * width + i);
                if (p.y) {
                    const f32x4 w = *(const f32x4*)(p.w_post + i);
#pragma unroll
                    for (int q = 0; q < 4; ++q) a[q] += v[j][q] * ry * w[q];
                }
                if (p.x_out) *(f32x4*)(p.x_out + t * width + i) = a;
            }
            v[j] = a;
            sv += a[0] * a[0] + a[1] * a[1] + a[2] * a[2] + a[3] * a[3];
        }
        if (!p.out) continue;
        sv = wave_sum(sv);
        if (lane == 0) red[1][wave] = sv;
        __syncthreads();
        const float rv = 1.0f / sqrtf((red[1][0] + red[1][1] + red[1][2] + red[1][3]) / (float)width + p.eps);
#pragma unroll
        for (int j = 0; j < V4; ++j) {
            const int i = 4 * (tid + 256 * j);
            if (i < width) {
                const f32x4 w = *(const f32x4*)(p.w_next + i);
                sts4_dt(p.out, p.out_dt, t * width + i, f32x4{v[j][0] * rv * w[0], v[j][1] * rv * w[1], v[j][2] * rv * w[2], v[j][3] * rv * w[3]});
            }
        }
    }
}

extern "C" int mi355_sandwich_rmsnorm(int64_t tokens, int width, const float* x, const void* y, int y_dt, int64_t ldy, const float* w_post, float* x_out,
                                      const float* w_next, float eps, void* out, int out_dt, void* stream) {
    MI355_REQUIRE(tokens > 0 && width > 0 && width <= 8192 && x, "sandwich_rmsnorm: bad arguments (width <= 8192)");
    MI355_REQUIRE(!y || (w_post && sand_dt_ok(y_dt) && ldy >= width), "sandwich_rmsnorm: a sublayer output needs its norm weight and a row pitch >= width");
    MI355_REQUIRE((out != nullptr) == (w_next != nullptr) && (!out || sand_dt_ok(out_dt)), "sandwich_rmsnorm: the normed output and its weight come together");
    MI355_REQUIRE(x_out || out, "sandwich_rmsnorm: nothing to write");
    SandwichArgs p;
    p.x = x, p.y = y, p.w_post = w_post, p.w_next = w_next, p.x_out = x_out, p.out = out, p.ldy = ldy, p.y_dt = y_dt, p.out_dt = out_dt, p.eps = eps;
    const bool vec = width % 4 == 0 && width > 256 && sand_al16(x) && (!y || (ldy % 4 == 0 && sand_al16(y) && sand_al16(w_post))) && (!x_out || sand_al16(x_out)) &&
                     (!out || (sand_al16(out) && sand_al16(w_next)));
    if (vec) {
        const int g = sand_grid(tokens, 1, 65535 * 16);
        const int v4 = (width + 1023) / 1024;
        if (v4 <= 1) sandwich_rmsnorm_wide_kernel<1><<<g, 256, 0, ST(stream)>>>(tokens, width, p);
        else if (v4 <= 2) sandwich_rmsnorm_wide_kernel<2><<<g, 256, 0, ST(stream)>>>(tokens, width, p);
        else if (v4 <= 4) sandwich_rmsnorm_wide_kernel<4><<<g, 256, 0, ST(stream)>>>(tokens, width, p);
        else sandwich_rmsnorm_wide_kernel<8><<<g, 256, 0, ST(stream)>>>(tokens, width, p);
    } else {
        const int g = sand_grid(tokens, 4, 65535 * 16);
        if (width <= 256) sandwich_rmsnorm_kernel<4><<<g, 256, 0, ST(stream)>>>(tokens, width, p);
        else if (width <= 1024) sandwich_rmsnorm_kernel<16><<<g, 256, 0, ST(stream)>>>(tokens, width, p);
        else if (width <= 2048) sandwich_rmsnorm_kernel<32><<<g, 256, 0, ST(stream)>>>(tokens, width, p);
        else sandwich_rmsnorm_kernel<128><<<g, 256, 0, ST(stream)>>>(tokens, width, p);
    }
    MI355_LAUNCH_CHECK("sandwich_rmsnorm");
    return 0;
}

// ------------------------------------------------------------------------------------------- pooled key / value rows
// Sequence s holds past[s] + n_new[s] cache rows after this step (rows cache_row0[s] + position).  Every block of `pool` positions that became complete in
// this step -- b in [past / pool, (past + n_new) / pool) -- gets its mean row: pooled[pool_row0[s] + b, :] = mean over the block's cache rows, summed in
// fp32 in position order and stored in the pooled buffer's dtype.
__global__ __launch_bounds__(256) void pool_rows_kernel(int width, int pool, const void* __restrict__ cache, int c_dt, int64_t ldc, void* __restrict__ pooled, int p_dt,
                                                        int64_t ldp, const int* __restrict__ cache_row0, const int* __restrict__ pool_row0, const int* __restrict__ past,
                                                        const int* __restrict__ n_new) {
    const int s = blockIdx.y;
    const int b0 = past[s] / pool, b1 = (past[s] + n_new[s]) / pool;
    const float inv = 1.0f / (float)pool;
    for (int b = b0 + blockIdx.x; b < b1; b += gridDim.x) {
        const int64_t r0 = (int64_t)cache_row0[s] + (int64_t)b * pool, dst = ((int64_t)pool_row0[s] + b) * ldp;
        for (int i = threadIdx.x; i < width; i += blockDim.x) {
            float acc = 0.f;
            for (int j = 0; j < pool; ++j) acc += lds_dt(cache, c_dt, (r0 + j) * ldc + i);
            sts_dt(pooled, p_dt, dst + i, acc * inv);
        }
    }
}

extern "C" int mi355_pool_rows_update(int n_seq, int max_blocks, int width, int pool, const void* cache, int c_dt, int64_t ldc, void* pooled, int p_dt, int64_t ldp,
                                      const int* cache_row0, const int* pool_row0, const int* past, const int* n_new, void* stream) {
    MI355_REQUIRE(n_seq > 0 && n_seq <= 65535 && max_blocks > 0 && width > 0 && pool > 0 && cache && pooled && sand_dt_ok(c_dt) && sand_dt_ok(p_dt) && ldc >= width && ldp >= width,
                  "pool_rows_update: bad arguments");
    MI355_REQUIRE(cache_row0 && pool_row0 && past && n_new, "pool_rows_update: sequence descriptors missing");
    dim3 grid((unsigned)(max_blocks > 4096 ? 4096 : max_blocks), (unsigned)n_seq);
    pool_rows_kernel<<<grid, width >= 256 ? 256 : 64, 0, ST(stream)>>>(width, pool, cache, c_dt, ldc, pooled, p_dt, ldp, cache_row0, pool_row0, past, n_new);
    MI355_LAUNCH_CHECK("pool_rows_update");
    return 0;
}

// ------------------------------------------------------------------------------------------- activations and gates on rows
// kind 0 (xIELU, params = two raw numbers p, q):  z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2.
// kind 1 (sigmoid gate): out = x * sigmoid(gate), gate rows of their own dtype and pitch.
__device__ __forceinline__ float softplus_f(float a) { return a > 20.f ? a : log1pf(expf(a)); }
// exp(z) - 1 - z for z <= 0 without cancellation: the series z^2 (1/2! + z/3! + ... + z^8/10!) down to -1/2, the exponential itself below
__device__ __forceinline__ float exp_minus_1_minus_z(float z) {
    if (z < -0.5f) return expf(z) - 1.0f - z;
    float s = 1.0f / 3628800.0f;
    s = fmaf(s, z, 1.0f / 362880.0f);
    s = fmaf(s, z, 1.0f / 40320.0f);
    s = fmaf(s, z, 1.0f / 5040.0f);
    s = fmaf(s, z, 1.0f / 720.0f);
    s = fmaf(s, z, 1.0f / 120.0f);
    s = fmaf(s, z, 1.0f / 24.0f);
    s = fmaf(s, z, 1.0f / 6.0f);
    s = fmaf(s, z, 0.5f);
    return z * z * s;
}
__device__ __forceinline__ float xielu_f(float z, float ap, float aq) { return z > 0.f ? ap * z * z + 0.5f * z : aq * exp_minus_1_minus_z(z) + 0.5f * z; }
// eight consecutive bf16 (16-byte aligned) <-> floats
__device__ __forceinline__ void ld8_bf(const void* p, int64_t i, float* v) {
    const u32x4 r = *(const u32x4*)((const bf16_t*)p + i);
#pragma unroll
    for (int q = 0; q < 4; ++q) v[2 * q] = __uint_as_float(r[q] << 16), v[2 * q + 1] = __uint_as_float(r[q] & 0xffff0000u);
}
__device__ __forceinline__ void st8_bf(void* p, int64_t i, const float* v) {
    *(u32x4*)((bf16_t*)p + i) = u32x4{pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3]), pack_bf2(v[4], v[5]), pack_bf2(v[6], v[7])};
}

// bf16 rows in and out, eight entries per thread (16-byte accesses); the gate may be bf16 or fp32
__global__ __launch_bounds__(256) void act_rows_bf8_kernel(int64_t R, int n, const void* __restrict__ x, int64_t ldx, const void* __restrict__ gate, int g_dt, int64_t ldg, int kind,
                                                           const float* __restrict__ params, void* __restrict__ out, int64_t ldo) {
    float ap = 0.f, aq = 0.f;
    if (kind == 0) ap = softplus_f(params[0]), aq = 0.5f + softplus_f(params[1]);
    const int nw = n / 8;
    const int64_t total = R * nw;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = e / nw;
        const int i = 8 * (int)(e % nw);
        float a[8], o[8];
        ld8_bf(x, r * ldx + i, a);
        if (kind == 0) {
#pragma unroll
            for (int q = 0; q < 8; ++q) o[q] = xielu_f(a[q], ap, aq);
        } else {
            float g[8];
            if (g_dt == MI355_DT_F32) {
                const f32x4 g0 = *(const f32x4*)((const float*)gate + r * ldg + i), g1 = *(const f32x4*)((const float*)gate + r * ldg + i + 4);
#pragma unroll
                for (int q = 0; q < 4; ++q) g[q] = g0[q], g[4 + q] = g1[q];
            } else {
                ld8_bf(gate, r * ldg + i, g);
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) o[q] = a[q] / (1.0f + expf(-g[q]));
        }
        st8_bf(out, r * ldo + i, o);
    }
}

template <bool VEC>
__global__ __launch_bounds__(256) void act_rows_kernel(int64_t R, int n, const void* __restrict__ x, int x_dt, int64_t ldx, const void* __restrict__ gate, int g_dt, int64_t ldg,
                                                       int kind, const float* __restrict__ params, void* __restrict__ out, int out_dt, int64_t ldo) {
    float ap = 0.f, aq = 0.f;
    if (kind == 0) ap = softplus_f(params[0]), aq = 0.5f + softplus_f(params[1]);
    constexpr int W = VEC ? 4 : 1;
    const int nw = n / W;
    const int64_t total = R * nw;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = e / nw;
        const int i = W * (int)(e % nw);
        if (VEC) {
            const f32x4 a = lds4_dt(x, x_dt, r * ldx + i);
            f32x4 o;
            if (kind == 0) {
#pragma unroll
                for (int q = 0; q < 4; ++q) o[q] = xielu_f(a[q], ap, aq);
            } else {
                const f32x4 g = lds4_dt(gate, g_dt, r * ldg + i);
#pragma unroll
                for (int q = 0; q < 4; ++q) o[q] = a[q] / (1.0f + expf(-g[q]));
            }
            sts4_dt(out, out_dt, r * ldo + i, o);
        } else {
            const float a = lds_dt(x, x_dt, r * ldx + i);
            sts_dt(out, out_dt, r * ldo + i, kind == 0 ? xielu_f(a, ap, aq) : a / (1.0f + expf(-lds_dt(gate, g_dt, r * ldg + i))));
        }
    }
}

extern "C" int mi355_act_rows(int64_t rows, int n, const void* x, int x_dt, int64_t ldx, const void* gate, int g_dt, int64_t ldg, int kind, const float* params,
                              void* out, int out_dt, int64_t ldo, void* stream) {
    MI355_REQUIRE(rows > 0 && n > 0 && x && out && sand_dt_ok(x_dt) && sand_dt_ok(out_dt) && ldx >= n && ldo >= n && (kind == 0 || kind == 1), "act_rows: bad arguments");
    MI355_REQUIRE(kind == 0 ? params != nullptr : (gate && sand_dt_ok(g_dt) && ldg >= n), "act_rows: xIELU needs its two numbers, a gate its rows");
    if (x_dt == MI355_DT_BF16 && out_dt == MI355_DT_BF16 && n % 8 == 0 && ldx % 8 == 0 && ldo % 8 == 0 && sand_al16(x) && sand_al16(out) &&
        (kind == 0 || (ldg % 8 == 0 && sand_al16(gate)))) {
        act_rows_bf8_kernel<<<sand_grid(rows * (n / 8), 256, 65535 * 8), 256, 0, ST(stream)>>>(rows, n, x, ldx, gate, g_dt, ldg, kind, params, out, ldo);
        MI355_LAUNCH_CHECK("act_rows");
        return 0;
    }
    const bool vec = n % 4 == 0 && ldx % 4 == 0 && ldo % 4 == 0 && sand_al16(x) && sand_al16(out) && (kind == 0 || (ldg % 4 == 0 && sand_al16(gate)));
    const int64_t total = rows * (vec ? n / 4 : n);
    const int g = sand_grid(total, 256, 65535 * 8);
    if (vec) act_rows_kernel<true><<<g, 256, 0, ST(stream)>>>(rows, n, x, x_dt, ldx, gate, g_dt, ldg, kind, params, out, out_dt, ldo);
    else act_rows_kernel<false><<<g, 256, 0, ST(stream)>>>(rows, n, x, x_dt, ldx, gate, g_dt, ldg, kind, params, out, out_dt, ldo);
    MI355_LAUNCH_CHECK("act_rows");
    return 0;
}
