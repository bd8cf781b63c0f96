// Row operations of the ragged-batch serving path (gfx950 only): hashed-bigram embedding, post-sum LayerNorm on an fp32 residual stream,
// strided RMSNorm, latent key/value rows (RMSNorm + interleaved rotary) written into a slot cache, interleaved rotary on strided heads,
// gated linear attention as a per-channel-decay recurrence with carried fp32 state, per-head RMSNorm with a SiLU output gate, and the
// grouped sigmoid router of a mixture of experts with its dispatch lists.
//
// Conventions: activations come as bf16 or fp32 (a MI355_DT_* code per operand); the residual stream, norm statistics, rotary angles,
// decays, recurrent state and router arithmetic are fp32 in both modes.  A "row" is a token of the packed batch; sequences are described
// by int32 device arrays.  One wave works on one row unless stated.
#include "common.h"

#define ST(s) ((hipStream_t)(s))

template <typename T> __device__ __forceinline__ float ldv(const T* p);
template <> __device__ __forceinline__ float ldv<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldv<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stv(T* p, float v);
template <> __device__ __forceinline__ void stv<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stv<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

// element i of a row of dtype code dt
__device__ __forceinline__ float ld_dt(const void* p, int dt, int64_t i) {
    return dt == MI355_DT_F32 ? ((const float*)p)[i] : bf2f(((const bf16_t*)p)[i]);
}
__device__ __forceinline__ void st_dt(void* p, int dt, int64_t i, float v) {
    if (dt == MI355_DT_F32) ((float*)p)[i] = v;
    else ((bf16_t*)p)[i] = f2bf(v);
}

static inline int rows_grid(int64_t rows, int per_block) {
    int64_t g = (rows + per_block - 1) / per_block;
    return (int)(g < 1 ? 1 : (g > 65535 * 16 ? 65535 * 16 : g));
}
static inline bool dt_ok(int dt) { return dt == MI355_DT_BF16 || dt == MI355_DT_F32; }

// ------------------------------------------------------------------------------------------- embedding + hashed bigram
// out[t] = table[tok[t]] * scale + bigram[row(t)],  row = (prev * mul_prev + tok * mul_cur) mod buckets, or `buckets` when prev < 0
__global__ __launch_bounds__(256) void embed_hash_kernel(int64_t T, int width, int vocab, const int* __restrict__ tok, const int* __restrict__ prev,
                                                         const bf16_t* __restrict__ table, float scale, const bf16_t* __restrict__ bigram, int buckets,
                                                         int mul_prev, int mul_cur, float* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += (int64_t)gridDim.x * 4) {
        const int id = tok[t];
        const bool ok = id >= 0 && id < vocab;
        const bf16_t* e = table + (int64_t)(ok ? id : 0) * width;
        const bf16_t* b = nullptr;
        if (bigram) {
            const int p = prev[t];
            int64_t row = buckets;
            if (p >= 0) row = ((int64_t)p * mul_prev + (int64_t)id * mul_cur) % buckets;
            if (row < 0) row += buckets;
            b = bigram + row * width;
        }
        for (int i = lane; i < width; i += 64) {
            float v = ok ? bf2f(e[i]) * scale : 0.f;
            if (b) v += bf2f(b[i]);
            out[t * width + i] = v;
        }
    }
}

extern "C" int mi355_embed_hash_fwd(int64_t tokens, int width, int vocab, const int* tok, const int* prev, const void* table, float scale,
                                    const void* bigram, int buckets, int mul_prev, int mul_cur, float* out, void* stream) {
    MI355_REQUIRE(tokens > 0 && width > 0 && vocab > 0 && tok && table && out, "embed_hash_fwd: bad arguments");
    MI355_REQUIRE(!bigram || (prev && buckets > 0), "embed_hash_fwd: a bigram table needs the previous tokens and a bucket count");
    embed_hash_kernel<<<rows_grid(tokens, 4), 256, 0, ST(stream)>>>(tokens, width, vocab, tok, prev, (const bf16_t*)table, scale, (const bf16_t*)bigram,
                                                                    buckets, mul_prev, mul_cur, out);
    MI355_LAUNCH_CHECK("embed_hash_fwd");
    return 0;
}

// ------------------------------------------------------------------------------------------- LayerNorm after the (scaled) residual sum
// v = alpha * x + sum_{p < parts} y[(t * parts + p)];  out = (v - mean) / sqrt(var + eps) * w + b, var = mean((v - mean)^2); all fp32.
// `cast` (optional) receives the same rows in dtype cast_dt (the operand of the projections that follow).
template <int EPL>
__global__ __launch_bounds__(256) void add_layernorm_kernel(int64_t T, int width, const float* __restrict__ x, float alpha, const void* __restrict__ y, int y_dt,
                                                            int64_t ldy, int parts, const float* __restrict__ w, const float* __restrict__ b, float eps,
                                                            float* __restrict__ out, void* __restrict__ cast, int cast_dt) {
    const int lane = threadIdx.x & 63;
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += (int64_t)gridDim.x * 4) {
        float v[EPL], s = 0.f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int i = lane + 64 * j;
            float a = 0.f;
            if (i < width) {
                a = alpha * x[t * width + i];
                if (y) {
                    float ys = 0.f;
                    for (int p = 0; p < parts; ++p) ys += ld_dt(y, y_dt, (t * parts + p) * ldy + i);
                    a += ys;
                }
            }
            v[j] = a;
            s += a;
        }
        const float mean = wave_sum(s) / (float)width;
        float q = 0.f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int i = lane + 64 * j;
            const float d = i < width ? v[j] - mean : 0.f;
            q += d * d;
        }
        const float r = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int i = lane + 64 * j;
            if (i < width) {
                const float o = (v[j] - mean) * r * w[i] + b[i];
                out[t * width + i] = o;
                if (cast) st_dt(cast, cast_dt, t * width + i, o);
            }
        }
    }
}

// The same for wide rows: one workgroup per row, 16-byte accesses (width % 4 == 0), thread t owns elements 4 (t + 256 j) .. + 4.
template <int V4>
__global__ __launch_bounds__(256) void add_layernorm_wide_kernel(int64_t T, int width, const float* __restrict__ x, float alpha, const void* __restrict__ y, int y_dt,
                                                                 int64_t ldy, int parts, const float* __restrict__ w, const float* __restrict__ b, float eps,
                                                                 float* __restrict__ out, void* __restrict__ cast, int cast_dt) {
    __shared__ float red[2][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int64_t t = blockIdx.x; t < T; t += gridDim.x) {
        f32x4 v[V4];
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < V4; ++j) {
            const int i = 4 * (tid + 256 * j);
            f32x4 a = {0.f, 0.f, 0.f, 0.f};
            if (i < width) {
                a = *(const f32x4*)(x + t * width + i) * alpha;
                if (y) {
                    f32x4 ys = {0.f, 0.f, 0.f, 0.f};
                    for (int pp = 0; pp < parts; ++pp) {
                        const int64_t o = (t * parts + pp) * ldy + i;
                        if (y_dt == MI355_DT_F32) ys += *(const f32x4*)((const float*)y + o);
                        else {
                            const u32x2 r = *(const u32x2*)((const bf16_t*)y + o);
                            ys += f32x4{__uint_as_float(r[0] << 16), __uint_as_float(r[0] & 0xffff0000u), __uint_as_float(r[1] << 16), __uint_as_float(r[1] & 0xffff0000u)};
                        }
                    }
                    a += ys;
                }
            }
            v[j] = a;
            s += (a[0] + a[1]) + (a[2] + a[3]);
        }
        s = wave_sum(s);
        if (lane == 0) red[0][wave] = s;
        __syncthreads();
        const float mean = ((red[0][0] + red[0][1]) + (red[0][2] + red[0][3])) / (float)width;
        float q = 0.f;
#pragma unroll
        for (int j = 0; j < V4; ++j) {
            if (4 * (tid + 256 * j) < width) {
                const f32x4 d = v[j] - mean;
                q += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
            }
        }
        q = wave_sum(q);
        if (lane == 0) red[1][wave] = q;
        __syncthreads();
        const float r = 1.0f / sqrtf(((red[1][0] + red[1][1]) + (red[1][2] + red[1][3])) / (float)width + eps);
#pragma unroll
        for (int j = 0; j < V4; ++j) {
            const int i = 4 * (tid + 256 * j);
            if (i < width) {
                const f32x4 o = (v[j] - mean) * r * *(const f32x4*)(w + i) + *(const f32x4*)(b + i);
                *(f32x4*)(out + t * width + i) = o;
                if (cast) {
                    if (cast_dt == MI355_DT_F32) *(f32x4*)((float*)cast + t * width + i) = o;
                    else *(u32x2*)((bf16_t*)cast + t * width + i) = u32x2{pack_bf2(o[0], o[1]), pack_bf2(o[2], o[3])};
                }
            }
        }
        __syncthreads();  // red[] is reused by the next row
    }
}

extern "C" int mi355_add_layernorm_fwd(int64_t tokens, int width, const float* x, float alpha, const void* y, int y_dt, int64_t ldy, int parts, const float* w,
                                       const float* b, float eps, float* out, void* cast, int cast_dt, void* stream) {
    MI355_REQUIRE(tokens > 0 && width > 0 && width <= 8192 && x && w && b && out, "add_layernorm_fwd: bad arguments (width <= 8192)");
    MI355_REQUIRE(!y || (dt_ok(y_dt) && parts >= 1 && ldy >= width), "add_layernorm_fwd: bad summand");
    MI355_REQUIRE(!cast || dt_ok(cast_dt), "add_layernorm_fwd: bad cast dtype");
    const bool aligned = width % 4 == 0 && (!y || (ldy % 4 == 0 && ((uintptr_t)y & 15) == 0)) && ((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0 &&
                         ((uintptr_t)w & 15) == 0 && ((uintptr_t)b & 15) == 0 && (!cast || ((uintptr_t)cast & 15) == 0);
    if (aligned && width > 512) {
        const int g = (int)(tokens < 65535 * 8 ? tokens : 65535 * 8);
#define LNW_CASE(V)                                                                                                                                            \
    if (width <= 1024 * V) {                                                                                                                                   \
        add_layernorm_wide_kernel<V><<<g, 256, 0, ST(stream)>>>(tokens, width, x, alpha, y, y_dt, ldy, parts, w, b, eps, out, cast, cast_dt);                \
        MI355_LAUNCH_CHECK("add_layernorm_fwd");                                                                                                               \
        return 0;                                                                                                                                              \
    }
        LNW_CASE(1) LNW_CASE(2) LNW_CASE(4) LNW_CASE(8)
#undef LNW_CASE
    }
    const int grid = rows_grid(tokens, 4);
#define LN_CASE(E)                                                                                                                                         \
    if (width <= 64 * E) {                                                                                                                                 \
        add_layernorm_kernel<E><<<grid, 256, 0, ST(stream)>>>(tokens, width, x, alpha, y, y_dt, ldy, parts, w, b, eps, out, cast, cast_dt);              \
        MI355_LAUNCH_CHECK("add_layernorm_fwd");                                                                                                           \
        return 0;                                                                                                                                          \
    }
    LN_CASE(2) LN_CASE(4) LN_CASE(8) LN_CASE(16) LN_CASE(32) LN_CASE(64) LN_CASE(128)
#undef LN_CASE
    return 1;
}

// ------------------------------------------------------------------------------------------- RMSNorm on strided rows
// out[t, i] = x[t, i] / sqrt(mean(x[t]^2) + eps) * w[i]   (i < n)
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(int64_t T, int n, const void* __restrict__ x, int x_dt, int64_t ldx, const float* __restrict__ w, float eps,
                                                           void* __restrict__ out, int out_dt, int64_t ldo) {
    const int lane = threadIdx.x & 63;
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += (int64_t)gridDim.x * 4) {
        float s = 0.f;
        for (int i = lane; i < n; i += 64) {
            const float a = ld_dt(x, x_dt, t * ldx + i);
            s += a * a;
        }
        const float r = 1.0f / sqrtf(wave_sum(s) / (float)n + eps);
        for (int i = lane; i < n; i += 64) st_dt(out, out_dt, t * ldo + i, ld_dt(x, x_dt, t * ldx + i) * r * w[i]);
    }
}

extern "C" int mi355_rmsnorm_rows(int64_t tokens, int n, const void* x, int x_dt, int64_t ldx, const float* w, float eps, void* out, int out_dt, int64_t ldo,
                                  void* stream) {
    MI355_REQUIRE(tokens > 0 && n > 0 && x && w && out && dt_ok(x_dt) && dt_ok(out_dt) && ldx >= n && ldo >= n, "rmsnorm_rows: bad arguments");
    rmsnorm_rows_kernel<<<rows_grid(tokens, 4), 256, 0, ST(stream)>>>(tokens, n, x, x_dt, ldx, w, eps, out, out_dt, ldo);
    MI355_LAUNCH_CHECK("rmsnorm_rows");
    return 0;
}

// ------------------------------------------------------------------------------------------- interleaved rotary embedding
// Entries (2i, 2i+1) of the rotated range turn by angle pos * freq[i]; angle, sine and cosine in fp32 (full-range sinf / cosf).
__device__ __forceinline__ void turn_pair(float u, float v, float ang, float& ou, float& ov) {
    const float c = cosf(ang), s = sinf(ang);
    ou = u * c - v * s;
    ov = v * c + u * s;
}

// Latent key/value row of token t: src[t] = [rank values | rot values].  dst row dst_row[t] of the cache receives
// [RMSNorm(first rank) * w | rotate(last rot)] (the first `dims` of the rot part turn, the rest pass).  layout 0: pair i = entries (2i, 2i+1);
// layout 1: pair i = entries (i, i + dims/2).
__global__ __launch_bounds__(256) void latent_kv_append_kernel(int64_t T, int rank, int rot, const void* __restrict__ src, int src_dt, int64_t lds_, const float* __restrict__ w,
                                                               float eps, const int* __restrict__ pos, const int* __restrict__ dst_row, const float* __restrict__ freq,
                                                               int dims, int layout, void* __restrict__ cache, int cache_dt, int64_t ldc) {
    const int lane = threadIdx.x & 63;
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += (int64_t)gridDim.x * 4) {
        const int64_t so = t * lds_, d0 = (int64_t)dst_row[t] * ldc;
        float s = 0.f;
        for (int i = lane; i < rank; i += 64) {
            const float a = ld_dt(src, src_dt, so + i);
            s += a * a;
        }
        const float r = 1.0f / sqrtf(wave_sum(s) / (float)rank + eps);
        for (int i = lane; i < rank; i += 64) st_dt(cache, cache_dt, d0 + i, ld_dt(src, src_dt, so + i) * r * w[i]);
        const float p = (float)pos[t];
        if (layout == 1) {
            for (int i = dims + lane; i < rot; i += 64) st_dt(cache, cache_dt, d0 + rank + i, ld_dt(src, src_dt, so + rank + i));
            for (int i = lane; i < dims / 2; i += 64) {
                float ou, ov;
                turn_pair(ld_dt(src, src_dt, so + rank + i), ld_dt(src, src_dt, so + rank + i + dims / 2), p * freq[i], ou, ov);
                st_dt(cache, cache_dt, d0 + rank + i, ou);
                st_dt(cache, cache_dt, d0 + rank + i + dims / 2, ov);
            }
            continue;
        }
        for (int i = lane; i < (rot + 1) / 2; i += 64) {
            const float u = ld_dt(src, src_dt, so + rank + 2 * i);
            const bool has_v = 2 * i + 1 < rot;
            const float v = has_v ? ld_dt(src, src_dt, so + rank + 2 * i + 1) : 0.f;
            float ou = u, ov = v;
            if (2 * i + 1 < dims) turn_pair(u, v, p * freq[i], ou, ov);
            st_dt(cache, cache_dt, d0 + rank + 2 * i, ou);
            if (has_v) st_dt(cache, cache_dt, d0 + rank + 2 * i + 1, ov);
        }
    }
}

extern "C" int mi355_latent_kv_append(int64_t tokens, int rank, int rot, const void* src, int src_dt, int64_t ld, const float* w, float eps, const int* pos,
                                      const int* dst_row, const float* freq, int dims, int layout, void* cache, int cache_dt, int64_t ldc, void* stream) {
    MI355_REQUIRE(tokens > 0 && rank > 0 && rot >= 0 && src && w && pos && dst_row && cache && dt_ok(src_dt) && dt_ok(cache_dt) && (layout == 0 || layout == 1), "latent_kv_append: bad arguments");
    MI355_REQUIRE(ld >= rank + rot && ldc >= rank + rot && dims >= 0 && dims <= rot && dims % 2 == 0 && (dims == 0 || freq), "latent_kv_append: bad row sizes");
    latent_kv_append_kernel<<<rows_grid(tokens, 4), 256, 0, ST(stream)>>>(tokens, rank, rot, src, src_dt, ld, w, eps, pos, dst_row, freq, dims, layout, cache, cache_dt, ldc);
    MI355_LAUNCH_CHECK("latent_kv_append");
    return 0;
}

// Copy n entries per head from src to dst (fp32) and turn the pairs of [rot_start, rot_start + dims) -- layout 0: neighbours (2i, 2i+1); layout 1: the
// two halves of the range, (i, i + dims/2):
// dst[t, h * dst_hs + dst_off + i] = src[t, h * src_hs + src_off + i]
__global__ __launch_bounds__(256) void rope_heads_kernel(int64_t T, int H, int n, const void* __restrict__ src, int src_dt, int64_t lds_, int src_hs, int src_off,
                                                         float* __restrict__ dst, int64_t ldd, int dst_hs, int dst_off, int rot_start, int dims, int layout,
                                                         const float* __restrict__ freq, const int* __restrict__ pos) {
    const int lane = threadIdx.x & 63;
    const int64_t items = T * H;
    for (int64_t it = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); it < items; it += (int64_t)gridDim.x * 4) {
        const int64_t t = it / H;
        const int h = (int)(it % H);
        const int64_t so = t * lds_ + (int64_t)h * src_hs + src_off, dof = t * ldd + (int64_t)h * dst_hs + dst_off;
        const float p = (float)pos[t];
        // the plain part: everything outside the rotated range
        for (int i = lane; i < n; i += 64)
            if (i < rot_start || i >= rot_start + dims) dst[dof + i] = ld_dt(src, src_dt, so + i);
        for (int i = lane; i < dims / 2; i += 64) {
            const int a = rot_start + (layout ? i : 2 * i), b = rot_start + (layout ? i + dims / 2 : 2 * i + 1);
            const float u = ld_dt(src, src_dt, so + a), v = ld_dt(src, src_dt, so + b);
            float ou, ov;
            turn_pair(u, v, p * freq[i], ou, ov);
            dst[dof + a] = ou;
            dst[dof + b] = ov;
        }
    }
}

extern "C" int mi355_rope_heads(int64_t tokens, int H, int n, const void* src, int src_dt, int64_t ld_src, int src_hs, int src_off, float* dst, int64_t ld_dst,
                                int dst_hs, int dst_off, int rot_start, int dims, int layout, const float* freq, const int* pos, void* stream) {
    MI355_REQUIRE(tokens > 0 && H > 0 && n > 0 && src && dst && pos && dt_ok(src_dt) && (layout == 0 || layout == 1), "rope_heads: bad arguments");
    MI355_REQUIRE(rot_start >= 0 && dims >= 0 && dims % 2 == 0 && rot_start + dims <= n && (dims == 0 || freq), "rope_heads: the rotated range must lie inside the head");
    MI355_REQUIRE(src_off >= 0 && dst_off >= 0 && ld_src >= (int64_t)(H - 1) * src_hs + src_off + n && ld_dst >= (int64_t)(H - 1) * dst_hs + dst_off + n, "rope_heads: rows too short");
    rope_heads_kernel<<<rows_grid(tokens * H, 4), 256, 0, ST(stream)>>>(tokens, H, n, src, src_dt, ld_src, src_hs, src_off, dst, ld_dst, dst_hs, dst_off, rot_start, dims,
                                                                      layout, freq, pos);
    MI355_LAUNCH_CHECK("rope_heads");
    return 0;
}

// ------------------------------------------------------------------------------------------- per-head RMSNorm with a SiLU gate
// out[t, h, i] = o[t, h, i] / sqrt(mean_i o^2 + eps) * w[i] * silu(gate[t, h, i]);  o fp32 [T, H*D]
__global__ __launch_bounds__(256) void gated_headnorm_kernel(int64_t T, int H, int D, const float* __restrict__ o, const float* __restrict__ w, const void* __restrict__ gate,
                                                             int g_dt, int64_t ldg, float eps, void* __restrict__ out, int out_dt, int64_t ldo) {
    const int lane = threadIdx.x & 63;
    const int64_t items = T * H;
    for (int64_t it = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); it < items; it += (int64_t)gridDim.x * 4) {
        const int64_t t = it / H;
        const int h = (int)(it % H);
        const float* row = o + it * D;
        float s = 0.f;
        for (int i = lane; i < D; i += 64) s += row[i] * row[i];
        const float r = 1.0f / sqrtf(wave_sum(s) / (float)D + eps);
        for (int i = lane; i < D; i += 64) {
            const float g = ld_dt(gate, g_dt, t * ldg + (int64_t)h * D + i);
            const float sg = g / (1.0f + expf(-g));
            st_dt(out, out_dt, t * ldo + (int64_t)h * D + i, row[i] * r * w[i] * sg);
        }
    }
}

extern "C" int mi355_gated_headnorm(int64_t tokens, int H, int D, const float* o, const float* w, const void* gate, int g_dt, int64_t ldg, float eps, void* out,
                                    int out_dt, int64_t ldo, void* stream) {
    MI355_REQUIRE(tokens > 0 && H > 0 && D > 0 && o && w && gate && out && dt_ok(g_dt) && dt_ok(out_dt) && ldg >= (int64_t)H * D && ldo >= (int64_t)H * D,
                  "gated_headnorm: bad arguments");
    gated_headnorm_kernel<<<rows_grid(tokens * H, 4), 256, 0, ST(stream)>>>(tokens, H, D, o, w, gate, g_dt, ldg, eps, out, out_dt, ldo);
    MI355_LAUNCH_CHECK("gated_headnorm");
    return 0;
}

// ------------------------------------------------------------------------------------------- gated linear attention
// Per head a state S [dk, dv] (fp32, carried per sequence slot):  S <- diag(a_t) S + k_t v_t^T,  o_t = S^T (q_t * qscale),
// a_t = sigmoid(z_t + zbias)^(inv_tau) = exp(inv_tau * logsigmoid(.)) in fp32 -- or, with head_decay, the constant head_decay[h] for every key channel
// of head h (retention: z / zbias are then unused).  k_t is multiplied by kscale.
// Block: 64 value columns x RC row chunks of GLA_R key channels; a thread keeps GLA_R state entries of one column in registers.
// Tokens go through in groups of GLA_TB: the group's q / k / decay rows are staged in LDS once, partial outputs of the row chunks meet in LDS.
#define GLA_R 16
#define GLA_TB 8
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

__global__ void gla_kernel(const int* __restrict__ seq_off, const int* __restrict__ slot, int H, int dk, int dv, const void* __restrict__ q, const void* __restrict__ k,
                           const void* __restrict__ v, const void* __restrict__ z, int dt, int z_dt, int v_dt, int64_t ldq, int64_t ldk, int64_t ldv_, int64_t ldz,
                           const float* __restrict__ zbias, float inv_tau, float qscale, const float* __restrict__ head_decay, float kscale,
                           float* __restrict__ state, float* __restrict__ o) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int RC = blockDim.x >> 6;
    float* sq = smem;                       // [TB][dk]
    float* sk = sq + GLA_TB * dk;           // [TB][dk]
    float* sa = sk + GLA_TB * dk;           // [TB][dk]
    float* sv = sa + GLA_TB * dk;           // [TB][64]
    float* sp = sv + GLA_TB * 64;           // [TB][RC][64]
    const int s = blockIdx.x, h = blockIdx.y, col = blockIdx.z * 64 + (threadIdx.x & 63), chunk = threadIdx.x >> 6;
    const int t0 = seq_off[s], t1 = seq_off[s + 1];
    const bool col_ok = col < dv;
    float* S = state + (((int64_t)slot[s] * H + h) * dk) * dv;
    float st[GLA_R];
#pragma unroll
    for (int r = 0; r < GLA_R; ++r) {
        const int i = chunk * GLA_R + r;
        st[r] = (col_ok && i < dk) ? S[(int64_t)i * dv + col] : 0.f;
    }
    // the next group's rows travel from memory into registers while the current group is worked on (a group's loads would otherwise cost a full
    // memory round trip between every eight tokens); dk <= 16 RC, so a thread carries at most 2 entries of q / k / z and 8 of v
    float rq[2], rk[2], rz[2], rv[8];
    auto fetch = [&](int tb) {
        const int nt = min(GLA_TB, t1 - tb);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int e = threadIdx.x + u * blockDim.x;
            rq[u] = rk[u] = rz[u] = 0.f;
            if (e < nt * dk) {
                const int j = e / dk, i = e % dk;
                const int64_t t = tb + j;
                rq[u] = ld_dt(q, dt, t * ldq + (int64_t)h * dk + i);
                rk[u] = ld_dt(k, dt, t * ldk + (int64_t)h * dk + i);
                if (!head_decay) rz[u] = ld_dt(z, z_dt, t * ldz + (int64_t)h * dk + i) + zbias[h * dk + i];
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int e = threadIdx.x + u * blockDim.x;
            rv[u] = 0.f;
            if (e < nt * 64) {
                const int j = e >> 6, c = blockIdx.z * 64 + (e & 63);
                if (c < dv) rv[u] = ld_dt(v, v_dt, (int64_t)(tb + j) * ldv_ + (int64_t)h * dv + c);
            }
        }
    };
    if (t0 < t1) fetch(t0);
    for (int tb = t0; tb < t1; tb += GLA_TB) {
        const int nt = min(GLA_TB, t1 - tb);
        __syncthreads();  // the previous group's rows and partial sums are consumed
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int e = threadIdx.x + u * blockDim.x;
            if (e < nt * dk) {
                sq[e] = rq[u] * qscale;
                sk[e] = rk[u] * kscale;
                sa[e] = head_decay ? head_decay[h] : expf(inv_tau * log_sigmoid(rz[u]));
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int e = threadIdx.x + u * blockDim.x;
            if (e < nt * 64) sv[e] = rv[u];
        }
        __syncthreads();
        if (tb + GLA_TB < t1) fetch(tb + GLA_TB);
        const bool full = chunk * GLA_R + GLA_R <= dk && dk % 4 == 0;
        for (int j = 0; j < nt; ++j) {
            const float vv = sv[j * 64 + (threadIdx.x & 63)];
            const float* qa = sq + j * dk + chunk * GLA_R;
            const float* ka = sk + j * dk + chunk * GLA_R;
            const float* aa = sa + j * dk + chunk * GLA_R;
            float acc = 0.f;
            if (full) {
#pragma unroll
                for (int r4 = 0; r4 < GLA_R / 4; ++r4) {
                    const f32x4 q4 = *(const f32x4*)(qa + 4 * r4), k4 = *(const f32x4*)(ka + 4 * r4), a4 = *(const f32x4*)(aa + 4 * r4);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        st[4 * r4 + i] = a4[i] * st[4 * r4 + i] + k4[i] * vv;
                        acc += st[4 * r4 + i] * q4[i];
                    }
                }
            } else {
#pragma unroll
                for (int r = 0; r < GLA_R; ++r) {
                    if (chunk * GLA_R + r < dk) {
                        st[r] = aa[r] * st[r] + ka[r] * vv;
                        acc += st[r] * qa[r];
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
                o[(int64_t)(tb + j) * H * dv + (int64_t)h * dv + c] = acc;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < GLA_R; ++r) {
        const int i = chunk * GLA_R + r;
        if (col_ok && i < dk) S[(int64_t)i * dv + col] = st[r];
    }
}

extern "C" int mi355_gla_fwd(int n_seq, const int* seq_off, const int* slot, int H, int dk, int dv, const void* q, const void* k, const void* v, const void* z, int dt,
                             int z_dt, int v_dt, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldz, const float* zbias, float inv_tau, float qscale, const float* head_decay, float kscale,
                             float* state, float* o, void* stream) {
    MI355_REQUIRE(n_seq > 0 && n_seq <= 65535 && seq_off && slot && H > 0 && H <= 65535 && dk > 0 && dk <= 16 * GLA_R && dv > 0 && q && k && v && state && o && dt_ok(dt) && dt_ok(v_dt),
                  "gla_fwd: bad arguments (key channels per head <= 256)");
    MI355_REQUIRE(head_decay || (z && zbias && dt_ok(z_dt) && ldz >= (int64_t)H * dk), "gla_fwd: the decay needs its rows and bias, or a constant per head");
    MI355_REQUIRE(ldq >= (int64_t)H * dk && ldk >= (int64_t)H * dk && ldv >= (int64_t)H * dv, "gla_fwd: rows too short");
    const int RC = (dk + GLA_R - 1) / GLA_R;
    const size_t lds_bytes = sizeof(float) * ((size_t)3 * GLA_TB * dk + (size_t)GLA_TB * 64 + (size_t)GLA_TB * RC * 64);
    MI355_REQUIRE(lds_bytes <= 64 * 1024, "gla_fwd: LDS budget exceeded");
    gla_kernel<<<dim3(n_seq, H, (dv + 63) / 64), 64 * RC, lds_bytes, ST(stream)>>>(seq_off, slot, H, dk, dv, q, k, v, z, dt, z_dt, v_dt, ldq, ldk, ldv, ldz, zbias, inv_tau, qscale,
                                                                                   head_decay, kscale, state, o);
    MI355_LAUNCH_CHECK("gla_fwd");
    return 0;
}

// ------------------------------------------------------------------------------------------- router logits
// logits[t, e] = sum_k x[t, k] * W[e, k]: fp32 rows against a small bf16 matrix, fp32 FMA.  One workgroup per token keeps the row in LDS; wave w takes
// experts w, w + 4, ...; a lane reads 8 weights (16 bytes) at a time when the rows allow it.
__global__ __launch_bounds__(256) void router_logits_kernel(int64_t T, int E, int Kd, const float* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ W, int64_t ldw,
                                                            float* __restrict__ out, int vec) {
    extern __shared__ __attribute__((aligned(16))) float xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int64_t t = blockIdx.x; t < T; t += gridDim.x) {
        __syncthreads();
        for (int k = tid; k < Kd; k += 256) xs[k] = x[t * ldx + k];
        __syncthreads();
        for (int e = wave; e < E; e += 4) {
            const bf16_t* wr = W + (int64_t)e * ldw;
            float acc = 0.f;
            if (vec) {
                for (int k = lane * 8; k < Kd; k += 512) {
                    const u32x4 r = *(const u32x4*)(wr + k);
                    const f32x4 a = *(const f32x4*)(xs + k), c = *(const f32x4*)(xs + k + 4);
                    acc = fmaf(a[0], __uint_as_float(r[0] << 16), acc);
                    acc = fmaf(a[1], __uint_as_float(r[0] & 0xffff0000u), acc);
                    acc = fmaf(a[2], __uint_as_float(r[1] << 16), acc);
                    acc = fmaf(a[3], __uint_as_float(r[1] & 0xffff0000u), acc);
                    acc = fmaf(c[0], __uint_as_float(r[2] << 16), acc);
                    acc = fmaf(c[1], __uint_as_float(r[2] & 0xffff0000u), acc);
                    acc = fmaf(c[2], __uint_as_float(r[3] << 16), acc);
                    acc = fmaf(c[3], __uint_as_float(r[3] & 0xffff0000u), acc);
                }
            } else {
                for (int k = lane; k < Kd; k += 64) acc = fmaf(xs[k], bf2f(wr[k]), acc);
            }
            acc = wave_sum(acc);
            if (lane == 0) out[t * E + e] = acc;
        }
    }
}

extern "C" int mi355_router_logits(int64_t tokens, int E, int K, const float* x, int64_t ldx, const void* W, int64_t ldw, float* out, void* stream) {
    MI355_REQUIRE(tokens > 0 && E > 0 && K > 0 && K <= 16384 && x && W && out && ldx >= K && ldw >= K, "router_logits: bad arguments (width <= 16384)");
    const int vec = K % 8 == 0 && ldw % 8 == 0 && ((uintptr_t)W & 15) == 0;
    const int g = (int)(tokens < 65535 * 8 ? tokens : 65535 * 8);
    router_logits_kernel<<<g, 256, sizeof(float) * K, ST(stream)>>>(tokens, E, K, x, ldx, (const bf16_t*)W, ldw, out, vec);
    MI355_LAUNCH_CHECK("router_logits");
    return 0;
}

// ------------------------------------------------------------------------------------------- grouped sigmoid router
// s = sigmoid(logits); choice = s + correction.  Experts form `groups` equal runs of neighbours; a group's score is the sum of its two largest
// choice scores; only experts of the `keep` best groups may be chosen; the `top` largest allowed choice scores win (ties: lowest index).
// weights = s of the winners / (their sum + 1e-20) * scale.  One wave per token, expert e on lane e % 64, register e / 64.
// mode 1 (softmax router): s = softmax(logits) over ALL experts, choice = s (no correction, no groups), weights = s of the winners * scale, not renormalised.
// mode 2 (softmax over the winners): as mode 1 on logits + correction (a bias that counts for choice and weight), the winners' s divided by their sum --
// the softmax over the chosen logits alone -- times scale.
template <int EPL>
__global__ __launch_bounds__(256) void moe_route_kernel(int64_t T, int E, int top, int groups, int keep, const float* __restrict__ logits, const float* __restrict__ corr,
                                                        float scale, int mode, int* __restrict__ ids, float* __restrict__ wts) {
    const int lane = threadIdx.x & 63;
    const float NEG = -__builtin_huge_valf();
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += (int64_t)gridDim.x * 4) {
        float s[EPL], c[EPL];
        if (mode >= 1) {
            float mx = NEG;
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                const int e = lane + 64 * j;
                s[j] = e < E ? logits[t * E + e] + (mode == 2 && corr ? corr[e] : 0.f) : NEG;
                mx = fmaxf(mx, s[j]);
            }
            mx = wave_max(mx);
            float den = 0.f;
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                s[j] = lane + 64 * j < E ? expf(s[j] - mx) : 0.f;
                den += s[j];
            }
            den = wave_sum(den);
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                s[j] = s[j] / den;
                c[j] = lane + 64 * j < E ? s[j] : NEG;
            }
        } else {
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                const int e = lane + 64 * j;
                if (e < E) {
                    const float zz = logits[t * E + e];
                    s[j] = 1.0f / (1.0f + expf(-zz));
                    c[j] = s[j] + (corr ? corr[e] : 0.f);
                } else {
                    s[j] = 0.f;
                    c[j] = NEG;
                }
            }
        }
        if (mode == 0 && groups > 1) {
            const int per = E / groups;
            // group scores: lane g keeps the score of group g (+ 64 * register)
            float gs[EPL];
#pragma unroll
            for (int j = 0; j < EPL; ++j) gs[j] = NEG;
            for (int g = 0; g < groups; ++g) {
                float best = NEG, second = NEG;
                int bi = -1;
#pragma unroll
                for (int j = 0; j < EPL; ++j) {
                    const int e = lane + 64 * j;
                    if (e < E && e / per == g && c[j] > best) best = c[j], bi = e;
                }
                // wave argmax (value, lowest index)
                for (int o = 32; o > 0; o >>= 1) {
                    const float ob = __shfl_xor(best, o, 64);
                    const int oi = __shfl_xor(bi, o, 64);
                    if (ob > best || (ob == best && oi >= 0 && (bi < 0 || oi < bi))) best = ob, bi = oi;
                }
#pragma unroll
                for (int j = 0; j < EPL; ++j) {
                    const int e = lane + 64 * j;
                    if (e < E && e / per == g && e != bi && c[j] > second) second = c[j];
                }
                second = wave_max(second);
                const float score = per > 1 ? best + second : best;
#pragma unroll
                for (int j = 0; j < EPL; ++j)
                    if (lane + 64 * j == g) gs[j] = score;
            }
            // the `keep` best groups stay; mark them in a bit per (lane, register)
            unsigned kept = 0;
            for (int n = 0; n < keep; ++n) {
                float best = NEG;
                int bi = -1;
#pragma unroll
                for (int j = 0; j < EPL; ++j) {
                    const int g = lane + 64 * j;
                    if (g < groups && !(kept >> j & 1) && (gs[j] > best || bi < 0)) best = gs[j], bi = g;
                }
                for (int o = 32; o > 0; o >>= 1) {
                    const float ob = __shfl_xor(best, o, 64);
                    const int oi = __shfl_xor(bi, o, 64);
                    if (oi >= 0 && (bi < 0 || ob > best || (ob == best && oi < bi))) best = ob, bi = oi;
                }
#pragma unroll
                for (int j = 0; j < EPL; ++j)
                    if (lane + 64 * j == bi) kept |= 1u << j;
            }
            // an expert is allowed iff its group was kept: ask the lane that holds the group's bit
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                const int e = lane + 64 * j;
                const int g = e < E ? e / per : 0;
                const unsigned kb = __shfl(kept, g & 63, 64);
                if (e < E && !(kb >> (g >> 6) & 1)) c[j] = NEG;
            }
        }
        float wsum = 0.f, mine = 0.f;
        int my_id = 0;
        for (int n = 0; n < top; ++n) {
            float best = NEG;
            int bi = -1;
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                const int e = lane + 64 * j;
                if (e < E && c[j] > best) best = c[j], bi = e;
            }
            for (int o = 32; o > 0; o >>= 1) {
                const float ob = __shfl_xor(best, o, 64);
                const int oi = __shfl_xor(bi, o, 64);
                if (oi >= 0 && (bi < 0 || ob > best || (ob == best && oi < bi))) best = ob, bi = oi;
            }
            float sv = 0.f;
#pragma unroll
            for (int j = 0; j < EPL; ++j)
                if (lane + 64 * j == bi) sv = s[j], c[j] = NEG;
            sv = wave_sum(sv);  // exactly one lane holds it (0 if no expert was left)
            wsum += sv;
            if (lane == n % 64 && n < 64) mine = sv, my_id = bi < 0 ? 0 : bi;
            else if (n >= 64 && lane == 0) {  // more than 64 winners per token: written one by one
                ids[t * top + n] = bi < 0 ? 0 : bi;
                wts[t * top + n] = sv;
            }
        }
        const float inv = mode == 1 ? scale : scale / (wsum + 1e-20f);
        if (lane < top && lane < 64) {
            ids[t * top + lane] = my_id;
            wts[t * top + lane] = mine * inv;
        }
        if (top > 64 && lane == 0)
            for (int n = 64; n < top; ++n) wts[t * top + n] *= inv;
    }
}

extern "C" int mi355_moe_route(int64_t tokens, int E, int top, int groups, int keep, const float* logits, const float* correction, float scale, int mode, int* ids,
                               float* wts, void* stream) {
    MI355_REQUIRE(tokens > 0 && E > 0 && E <= 512 && top > 0 && top <= E && logits && ids && wts && mode >= 0 && mode <= 2, "moe_route: bad arguments (experts <= 512)");
    MI355_REQUIRE(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && (int64_t)keep * (E / groups) >= top, "moe_route: the kept groups must hold the experts to choose");
    const int grid = rows_grid(tokens, 4);
    if (E <= 64) moe_route_kernel<1><<<grid, 256, 0, ST(stream)>>>(tokens, E, top, groups, keep, logits, correction, scale, mode, ids, wts);
    else if (E <= 128) moe_route_kernel<2><<<grid, 256, 0, ST(stream)>>>(tokens, E, top, groups, keep, logits, correction, scale, mode, ids, wts);
    else if (E <= 256) moe_route_kernel<4><<<grid, 256, 0, ST(stream)>>>(tokens, E, top, groups, keep, logits, correction, scale, mode, ids, wts);
    else moe_route_kernel<8><<<grid, 256, 0, ST(stream)>>>(tokens, E, top, groups, keep, logits, correction, scale, mode, ids, wts);
    MI355_LAUNCH_CHECK("moe_route");
    return 0;
}

// Dispatch lists: entries (token, choice) sorted by expert.  offs[e] .. offs[e+1] are expert e's rows of `perm`, perm[r] = token * top + choice.
// One workgroup: histogram in LDS, scan, then positions in token order (rows of an expert stay in token order: a fixed layout, no atomics).
__global__ __launch_bounds__(1024) void moe_dispatch_kernel(int64_t n, int E, const int* __restrict__ ids, int* __restrict__ offs, int* __restrict__ perm) {
    extern __shared__ int cnt[];  // [E + 1] counts, then running offsets
    for (int e = threadIdx.x; e <= E; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
        const int e = ids[i];
        if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int e = 0; e < E; ++e) {
            const int c = cnt[e];
            cnt[e] = run;
            offs[e] = run;
            run += c;
        }
        offs[E] = run;
    }
    __syncthreads();
    // wave e walks the entries 64 at a time and places its expert's rows by ballot + prefix count
    const int lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    for (int e = threadIdx.x >> 6; e < E; e += nw) {
        int at = cnt[e];
        for (int64_t i0 = 0; i0 < n; i0 += 64) {
            const int64_t i = i0 + lane;
            const bool m = i < n && ids[i] == e;
            const unsigned long long b = __ballot(m);
            if (m) perm[at + __popcll(b & ((1ull << lane) - 1ull))] = (int)i;
            at += __popcll(b);
        }
    }
}

extern "C" int mi355_moe_dispatch(int64_t entries, int E, const int* ids, int* offs, int* perm, void* stream) {
    MI355_REQUIRE(entries > 0 && entries < (int64_t)1 << 31 && E > 0 && E <= 4096 && ids && offs && perm, "moe_dispatch: bad arguments");
    moe_dispatch_kernel<<<1, 1024, sizeof(int) * (E + 1), ST(stream)>>>(entries, E, ids, offs, perm);
    MI355_LAUNCH_CHECK("moe_dispatch");
    return 0;
}
