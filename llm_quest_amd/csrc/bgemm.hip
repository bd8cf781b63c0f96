// Batched / grouped matrix products with general strides (gfx950 only).
//
//   C[b][m, n] = epi( sum_k A[b][m, k] * B[b][n, k] )        b < batch
//
// A element (m, k) of batch b:  A[b * a_bs + row(m) * lda + k]
// B element (n, k) of batch b:  B[b * b_bs + n * sbn + k * sbk]      (sbk == 1: weight stored [out, in]; sbn == 1: stored [in, out])
// C element (m, n) of batch b:  C[b * c_bs + crow(m) * ldc + n]
//
// Uses: the per-head products of latent attention with the key / value up-projections folded onto the query and the output side;
// the experts of a mixture (batch = expert, a batch's rows given by device-side offsets, A rows gathered through a dispatch list,
// C rows scattered back and scaled by the routing weight); and every linear layer of the true-fp32 mode (fp32 activations,
// weights kept in bf16 -- exactly representable -- and widened on load, fp32 FMA accumulation in a fixed k order, so a row's result does not depend
// on which other rows share its tile).
//
// Two compute paths:
//   * FMA: 64 x 64 tile, 256 threads, 4 x 4 outputs per thread, k in steps of 16 through LDS (any operand type);
//   * MFMA (bf16 A and B): the same tile, four waves of 32 x 32 on v_mfma_f32_32x32x8_bf16_1k, k in steps of 32.
#include "common.h"

#define ST(s) ((hipStream_t)(s))

struct BgemmArgs {
    const void* A;
    const void* B;
    void* C;
    int64_t lda, a_bs, sbn, sbk, b_bs, ldc, c_bs;
    int M, N, K;
    const int* grp_offs;     // [batch + 1] or null: rows of batch b are the sorted rows [grp_offs[b], grp_offs[b+1]) (then M is the tile bound)
    const int* a_rows;       // or null: sorted row r reads A row a_rows[r] / a_div
    int a_div;
    const int* c_rows;       // or null: sorted row r writes C row c_rows[r]
    const float* row_scale;  // or null: C row (after c_rows) is multiplied by row_scale[that row]
    const float* bias;       // or null: bias[n] is added to column n before the epilogue
    int epi;                 // 0 none, 1 relu(x)^2, 2 / 3 / 4 gated (see gated_act): B's rows come in blocks of 64 = [32 gate rows | 32 up rows], C has n_out columns
    float limit;
    int n_out;
    int a_dt, b_dt, c_dt;
};

// Gated activations of a feed-forward's [gate | up] product.  2: g = min(gate, limit), u = clamp(up, -limit, limit), g sigmoid(1.702 g) (u + 1).
// 3: gelu_tanh(gate) * up.  4: silu(gate) * up.
__device__ __forceinline__ float gated_act(int epi, float g, float u, float limit) {
    if (epi == 2) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
    }
    if (epi == 4) return g / (1.0f + expf(-g)) * u;
    return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
}

__device__ __forceinline__ float ldx(const void* p, int dt, int64_t i) { return dt == MI355_DT_F32 ? ((const float*)p)[i] : bf2f(((const bf16_t*)p)[i]); }

#define BM 64
#define BN 64
#define BK 16

__global__ __launch_bounds__(256) void bgemm_fma_kernel(BgemmArgs p) {
    __shared__ float As[BK][BM + 4];
    __shared__ float Bs[BK][BN + 4];
    const int b = blockIdx.z;
    int row0 = 0, rows = p.M;
    if (p.grp_offs) {
        row0 = p.grp_offs[b];
        rows = p.grp_offs[b + 1] - row0;
    }
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    if (m0 >= rows) return;
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    // loader roles: A element (m = tid / 4 + {0}, k = (tid % 4) * 4 .. +4): 64 rows x 16 k
    const int am = tid >> 2, ak = (tid & 3) * 4;
    int64_t a_base = -1;
    if (m0 + am < rows) {
        const int r = row0 + m0 + am;
        const int64_t arow = p.a_rows ? p.a_rows[r] / p.a_div : r;
        a_base = (int64_t)b * p.a_bs + arow * p.lda;
    }
    // B loader: if sbk == 1 the same (n = tid / 4, k chunk) shape as A; if sbn == 1, n runs fastest: (k = tid / 16, n = (tid % 16) * 4 .. +4)
    const bool b_kfast = p.sbk == 1;
    const int bn = b_kfast ? tid >> 2 : (tid & 15) * 4, bk = b_kfast ? (tid & 3) * 4 : tid >> 4;
    const int64_t b_base = (int64_t)b * p.b_bs;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < p.K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + ak + i;
            As[ak + i][am] = (a_base >= 0 && k < p.K) ? ldx(p.A, p.a_dt, a_base + k) : 0.f;
        }
        if (b_kfast) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int k = k0 + bk + i, n = n0 + bn;
                Bs[bk + i][bn] = (n < p.N && k < p.K) ? ldx(p.B, p.b_dt, b_base + (int64_t)n * p.sbn + k) : 0.f;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int k = k0 + bk, n = n0 + bn + i;
                Bs[bk][bn + i] = (n < p.N && k < p.K) ? ldx(p.B, p.b_dt, b_base + (int64_t)n * p.sbn + (int64_t)k * p.sbk) : 0.f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float a[4], bb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i], bb[i] = Bs[k][(i >> 1) * 32 + tx * 2 + (i & 1)];  // columns 2 tx, 2 tx + 1 and the same + 32: a gate and its up
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], bb[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= rows) continue;
        const int r = row0 + m;
        const int64_t crow = p.c_rows ? p.c_rows[r] : r;
        const float sc = p.row_scale ? p.row_scale[crow] : 1.0f;
        const int64_t cb = (int64_t)b * p.c_bs + crow * p.ldc;
        if (p.epi >= 2) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int n = (n0 >> 1) + tx * 2 + j;  // gate column n0 + 2 tx + j, up column 32 further
                if (n >= p.n_out) continue;
                const float v = gated_act(p.epi, acc[i][j], acc[i][j + 2], p.limit) * sc;
                if (p.c_dt == MI355_DT_F32) ((float*)p.C)[cb + n] = v;
                else ((bf16_t*)p.C)[cb + n] = f2bf(v);
            }
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + (j >> 1) * 32 + tx * 2 + (j & 1);
            if (n >= p.N) continue;
            float v = acc[i][j] + (p.bias ? p.bias[n] : 0.f);
            if (p.epi == 1) v = v > 0.f ? v * v : 0.f;
            v *= sc;
            if (p.c_dt == MI355_DT_F32) ((float*)p.C)[cb + n] = v;
            else ((bf16_t*)p.C)[cb + n] = f2bf(v);
        }
    }
}

// ---- MFMA path: bf16 A and B.  LDS tiles [64][32 + 8] bf16 (k contiguous; the 16-byte pad keeps the 8-byte fragment reads off one bank group).
// Wave w computes the 32 x 32 block (w / 2, w % 2).  v_mfma_f32_32x32x8_bf16_1k: lane l supplies A[m = l % 32][k = 4 * (l / 32) .. +4] and
// B[n = l % 32][same k]; accumulator register 4 * g + i of lane l is C[m = 8 * g + 4 * (l / 32) + i][n = l % 32].
#define MK 32
#define MPAD 8
__global__ __launch_bounds__(256) void bgemm_mfma_kernel(BgemmArgs p) {
    __shared__ bf16_t As[BM][MK + MPAD];
    __shared__ bf16_t Bs[BN][MK + MPAD];
    const int b = blockIdx.z;
    int row0 = 0, rows = p.M;
    if (p.grp_offs) {
        row0 = p.grp_offs[b];
        rows = p.grp_offs[b + 1] - row0;
    }
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    if (m0 >= rows) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bf16_t* A = (const bf16_t*)p.A;
    const bf16_t* B = (const bf16_t*)p.B;
    // loaders: 64 rows x 32 k = 2048 elements, 8 per thread: (row = tid / 4, k = (tid % 4) * 8 .. +8)
    const int lr = tid >> 2, lk = (tid & 3) * 8;
    int64_t a_base = -1;
    if (m0 + lr < rows) {
        const int r = row0 + m0 + lr;
        const int64_t arow = p.a_rows ? p.a_rows[r] / p.a_div : r;
        a_base = (int64_t)b * p.a_bs + arow * p.lda;
    }
    const bool b_kfast = p.sbk == 1;
    const int64_t b_base = (int64_t)b * p.b_bs;
    const bool a_vec = (p.lda % 8 == 0) && (p.a_bs % 8 == 0) && (((uintptr_t)p.A & 15) == 0);
    const bool b_vec = b_kfast && (p.sbn % 8 == 0) && (p.b_bs % 8 == 0) && (((uintptr_t)p.B & 15) == 0);
    f32x16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    for (int k0 = 0; k0 < p.K; k0 += MK) {
        // A tile
        if (a_base >= 0 && a_vec && k0 + lk + 8 <= p.K) {
            *(u32x4*)&As[lr][lk] = *(const u32x4*)(A + a_base + k0 + lk);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) As[lr][lk + i] = (a_base >= 0 && k0 + lk + i < p.K) ? A[a_base + k0 + lk + i] : (bf16_t)0;
        }
        // B tile
        if (b_kfast) {
            const int n = n0 + lr;
            if (n < p.N && b_vec && k0 + lk + 8 <= p.K) {
                *(u32x4*)&Bs[lr][lk] = *(const u32x4*)(B + b_base + (int64_t)n * p.sbn + k0 + lk);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) Bs[lr][lk + i] = (n < p.N && k0 + lk + i < p.K) ? B[b_base + (int64_t)n * p.sbn + k0 + lk + i] : (bf16_t)0;
            }
        } else {  // n runs fastest in memory: thread (k = tid / 8, n = (tid % 8) * 8 .. +8)
            const int k = k0 + (tid >> 3), nb = (tid & 7) * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int n = n0 + nb + i;
                Bs[nb + i][tid >> 3] = (n < p.N && k < p.K) ? B[b_base + (int64_t)n * p.sbn + (int64_t)k * p.sbk] : (bf16_t)0;
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < MK; kk += 8) {
            const bf16x4 a = *(const bf16x4*)&As[wm + (lane & 31)][kk + 4 * (lane >> 5)];
            const bf16x4 bb = *(const bf16x4*)&Bs[wn + (lane & 31)][kk + 4 * (lane >> 5)];
            acc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a, bb, acc, 0, 0, 0);
        }
        __syncthreads();
    }
    const int n = n0 + wn + (lane & 31);
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + wm + 8 * g + 4 * (lane >> 5) + i;
            if (m >= rows || n >= p.N) continue;
            const int r = row0 + m;
            const int64_t crow = p.c_rows ? p.c_rows[r] : r;
            const float sc = p.row_scale ? p.row_scale[crow] : 1.0f;
            float v = acc[4 * g + i] + (p.bias ? p.bias[n] : 0.f);
            if (p.epi == 1) v = v > 0.f ? v * v : 0.f;
            v *= sc;
            const int64_t ci = (int64_t)b * p.c_bs + crow * p.ldc + n;
            if (p.c_dt == MI355_DT_F32) ((float*)p.C)[ci] = v;
            else ((bf16_t*)p.C)[ci] = f2bf(v);
        }
}

// ---- MFMA path, 128 x 128 tile: four waves of 64 x 64 (2 x 2 blocks of 32 x 32), k in steps of 32; the next step's operands are fetched into registers
// while the current step multiplies from LDS (one LDS stage, two barriers per step).  Four LDS fragment reads feed four MFMAs.
#define TM 128
__global__ __launch_bounds__(256) void bgemm_mfma128_kernel(BgemmArgs p) {
    __shared__ __attribute__((aligned(16))) bf16_t As[TM][MK + MPAD];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[TM][MK + MPAD];
    const int b = blockIdx.z;
    int row0 = 0, rows = p.M;
    if (p.grp_offs) {
        row0 = p.grp_offs[b];
        rows = p.grp_offs[b + 1] - row0;
    }
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TM;
    if (m0 >= rows) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, ln = lane & 31, hf = lane >> 5;
    const bf16_t* A = (const bf16_t*)p.A;
    const bf16_t* B = (const bf16_t*)p.B;
    const bool b_kfast = p.sbk == 1;
    const int64_t b_base = (int64_t)b * p.b_bs;
    const bool a_vec = (p.lda % 8 == 0) && (p.a_bs % 8 == 0) && (((uintptr_t)p.A & 15) == 0);
    const bool b_vec = b_kfast && (p.sbn % 8 == 0) && (p.b_bs % 8 == 0) && (((uintptr_t)p.B & 15) == 0);
    // loader roles: chunk c = tid + 256 i (i < 2): row c / 4, k offset (c % 4) * 8
    int64_t a_base[2];
    int lr[2], lk[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int c = tid + 256 * i;
        lr[i] = c >> 2, lk[i] = (c & 3) * 8;
        a_base[i] = -1;
        if (m0 + lr[i] < rows) {
            const int r = row0 + m0 + lr[i];
            const int64_t arow = p.a_rows ? p.a_rows[r] / p.a_div : r;
            a_base[i] = (int64_t)b * p.a_bs + arow * p.lda;
        }
    }
    u32x4 ra[2], rb[2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            u32x4 va = {0u, 0u, 0u, 0u}, vb = {0u, 0u, 0u, 0u};
            if (a_base[i] >= 0) {
                if (a_vec && k0 + lk[i] + 8 <= p.K) va = *(const u32x4*)(A + a_base[i] + k0 + lk[i]);
                else {
                    bf16_t e[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) e[j] = k0 + lk[i] + j < p.K ? A[a_base[i] + k0 + lk[i] + j] : (bf16_t)0;
                    va = u32x4{(unsigned)e[0] | ((unsigned)e[1] << 16), (unsigned)e[2] | ((unsigned)e[3] << 16), (unsigned)e[4] | ((unsigned)e[5] << 16), (unsigned)e[6] | ((unsigned)e[7] << 16)};
                }
            }
            const int n = n0 + lr[i];
            if (n < p.N) {
                if (b_vec && k0 + lk[i] + 8 <= p.K) vb = *(const u32x4*)(B + b_base + (int64_t)n * p.sbn + k0 + lk[i]);
                else {
                    bf16_t e[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) e[j] = k0 + lk[i] + j < p.K ? B[b_base + (int64_t)n * p.sbn + (int64_t)(k0 + lk[i] + j) * p.sbk] : (bf16_t)0;
                    vb = u32x4{(unsigned)e[0] | ((unsigned)e[1] << 16), (unsigned)e[2] | ((unsigned)e[3] << 16), (unsigned)e[4] | ((unsigned)e[5] << 16), (unsigned)e[6] | ((unsigned)e[7] << 16)};
                }
            }
            ra[i] = va, rb[i] = vb;
        }
    };
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    fetch(0);
    for (int k0 = 0; k0 < p.K; k0 += MK) {
        __syncthreads();  // the previous step's fragments are read
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            *(u32x4*)&As[lr[i]][lk[i]] = ra[i];
            *(u32x4*)&Bs[lr[i]][lk[i]] = rb[i];
        }
        __syncthreads();
        if (k0 + MK < p.K) fetch(k0 + MK);
#pragma unroll
        for (int kk = 0; kk < MK; kk += 8) {
            const bf16x4 a0 = *(const bf16x4*)&As[wm + ln][kk + 4 * hf], a1 = *(const bf16x4*)&As[wm + 32 + ln][kk + 4 * hf];
            const bf16x4 b0 = *(const bf16x4*)&Bs[wn + ln][kk + 4 * hf], b1 = *(const bf16x4*)&Bs[wn + 32 + ln][kk + 4 * hf];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a1, b1, acc[1][1], 0, 0, 0);
        }
    }
#pragma unroll
    for (int bi = 0; bi < 2; ++bi)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = m0 + wm + 32 * bi + 8 * g + 4 * hf + i;
                if (m >= rows) continue;
                const int r = row0 + m;
                const int64_t crow = p.c_rows ? p.c_rows[r] : r;
                const float sc = p.row_scale ? p.row_scale[crow] : 1.0f;
                const int64_t cb = (int64_t)b * p.c_bs + crow * p.ldc;
                if (p.epi >= 2) {  // this wave's 64 columns are one [32 gates | 32 ups] block: the lane holds a gate (bj = 0) and its up (bj = 1)
                    const int n = ((n0 + wn) >> 1) + ln;
                    if (n < p.n_out) {
                        const float v = gated_act(p.epi, acc[bi][0][4 * g + i], acc[bi][1][4 * g + i], p.limit) * sc;
                        if (p.c_dt == MI355_DT_F32) ((float*)p.C)[cb + n] = v;
                        else ((bf16_t*)p.C)[cb + n] = f2bf(v);
                    }
                    continue;
                }
#pragma unroll
                for (int bj = 0; bj < 2; ++bj) {
                    const int n = n0 + wn + 32 * bj + ln;
                    if (n >= p.N) continue;
                    float v = acc[bi][bj][4 * g + i] + (p.bias ? p.bias[n] : 0.f);
                    if (p.epi == 1) v = v > 0.f ? v * v : 0.f;
                    v *= sc;
                    if (p.c_dt == MI355_DT_F32) ((float*)p.C)[cb + n] = v;
                    else ((bf16_t*)p.C)[cb + n] = f2bf(v);
                }
            }
}

extern "C" int mi355_bgemm(int batch, int M, int N, int K, const void* A, int a_dt, int64_t lda, int64_t a_bs, const void* B, int b_dt, int64_t sbn, int64_t sbk,
                           int64_t b_bs, void* C, int c_dt, int64_t ldc, int64_t c_bs, const int* grp_offs, const int* a_rows, int a_div, const int* c_rows,
                           const float* row_scale, int epi, int use_mfma, const float* bias, float limit, int n_out, void* stream) {
    MI355_REQUIRE(batch > 0 && batch <= 65535 && M > 0 && N > 0 && K > 0 && A && B && C, "bgemm: bad arguments");
    MI355_REQUIRE((a_dt == MI355_DT_BF16 || a_dt == MI355_DT_F32) && (b_dt == MI355_DT_BF16 || b_dt == MI355_DT_F32) && (c_dt == MI355_DT_BF16 || c_dt == MI355_DT_F32),
                  "bgemm: bad dtype");
    MI355_REQUIRE(epi >= 0 && epi <= 4, "bgemm: bad epilogue");
    MI355_REQUIRE(epi < 2 || (N % 64 == 0 && n_out > 0 && n_out <= N / 2 && !bias), "bgemm: a gated epilogue takes B rows in [32 gate | 32 up] blocks (N a multiple of 64), n_out <= N / 2 columns, no bias");
    MI355_REQUIRE(!a_rows || a_div >= 1, "bgemm: gathered rows need a divisor >= 1");
    MI355_REQUIRE(sbn >= 1 && sbk >= 1 && (sbn == 1 || sbk == 1), "bgemm: one of B's strides must be 1");
    MI355_REQUIRE(!use_mfma || (a_dt == MI355_DT_BF16 && b_dt == MI355_DT_BF16), "bgemm: the MFMA path takes bf16 operands");
    BgemmArgs p;
    p.A = A, p.B = B, p.C = C;
    p.lda = lda, p.a_bs = a_bs, p.sbn = sbn, p.sbk = sbk, p.b_bs = b_bs, p.ldc = ldc, p.c_bs = c_bs;
    p.M = M, p.N = N, p.K = K;
    p.grp_offs = grp_offs, p.a_rows = a_rows, p.a_div = a_rows ? a_div : 1, p.c_rows = c_rows, p.row_scale = row_scale;
    p.bias = bias;
    p.limit = limit, p.n_out = n_out;
    p.epi = epi, p.a_dt = a_dt, p.b_dt = b_dt, p.c_dt = c_dt;
    if (use_mfma && ((sbk == 1 && N >= 128 && K >= 64) || epi >= 2)) {  // (a gated epilogue needs a gate and its up in one lane: this kernel's 64 columns per wave)  // the large tile: weights stored [out, in], enough columns to fill it
        const int64_t my128 = ((int64_t)M + TM - 1) / TM;
        MI355_REQUIRE(my128 <= 65535, "bgemm: too many row tiles");
        bgemm_mfma128_kernel<<<dim3((N + TM - 1) / TM, (unsigned)my128, batch), 256, 0, ST(stream)>>>(p);
        MI355_LAUNCH_CHECK("bgemm");
        return 0;
    }
    const int64_t my = ((int64_t)M + BM - 1) / BM;
    MI355_REQUIRE(my <= 65535, "bgemm: too many row tiles");
    const dim3 grid((N + BN - 1) / BN, (unsigned)my, batch);
    if (use_mfma) bgemm_mfma_kernel<<<grid, 256, 0, ST(stream)>>>(p);
    else bgemm_fma_kernel<<<grid, 256, 0, ST(stream)>>>(p);
    MI355_LAUNCH_CHECK("bgemm");
    return 0;
}
