// Causal softmax attention whose keys come in two parts -- a main part (per head, or one shared by all heads) and a rotated part shared by
// all heads -- over ragged batches (gfx950 only).  It serves multi-head latent attention in both of its forms:
//   * expanded (prompts): K1 = the per-head keys and V = the per-head values rebuilt from the latent rows of this step, K2 = the rotated key part;
//   * folded (one-token steps): the key up-projection is folded into the query and the value up-projection is applied after the attention, so
//     K1 = V = the cached latent rows themselves (head stride 0), K2 = the cached rotated part: the cache is read once for all heads.
//
// score(row, j) = scale * ( Q[row, :D1] . K1[j, head, :] + Q[row, D1:] . K2[j, :] ),  softmax over j <= past + token index, out = sum_j p V[j].
// The same kernels serve grouped-query attention (kv_rep query heads per key / value head, D2 = 0) and a sliding window that keeps the first tokens
// (window, keep_first): key steps that no row of a tile can see are skipped.  Further options: tanh-capped scores (softcap), a per-head sink that
// only enters the softmax denominator, and POOLED blocks in front of a window -- one mean key / value row per `pool` tokens, kept by the caller in a
// second buffer; the query at position i sees block b iff all of its tokens have left the window, (b + 1) pool <= i - window + 1.  Pooled rows
// and tokens share one softmax: the key loop simply runs over the pooled rows first.
// Scores, softmax statistics and the output accumulators are fp32.  A tile is `tm` tokens x `hm` heads = 32 query rows (hm > 1 only with shared
// keys and values) against 64 keys at a time.
//
// Two compute paths: fp32 FMA through LDS (any operand type: the true-fp32 mode), and bf16 MFMA (v_mfma_f32_32x32x8_bf16_1k) for bf16 keys / values.
#include "common.h"

#define ST(s) ((hipStream_t)(s))

struct LatAttnArgs {
    const float* Q;
    const void* K1;
    const void* K2;
    const void* V;
    void* O;
    int64_t ldq, ldk1, ldk2, ldv, ldo;
    int q_hs, k1_hs, v_hs, o_hs;
    int D1, D2, DV, H, hm, dt;
    const int *q_row0, *n_new, *past, *k1_row0, *k2_row0, *v_row0;
    float scale;
    int splits;  // MFMA path: a tile's keys are dealt to `splits` workgroups; partial (max, sum, output) rows go to ws and latent_attn_combine_kernel joins them
    float* ws;   // per (sequence, head tile, token tile, split): 128 maxima | 128 sums | 128 x DVP unnormalised outputs
    int kv_rep;  // query heads per key / value head (grouped queries): head h reads key / value head h / kv_rep
    int window;  // > 0: a query at position i sees key j <= i only if i - j < window or j < keep_first (sliding window that keeps the first tokens)
    int keep_first;
    int chunk;  // > 0: positions are cut into chunks of this many, counted from the sequence's first token; a query sees only the keys of its own chunk
    float softcap;      // > 0: score <- softcap * tanh(score / softcap) after the scale
    const float* sink;  // fp32 [H] or NULL: exp(sink[h]) joins the denominator of head h (no key, no value, not scaled)
    int pool;           // > 0: one pooled key / value row per `pool` tokens (needs window > 0, D2 == 0); rows PK / PV, first row of sequence s = pool_row0[s]
    const void *PK, *PV;
    int64_t ldp;
    const int* pool_row0;
};

// pooled blocks the query at position lim sees: those that end at or before lim - window
__device__ __forceinline__ int pooled_visible(int lim, int window, int pool) {
    const int gone = lim - window + 1;  // tokens that have left the window
    return gone > 0 ? gone / pool : 0;
}
// the capped score (natural units)
__device__ __forceinline__ float cap_score(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }

// key j for the query at position lim (lim < 0: a padding row that sees nothing)
__device__ __forceinline__ bool key_visible(int j, int lim, int window, int keep_first, int chunk) {
    return j <= lim && (window <= 0 || lim - j < window || j < keep_first) && (chunk <= 0 || j >= lim / chunk * chunk);
}
// keys below this one are seen by no row of a tile whose first row stands at position pos0 (rows of a tile are consecutive positions)
__device__ __forceinline__ int tile_key_floor(int pos0, int window, int chunk) {
    const int w = window > 0 ? pos0 - window + 1 : 0, c = chunk > 0 ? pos0 / chunk * chunk : 0;
    return max(w, c);
}

__device__ __forceinline__ float lda_dt(const void* p, int dt, int64_t i) { return dt == MI355_DT_F32 ? ((const float*)p)[i] : bf2f(((const bf16_t*)p)[i]); }

#define AM 32  // query rows per tile
#define AN 64  // keys per step
#define AC 32  // feature chunk of the score product

template <int NC>
__global__ __launch_bounds__(256) void latent_attn_fma_kernel(LatAttnArgs p) {
    __shared__ float Qs[AM][AC + 1];
    __shared__ float Ks[AN][AC + 1];
    __shared__ float Ps[AM][AN + 4];
    __shared__ float fs[AM], ls[AM];
    const int s = blockIdx.z, tm = AM / p.hm;
    const int tok0 = blockIdx.x * tm, head0 = blockIdx.y * p.hm;
    const int n_new = p.n_new[s], past = p.past[s];
    if (tok0 >= n_new) return;
    const int64_t qr0 = p.q_row0[s], k1r0 = p.k1_row0[s], k2r0 = p.k2_row0[s], vr0 = p.v_row0[s];
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int DK = p.D1 + p.D2;
    const int n_keys = past + min(tok0 + tm, n_new);  // keys any row of the tile may see
    // S layout: rows 2 ty, 2 ty + 1; keys tx + 16 i
    int lim[2];
    float m_run[2] = {-__builtin_huge_valf(), -__builtin_huge_valf()}, l_run[2] = {0.f, 0.f};
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const int r = 2 * ty + a, tok = tok0 + r / p.hm, head = head0 + r % p.hm;
        lim[a] = (tok < n_new && head < p.H) ? past + tok : -1;
    }
    // PV layout: rows 8 rg .. +8, columns c + 64 i
    const int rg = tid >> 6, c = tid & 63;
    float o[8][NC];
#pragma unroll
    for (int r = 0; r < 8; ++r)
#pragma unroll
        for (int i = 0; i < NC; ++i) o[r][i] = 0.f;

    const int kvh = head0 / p.kv_rep;
    const int win_lo = tile_key_floor(past + tok0, p.window, p.chunk);  // keys below it are outside the window (or chunk) of every row of the tile
    const int n_pool = p.pool > 0 ? pooled_visible(n_keys - 1, p.window, p.pool) : 0;  // pooled rows any row of the tile may see
    const int pool_steps = (n_pool + AN - 1) / AN;
    const int64_t pr0 = p.pool > 0 ? p.pool_row0[s] : 0;
    int npv[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) npv[a] = p.pool > 0 ? pooled_visible(lim[a], p.window, p.pool) : 0;
    for (int it = -pool_steps;; ++it) {
        const bool seg = it < 0;  // the pooled rows come first
        const int j0 = seg ? (it + pool_steps) * AN : it * AN;
        const int n_here = seg ? n_pool : n_keys;
        if (!seg) {
            if (j0 >= n_keys) break;
            if (j0 + AN <= win_lo && j0 >= p.keep_first) continue;  // block-uniform: no row sees a key of this step
        }
        const void* Kp = seg ? p.PK : p.K1;
        const void* Vp = seg ? p.PV : p.V;
        const int64_t kr = seg ? pr0 : k1r0, vr = seg ? pr0 : vr0, ldk = seg ? p.ldp : p.ldk1, ldvv = seg ? p.ldp : p.ldv;
        float acc[2][4] = {};
        for (int d0 = 0; d0 < DK; d0 += AC) {
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 4; ++i) {  // Q chunk: 32 rows x 32 features
                const int e = tid + 256 * i, d = d0 + (e & 31), r = e >> 5;
                const int tok = tok0 + r / p.hm, head = head0 + r % p.hm;
                Qs[r][e & 31] = (d < DK && tok < n_new && head < p.H) ? p.Q[(qr0 + tok) * p.ldq + (int64_t)head * p.q_hs + d] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {  // K chunk: 64 keys x 32 features
                const int e = tid + 256 * i, d = d0 + (e & 31), j = j0 + (e >> 5);
                float v = 0.f;
                if (j < n_here && d < DK)
                    v = d < p.D1 ? lda_dt(Kp, p.dt, (kr + j) * ldk + (int64_t)kvh * p.k1_hs + d) : lda_dt(p.K2, p.dt, (k2r0 + j) * p.ldk2 + (d - p.D1));
                Ks[e >> 5][e & 31] = v;
            }
            __syncthreads();
#pragma unroll
            for (int d = 0; d < AC; ++d) {
                const float q0 = Qs[2 * ty][d], q1 = Qs[2 * ty + 1][d];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float kv = Ks[tx + 16 * i][d];
                    acc[0][i] = fmaf(q0, kv, acc[0][i]);
                    acc[1][i] = fmaf(q1, kv, acc[1][i]);
                }
            }
        }
        // online softmax over this step's keys
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            float mx = -__builtin_huge_valf();
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = j0 + tx + 16 * i;
                const bool vis = seg ? j < npv[a] : key_visible(j, lim[a], p.window, p.keep_first, p.chunk);
                acc[a][i] = vis ? cap_score(acc[a][i] * p.scale, p.softcap) : -__builtin_huge_valf();
                mx = fmaxf(mx, acc[a][i]);
            }
#pragma unroll
            for (int of = 8; of > 0; of >>= 1) mx = fmaxf(mx, __shfl_xor(mx, of, 64));
            const float m_new = fmaxf(m_run[a], mx);
            const float base = m_new == -__builtin_huge_valf() ? 0.f : m_new;
            const float f = expf(m_run[a] - base);
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = expf(acc[a][i] - base);
                Ps[2 * ty + a][tx + 16 * i] = e;
                sum += e;
            }
#pragma unroll
            for (int of = 8; of > 0; of >>= 1) sum += __shfl_xor(sum, of, 64);
            l_run[a] = l_run[a] * f + sum;
            m_run[a] = m_new;
            if (tx == 0) fs[2 * ty + a] = f;
        }
        __syncthreads();
        // O <- O * f + P V
        const int nk = min(AN, n_here - j0);
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const float f = fs[8 * rg + r];
#pragma unroll
            for (int i = 0; i < NC; ++i) o[r][i] *= f;
        }
        for (int j = 0; j < nk; ++j) {
            float vv[NC];
#pragma unroll
            for (int i = 0; i < NC; ++i) {
                const int col = c + 64 * i;
                vv[i] = col < p.DV ? lda_dt(Vp, p.dt, (vr + j0 + j) * ldvv + (int64_t)kvh * p.v_hs + col) : 0.f;
            }
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const float pj = Ps[8 * rg + r][j];
#pragma unroll
                for (int i = 0; i < NC; ++i) o[r][i] = fmaf(pj, vv[i], o[r][i]);
            }
        }
    }
    __syncthreads();
    if (tx == 0) {
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            const int r = 2 * ty + a, head = head0 + r % p.hm;
            float l = l_run[a], f = 1.0f;
            if (p.sink && head < p.H) {  // the sink joins the denominator: out = O f / (l f + exp(sink - m'))
                const float sk = p.sink[head], m2 = fmaxf(m_run[a], sk);
                f = expf(m_run[a] - m2);
                l = l * f + expf(sk - m2);
            }
            ls[r] = l, fs[r] = f;
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const int row = 8 * rg + r, tok = tok0 + row / p.hm, head = head0 + row % p.hm;
        if (tok >= n_new || head >= p.H) continue;
        const float inv = fs[row] / ls[row];
        const int64_t ob = (qr0 + tok) * p.ldo + (int64_t)head * p.o_hs;
#pragma unroll
        for (int i = 0; i < NC; ++i) {
            const int col = c + 64 * i;
            if (col >= p.DV) continue;
            const float v = o[r][i] * inv;
            if (p.dt == MI355_DT_F32) ((float*)p.O)[ob + col] = v;
            else ((bf16_t*)p.O)[ob + col] = f2bf(v);
        }
    }
}


// ---- MFMA path (bf16 keys / values).  A workgroup is four waves; wave w owns query rows 32 w .. 32 w + 31 of a 128-row tile and keeps their Q fragments
// (bf16) in registers.  Scores are computed transposed, S^T = K Q^T (v_mfma_f32_32x32x8_bf16_1k: A = 32 keys x 8 features from LDS, B = the lane's own
// query), so a lane holds 16 of every 32 keys of ONE query: the softmax statistics are lane-local plus one exchange with lane ^ 32, the rescale factor
// of the transposed output O^T = V^T P^T is lane-local too, and P (bf16) is the B operand of that product as it stands in registers.  The key tile lies in
// LDS as [64 keys][DKP] (main part and rotated part side by side, zero padded), the value tile transposed as [DVP][64 keys].
#define MQ 128
#define MKT 64
template <int DKS, int NVB>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(LatAttnArgs p, int vec_ok) {
    constexpr int DKP = DKS * 8, DVP = NVB * 32, KLD = DKP + 4, VLD = MKT + 4;
    __shared__ __attribute__((aligned(16))) bf16_t Ks[MKT * KLD];
    __shared__ __attribute__((aligned(16))) bf16_t Vt[DVP * VLD];
    const int s = blockIdx.z, tm = MQ / p.hm;
    const int tile = blockIdx.x / p.splits, split = blockIdx.x % p.splits;
    const int tok0 = tile * tm, head0 = blockIdx.y * p.hm;
    const int n_new = p.n_new[s], past = p.past[s];
    if (tok0 >= n_new) return;
    const int64_t qr0 = p.q_row0[s], k1r0 = p.k1_row0[s], k2r0 = p.k2_row0[s], vr0 = p.v_row0[s];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, ln = lane & 31, hf = lane >> 5;
    const int DK = p.D1 + p.D2;
    const bf16_t* K1 = (const bf16_t*)p.K1;
    const bf16_t* K2 = (const bf16_t*)p.K2;
    const bf16_t* V = (const bf16_t*)p.V;
    // this lane's query
    const int row = 32 * wave + ln, tok = tok0 + row / p.hm, head = head0 + row % p.hm;
    const bool row_ok = tok < n_new && head < p.H;
    const int lim = row_ok ? past + tok : -1;
    bf16x4 qf[DKS];
    {
        const float* qrow = p.Q + (qr0 + (row_ok ? tok : 0)) * p.ldq + (int64_t)(row_ok ? head : 0) * p.q_hs;
#pragma unroll
        for (int st = 0; st < DKS; ++st) {
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int d = 8 * st + 4 * hf + j;
                v[j] = (row_ok && d < DK) ? qrow[d] : 0.f;
            }
            const unsigned lo = pack_bf2(v[0], v[1]), hi = pack_bf2(v[2], v[3]);
            u32x2 pk = {lo, hi};
            qf[st] = __builtin_bit_cast(bf16x4, pk);
        }
    }
    const int n_keys = past + min(tok0 + tm, n_new);
    const int win_lo = tile_key_floor(past + tok0, p.window, p.chunk);  // keys below it are outside the window (or chunk) of every row of the tile
    // The tile's work is a list of 64-row steps: first the pooled rows any of its rows may see, then the keys from key_lo on (under a plain window dealt
    // out to several workgroups that is the window's lower edge, else 0: steps below a window are skipped one by one).  Workgroup `split` takes its share.
    const int n_pool = p.pool > 0 ? pooled_visible(n_keys - 1, p.window, p.pool) : 0;
    const int pool_steps = (n_pool + MKT - 1) / MKT;
    const int key_lo = (p.splits > 1 && p.keep_first == 0 && win_lo > 0) ? win_lo / MKT * MKT : 0;
    const int all_steps = pool_steps + (n_keys - key_lo + MKT - 1) / MKT;
    int v_lo = 0, v_hi = all_steps;
    if (p.splits > 1) {
        const int per = (all_steps + p.splits - 1) / p.splits;
        v_lo = split * per;
        v_hi = min(all_steps, v_lo + per);
    }
    // the last key any row of this WAVE may see (its rows are consecutive, so its last valid row has the largest limit)
    int wave_lim = lim;
#pragma unroll
    for (int of = 32; of > 0; of >>= 1) wave_lim = max(wave_lim, __shfl_xor(wave_lim, of, 64));
    f32x16 oacc[NVB];
#pragma unroll
    for (int vb = 0; vb < NVB; ++vb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[vb][i] = 0.f;
    const float NEG = -__builtin_huge_valf();
    float m_run = NEG, l_run = 0.f;
    const float sc2 = p.scale * 1.4426950408889634f;

    const int kvh = head0 / p.kv_rep;
    const int npv = p.pool > 0 ? pooled_visible(lim, p.window, p.pool) : 0;  // the pooled rows this lane's query sees
    const int64_t pr0 = p.pool > 0 ? p.pool_row0[s] : 0;
    const float capl = p.softcap * 1.4426950408889634f;
    for (int v = v_lo; v < v_hi; ++v) {
        const bool seg = v < pool_steps;  // the pooled rows come first
        const int j0 = seg ? v * MKT : key_lo + (v - pool_steps) * MKT;
        const int n_here = seg ? n_pool : n_keys;
        if (!seg && j0 + MKT <= win_lo && j0 >= p.keep_first) continue;  // block-uniform: no row sees a key of this step
        const bf16_t* Kp = seg ? (const bf16_t*)p.PK : K1;
        const bf16_t* Vp = seg ? (const bf16_t*)p.PV : V;
        const int64_t kr = seg ? pr0 : k1r0, vr = seg ? pr0 : vr0, ldk = seg ? p.ldp : p.ldk1, ldvv = seg ? p.ldp : p.ldv;
        __syncthreads();
        // ---- key tile -> LDS
        for (int c = tid; c < MKT * DKS; c += 256) {
            const int key = c / DKS, d0 = (c % DKS) * 8, j = j0 + key;
            u32x4 val = {0u, 0u, 0u, 0u};
            if (j < n_here) {
                if (vec_ok && d0 + 8 <= p.D1) {
                    val = *(const u32x4*)(Kp + (kr + j) * ldk + (int64_t)kvh * p.k1_hs + d0);
                } else if (vec_ok && d0 >= p.D1 && d0 + 8 <= DK) {
                    val = *(const u32x4*)(K2 + (k2r0 + j) * p.ldk2 + (d0 - p.D1));
                } else {
                    bf16_t e[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const int d = d0 + i;
                        e[i] = d < p.D1 ? Kp[(kr + j) * ldk + (int64_t)kvh * p.k1_hs + d] : (d < DK ? K2[(k2r0 + j) * p.ldk2 + (d - p.D1)] : (bf16_t)0);
                    }
                    val = u32x4{(unsigned)e[0] | ((unsigned)e[1] << 16), (unsigned)e[2] | ((unsigned)e[3] << 16), (unsigned)e[4] | ((unsigned)e[5] << 16),
                                (unsigned)e[6] | ((unsigned)e[7] << 16)};
                }
            }
            u32x2* dst = (u32x2*)&Ks[key * KLD + d0];  // rows are 8-byte aligned (KLD % 4 == 0)
            dst[0] = u32x2{val[0], val[1]};
            dst[1] = u32x2{val[2], val[3]};
        }
        // ---- value tile -> LDS, transposed
        for (int c = tid; c < MKT * (DVP / 8); c += 256) {
            const int key = c % MKT, v0 = (c / MKT) * 8, j = j0 + key;
            bf16_t e[8];
            if (j < n_here && vec_ok && v0 + 8 <= p.DV) {
                const u32x4 val = *(const u32x4*)(Vp + (vr + j) * ldvv + (int64_t)kvh * p.v_hs + v0);
#pragma unroll
                for (int i = 0; i < 4; ++i) e[2 * i] = (bf16_t)(val[i] & 0xffffu), e[2 * i + 1] = (bf16_t)(val[i] >> 16);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) e[i] = (j < n_here && v0 + i < p.DV) ? Vp[(vr + j) * ldvv + (int64_t)kvh * p.v_hs + v0 + i] : (bf16_t)0;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) Vt[(v0 + i) * VLD + key] = e[i];
        }
        __syncthreads();
        if (!seg && j0 > wave_lim) continue;  // every key of this step lies behind the wave's rows (the barriers above are still reached by all)
        // ---- S^T = K Q^T: two blocks of 32 keys
        f32x16 sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) sacc[kb][i] = 0.f;
#pragma unroll
            for (int st = 0; st < DKS; ++st) {
                const bf16x4 a = *(const bf16x4*)&Ks[(kb * 32 + ln) * KLD + 8 * st + 4 * hf];
                sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a, qf[st], sacc[kb], 0, 0, 0);
            }
        }
        // ---- online softmax for the lane's query (keys kb * 32 + 8 g + 4 hf + i)
        float mx = NEG;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int j = j0 + kb * 32 + 8 * (r >> 2) + 4 * hf + (r & 3);
                const bool vis = seg ? j < npv : (key_visible(j, lim, p.window, p.keep_first, p.chunk) && j < n_keys);
                const float v = !vis ? NEG : (p.softcap > 0.f ? capl * tanhf(sacc[kb][r] * p.scale / p.softcap) : sacc[kb][r] * sc2);
                sacc[kb][r] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        const float base = m_new == NEG ? 0.f : m_new;
        const float f = exp2f(m_run - base);
        float sum = 0.f;
        bf16x4 pf[8];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float e[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    e[i] = exp2f(sacc[kb][4 * g + i] - base);
                    sum += e[i];
                }
                u32x2 pk = {pack_bf2(e[0], e[1]), pack_bf2(e[2], e[3])};
                pf[kb * 4 + g] = __builtin_bit_cast(bf16x4, pk);
            }
        sum += __shfl_xor(sum, 32, 64);
        l_run = l_run * f + sum;
        m_run = m_new;
        // ---- O^T <- O^T * f + V^T P^T
#pragma unroll
        for (int vb = 0; vb < NVB; ++vb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[vb][i] *= f;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const bf16x4 a = *(const bf16x4*)&Vt[(vb * 32 + ln) * VLD + 8 * ks + 4 * hf];
                oacc[vb] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a, pf[ks], oacc[vb], 0, 0, 0);
            }
        }
    }
    if (p.splits > 1) {  // partial results; rows that see nothing keep max = -inf and sum = 0
        const int64_t blk = (((int64_t)s * gridDim.y + blockIdx.y) * (gridDim.x / p.splits) + tile) * p.splits + split;
        float* base = p.ws + blk * (int64_t)(MQ * (2 + DVP));
        if (hf == 0) base[row] = m_run, base[MQ + row] = l_run;
#pragma unroll
        for (int vb = 0; vb < NVB; ++vb)
#pragma unroll
            for (int r = 0; r < 16; ++r) base[2 * MQ + (int64_t)row * DVP + vb * 32 + 8 * (r >> 2) + 4 * hf + (r & 3)] = oacc[vb][r];
        return;
    }
    if (!row_ok) return;
    float inv = 1.0f / l_run;
    if (p.sink) {  // the sink joins the denominator (statistics are in base-2 units)
        const float sk = p.sink[head] * 1.4426950408889634f, m2 = fmaxf(m_run, sk), f = exp2f(m_run - m2);
        inv = f / (l_run * f + exp2f(sk - m2));
    }
    bf16_t* orow = (bf16_t*)p.O + (qr0 + tok) * p.ldo + (int64_t)head * p.o_hs;
#pragma unroll
    for (int vb = 0; vb < NVB; ++vb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int dv = vb * 32 + 8 * (r >> 2) + 4 * hf + (r & 3);
            if (dv < p.DV) orow[dv] = f2bf(oacc[vb][r] * inv);
        }
}

// Joins the partial results of a tile's key splits: one wave per query row.
__global__ __launch_bounds__(256) void latent_attn_combine_kernel(LatAttnArgs p, int DVP, int tiles, int gy, int n_seq) {
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (sequence, head tile, token tile, row)
    const int row = (int)(item % MQ);
    int64_t rest = item / MQ;
    const int tile = (int)(rest % tiles);
    rest /= tiles;
    const int by = (int)(rest % gy), s = (int)(rest / gy);
    if (s >= n_seq) return;
    const int tm = MQ / p.hm, tok = tile * tm + row / p.hm, head = by * p.hm + row % p.hm;
    if (tok >= p.n_new[s] || head >= p.H) return;
    const int64_t blk0 = (((int64_t)s * gy + by) * tiles + tile) * p.splits;
    const int64_t stride = (int64_t)MQ * (2 + DVP);
    float m = -__builtin_huge_valf();
    for (int i = 0; i < p.splits; ++i) m = fmaxf(m, p.ws[(blk0 + i) * stride + row]);
    float l = 0.f;
    if (p.sink) {
        const float sk = p.sink[head] * 1.4426950408889634f;
        m = fmaxf(m, sk);
        l = exp2f(sk - m);
    }
    for (int i = 0; i < p.splits; ++i) {
        const float mi = p.ws[(blk0 + i) * stride + row];
        if (mi != -__builtin_huge_valf()) l += p.ws[(blk0 + i) * stride + MQ + row] * exp2f(mi - m);
    }
    bf16_t* orow = (bf16_t*)p.O + ((int64_t)p.q_row0[s] + tok) * p.ldo + (int64_t)head * p.o_hs;
    for (int dv = lane; dv < p.DV; dv += 64) {
        float acc = 0.f;
        for (int i = 0; i < p.splits; ++i) {
            const float mi = p.ws[(blk0 + i) * stride + row];
            if (mi != -__builtin_huge_valf()) acc += p.ws[(blk0 + i) * stride + 2 * MQ + (int64_t)row * DVP + dv] * exp2f(mi - m);
        }
        orow[dv] = f2bf(acc / l);
    }
}

template <int DKS>
static int launch_mfma(const LatAttnArgs& p, dim3 grid, int vec_ok, hipStream_t st) {
    if (p.DV <= 32) latent_attn_mfma_kernel<DKS, 1><<<grid, 256, 0, st>>>(p, vec_ok);
    else if (p.DV <= 64) latent_attn_mfma_kernel<DKS, 2><<<grid, 256, 0, st>>>(p, vec_ok);
    else if (p.DV <= 128) latent_attn_mfma_kernel<DKS, 4><<<grid, 256, 0, st>>>(p, vec_ok);
    else latent_attn_mfma_kernel<DKS, 8><<<grid, 256, 0, st>>>(p, vec_ok);
    return 0;
}

extern "C" int mi355_latent_attn(int n_seq, int max_new, int H, int hm, int D1, int D2, int DV, const float* Q, int64_t ldq, int q_hs, const void* K1, int64_t ldk1,
                                 int k1_hs, const void* K2, int64_t ldk2, const void* V, int64_t ldv, int v_hs, void* O, int64_t ldo, int o_hs, int dt,
                                 const int* q_row0, const int* n_new, const int* past, const int* k1_row0, const int* k2_row0, const int* v_row0, float scale,
                                 int use_mfma, int splits, float* ws, int64_t ws_floats, int kv_rep, int window, int keep_first, float softcap, const float* sink,
                                 int pool, const void* PK, const void* PV, int64_t ldp, const int* pool_row0, int chunk, void* stream) {
    MI355_REQUIRE(n_seq > 0 && n_seq <= 65535 && max_new > 0 && H > 0 && D1 > 0 && D2 >= 0 && DV > 0 && DV <= 512 && Q && K1 && V && O && (D2 == 0 || K2),
                  "latent_attn: bad arguments (value width <= 512)");
    MI355_REQUIRE(dt == MI355_DT_BF16 || dt == MI355_DT_F32, "latent_attn: bad dtype");
    MI355_REQUIRE(kv_rep >= 1 && H % kv_rep == 0 && window >= 0 && keep_first >= 0, "latent_attn: bad head grouping or window");
    MI355_REQUIRE(hm >= 1 && hm <= AM && AM % hm == 0 && (hm == 1 || (k1_hs == 0 && v_hs == 0) || kv_rep % hm == 0),
                  "latent_attn: several heads per tile (a power of two <= 32) need shared keys and values (head stride 0, or one key / value head for the tile's heads)");
    MI355_REQUIRE(!use_mfma || dt == MI355_DT_BF16, "latent_attn: the MFMA path takes bf16 keys and values");
    MI355_REQUIRE(softcap >= 0.f && pool >= 0, "latent_attn: bad softcap or pool");
    MI355_REQUIRE(chunk >= 0 && (chunk == 0 || (keep_first == 0 && pool == 0)), "latent_attn: chunks combine with neither kept first tokens nor pooled blocks");
    MI355_REQUIRE(pool == 0 || (window > 0 && keep_first == 0 && D2 == 0 && PK && PV && pool_row0 && ldp >= (int64_t)((H - 1) / kv_rep) * k1_hs + D1 &&
                                ldp >= (int64_t)((H - 1) / kv_rep) * v_hs + DV),
                  "latent_attn: pooled blocks need a window, one-part keys and the pooled rows (laid out like the key / value rows)");
    MI355_REQUIRE(q_row0 && n_new && past && k1_row0 && k2_row0 && v_row0, "latent_attn: sequence descriptors missing");
    MI355_REQUIRE(ldq >= (int64_t)(H - 1) * q_hs + D1 + D2 && ldo >= (int64_t)(H - 1) * o_hs + DV && ldk1 >= (int64_t)((H - 1) / kv_rep) * k1_hs + D1 && ldv >= (int64_t)((H - 1) / kv_rep) * v_hs + DV &&
                      (D2 == 0 || ldk2 >= D2),
                  "latent_attn: rows too short");
    LatAttnArgs p;
    p.Q = Q, p.K1 = K1, p.K2 = K2, p.V = V, p.O = O;
    p.ldq = ldq, p.ldk1 = ldk1, p.ldk2 = ldk2, p.ldv = ldv, p.ldo = ldo;
    p.q_hs = q_hs, p.k1_hs = k1_hs, p.v_hs = v_hs, p.o_hs = o_hs;
    p.D1 = D1, p.D2 = D2, p.DV = DV, p.H = H, p.hm = hm, p.dt = dt;
    p.q_row0 = q_row0, p.n_new = n_new, p.past = past, p.k1_row0 = k1_row0, p.k2_row0 = k2_row0, p.v_row0 = v_row0;
    p.scale = scale;
    p.kv_rep = kv_rep, p.window = window, p.keep_first = keep_first, p.chunk = chunk;
    p.softcap = softcap, p.sink = sink, p.pool = pool, p.PK = PK, p.PV = PV, p.ldp = ldp, p.pool_row0 = pool_row0;
    p.splits = 1, p.ws = nullptr;
    const bool mfma = use_mfma && D1 + D2 <= 320 && DV <= 256;  // what the MFMA kernel keeps in registers; larger heads take the FMA path
    const int tm = (mfma ? MQ : AM) / hm;
    const int64_t gx = ((int64_t)max_new + tm - 1) / tm, gy = (H + hm - 1) / hm;
    MI355_REQUIRE(gy <= 65535 && gx < ((int64_t)1 << 31), "latent_attn: grid too large");
    dim3 grid((unsigned)gx, (unsigned)gy, n_seq);
    if (mfma && splits > 1) {
        const int DVPh = DV <= 32 ? 32 : DV <= 64 ? 64 : DV <= 128 ? 128 : 256;
        const int64_t need = (int64_t)n_seq * gy * gx * splits * MQ * (2 + DVPh);
        MI355_REQUIRE(splits <= 64 && ws && ws_floats >= need && gx * splits < ((int64_t)1 << 31), "latent_attn: key splits need a workspace of %lld floats", (long long)need);
        p.splits = splits, p.ws = ws;
        grid.x = (unsigned)(gx * splits);
    }
    if (mfma) {
        const int vec_ok = D1 % 8 == 0 && D2 % 8 == 0 && DV % 8 == 0 && ldk1 % 8 == 0 && ldk2 % 8 == 0 && ldv % 8 == 0 && k1_hs % 8 == 0 && v_hs % 8 == 0 &&
                           ((uintptr_t)K1 & 15) == 0 && ((uintptr_t)K2 & 15) == 0 && ((uintptr_t)V & 15) == 0 &&
                           (pool == 0 || (ldp % 8 == 0 && ((uintptr_t)PK & 15) == 0 && ((uintptr_t)PV & 15) == 0));
        const int DK = D1 + D2;
        if (DK <= 64) launch_mfma<8>(p, grid, vec_ok, ST(stream));
        else if (DK <= 128) launch_mfma<16>(p, grid, vec_ok, ST(stream));
        else if (DK <= 192) launch_mfma<24>(p, grid, vec_ok, ST(stream));
        else launch_mfma<40>(p, grid, vec_ok, ST(stream));
        MI355_LAUNCH_CHECK("latent_attn(mfma)");
        if (p.splits > 1) {
            const int DVPh = DV <= 32 ? 32 : DV <= 64 ? 64 : DV <= 128 ? 128 : 256;
            const int64_t items = (int64_t)n_seq * gy * gx * MQ;
            latent_attn_combine_kernel<<<(unsigned)((items + 3) / 4), 256, 0, ST(stream)>>>(p, DVPh, (int)gx, (int)gy, n_seq);
            MI355_LAUNCH_CHECK("latent_attn(combine)");
        }
        return 0;
    }
    if (DV <= 64) latent_attn_fma_kernel<1><<<grid, 256, 0, ST(stream)>>>(p);
    else if (DV <= 128) latent_attn_fma_kernel<2><<<grid, 256, 0, ST(stream)>>>(p);
    else if (DV <= 256) latent_attn_fma_kernel<4><<<grid, 256, 0, ST(stream)>>>(p);
    else latent_attn_fma_kernel<8><<<grid, 256, 0, ST(stream)>>>(p);
    MI355_LAUNCH_CHECK("latent_attn");
    return 0;
}
