// Attention forward: O = softmax(scale * Q K^T + bias) V, LSE = logsumexp of the logits.
//
// One workgroup = 4 wavefronts = 128 query rows of one (batch, head); each wavefront owns 32 query
// rows and walks the keys in tiles of 64.  Everything is computed transposed so that a query row
// lives in ONE lane column (lane % 32) for both matrix products:
//     S^T (keys x queries) = K (keys x d) . Q^T (d x queries)      A = K tile from LDS, B = Q in registers
//     O^T (d x queries)   += V^T (d x keys) . P^T (keys x queries)  A = V^T tile from LDS, B = P in registers
// The accumulator layout of S^T is exactly the B-operand layout of the second product, so the
// probabilities never leave registers, the online-softmax state (running max, running sum) is one
// value per lane, and the row reductions are 31 in-lane ops plus one exchange with lane ^ 32.
// K (row-major) and V (transposed on the way in) are staged through double-buffered LDS tiles;
// global loads of tile j+1 are in flight while tile j is in the matrix cores.  The bias tile is read
// straight from HBM as 16-element contiguous runs per lane (32 or 64 bytes) and is touched once.
#pragma once

#include "attn_common.h"

constexpr int ATTN_BM = 128;  // query rows per workgroup
constexpr int ATTN_BN = 64;   // keys per tile
constexpr int ATTN_THREADS = 256;

struct AttnFwdParams {
    AttnTensor q, k, v, bias, o;
    float* lse;
    int B, H, Tq, Tk, D, Tq_rounded, nqb;
    int bias_kind, bias_dtype, bias_vec, causal, vec;
    float scale_log2;  // softmax_scale * log2(e)
};

template <int DPAD> struct AttnFwdSmem {
    static constexpr int KS = DPAD + 8;     // K tile row stride (elements)
    static constexpr int VS = ATTN_BN + 8;  // V^T tile row stride (elements)
    static constexpr int K_ELEMS = ATTN_BN * KS;
    static constexpr int V_ELEMS = DPAD * VS;
    static constexpr size_t BYTES = 2 * (K_ELEMS + V_ELEMS) * 2;
};

template <typename T, int DPAD, bool HAS_BIAS>
__global__ __launch_bounds__(ATTN_THREADS) void attn_fwd_kernel(const AttnFwdParams p) {
    typedef Mfma<T> MM;
    typedef AttnFwdSmem<DPAD> SM;
    constexpr int NC = DPAD / 16;   // d chunks of the first product
    constexpr int NDB = DPAD / 32;  // 32-row blocks of O^T
    constexpr int CPR = DPAD / 8;   // 16-byte chunks per K/V row
    constexpr int K_LOADS = ATTN_BN * CPR / ATTN_THREADS;        // per thread, per tile
    constexpr int V_TASKS = (ATTN_BN / 2) * CPR;  // (key pair, chunk) items per tile
    constexpr int V_LOADS = (V_TASKS + ATTN_THREADS - 1) / ATTN_THREADS;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T* const ks_base = reinterpret_cast<T*>(smem_raw);
    T* const vt_base = ks_base + 2 * SM::K_ELEMS;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 31;
    const int g = lane >> 5;

    const int qb = blockIdx.x % p.nqb;
    const int bh = blockIdx.x / p.nqb;
    const int b = bh / p.H;
    const int h = bh - b * p.H;

    const int q_row = qb * ATTN_BM + wave * 32 + li;  // this lane's query row
    const bool q_valid = q_row < p.Tq;
    const int q_ld = q_valid ? q_row : p.Tq - 1;

    const T* qp = static_cast<const T*>(p.q.ptr) + b * p.q.sb + h * p.q.sh + (int64_t)q_ld * p.q.sn;
    const T* kp = static_cast<const T*>(p.k.ptr) + b * p.k.sb + h * p.k.sh;
    const T* vp = static_cast<const T*>(p.v.ptr) + b * p.v.sb + h * p.v.sh;
    const bool vec = p.vec != 0;

    typename MM::V8 qreg[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) qreg[c] = as_v8<T>(load8<T>(qp, c * 16 + g * 8, p.D, true, vec));

    f32x16 oacc[NDB];
#pragma unroll
    for (int d = 0; d < NDB; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[d][v] = 0.f;
    float m_run = -INFINITY;  // running max of the scaled logits (log2 domain)
    float l_run = 0.f;        // running sum over this lane's keys

    int ntiles = (p.Tk + ATTN_BN - 1) / ATTN_BN;
    if (p.causal) ntiles = min(ntiles, (min(p.Tq, (qb + 1) * ATTN_BM) + ATTN_BN - 1) / ATTN_BN);

    u32x4 kst[K_LOADS];
    u32x4 vst[V_LOADS][2];

    auto issue_loads = [&](int tile) {
        const int key0 = tile * ATTN_BN;
#pragma unroll
        for (int i = 0; i < K_LOADS; ++i) {
            const int id = tid + i * ATTN_THREADS;
            const int key = id / CPR, dc = id % CPR;
            kst[i] = load8<T>(kp + (int64_t)(key0 + key) * p.k.sn, dc * 8, p.D, key0 + key < p.Tk, vec);
        }
#pragma unroll
        for (int i = 0; i < V_LOADS; ++i) {
            const int id = tid + i * ATTN_THREADS;
            const int kpair = id / CPR, dc = id % CPR;
            const int key = key0 + 2 * kpair;
            const bool live = id < V_TASKS;
            vst[i][0] = load8<T>(vp + (int64_t)key * p.v.sn, dc * 8, p.D, live && key < p.Tk, vec);
            vst[i][1] = load8<T>(vp + (int64_t)(key + 1) * p.v.sn, dc * 8, p.D, live && key + 1 < p.Tk, vec);
        }
    };
    auto store_tiles = [&](int buf) {
        T* ks = ks_base + buf * SM::K_ELEMS;
        T* vt = vt_base + buf * SM::V_ELEMS;
#pragma unroll
        for (int i = 0; i < K_LOADS; ++i) {
            const int id = tid + i * ATTN_THREADS;
            const int key = id / CPR, dc = id % CPR;
            *reinterpret_cast<u32x4*>(ks + key * SM::KS + dc * 8) = kst[i];
        }
#pragma unroll
        for (int i = 0; i < V_LOADS; ++i) {
            const int id = tid + i * ATTN_THREADS;
            const int kpair = id / CPR, dc = id % CPR;
            if (id >= V_TASKS) continue;
            Pack16 a, c;
            a.v = vst[i][0];
            c.v = vst[i][1];
            uint32_t* vt32 = reinterpret_cast<uint32_t*>(vt);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // (key, d) and (key+1, d) side by side in row d of the transposed tile
                const uint32_t lo = __builtin_amdgcn_perm(c.w[e], a.w[e], 0x05040100);  // low halves
                const uint32_t hi = __builtin_amdgcn_perm(c.w[e], a.w[e], 0x07060302);  // high halves
                vt32[((dc * 8 + 2 * e) * SM::VS) / 2 + kpair] = lo;
                vt32[((dc * 8 + 2 * e + 1) * SM::VS) / 2 + kpair] = hi;
            }
        }
    };

    if (ntiles > 0) {
        issue_loads(0);
        store_tiles(0);
    }
    __syncthreads();

    const int krow = mfma_row_perm(li);  // matrix row this lane reads for an A operand
    const char* bias_base = nullptr;
    int64_t bias_row = 0;
    if constexpr (HAS_BIAS) {
        bias_base = static_cast<const char*>(p.bias.ptr);
        bias_row = b * p.bias.sb + h * p.bias.sh + (int64_t)q_ld * p.bias.sn;
    }

    for (int j = 0; j < ntiles; ++j) {
        const int buf = j & 1;
        const int key0 = j * ATTN_BN;
        if (j + 1 < ntiles) issue_loads(j + 1);

        const bool tail = key0 + ATTN_BN > p.Tk;
        float bias_v[2][16];
        if constexpr (HAS_BIAS) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
                load_bias16(bias_base, bias_row, p.bias_dtype, key0 + kb * 32 + g * 16, p.Tk, p.bias_vec && !tail, kLog2e,
                            bias_v[kb]);
        }

        // ---- S^T = K . Q^T ----
        const T* ks = ks_base + buf * SM::K_ELEMS;
        f32x16 s[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) s[kb][v] = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const u32x4 a = *reinterpret_cast<const u32x4*>(ks + (kb * 32 + krow) * SM::KS + c * 16 + g * 8);
                s[kb] = MM::run(as_v8<T>(a), qreg[c], s[kb]);
            }
        }

        // ---- logits in the log2 domain, masks ----
        const bool diag = p.causal && (key0 + ATTN_BN - 1 > qb * ATTN_BM + wave * 32);
        float mt = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float x = HAS_BIAS ? fmaf(s[kb][v], p.scale_log2, bias_v[kb][v]) : s[kb][v] * p.scale_log2;
                if (tail || diag) {
                    const int key = key0 + kb * 32 + g * 16 + v;
                    if (key >= p.Tk || (p.causal && key > q_row)) x = -INFINITY;
                }
                s[kb][v] = x;
                mt = fmaxf(mt, x);
            }
        mt = fmaxf(mt, lane_xor32(mt));
        const float m_new = fmaxf(m_run, mt);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
        m_run = m_new;

        float lsum = 0.f;
        uint32_t pk[2][8];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                const float p0 = __builtin_amdgcn_exp2f(s[kb][v] - m_safe);
                const float p1 = __builtin_amdgcn_exp2f(s[kb][v + 1] - m_safe);
                lsum += p0 + p1;
                pk[kb][v / 2] = pack2<T>(p0, p1);
            }
        l_run = l_run * alpha + lsum;
#pragma unroll
        for (int d = 0; d < NDB; ++d)
#pragma unroll
            for (int v = 0; v < 16; ++v) oacc[d][v] *= alpha;

        // ---- O^T += V^T . P^T ----
        const T* vt = vt_base + buf * SM::V_ELEMS;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int kb = t >> 1, jj = t & 1;
            const u32x4 praw = {pk[kb][jj * 4 + 0], pk[kb][jj * 4 + 1], pk[kb][jj * 4 + 2], pk[kb][jj * 4 + 3]};
            const typename MM::V8 pb = as_v8<T>(praw);
#pragma unroll
            for (int d = 0; d < NDB; ++d) {
                const u32x4 a =
                    *reinterpret_cast<const u32x4*>(vt + (d * 32 + krow) * SM::VS + kb * 32 + g * 16 + jj * 8);
                oacc[d] = MM::run(as_v8<T>(a), pb, oacc[d]);
            }
        }

        if (j + 1 < ntiles) store_tiles(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: normalise, write O and LSE ----
    const float l_tot = l_run + lane_xor32(l_run);
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    T* op = static_cast<T*>(const_cast<void*>(p.o.ptr)) + b * p.o.sb + h * p.o.sh + (int64_t)q_row * p.o.sn;
    if (q_valid) {
#pragma unroll
        for (int d = 0; d < NDB; ++d) {
            const int col = d * 32 + g * 16;
            if (vec) {
                if (col < p.D) {
                    Pack16 lo, hi;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        lo.w[e] = pack2<T>(oacc[d][2 * e] * inv, oacc[d][2 * e + 1] * inv);
                        hi.w[e] = pack2<T>(oacc[d][8 + 2 * e] * inv, oacc[d][8 + 2 * e + 1] * inv);
                    }
                    *reinterpret_cast<u32x4*>(op + col) = lo.v;
                    if (col + 8 < p.D) *reinterpret_cast<u32x4*>(op + col + 8) = hi.v;
                }
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (col + v < p.D) op[col + v] = static_cast<T>(oacc[d][v] * inv);
            }
        }
    }
    if (g == 0 && q_row < p.Tq_rounded) {
        // natural-log logsumexp; padding rows get a fixed value
        const float lse = q_valid ? (m_run + __builtin_amdgcn_logf(l_tot)) * kLn2 : 0.f;
        p.lse[(int64_t)bh * p.Tq_rounded + q_row] = lse;
    }
}
