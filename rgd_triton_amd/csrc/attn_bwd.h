// Attention backward as two deterministic kernels (no atomics, every gradient element written once):
//
//   attn_bwd_dq_kernel    one workgroup = 128 query rows; walks the keys.  Also produces
//                         delta = rowsum(O * dO) for the second kernel.
//       S^T  = K . Q^T              A = K tile (LDS, row-major)       B = Q  (registers)
//       dP^T = V . dO^T             A = V tile (LDS, row-major)       B = dO (registers)
//       dS^T = P^T * (dP^T - delta) * scale,   P^T = exp2(S^T*c + bias*log2e - lse*log2e)
//       dQ^T += K^T . dS^T          A = K^T via transposing LDS reads  B = dS^T (registers)
//
//   attn_bwd_dkv_kernel   one workgroup = 128 keys; walks the query rows.
//       S  = Q . K^T                A = Q tile  (LDS, row-major)      B = K (registers)
//       dP = dO . V^T               A = dO tile (LDS, row-major)      B = V (registers)
//       dV^T += dO^T . P            A = dO^T via transposing reads    B = P  (registers)
//       dK^T += Q^T . dS            A = Q^T  via transposing reads    B = dS (registers)
//
// In both kernels the row/column that owns the output (query row for dQ, key for dK/dV) sits in one
// lane column (lane % 32), so P and dS go from accumulator registers straight into the next matrix
// product, and all LDS tiles are stored row-major exactly as they arrive from HBM.  Transposed
// operands are fetched with ds_read_b64_tr_b16: inside each group of 16 lanes, result lane i gets
// element (i % 4) of the 8-byte pieces addressed by lanes i/4, 4 + i/4, 8 + i/4 and 12 + i/4.
#pragma once

#include "attn_common.h"

constexpr int BWD_THREADS = 256;
constexpr int BWD_BM = 128;  // rows (queries or keys) owned by a workgroup

struct AttnBwdParams {
    AttnTensor q, k, v, o, dout, bias, dq, dk, dv;
    const float* lse;
    float* delta;
    int B, H, Tq, Tk, D, Tq_rounded, nblk;
    int bias_kind, bias_dtype, bias_vec, causal, vec;
    float scale, scale_log2;
};

template <int DPAD> struct BwdTile {
    static constexpr int S = DPAD + 8;  // row stride of every staged tile (elements)
};

// ------------------------------------------------------------------------------------------------
// dQ kernel
// ------------------------------------------------------------------------------------------------
template <int DPAD> struct DqSmem {
    static constexpr int BN = 64;
    static constexpr int TILE = BN * BwdTile<DPAD>::S;
    static constexpr size_t BYTES = 2 * 2 * TILE * 2;  // K and V, double buffered
};

template <typename T, int DPAD, bool HAS_BIAS>
__global__ __launch_bounds__(BWD_THREADS) void attn_bwd_dq_kernel(const AttnBwdParams p) {
    typedef Mfma<T> MM;
    constexpr int BN = DqSmem<DPAD>::BN;
    constexpr int ST = BwdTile<DPAD>::S;
    constexpr int TILE = DqSmem<DPAD>::TILE;
    constexpr int NC = DPAD / 16;
    constexpr int NDB = DPAD / 32;
    constexpr int CPR = DPAD / 8;
    constexpr int LOADS = BN * CPR / BWD_THREADS;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T* const ks_base = reinterpret_cast<T*>(smem_raw);
    T* const vs_base = ks_base + 2 * TILE;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 31, g = lane >> 5;
    const int qb = blockIdx.x % p.nblk;
    const int bh = blockIdx.x / p.nblk;
    const int b = bh / p.H, h = bh - b * p.H;
    const int q_row = qb * BWD_BM + wave * 32 + li;
    const bool q_valid = q_row < p.Tq;
    const int q_ld = q_valid ? q_row : p.Tq - 1;
    const bool vec = p.vec != 0;

    const T* qp = static_cast<const T*>(p.q.ptr) + b * p.q.sb + h * p.q.sh + (int64_t)q_ld * p.q.sn;
    const T* dop = static_cast<const T*>(p.dout.ptr) + b * p.dout.sb + h * p.dout.sh + (int64_t)q_ld * p.dout.sn;
    const T* op = static_cast<const T*>(p.o.ptr) + b * p.o.sb + h * p.o.sh + (int64_t)q_ld * p.o.sn;
    const T* kp = static_cast<const T*>(p.k.ptr) + b * p.k.sb + h * p.k.sh;
    const T* vp = static_cast<const T*>(p.v.ptr) + b * p.v.sb + h * p.v.sh;

    typename MM::V8 qreg[NC], doreg[NC];
    float dsum = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        qreg[c] = as_v8<T>(load8<T>(qp, c * 16 + g * 8, p.D, q_valid, vec));
        const u32x4 draw = load8<T>(dop, c * 16 + g * 8, p.D, q_valid, vec);
        const u32x4 oraw = load8<T>(op, c * 16 + g * 8, p.D, q_valid, vec);
        doreg[c] = as_v8<T>(draw);
        const typename MM::V8 ov = as_v8<T>(oraw);
#pragma unroll
        for (int e = 0; e < 8; ++e) dsum += static_cast<float>(doreg[c][e]) * static_cast<float>(ov[e]);
    }
    const float delta = dsum + lane_xor32(dsum);
    const float lse = p.lse[(int64_t)bh * p.Tq_rounded + min(q_row, p.Tq_rounded - 1)];
    // rows that do not exist, and rows whose logits are all -inf, get probability 0 everywhere
    const float lse_l2 = (q_valid && lse != -INFINITY) ? lse * kLog2e : INFINITY;
    if (g == 0 && q_row < p.Tq_rounded) p.delta[(int64_t)bh * p.Tq_rounded + q_row] = q_valid ? delta : 0.f;

    f32x16 acc[NDB];
#pragma unroll
    for (int d = 0; d < NDB; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[d][v] = 0.f;

    int ntiles = (p.Tk + BN - 1) / BN;
    if (p.causal) ntiles = min(ntiles, (min(p.Tq, (qb + 1) * BWD_BM) + BN - 1) / BN);

    u32x4 kst[LOADS], vst[LOADS];
    auto issue_loads = [&](int tile) {
        const int key0 = tile * BN;
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int id = tid + i * BWD_THREADS;
            const int key = id / CPR, dc = id % CPR;
            const bool ok = key0 + key < p.Tk;
            kst[i] = load8<T>(kp + (int64_t)(key0 + key) * p.k.sn, dc * 8, p.D, ok, vec);
            vst[i] = load8<T>(vp + (int64_t)(key0 + key) * p.v.sn, dc * 8, p.D, ok, vec);
        }
    };
    auto store_tiles = [&](int buf) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int id = tid + i * BWD_THREADS;
            const int key = id / CPR, dc = id % CPR;
            *reinterpret_cast<u32x4*>(ks_base + buf * TILE + key * ST + dc * 8) = kst[i];
            *reinterpret_cast<u32x4*>(vs_base + buf * TILE + key * ST + dc * 8) = vst[i];
        }
    };
    if (ntiles > 0) {
        issue_loads(0);
        store_tiles(0);
    }
    __syncthreads();

    const int krow = mfma_row_perm(li);
    const char* bias_base = nullptr;
    int64_t bias_row = 0;
    if constexpr (HAS_BIAS) {
        bias_base = static_cast<const char*>(p.bias.ptr);
        bias_row = b * p.bias.sb + h * p.bias.sh + (int64_t)q_ld * p.bias.sn;
    }

    for (int j = 0; j < ntiles; ++j) {
        const int buf = j & 1;
        const int key0 = j * BN;
        if (j + 1 < ntiles) issue_loads(j + 1);
        const bool tail = key0 + BN > p.Tk;
        float bias_v[2][16];
        if constexpr (HAS_BIAS) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
                load_bias16(bias_base, bias_row, p.bias_dtype, key0 + kb * 32 + g * 16, p.Tk, p.bias_vec && !tail, kLog2e,
                            bias_v[kb]);
        }
        const T* ks = ks_base + buf * TILE;
        const T* vs = vs_base + buf * TILE;
        f32x16 s[2], dp[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                s[kb][v] = 0.f;
                dp[kb][v] = 0.f;
            }
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const u32x4 ka = *reinterpret_cast<const u32x4*>(ks + (kb * 32 + krow) * ST + c * 16 + g * 8);
                s[kb] = MM::run(as_v8<T>(ka), qreg[c], s[kb]);
                const u32x4 va = *reinterpret_cast<const u32x4*>(vs + (kb * 32 + krow) * ST + c * 16 + g * 8);
                dp[kb] = MM::run(as_v8<T>(va), doreg[c], dp[kb]);
            }
        }
        const bool diag = p.causal && (key0 + BN - 1 > qb * BWD_BM + wave * 32);
        uint32_t dsk[2][8];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                float dsv[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    float x = HAS_BIAS ? fmaf(s[kb][v + e], p.scale_log2, bias_v[kb][v + e]) : s[kb][v + e] * p.scale_log2;
                    if (tail || diag) {
                        const int key = key0 + kb * 32 + g * 16 + v + e;
                        if (key >= p.Tk || (p.causal && key > q_row)) x = -INFINITY;
                    }
                    const float pr = __builtin_amdgcn_exp2f(x - lse_l2);
                    dsv[e] = pr * (dp[kb][v + e] - delta) * p.scale;
                }
                dsk[kb][v / 2] = pack2<T>(dsv[0], dsv[1]);
            }
        // dQ^T += K^T . dS^T
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int kb = t >> 1, jj = t & 1;
            const u32x4 raw = {dsk[kb][jj * 4 + 0], dsk[kb][jj * 4 + 1], dsk[kb][jj * 4 + 2], dsk[kb][jj * 4 + 3]};
            const typename MM::V8 bop = as_v8<T>(raw);
#pragma unroll
            for (int d = 0; d < NDB; ++d) {
                const typename MM::V8 a = load_a_transposed<T>(ks, ST, kb * 32 + g * 16 + jj * 8, d * 32, lane);
                acc[d] = MM::run(a, bop, acc[d]);
            }
        }
        if (j + 1 < ntiles) store_tiles(buf ^ 1);
        __syncthreads();
    }

    if (q_valid) {
        T* dqp = static_cast<T*>(const_cast<void*>(p.dq.ptr)) + b * p.dq.sb + h * p.dq.sh + (int64_t)q_row * p.dq.sn;
#pragma unroll
        for (int d = 0; d < NDB; ++d) {
            const int col = d * 32 + g * 16;
            if (vec) {
                if (col < p.D) {
                    Pack16 lo, hi;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        lo.w[e] = pack2<T>(acc[d][2 * e], acc[d][2 * e + 1]);
                        hi.w[e] = pack2<T>(acc[d][8 + 2 * e], acc[d][8 + 2 * e + 1]);
                    }
                    *reinterpret_cast<u32x4*>(dqp + col) = lo.v;
                    if (col + 8 < p.D) *reinterpret_cast<u32x4*>(dqp + col + 8) = hi.v;
                }
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (col + v < p.D) dqp[col + v] = static_cast<T>(acc[d][v]);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// dK / dV kernel
// ------------------------------------------------------------------------------------------------
template <int DPAD> struct DkvSmem {
    static constexpr int BQ = DPAD <= 64 ? 64 : 32;  // query rows per tile
    static constexpr int TILE = BQ * BwdTile<DPAD>::S;
    // per buffer: Q tile, dO tile, then BQ floats of lse*log2e and BQ floats of delta
    static constexpr int BUF_BYTES = 2 * TILE * 2 + 2 * BQ * 4;
    static constexpr size_t BYTES = 2 * BUF_BYTES;
};

template <typename T, int DPAD, bool HAS_BIAS>
__global__ __launch_bounds__(BWD_THREADS) void attn_bwd_dkv_kernel(const AttnBwdParams p) {
    typedef Mfma<T> MM;
    constexpr int BQ = DkvSmem<DPAD>::BQ;
    constexpr int NQB = BQ / 32;
    constexpr int ST = BwdTile<DPAD>::S;
    constexpr int TILE = DkvSmem<DPAD>::TILE;
    constexpr int BUFB = DkvSmem<DPAD>::BUF_BYTES;
    constexpr int NC = DPAD / 16;
    constexpr int NDB = DPAD / 32;
    constexpr int CPR = DPAD / 8;
    constexpr int TASKS = BQ * CPR;
    constexpr int LOADS = (TASKS + BWD_THREADS - 1) / BWD_THREADS;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 31, g = lane >> 5;
    const int kblk = blockIdx.x % p.nblk;
    const int bh = blockIdx.x / p.nblk;
    const int b = bh / p.H, h = bh - b * p.H;
    const int key = kblk * BWD_BM + wave * 32 + li;  // this lane's key
    const bool k_valid = key < p.Tk;
    const int k_ld = k_valid ? key : p.Tk - 1;
    const bool vec = p.vec != 0;

    const T* kp = static_cast<const T*>(p.k.ptr) + b * p.k.sb + h * p.k.sh + (int64_t)k_ld * p.k.sn;
    const T* vp = static_cast<const T*>(p.v.ptr) + b * p.v.sb + h * p.v.sh + (int64_t)k_ld * p.v.sn;
    const T* qp = static_cast<const T*>(p.q.ptr) + b * p.q.sb + h * p.q.sh;
    const T* dop = static_cast<const T*>(p.dout.ptr) + b * p.dout.sb + h * p.dout.sh;
    const float* lsep = p.lse + (int64_t)bh * p.Tq_rounded;
    const float* deltap = p.delta + (int64_t)bh * p.Tq_rounded;

    typename MM::V8 kreg[NC], vreg[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        kreg[c] = as_v8<T>(load8<T>(kp, c * 16 + g * 8, p.D, k_valid, vec));
        vreg[c] = as_v8<T>(load8<T>(vp, c * 16 + g * 8, p.D, k_valid, vec));
    }
    f32x16 dk_acc[NDB], dv_acc[NDB];
#pragma unroll
    for (int d = 0; d < NDB; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            dk_acc[d][v] = 0.f;
            dv_acc[d][v] = 0.f;
        }

    const int ntiles = (p.Tq + BQ - 1) / BQ;
    const int tile_begin = p.causal ? min(ntiles, (kblk * BWD_BM) / BQ) : 0;

    u32x4 qst[LOADS], dst[LOADS];
    float lse_st = 0.f, delta_st = 0.f;
    auto issue_loads = [&](int tile) {
        const int q0 = tile * BQ;
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int id = tid + i * BWD_THREADS;
            const int r = id / CPR, dc = id % CPR;
            const bool ok = id < TASKS && q0 + r < p.Tq;
            qst[i] = load8<T>(qp + (int64_t)(q0 + r) * p.q.sn, dc * 8, p.D, ok, vec);
            dst[i] = load8<T>(dop + (int64_t)(q0 + r) * p.dout.sn, dc * 8, p.D, ok, vec);
        }
        if (tid < BQ) {
            const int q = q0 + tid;
            const float l = q < p.Tq ? lsep[q] : 0.f;
            lse_st = (q < p.Tq && l != -INFINITY) ? l * kLog2e : INFINITY;
            delta_st = q < p.Tq ? deltap[q] : 0.f;
        }
    };
    auto store_tiles = [&](int buf) {
        T* qs = reinterpret_cast<T*>(smem_raw + buf * BUFB);
        T* ds = qs + TILE;
        float* st = reinterpret_cast<float*>(smem_raw + buf * BUFB + 2 * TILE * 2);
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int id = tid + i * BWD_THREADS;
            const int r = id / CPR, dc = id % CPR;
            if (id < TASKS) {
                *reinterpret_cast<u32x4*>(qs + r * ST + dc * 8) = qst[i];
                *reinterpret_cast<u32x4*>(ds + r * ST + dc * 8) = dst[i];
            }
        }
        if (tid < BQ) {
            st[tid] = lse_st;
            st[BQ + tid] = delta_st;
        }
    };
    if (tile_begin < ntiles) {
        issue_loads(tile_begin);
        store_tiles(tile_begin & 1);
    }
    __syncthreads();

    const int arow = mfma_row_perm(li);
    const int besz = p.bias_dtype == RGD_F32 ? 4 : 2;
    const char* bias_base = nullptr;
    float bias_vector = 0.f;
    if constexpr (HAS_BIAS) {
        bias_base = static_cast<const char*>(p.bias.ptr) + (b * p.bias.sb + h * p.bias.sh + k_ld) * besz;
        if (p.bias_kind == RGD_BIAS_VECTOR) {
            float t[1];
            load_chunk_dyn<1, false>(bias_base, p.bias_dtype, 0, 1, t);
            bias_vector = t[0] * kLog2e;
        }
    }

    for (int j = tile_begin; j < ntiles; ++j) {
        const int buf = j & 1;
        const int q0 = j * BQ;
        if (j + 1 < ntiles) issue_loads(j + 1);

        const T* qs = reinterpret_cast<const T*>(smem_raw + buf * BUFB);
        const T* ds_t = qs + TILE;
        const float* st = reinterpret_cast<const float*>(smem_raw + buf * BUFB + 2 * TILE * 2);

        f32x16 s[NQB], dp[NQB];
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                s[qb][v] = 0.f;
                dp[qb][v] = 0.f;
            }
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const u32x4 qa = *reinterpret_cast<const u32x4*>(qs + (qb * 32 + arow) * ST + c * 16 + g * 8);
                s[qb] = MM::run(as_v8<T>(qa), kreg[c], s[qb]);
                const u32x4 da = *reinterpret_cast<const u32x4*>(ds_t + (qb * 32 + arow) * ST + c * 16 + g * 8);
                dp[qb] = MM::run(as_v8<T>(da), vreg[c], dp[qb]);
            }
        }
        const bool diag = p.causal && (q0 < kblk * BWD_BM + wave * 32 + 32);
        uint32_t pk[NQB][8], dsk[NQB][8];
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            float lse_r[16], delta_r[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f32x4 a = *reinterpret_cast<const f32x4*>(st + qb * 32 + g * 16 + 4 * i);
                const f32x4 c = *reinterpret_cast<const f32x4*>(st + BQ + qb * 32 + g * 16 + 4 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    lse_r[4 * i + e] = a[e];
                    delta_r[4 * i + e] = c[e];
                }
            }
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                float pv[2], dsv[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int q = q0 + qb * 32 + g * 16 + v + e;
                    float x = s[qb][v + e] * p.scale_log2;
                    if constexpr (HAS_BIAS) {
                        if (p.bias_kind == RGD_BIAS_VECTOR) {
                            x += bias_vector;
                        } else {
                            float t[1] = {0.f};
                            if (q < p.Tq) load_chunk_dyn<1, false>(bias_base + (int64_t)q * p.bias.sn * besz, p.bias_dtype, 0, 1, t);
                            x = fmaf(t[0], kLog2e, x);
                        }
                    }
                    if (!k_valid || (diag && key > q)) x = -INFINITY;
                    pv[e] = __builtin_amdgcn_exp2f(x - lse_r[v + e]);
                    dsv[e] = pv[e] * (dp[qb][v + e] - delta_r[v + e]) * p.scale;
                }
                pk[qb][v / 2] = pack2<T>(pv[0], pv[1]);
                dsk[qb][v / 2] = pack2<T>(dsv[0], dsv[1]);
            }
        }
        // dV^T += dO^T . P ;  dK^T += Q^T . dS
#pragma unroll
        for (int t = 0; t < 2 * NQB; ++t) {
            const int qb = t >> 1, jj = t & 1;
            const u32x4 praw = {pk[qb][jj * 4 + 0], pk[qb][jj * 4 + 1], pk[qb][jj * 4 + 2], pk[qb][jj * 4 + 3]};
            const u32x4 draw = {dsk[qb][jj * 4 + 0], dsk[qb][jj * 4 + 1], dsk[qb][jj * 4 + 2], dsk[qb][jj * 4 + 3]};
            const typename MM::V8 pb = as_v8<T>(praw), db = as_v8<T>(draw);
            const int row0 = qb * 32 + g * 16 + jj * 8;
#pragma unroll
            for (int d = 0; d < NDB; ++d) {
                const typename MM::V8 at = load_a_transposed<T>(ds_t, ST, row0, d * 32, lane);
                dv_acc[d] = MM::run(at, pb, dv_acc[d]);
                const typename MM::V8 qt = load_a_transposed<T>(qs, ST, row0, d * 32, lane);
                dk_acc[d] = MM::run(qt, db, dk_acc[d]);
            }
        }
        if (j + 1 < ntiles) store_tiles(buf ^ 1);
        __syncthreads();
    }

    if (k_valid) {
        T* dkp = static_cast<T*>(const_cast<void*>(p.dk.ptr)) + b * p.dk.sb + h * p.dk.sh + (int64_t)key * p.dk.sn;
        T* dvp = static_cast<T*>(const_cast<void*>(p.dv.ptr)) + b * p.dv.sb + h * p.dv.sh + (int64_t)key * p.dv.sn;
#pragma unroll
        for (int d = 0; d < NDB; ++d) {
            const int col = d * 32 + g * 16;
            if (vec) {
                if (col < p.D) {
                    Pack16 a, c, e2, f;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        a.w[e] = pack2<T>(dk_acc[d][2 * e], dk_acc[d][2 * e + 1]);
                        c.w[e] = pack2<T>(dk_acc[d][8 + 2 * e], dk_acc[d][8 + 2 * e + 1]);
                        e2.w[e] = pack2<T>(dv_acc[d][2 * e], dv_acc[d][2 * e + 1]);
                        f.w[e] = pack2<T>(dv_acc[d][8 + 2 * e], dv_acc[d][8 + 2 * e + 1]);
                    }
                    *reinterpret_cast<u32x4*>(dkp + col) = a.v;
                    *reinterpret_cast<u32x4*>(dvp + col) = e2.v;
                    if (col + 8 < p.D) {
                        *reinterpret_cast<u32x4*>(dkp + col + 8) = c.v;
                        *reinterpret_cast<u32x4*>(dvp + col + 8) = f.v;
                    }
                }
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (col + v < p.D) {
                        dkp[col + v] = static_cast<T>(dk_acc[d][v]);
                        dvp[col + v] = static_cast<T>(dv_acc[d][v]);
                    }
            }
        }
    }
}
