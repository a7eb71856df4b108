// Attention backward as two deterministic kernels (no atomics, every gradient element written once):
//
//   attn_bwd_dq_kernel    one workgroup = 128 query rows; walks the keys in tiles of 64.  Also produces
//                         delta = rowsum(O * dO) for the second kernel.
//       S^T  = K . Q^T              A = K tile (LDS, row-major)       B = Q  (registers)
//       dP^T = V . dO^T             A = V tile (LDS, row-major)       B = dO (registers)
//       dS^T = P^T * (dP^T - delta),   P^T = exp2(S^T*c + bias*log2e - lse*log2e)
//       dQ^T += K^T . dS^T          A = K^T via transposing LDS reads  B = dS^T (registers)
//
//   attn_bwd_dkv_kernel   one workgroup = 128 keys; walks the query rows in tiles of 32.
//       S  = Q . K^T                A = Q tile  (LDS, row-major)      B = K (registers)
//       dP = dO . V^T               A = dO tile (LDS, row-major)      B = V (registers)
//       dV^T += dO^T . P            A = dO^T via transposing reads    B = P  (registers)
//       dK^T += Q^T . dS            A = Q^T  via transposing reads    B = dS (registers)
//
//   attn_bwd_dkv_kernel<..., FUSED = true>   the same kernel also produces dQ (one pass, five products instead of
//                         seven): every wavefront leaves its dS block in LDS, and after the step's barrier the
//                         wavefronts share out  dQ (32 queries x d) += dS (32 x 128 keys) . K (128 x d),
//                         A = dS via transposing reads, B = K^T held in registers, and add the result to an fp32
//                         dq_accum with atomics.  delta comes from attn_bwd_prep_kernel (which also clears dq_accum),
//                         dQ is rounded and scaled by attn_bwd_dq_convert_kernel.  dK and dV are as deterministic as
//                         in the two-kernel form; dQ depends on the order in which the key blocks' atomics arrive.
//                         Measured on MI355X, (4,4096,16,64) bf16: 1.79 ms against 0.93 ms for the two kernels.  The
//                         atomics are 2.1 GB of fp32 additions (T^2*d*4/128 bytes per batch and head) and the L2 takes
//                         about 3.2 TB/s of them: 0.66 ms that the rest of the kernel does not hide (timing-only builds:
//                         0.72 ms without any dQ work, 0.83 with the dS stores, 1.13 with the dQ product, 1.79 with the
//                         atomics).  It is therefore selectable, not the default.
//
// In both kernels the row/column that owns the output (query row for dQ, key for dK/dV) sits in one
// lane column (lane % 32), so P and dS go from accumulator registers straight into the next matrix
// product, and all LDS tiles are stored row-major exactly as they arrive from HBM.  The softmax scale
// is applied once to the finished dQ / dK accumulators instead of to every dS element.
#pragma once

#include "attn_common.h"
#include "attn_classes.h"

#include <type_traits>

constexpr int BWD_THREADS = 256;
constexpr int BWD_BM = 128;  // rows (queries or keys) owned by a workgroup

struct AttnBwdParams {
    AttnTensor q, k, v, o, dout, bias, dq, dk, dv;
    const float* lse;
    float* delta;
    int B, H, Tq, Tk, D, Tq_rounded, nblk;
    int bias_kind, bias_dtype, bias_vec, causal, vec;
    float scale, scale_log2;
    // split of the last round of workgroups (AttnSplit), set separately for the dQ and the dK/dV launch:
    // hardware blocks >= split_full are part (id % split_s) of item split_full + id / split_s and leave fp32
    // partial sums in `part`, (parts, 128, DPAD) for dQ and (parts, 2, 128, DPAD) for dK, dV
    int split_full, split_s;
    int group_lg;  // dQ launch: see row_block_of
    int trim;      // this launch looks for leading (dK/dV) or trailing (dQ) all -inf bias tiles first
    // Key ranges seen by the dQ launch, read by the dK/dV launch of the same call (or null): for every 32 query rows
    // (B * H * nrows32 entries of two ints) the first key and the end of the last key of the 32-key blocks in which some
    // pair of those rows had a bias above -inf.  Outside that range P = 0 for those rows.
    int* ranges;
    int nrows32;   // entries per (batch, head): 4 * ceil(Tq / 128)
    float* part;
    float* dq_accum;  // one-pass form: fp32 (B, H, Tq_rounded, DPAD), cleared by attn_bwd_prep_kernel
    // bias gradient (optional, dQ kernel): dS = P * (dP - delta) of every (query, key) pair, in the bias dtype, as a
    // full (B, H, Tq, Tk) tensor whose rows are padded to whole 64-key tiles (the caller sums broadcast dims)
    AttnTensor dbias;
    // Tile classes of a bias shared by the heads (or words == null), read by the CLS variants of the kernels, and which
    // workgroups this launch serves when the classes came with two launches (see cls_batch_dense): 0 all, 1 only batch
    // elements whose bias is mostly ZERO / NEG tiles, 2 only the others.
    BiasClasses cls;
    int cls_take;  // dK/dV launches: 1 only the "key mask" blocks of the classes' summary, 2 only the others
};

// block id -> (logical item, part, number of parts, part id)
struct BwdItem {
    int bid, part, nparts, part_id;
};
__device__ __forceinline__ BwdItem bwd_item(const AttnBwdParams& p) {
    BwdItem it{0, 0, 1, 0};
    if (p.split_s <= 1) {
        it.bid = xcd_remap(blockIdx.x, gridDim.x);
    } else if ((int)blockIdx.x < p.split_full) {
        it.bid = xcd_remap(blockIdx.x, p.split_full);
    } else {
        it.part_id = blockIdx.x - p.split_full;
        it.bid = p.split_full + it.part_id / p.split_s;
        it.part = it.part_id % p.split_s;
        it.nparts = p.split_s;
    }
    return it;
}

#ifndef RGD_DKV_SKIP_PREFIX
#define RGD_DKV_SKIP_PREFIX 1
#endif
#ifndef RGD_DKV_GROUP
#define RGD_DKV_GROUP 4
#endif
// Item of the dK/dV launch -> (key block, batch*head).  Items run through groups of RGD_DKV_GROUP (batch, head) pairs
// key block by key block: where the work of a key block falls with its index (causal launches, block-causal biases: the
// first key blocks see every query row) the launch then starts with the long workgroups of several heads and ends on
// the short ones, instead of giving a late, long workgroup to the compute unit that finished a short one first.
__device__ __forceinline__ void dkv_block_of(int item, const AttnBwdParams& p, int& kblk, int& bh) {
    const int nbh = p.B * p.H;
    const int per = RGD_DKV_GROUP * p.nblk;
    const int grp = item / per, local = item - grp * per;
    const int heads = min(RGD_DKV_GROUP, nbh - grp * RGD_DKV_GROUP);
    kblk = local / heads;
    bh = grp * RGD_DKV_GROUP + local - kblk * heads;
}

// 16 contiguous columns of one row of an fp32 partial tile
__device__ __forceinline__ void store_part16(float* row, int col, const f32x16& acc) {
#pragma unroll
    for (int e = 0; e < 16; e += 4) *reinterpret_cast<f32x4*>(row + col + e) = f32x4{acc[e], acc[e + 1], acc[e + 2], acc[e + 3]};
}

template <int DPAD> struct BwdTile {
    static constexpr int S = attn_lds_stride(DPAD);  // row stride of every staged tile (elements)
};

// writes 16 contiguous columns (two 16-byte stores on the vector path) of one output row
template <typename T>
__device__ __forceinline__ void store_row16(T* row, int col, int D, bool vec, const f32x16& acc, float mul) {
    if (vec) {
        if (col < D) {
            Pack16 lo, hi;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                lo.w[e] = pack2<T>(acc[2 * e] * mul, acc[2 * e + 1] * mul);
                hi.w[e] = pack2<T>(acc[8 + 2 * e] * mul, acc[8 + 2 * e + 1] * mul);
            }
            *reinterpret_cast<u32x4*>(row + col) = lo.v;
            if (col + 8 < D) *reinterpret_cast<u32x4*>(row + col + 8) = hi.v;
        }
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v)
            if (col + v < D) row[col + v] = static_cast<T>(acc[v] * mul);
    }
}

// ------------------------------------------------------------------------------------------------
// dQ kernel
// ------------------------------------------------------------------------------------------------
#ifndef RGD_DQ_BN128
#define RGD_DQ_BN128 32
#endif
#ifndef RGD_DQ_TRIM
#define RGD_DQ_TRIM 1
#endif
#ifndef RGD_DQ_SKIP_EARLY
#define RGD_DQ_SKIP_EARLY 1
#endif
// 1: the main loop of the dQ kernel without bias (d <= 64) fetches two tiles ahead
#ifndef RGD_DQ_PREFETCH2
#define RGD_DQ_PREFETCH2 1
#endif
template <int DPAD> struct DqSmem {
    // keys per tile: 32 at d = 128, where the smaller staging and logit registers let two wavefronts share a SIMD
    static constexpr int BN = DPAD == 128 ? RGD_DQ_BN128 : 64;
    static constexpr int TILE = BN * BwdTile<DPAD>::S;
    static constexpr size_t BYTES = 2 * 2 * TILE * 2;  // K and V, double buffered
};

// DBIAS: also write the bias gradient (a variant of its own: the kernels for head dims above 64 have no register to
// spare, and a pointer that is only tested at run time already costs them spills in the main loop: config-4-sized
// backward 0.31 -> 0.57 ms when it was a run-time option)
// CLS: the bias comes with tile classes (attn_classes.h); the kernel is laid out like the one without bias, runs the
// instructions of a tile without bias on ZERO tiles, leaves NEG tiles out and reads the bias of a MIXED tile in its step.
template <typename T, int DPAD, int BIAS, bool DBIAS = false, bool CLS = false>
__global__ __launch_bounds__(BWD_THREADS, (DPAD <= 64 || DqSmem<DPAD>::BN == 32) ? 2 : 1) void attn_bwd_dq_kernel(const AttnBwdParams p) {
    constexpr bool HAS_BIAS = BIAS != BIAS_OFF;
    static_assert(!DBIAS || HAS_BIAS, "a bias gradient needs a bias");
    static_assert(!CLS || (HAS_BIAS && !DBIAS && DPAD <= 64), "tile classes: head dims up to 64, with a bias, no bias gradient");
    constexpr bool BIAS_AHEAD = HAS_BIAS && !CLS;  // bias registers fetched one tile ahead of use
    typedef typename BiasElem<T, BIAS>::type TB;
    typedef Mfma<T> MM;
    constexpr int BN = DqSmem<DPAD>::BN;
    constexpr int NKB = BN / 32;  // 32-key halves per tile
    // starting the dP accumulators from -delta takes 16 registers; the bias variants at two wavefronts per
    // SIMD have none to spare and subtract delta per element instead
    constexpr bool DP_INIT = BIAS == BIAS_OFF || CLS || (DPAD > 64 && DqSmem<DPAD>::BN == 64);
    constexpr int ST = BwdTile<DPAD>::S;
    constexpr int TILE = DqSmem<DPAD>::TILE;
    constexpr int NC = DPAD / 16;
    constexpr int NDB = DPAD / 32;
    constexpr int CPR = DPAD / 8;
    constexpr int TASKS = BN * CPR;
    static_assert(TASKS % BWD_THREADS == 0, "tile chunks must divide evenly over the workgroup");
    constexpr int LOADS = TASKS / BWD_THREADS;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T* const ks_base = reinterpret_cast<T*>(smem_raw);
    T* const vs_base = ks_base + 2 * TILE;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 31, g = lane >> 5;
    const BwdItem item = bwd_item(p);
    int qb, bh;
    row_block_of(item.bid, p.nblk, p.group_lg, p.causal != 0, qb, bh);  // causal: longest row blocks first
    const int b = bh / p.H, h = bh - b * p.H;
    if constexpr (HAS_BIAS && !DBIAS && DPAD <= 64) {
        // classes came with two launches over the same grid: this one serves the batch elements of its kind
        if (p.cls_take != 0) {
            if (cls_batch_dense(p.cls, b) != (p.cls_take == 2)) return;
        }
    }
    const int q_row = qb * BWD_BM + wave * 32 + li;
    const bool q_valid = q_row < p.Tq;
    const int q_ld = q_valid ? q_row : p.Tq - 1;
    const bool vec = p.vec != 0;

    const T* qp = static_cast<const T*>(p.q.ptr) + b * p.q.sb + h * p.q.sh + (int64_t)q_ld * p.q.sn;
    const T* dop = static_cast<const T*>(p.dout.ptr) + b * p.dout.sb + h * p.dout.sh + (int64_t)q_ld * p.dout.sn;
    const T* op = static_cast<const T*>(p.o.ptr) + b * p.o.sb + h * p.o.sh + (int64_t)q_ld * p.o.sn;

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
    const float neg_lse_l2 = (q_valid && lse != -INFINITY) ? -lse * kLog2e : -INFINITY;
    if (g == 0 && q_row < p.Tq_rounded && item.part == 0) p.delta[(int64_t)bh * p.Tq_rounded + q_row] = q_valid ? delta : 0.f;
    f32x16 dp_init;  // -delta in every element: what the dP accumulators start from
#pragma unroll
    for (int v = 0; v < 16; ++v) dp_init[v] = -delta;

    f32x16 acc[NDB];
#pragma unroll
    for (int d = 0; d < NDB; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[d][v] = 0.f;

    int ntiles = (p.Tk + BN - 1) / BN;
    if (p.causal) ntiles = min(ntiles, (min(p.Tq, (qb + 1) * BWD_BM) + BN - 1) / BN);
    // this workgroup's share of the key tiles (all of them unless the item is split)
    const int t_begin = (int)((int64_t)ntiles * item.part / item.nparts);
    int t_end = (int)((int64_t)ntiles * (item.part + 1) / item.nparts);
    // trailing key tiles with nothing but -inf in the bias are left out (not when the bias gradient is written: it has
    // zeros to put there)
    if constexpr (attn_skip_masked(DPAD, BIAS) && !DBIAS && RGD_DQ_TRIM) {
        if (p.trim && p.bias_vec && !p.causal && p.Tk % BN == 0 && t_begin < t_end) {
            const int row0 = qb * BWD_BM + __builtin_amdgcn_readfirstlane(wave) * 32;
            const TB* bh_rows = static_cast<const TB*>(p.bias.ptr) + b * p.bias.sb + h * p.bias.sh;
            const TB* rows = bh_rows + (int64_t)min(row0, p.Tq - 1) * p.bias.sn;
            t_end = bias_trim_end<TB, BN>(bh_rows + (int64_t)(qb * BWD_BM) * p.bias.sn, min(BWD_BM, p.Tq - qb * BWD_BM), rows, p.bias.sn,
                                          min(32, p.Tq - row0), t_begin, t_end, lane, tid, reinterpret_cast<int*>(smem_raw));
        }
    }

    // scalars the loop works with: copies of their own (see own_scalar)
    struct {
        int64_t ksn, vsn;
        int Tk, Tq, D, causal;
        float scale_log2;
    } L = {own_scalar(p.k.sn), own_scalar(p.v.sn), own_scalar(p.Tk), own_scalar(p.Tq), own_scalar(p.D), own_scalar(p.causal),
           own_scalar(p.scale_log2)};
    const T* kbase = static_cast<const T*>(p.k.ptr) + b * p.k.sb + h * p.k.sh;
    const T* vbase = static_cast<const T*>(p.v.ptr) + b * p.v.sb + h * p.v.sh;
    // A head dim below the padded one (40, 80, 112, ...) leaves whole chunks past the end of a row: the fast loader
    // reads chunk 0 of the row in their place and store_tiles writes zeros (pad_mask bit i = chunk i).
    const bool padded = L.D != DPAD;
    uint32_t pad_mask = 0;
    int ld_key[LOADS], ld_dc[LOADS], koff[LOADS], voff[LOADS], soff[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int id = tid + i * BWD_THREADS;
        ld_key[i] = id / CPR;
        ld_dc[i] = id % CPR;
        const bool pad = ld_dc[i] * 8 >= L.D;
        pad_mask |= (pad ? 1u : 0u) << i;
        koff[i] = ld_key[i] * (int)L.ksn + (pad ? 0 : ld_dc[i] * 8);
        voff[i] = ld_key[i] * (int)L.vsn + (pad ? 0 : ld_dc[i] * 8);
        soff[i] = ld_key[i] * ST + ld_dc[i] * 8;
    }
    const bool fast_tiles = vec;  // rows made of whole 16-byte chunks
    // two staging register sets when the main loop fetches two tiles ahead (PF2), else one
    constexpr bool PF2 = RGD_DQ_PREFETCH2 && DPAD <= 64 && (!HAS_BIAS || CLS);
    u32x4 kst_[PF2 ? 2 : 1][LOADS], vst_[PF2 ? 2 : 1][LOADS];
    // FAST (compile time): the tile is known to be full and on the 16-byte path.  The main loop runs on FAST steps
    // only; with the element-wise loader of ragged tiles in the same loop the compiler waits for every outstanding
    // load before a tile's first matrix instruction, and the prefetch hides nothing.
    auto issue_loads = [&](int tile, auto FAST, auto SET) __attribute__((always_inline)) {
        u32x4(&kst)[LOADS] = kst_[PF2 ? decltype(SET)::value : 0];
        u32x4(&vst)[LOADS] = vst_[PF2 ? decltype(SET)::value : 0];
        const int key0 = tile * BN;
        const T* kt = kbase + (int64_t)key0 * L.ksn;
        const T* vt = vbase + (int64_t)key0 * L.vsn;
        if (decltype(FAST)::value || (fast_tiles && key0 + BN <= L.Tk)) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                kst[i] = *reinterpret_cast<const u32x4*>(kt + koff[i]);
                vst[i] = *reinterpret_cast<const u32x4*>(vt + voff[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const bool ok = key0 + ld_key[i] < L.Tk;
                kst[i] = load8<T>(kt + (int64_t)ld_key[i] * L.ksn, ld_dc[i] * 8, L.D, ok, vec);
                vst[i] = load8<T>(vt + (int64_t)ld_key[i] * L.vsn, ld_dc[i] * 8, L.D, ok, vec);
            }
        }
    };
    auto store_tiles = [&](int buf, auto SET) __attribute__((always_inline)) {
        u32x4(&kst)[LOADS] = kst_[PF2 ? decltype(SET)::value : 0];
        u32x4(&vst)[LOADS] = vst_[PF2 ? decltype(SET)::value : 0];
        if (padded) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i)
                if (pad_mask >> i & 1u) kst[i] = vst[i] = u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            *reinterpret_cast<u32x4*>(ks_base + buf * TILE + soff[i]) = kst[i];
            *reinterpret_cast<u32x4*>(vs_base + buf * TILE + soff[i]) = vst[i];
        }
    };
    const int a_off = mfma_row_perm(li) * ST + g * 8;
    const int tr_off = ((lane & 15) >> 2) * ST + mfma_row_perm(((lane >> 4) & 1) * 16 + (lane & 3) * 4) + g * 16 * ST;
    const TB* bias_row = nullptr;
    TB* dbias_row = nullptr;  // this lane's row of the bias gradient (DBIAS)
    BiasRuns<TB, NKB> bias_cur, bias_nxt;  // fetched one tile ahead of use
    if constexpr (HAS_BIAS) {
        if constexpr (DBIAS)
            dbias_row = static_cast<TB*>(const_cast<void*>(p.dbias.ptr)) + b * p.dbias.sb + h * p.dbias.sh + (int64_t)q_ld * p.dbias.sn;
        if constexpr (!CLS) bias_row = static_cast<const TB*>(p.bias.ptr) + b * p.bias.sb + h * p.bias.sh + (int64_t)q_ld * p.bias.sn;
    }
    const uint8_t* const cls_lds = smem_raw + DqSmem<DPAD>::BYTES;  // CLS: class of every key tile for the workgroup's 128 rows
    if constexpr (CLS)
        cls_tiles_to_lds(p.cls, b, qb * (BWD_BM / CLS_ROWS), BWD_BM / CLS_ROWS, (L.Tk + BN - 1) / BN, smem_raw + DqSmem<DPAD>::BYTES, tid);
    int run_end = t_end;  // end of the run of tiles that is being worked on (all of them unless CLS)
    // CLS: class of the tile of the next step, read from the table in LDS a step ahead (in a register of every lane; the
    // step makes a scalar of it)
    int cls_ahead = CLS_ZERO;

    // One key tile.  FAST: tiles j and j+1 are full tiles on the 16-byte path (and the bias, if any, is aligned).
    // AHEAD 0: the step fetches tile j+1 and stores it at its end.  AHEAD 1 / 2 (j even / odd): it fetches tile j+2
    // tiles of this wavefront with a bias above -inf somewhere (wavefront-uniform): first, and end of the last
    constexpr bool RECORD = attn_skip_masked(DPAD, BIAS) && !DBIAS;
    int live_first = 0x7fffffff, live_end = 0;
    // into the staging set of j's parity and stores tile j+1, fetched by the step before, from the other set.
    // WBIAS: the tiles of the run have a bias (always, unless the tile classes say that they are ZERO).
    auto tile_step = [&](const int j, auto FAST, auto AHEAD, auto WBIAS, const int tc) __attribute__((always_inline)) {
        constexpr bool F = decltype(FAST)::value != 0;
        constexpr int AH = decltype(AHEAD)::value;
        const int buf = j & 1;
        const int key0 = j * BN;
        const bool tail = !F && key0 + BN > L.Tk;
        // the fetch of the next tile(s).  CLS: issued inside either arm of the class test below, so that each arm is one
        // block of loads, address arithmetic, products and the first use of their results, as in the kernel without bias
        auto fetch = [&]() __attribute__((always_inline)) {
            if (F || j + 1 < run_end) {
                if constexpr (AH == 0) issue_loads(j + 1, FAST, IntC<0>{});
                else issue_loads(j + 2, FAST, IntC<AH - 1>{});
                if constexpr (BIAS_AHEAD)
                    bias_nxt.load(bias_row, key0 + BN, g, L.Tk, F || (p.bias_vec && key0 + 2 * BN <= L.Tk));
            }
        };
        if constexpr (!CLS) fetch();
        // WB: the tile has a bias: the registers fetched a step ago, or (CLS: a run of MIXED tiles, which are few) read
        // here, at the start of the tile's own step
        auto body = [&](auto WB) __attribute__((always_inline)) {
        constexpr bool WITH_BIAS = decltype(WB)::value != 0;
        const BiasRuns<TB, NKB>& bias_use = bias_cur;

        const T* ks = ks_base + buf * TILE + a_off;
        const T* vs = vs_base + buf * TILE + a_off;
        // A tile whose bias is -inf for every (query, key) pair of this wavefront has P = 0 and dS = 0: the step is left
        // out.  RGD_DQ_SKIP_EARLY 1: tested before the first two products (the bias was requested a step earlier), 0: after.
        bool masked_tile = false;
#if RGD_DQ_SKIP_EARLY
        if constexpr (attn_skip_masked(DPAD, BIAS)) masked_tile = bias_use.all_neg_inf(0, NKB);
#endif
        if constexpr (RGD_DQ_SKIP_EARLY && RECORD) {
            if (!masked_tile) {
                live_first = min(live_first, j);
                live_end = j + 1;
            }
        }
        // the dP accumulators start from -delta, so that product comes out as dP - delta
        f32x16 s[NKB], dp[NKB];
        if (!masked_tile) {
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb) {
            if constexpr (DP_INIT) {
                dp[kb] = dp_init;
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v) dp[kb][v] = 0.f;
            }
        }
        auto products = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb) {
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const u32x4 ka = *reinterpret_cast<const u32x4*>(ks + kb * 32 * ST + c * 16);
                    s[kb] = MM::run(as_v8<T>(ka), qreg[c], s[kb]);
                    const u32x4 va = *reinterpret_cast<const u32x4*>(vs + kb * 32 * ST + c * 16);
                    dp[kb] = MM::run(as_v8<T>(va), doreg[c], dp[kb]);
                }
            }
        };
        // t = logit - lse (log2 domain), for tiles whose bias, if any, is already inside s
        auto logits = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) s[kb][v] = fmaf(s[kb][v], L.scale_log2, neg_lse_l2);
        };
        auto from_zero = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) s[kb][v] = 0.f;
            products();
        };
        if constexpr (CLS) {
            // A MIXED or COLUMN tile (few; tc is its class): the first product starts from the bias, in units of the raw
            // scores, instead of from zero, and the tile goes on like every other tile.  The bias is read here, straight
            // into the accumulators: no register is held for it while other tiles run, and the row address is formed here
            // for the same reason.  COLUMN: every row of the tile is the first row of this wavefront's 32, which all its
            // lanes read.  The products are written out twice, so that the one that starts from zero keeps its zero inside
            // its first matrix instructions instead of in 32 registers that something has to clear.
            if (__builtin_expect(tc == CLS_ZERO, 1)) {
                fetch();
                from_zero();
                logits();
            } else {
                // (the class as a value of its own: the compiler otherwise threads the choice of the row through the test
                // above, which puts four branches in front of every tile)
                int tcc = tc;
                asm volatile("" : "+s"(tcc));
                int row = tcc == CLS_COLUMN ? min(qb * BWD_BM + wave * 32, L.Tq - 1) : q_ld;
                asm volatile("" : "+v"(row));
                // the bias tensor is read from the kernel's argument memory here, not kept in scalar registers through the loop
                const AttnTensor& bt = cold_params<AttnBwdParams>().bias;
                const TB* here = static_cast<const TB*>(bt.ptr) + b * bt.sb + h * bt.sh + (int64_t)row * bt.sn;
                const float per_score = kLog2e / L.scale_log2;
                fetch();
#pragma unroll
                for (int kb = 0; kb < NKB; ++kb) {
                    BiasRuns<TB, 1> half;
                    half.load(here, key0 + kb * 32, g, L.Tk, key0 + BN <= L.Tk);
                    float bias_h[16];
                    half.decode_run(0, bias_h);
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[kb][v] = bias_h[v] * per_score;
                }
                products();
                logits();
                asm volatile("" ::: "memory");  // (keeps the two copies apart)
            }
        } else {
            from_zero();
        }
        }
#if !RGD_DQ_SKIP_EARLY
        if constexpr (attn_skip_masked(DPAD, BIAS)) masked_tile = bias_use.all_neg_inf(0, NKB);
#endif
        if constexpr (!RGD_DQ_SKIP_EARLY && RECORD) {
            if (!masked_tile) {
                live_first = min(live_first, j);
                live_end = j + 1;
            }
        }
        if (!masked_tile) {
        // t = logit - lse (log2 domain)
        if constexpr (!CLS) {
            float bias_v[NKB][16];
            if constexpr (WITH_BIAS && !CLS) bias_use.decode(bias_v);
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    if constexpr (WITH_BIAS && !CLS)
                        s[kb][v] = fmaf(s[kb][v], L.scale_log2, fmaf(bias_v[kb][v], kLog2e, neg_lse_l2));
                    else
                        s[kb][v] = fmaf(s[kb][v], L.scale_log2, neg_lse_l2);
                }
        }
        const bool diag = L.causal && (key0 + BN - 1 > qb * BWD_BM + wave * 32);
        if (tail || diag) {
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int key = key0 + kb * 32 + g * 16 + v;
                    if (key >= L.Tk || (L.causal && key > q_row)) s[kb][v] = -INFINITY;
                }
        }
        uint32_t dsk[NKB][8];
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                const float p0 = __builtin_amdgcn_exp2f(s[kb][v]);
                const float p1 = __builtin_amdgcn_exp2f(s[kb][v + 1]);
                const float ds0 = DP_INIT ? p0 * dp[kb][v] : p0 * (dp[kb][v] - delta);
                const float ds1 = DP_INIT ? p1 * dp[kb][v + 1] : p1 * (dp[kb][v + 1] - delta);
                dsk[kb][v / 2] = pack2<T>(ds0, ds1);
                if constexpr (DBIAS && BIAS == BIAS_F32) {  // the fp32 values are only needed for an fp32 bias gradient
                    s[kb][v] = ds0;
                    s[kb][v + 1] = ds1;
                }
            }
        if constexpr (DBIAS) {
            if (q_valid) {
                // bias gradient: this lane's query row, 16 consecutive keys per 32-key half (rows are padded to whole
                // tiles, so the runs of a ragged last tile stay inside the row)
#pragma unroll
                for (int kb = 0; kb < NKB; ++kb) {
                    TB* dst = dbias_row + key0 + kb * 32 + g * 16;
                    if constexpr (BIAS == BIAS_F32) {
#pragma unroll
                        for (int e = 0; e < 16; e += 4)
                            *reinterpret_cast<f32x4*>(dst + e) = f32x4{s[kb][e], s[kb][e + 1], s[kb][e + 2], s[kb][e + 3]};
                    } else {
                        *reinterpret_cast<u32x4*>(dst) = u32x4{dsk[kb][0], dsk[kb][1], dsk[kb][2], dsk[kb][3]};
                        *reinterpret_cast<u32x4*>(dst + 8) = u32x4{dsk[kb][4], dsk[kb][5], dsk[kb][6], dsk[kb][7]};
                    }
                }
            }
        }
        // dQ^T += K^T . dS^T
        const T* kt = ks_base + buf * TILE + tr_off;
#pragma unroll
        for (int t = 0; t < 2 * NKB; ++t) {
            const int kb = t >> 1, jj = t & 1;
            const u32x4 raw = {dsk[kb][jj * 4 + 0], dsk[kb][jj * 4 + 1], dsk[kb][jj * 4 + 2], dsk[kb][jj * 4 + 3]};
            const typename MM::V8 bop = as_v8<T>(raw);
#pragma unroll
            for (int d = 0; d < NDB; ++d) {
                const T* src = kt + (kb * 32 + jj * 8) * ST + d * 32;
                const u32x2 lo = lds_read_tr<T>(src);
                const u32x2 hi = lds_read_tr<T>(src + 4 * ST);
                const u32x4 a = {lo[0], lo[1], hi[0], hi[1]};
                acc[d] = MM::run(as_v8<T>(a), bop, acc[d]);
            }
        }
        } else if constexpr (DBIAS) {
            if (q_valid) {  // a block that was left out has dS = 0
#pragma unroll
                for (int kb = 0; kb < NKB; ++kb) {
                    u32x4* dst = reinterpret_cast<u32x4*>(dbias_row + key0 + kb * 32 + g * 16);
#pragma unroll
                    for (int i = 0; i < (int)(16 * sizeof(TB) / 16); ++i) dst[i] = u32x4{0u, 0u, 0u, 0u};
                }
            }
        }
        };  // body
        body(WBIAS);
        if (F || j + 1 < run_end) {
            store_tiles(buf ^ 1, IntC<(AH == 0 ? 0 : 2 - AH)>{});
            if constexpr (BIAS_AHEAD) bias_cur = bias_nxt;
        }
        __syncthreads();
    };
    // CLS: the class of the tile goes into the step as a scalar (read from LDS a step ahead)
    auto step = [&](const int j, auto FAST, auto AHEAD, auto WBIAS) __attribute__((always_inline)) {
        if constexpr (CLS) {
            const int tc = __builtin_amdgcn_readfirstlane(cls_ahead);
            cls_ahead = cls_lds[min(j + 1, CLS_MAX_TILES - 1)];
            tile_step(j, FAST, AHEAD, IntC<0>{}, tc);
        } else {
            tile_step(j, FAST, AHEAD, WBIAS, 0);
        }
    };
    // The tiles [rb, re), one after the other: the first tile is loaded and stored to LDS here, every step then works a
    // tile (or two) ahead.  A kernel without tile classes has one run, all its tiles.
    auto run_tiles = [&](const int rb, const int re, auto WBIAS) __attribute__((always_inline)) {
        run_end = re;
        if constexpr (CLS) cls_ahead = cls_lds[rb];
        if (rb < re) {
            issue_loads(rb, IntC<0>{}, IntC<0>{});
            store_tiles(rb & 1, IntC<0>{});
            if constexpr (BIAS_AHEAD) bias_cur.load(bias_row, rb * BN, g, L.Tk, p.bias_vec && (rb + 1) * BN <= L.Tk);
        }
        __syncthreads();
        // tiles below n_fast are full and take the 16-byte path; a FAST step also prefetches tile j+1
        const bool fast_ok = fast_tiles && (!HAS_BIAS || p.bias_vec);
        const int n_fast = fast_ok ? min(re, L.Tk / BN) : rb;
        int j = rb;
        if constexpr (PF2) {
            if (n_fast - j >= 4) {
                // tile j is in LDS; tile j+1 goes into flight here, each step then fetches two tiles ahead
                if (j & 1) {
                    issue_loads(j + 1, IntC<1>{}, IntC<0>{});
                    step(j, IntC<1>{}, IntC<2>{}, WBIAS);
                    ++j;
                } else {
                    issue_loads(j + 1, IntC<1>{}, IntC<1>{});
                }
                for (; j + 3 < n_fast; j += 2) {
                    step(j, IntC<1>{}, IntC<1>{}, WBIAS);
                    step(j + 1, IntC<1>{}, IntC<2>{}, WBIAS);
                }
                // tile j is in LDS and tile j+1 in flight; the steps below fetch it again
            }
        }
        for (; j + 1 < n_fast; ++j) step(j, IntC<1>{}, IntC<0>{}, WBIAS);
        for (; j < re; ++j) step(j, IntC<0>{}, IntC<0>{}, WBIAS);
    };
    if constexpr (CLS) {
        // Runs of tiles that are not NEG go through the loop (the loop of the kernel without bias, plus the addition of the
        // bias on MIXED tiles); NEG runs (P = 0 and dS = 0) are left out, K/V loads and all.
        int j = cls_next_tile(cls_lds, t_begin, t_end, false);
        while (j < t_end) {
            const int e = cls_next_tile(cls_lds, j + 1, t_end, true);
            run_tiles(j, e, IntC<0>{});
            j = cls_next_tile(cls_lds, e, t_end, false);
        }
    } else {
        run_tiles(t_begin, t_end, IntC<(HAS_BIAS ? 1 : 0)>{});
    }

    // CLS: what only the epilogue needs is read from the kernel's argument memory here instead of sitting in scalar
    // registers through the loop, which has none to spare
    const AttnBwdParams& pe = CLS ? cold_params<AttnBwdParams>() : p;
    if constexpr (RECORD) {
        if (p.ranges != nullptr && lane == 0 && item.part == 0) {
            // a part of a split item has seen a part of the keys: its rows are noted as having all of them
            const bool whole = item.nparts > 1;
            int* r = p.ranges + (((int64_t)bh * p.nrows32) + qb * (BWD_BM / 32) + wave) * 2;
            r[0] = whole ? 0 : (live_end > 0 ? live_first * BN : p.Tk);
            r[1] = whole ? p.Tk : min(live_end * BN, p.Tk);
        }
    }
    if (item.nparts > 1) {  // part of a split item: leave the unscaled fp32 sums
        float* row = pe.part + ((int64_t)item.part_id * BWD_BM + wave * 32 + li) * DPAD;
#pragma unroll
        for (int d = 0; d < NDB; ++d) store_part16(row, d * 32 + g * 16, acc[d]);
        return;
    }
    if (q_valid) {
        T* dqp = static_cast<T*>(const_cast<void*>(pe.dq.ptr)) + b * pe.dq.sb + h * pe.dq.sh + (int64_t)q_row * pe.dq.sn;
#pragma unroll
        for (int d = 0; d < NDB; ++d) store_row16<T>(dqp, d * 32 + g * 16, pe.D, vec, acc[d], pe.scale);
    }
}

// ------------------------------------------------------------------------------------------------
// dK / dV kernel
// ------------------------------------------------------------------------------------------------
// 1: LDS operand reads of the dK/dV kernel run one step ahead of the matrix instructions (head dims above 64)
#ifndef RGD_DKV_READ_AHEAD
#define RGD_DKV_READ_AHEAD 1
#endif
#ifndef RGD_DKV_OCC
#define RGD_DKV_OCC 2  // wavefronts per SIMD of the dK/dV kernel without bias at head dims <= 64
#endif
#ifndef RGD_DKV_NSUB
#define RGD_DKV_NSUB 2
#endif
// Query rows per loop iteration of the dK/dV kernel = 32 * dkv_nsub: each wavefront works on dkv_nsub
// independent 32-row sub-tiles between two barriers, which gives the scheduler matrix work of one sub-tile
// to put beside the exponentials of the other.  A bias costs the registers that would take.
#ifndef RGD_DKV_NSUB_BIAS_WIDE
#define RGD_DKV_NSUB_BIAS_WIDE 2  // sub-tiles per step with a bias at head dims above 64
#endif
#ifndef RGD_FUSED_NSUB_BIAS
#define RGD_FUSED_NSUB_BIAS 2
#endif
#ifndef RGD_FUSED_OCC
#define RGD_FUSED_OCC 1  // wavefronts per SIMD of the one-pass kernel
#endif

constexpr int dkv_nsub(int dpad, int bias, bool fused = false) {
    return fused ? (bias == BIAS_OFF ? 2 : RGD_FUSED_NSUB_BIAS)
                 : (bias == BIAS_OFF ? RGD_DKV_NSUB : (dpad > 64 ? RGD_DKV_NSUB_BIAS_WIDE : 1));
}
constexpr int dkv_occupancy(int dpad, int bias, bool fused) {
    return fused ? RGD_FUSED_OCC : (dpad <= 64 ? (bias == BIAS_OFF ? RGD_DKV_OCC : 2) : 1);
}
template <int DPAD, int NSUB, bool FUSED = false> struct DkvSmem {
    static constexpr int BQ = 32 * NSUB;  // query rows per tile
    static constexpr int TILE = BQ * BwdTile<DPAD>::S;
    // per buffer: Q tile, dO tile, then BQ floats of -lse*log2e and BQ floats of -delta
    static constexpr int BUF_BYTES = 2 * TILE * 2 + 2 * BQ * 4;
    // one-pass form: dS sub-tiles, [128 keys][32 queries + 8] elements each, NSUB per step, two steps deep
    static constexpr int DS_STRIDE = 40;
    static constexpr int DS_TILE = BWD_BM * DS_STRIDE;
    static constexpr int DS_BYTES = FUSED ? 2 * NSUB * DS_TILE * 2 : 0;
    static constexpr size_t BYTES = 2 * BUF_BYTES + DS_BYTES;
    // the K tile of the workgroup ([128][S] elements) passes through the Q/dO buffers once, before the first step
    static_assert(!FUSED || 2 * BUF_BYTES >= BWD_BM * BwdTile<DPAD>::S * 2, "K tile must fit the staging buffers");
};

// 16 bias values of one key column (16 consecutive rows of the bias matrix) in the "key per lane" layout.
// load() only issues the reads so it can run a tile ahead of decode().  `tile_rows` points at the first
// bias row of the query tile and is the same for the whole wavefront, `lane_off` is this lane's element
// offset from there (its key column plus 16*g rows).  The reads are buffer loads: one descriptor on the tile,
// the lane offset in ONE register for all rows, and the row offset v*sn in a scalar register, so no per-lane
// address arithmetic or address registers per row are needed.  A ragged last tile (rows_ok false) reads
// the last existing row instead of rows >= Tq; the caller masks those.
template <typename TB> struct BiasColumn {
    TB raw[16];
    __device__ __forceinline__ void load(const TB* __restrict__ tile_rows, int64_t sn, uint32_t lane_off, int row0,
                                         int Tq, bool rows_ok) {
        if (rows_ok) {
            // raw buffer over the tile: offsets stay below 2^31 bytes because row strides are below 2^24 elements
            const __amdgpu_buffer_rsrc_t rsrc =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<TB*>(tile_rows), 0, 0xffffffffu, 0x00020000);
            const uint32_t voff = lane_off * (uint32_t)sizeof(TB);
            const uint32_t row_bytes = (uint32_t)sn * (uint32_t)sizeof(TB);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                if constexpr (sizeof(TB) == 2) {
                    const uint16_t bits = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc, voff, v * row_bytes, 0);
                    raw[v] = __builtin_bit_cast(TB, bits);
                } else {
                    const uint32_t bits = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, voff, v * row_bytes, 0);
                    raw[v] = __builtin_bit_cast(TB, bits);
                }
            }
        } else {
            // rows_ok is false at most once per workgroup.  `last` is the one per-lane quantity (written so that
            // the loop around this call carries one value for this branch, not one per row).
            const TB* col = tile_rows + lane_off;
            const int last = Tq - 1 - row0;  // last existing row relative to this lane's first row (may be < 0)
#pragma unroll
            for (int v = 0; v < 16; ++v) raw[v] = col[(int64_t)min(v, last) * sn];
        }
    }
    __device__ __forceinline__ void decode(float (&out)[16]) const {
#pragma unroll
        for (int v = 0; v < 16; ++v) out[v] = static_cast<float>(raw[v]);
    }
    // per lane: every one of the 16 values is -inf (the caller combines lanes and sub-tiles)
    __device__ __forceinline__ bool first_is_neg_inf() const { return bits(0) == NEG_INF; }
    __device__ __forceinline__ bool lane_all_neg_inf() const {
        bool all = true;
#pragma unroll
        for (int v = 0; v < 16; ++v) all = all && bits(v) == NEG_INF;
        return all;
    }
    typedef typename std::conditional<sizeof(TB) == 2, uint16_t, uint32_t>::type Bits;
    static constexpr Bits NEG_INF = (Bits)(NegInfBits<TB>::value & (sizeof(TB) == 2 ? 0xFFFFu : 0xFFFFFFFFu));
    __device__ __forceinline__ Bits bits(int v) const { return __builtin_bit_cast(Bits, raw[v]); }
};

// CLS: the bias comes with tile classes (attn_classes.h).  The kernel is the one without bias (same loop, two 32-row
// sub-tiles per step); it serves the key blocks that a padding mask leaves as "key mask" blocks (cls_key_mask_block): their
// hidden keys are treated like keys that do not exist.  Every other key block leaves at once and runs in the ordinary biased
// kernel, which is launched over the same grid (cls_take == 2) and leaves the key mask blocks alone.
template <typename T, int DPAD, int BIAS, bool FUSED = false, bool CLS = false>
__global__ __launch_bounds__(BWD_THREADS, dkv_occupancy(DPAD, CLS ? BIAS_OFF : BIAS, FUSED)) void attn_bwd_dkv_kernel(const AttnBwdParams p) {
    constexpr bool HAS_BIAS = BIAS != BIAS_OFF;
    static_assert(!CLS || (HAS_BIAS && !FUSED && DPAD <= 64), "tile classes: head dims up to 64, with a bias, two-kernel form");
    constexpr bool BIAS_AHEAD = HAS_BIAS && !CLS;  // bias registers fetched one step ahead of use
    typedef typename BiasElem<T, BIAS>::type TB;
    typedef Mfma<T> MM;
    constexpr int NSUB = dkv_nsub(DPAD, CLS ? BIAS_OFF : BIAS, FUSED);
    typedef DkvSmem<DPAD, NSUB, FUSED> SM;
    static_assert(!FUSED || DPAD <= 64, "the one-pass form keeps K^T in registers: head dims up to 64");
    constexpr int DS_ST = SM::DS_STRIDE;
    constexpr int DS_TILE = SM::DS_TILE;
    // dQ work of one step: NSUB query sub-tiles x NDB_ blocks of 32 channels, one item per wavefront
    constexpr int DQ_ITEMS = FUSED ? NSUB * (DPAD / 32) : 0;
    static_assert(DQ_ITEMS <= 4, "one dQ item per wavefront");
    constexpr int BQ = SM::BQ;
    constexpr int ST = BwdTile<DPAD>::S;
    constexpr int TILE = SM::TILE;
    constexpr int BUFB = SM::BUF_BYTES;
    constexpr int NC = DPAD / 16;
    constexpr int NDB = DPAD / 32;
    constexpr int CPR = DPAD / 8;
    constexpr int TASKS = BQ * CPR;  // 16-byte chunks of one tile: 128 .. 1024
    constexpr int LOADS = (TASKS + BWD_THREADS - 1) / BWD_THREADS;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 31, g = lane >> 5;
    const BwdItem item = bwd_item(p);
    int kblk, bh;
    dkv_block_of(item.bid, p, kblk, bh);
    const int b = bh / p.H, h = bh - b * p.H;
    const int key = kblk * BWD_BM + wave * 32 + li;  // this lane's key
    bool k_valid = key < p.Tk;
    const int k_ld = k_valid ? key : p.Tk - 1;
    bool no_key_hidden = true;    // CLS: no key of the workgroup is hidden by the bias
    bool all_keys_hidden = false;  // CLS: every one is (a fully padded key block): dK = dV = 0 without a single step
    if constexpr (HAS_BIAS && !FUSED && DPAD <= 64) {
        // classes came with two launches over the same grid: key mask blocks run here when CLS, all others when not
        if (p.cls_take != 0) {
            static_assert(BWD_BM == CLS_KEY_BLOCK, "one summary entry per workgroup of this kernel");
            const uint32_t* entry = cls_key_block(p.cls, b, kblk);
            const uint32_t flags = entry[4];
            if (((flags & CLS_KB_PURE) != 0) != CLS) return;
            if constexpr (CLS) {
                const int kl = wave * 32 + li;  // this lane's key within the block
                const bool hidden = ((entry[kl >> 5] >> (kl & 31)) & 1u) != 0;
                k_valid = k_valid && !hidden;
                no_key_hidden = (flags & CLS_KB_ANY_HIDDEN) == 0;
                all_keys_hidden = (flags & CLS_KB_ALL_HIDDEN) != 0;
            }
        }
    }
    const bool vec = p.vec != 0;

    const T* kp = static_cast<const T*>(p.k.ptr) + b * p.k.sb + h * p.k.sh + (int64_t)k_ld * p.k.sn;
    const T* vp = static_cast<const T*>(p.v.ptr) + b * p.v.sb + h * p.v.sh + (int64_t)k_ld * p.v.sn;
    const T* qbase = static_cast<const T*>(p.q.ptr) + b * p.q.sb + h * p.q.sh;
    const T* dobase = static_cast<const T*>(p.dout.ptr) + b * p.dout.sb + h * p.dout.sh;
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

    // ---- one-pass form: K^T of the workgroup's 128 keys as the B operand of the dQ product, dS tiles in LDS ----
    T* const ds_base = reinterpret_cast<T*>(smem_raw + 2 * BUFB);
    const int dq_u = wave / NDB, dq_db = wave % NDB;  // this wavefront's dQ item: query sub-tile, block of 32 channels
    typename MM::V8 ktreg[FUSED ? BWD_BM / 16 : 1];
    float* dq_dst = nullptr;  // &dq_accum[b, h, 16 * g, this lane's channel]
    if constexpr (FUSED) {
        T* kt = reinterpret_cast<T*>(smem_raw);
        const T* krows = static_cast<const T*>(p.k.ptr) + b * p.k.sb + h * p.k.sh;
        for (int id = tid; id < BWD_BM * CPR; id += BWD_THREADS) {
            const int row = id / CPR, dc = id - row * CPR;
            const int kr = kblk * BWD_BM + row;
            const u32x4 raw = load8<T>(krows + (int64_t)min(kr, p.Tk - 1) * p.k.sn, dc * 8, p.D, kr < p.Tk, vec);
            *reinterpret_cast<u32x4*>(kt + row * ST + dc * 8) = raw;
        }
        // both parities of the dS tiles start from zero: the first step's dQ phase works on the tile "before" it
        for (int id = tid; id < SM::DS_BYTES / 16; id += BWD_THREADS)
            reinterpret_cast<u32x4*>(ds_base)[id] = u32x4{0u, 0u, 0u, 0u};
        __syncthreads();
        if (DQ_ITEMS == 4 || wave < DQ_ITEMS) {
#pragma unroll
            for (int kk = 0; kk < BWD_BM / 16; ++kk) ktreg[kk] = load_a_transposed<T>(kt, ST, 16 * kk + 8 * g, 32 * dq_db, lane);
        }
        __syncthreads();  // the buffers are about to receive the first Q / dO tile
        dq_dst = p.dq_accum + ((int64_t)bh * p.Tq_rounded + dq_u * 32 + 16 * g) * DPAD + 32 * dq_db + mfma_row_perm(li);
    }
    // dQ of the query tile `jprev` (whose dS every wavefront finished before the last barrier):
    //   dQ (32 x 32 block of this wavefront) = dS (32 queries x 128 keys) . K (128 x 32 channels), added to dq_accum.
    // Accumulator value v of lane (li, g) is query 16g + v, channel 32 * dq_db + perm(li): for every v the 32 lanes of a
    // half write 32 consecutive floats.  jprev = -1 (before the first tile) adds the zeros the tiles start from.
    auto dq_phase = [&](const int jprev) __attribute__((always_inline)) {
        if constexpr (FUSED) {
            if (DQ_ITEMS == 4 || wave < DQ_ITEMS) {
                const T* ds = ds_base + ((jprev & 1) * NSUB + dq_u) * DS_TILE;
                f32x16 acc;
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
                for (int kk = 0; kk < BWD_BM / 16; ++kk)
                    acc = MM::run(load_a_transposed<T>(ds, DS_ST, 16 * kk + 8 * g, 0, lane), ktreg[kk], acc);
                float* dst = dq_dst + (int64_t)(max(jprev, 0) * BQ) * DPAD;
#pragma unroll
                for (int v = 0; v < 16; ++v) unsafeAtomicAdd(dst + v * DPAD, acc[v]);
            }
        }
    };

    // this workgroup's share of the query tiles (all of them unless the item is split)
    const int ntiles_all = (p.Tq + BQ - 1) / BQ;
    const int tile_first = p.causal ? min(ntiles_all, (kblk * BWD_BM) / BQ) : 0;
    int tile_begin = tile_first + (int)((int64_t)(ntiles_all - tile_first) * item.part / item.nparts);
    int ntiles = tile_first + (int)((int64_t)(ntiles_all - tile_first) * (item.part + 1) / item.nparts);
    if (all_keys_hidden) ntiles = tile_begin;

    // Leading query tiles whose bias is -inf for every (query, key) pair of the workgroup give P = 0 and add nothing to dK
    // and dV (a block-causal bias: all queries before the key block).  They are found here, before anything else is
    // loaded, and left out of the loop altogether: every wavefront reads its [BQ rows][32 keys] bias blocks four steps at
    // a time, 16 bytes per lane, until it meets a value above -inf; the workgroup starts at the earliest such step.
    // (Inside the loop such a step still costs its tile loads, its first two products and a barrier.)
    if constexpr (attn_skip_masked(DPAD, BIAS) && !FUSED && RGD_DKV_SKIP_PREFIX) {
        if (p.ranges != nullptr && !p.causal && tile_begin < ntiles) {
            // the dQ launch of this call has left, for every 32 query rows, the range of keys with a bias above -inf:
            // the first and the last step that have such rows for this key block, without reading the bias
            constexpr int PER = BQ / 32;
            const int* rg = p.ranges + (int64_t)bh * p.nrows32 * 2;
            const int k0 = kblk * BWD_BM, k1 = min(p.Tk, k0 + BWD_BM);
            int* slot = reinterpret_cast<int*>(smem_raw);
            if (tid == 0) {
                slot[0] = ntiles;      // first live step
                slot[1] = tile_begin;  // end of the last live step
            }
            __syncthreads();
            const int r_end = min(ntiles * PER, p.nrows32);
            for (int r0 = tile_begin * PER; r0 < r_end; r0 += BWD_THREADS) {
                const int r = r0 + tid;
                const bool live = r < r_end && rg[2 * r] < k1 && rg[2 * r + 1] > k0;
                const uint64_t m = __builtin_amdgcn_ballot_w64(live);
                if (m != 0 && lane == 0) {
                    atomicMin(&slot[0], (r + (int)__builtin_ctzll(m)) / PER);
                    atomicMax(&slot[1], (r + 63 - (int)__builtin_clzll(m)) / PER + 1);
                }
            }
            __syncthreads();
            tile_begin = max(tile_begin, slot[0]);
            ntiles = min(ntiles, max(slot[1], tile_begin));
            __syncthreads();  // the tile buffers are written next
        } else if (p.trim && p.bias_vec && !p.causal && (kblk + 1) * BWD_BM <= p.Tk && tile_begin < ntiles) {
            constexpr int EPC = 16 / (int)sizeof(TB);  // bias elements per 16 bytes
            constexpr int CPW = 32 / EPC;              // 16-byte chunks of the wavefront's 32 keys in a row
            constexpr int RPL = 64 / CPW;              // rows per load instruction
            constexpr int LPS = BQ / RPL;              // load instructions per step
            constexpr int BATCH = 4;
            constexpr uint32_t PAT = NegInfBits<TB>::value;
            const TB* col = static_cast<const TB*>(p.bias.ptr) + b * p.bias.sb + h * p.bias.sh + kblk * BWD_BM + wave * 32 +
                            (lane % CPW) * EPC;
            const int rsub = lane / CPW;
            int live = ntiles;  // this wavefront's first step with a value above -inf
            for (int t0 = tile_begin; t0 < ntiles && live == ntiles; t0 += BATCH) {
                u32x4 v[BATCH][LPS];
#pragma unroll
                for (int bi = 0; bi < BATCH; ++bi)
#pragma unroll
                    for (int i = 0; i < LPS; ++i) {
                        const int row = min(min(t0 + bi, ntiles - 1) * BQ + i * RPL + rsub, p.Tq - 1);
                        v[bi][i] = *reinterpret_cast<const u32x4*>(col + (int64_t)row * p.bias.sn);
                    }
#pragma unroll
                for (int bi = BATCH - 1; bi >= 0; --bi) {
                    uint32_t all_and = PAT, all_or = PAT;
#pragma unroll
                    for (int i = 0; i < LPS; ++i)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            all_and &= v[bi][i][e];
                            all_or |= v[bi][i][e];
                        }
                    const bool some = __builtin_amdgcn_ballot_w64(all_and != PAT || all_or != PAT) != 0;
                    if (some && t0 + bi < ntiles) live = t0 + bi;
                }
            }
            int* first_live = reinterpret_cast<int*>(smem_raw);
            if (tid == 0) *first_live = ntiles;
            __syncthreads();
            if (lane == 0) atomicMin(first_live, live);
            __syncthreads();
            tile_begin = *first_live;
            __syncthreads();  // the tile buffers are written next
        }
    }

    // chunks past the end of a row (head dim below the padded one): as in the dQ kernel
    const bool padded = p.D != DPAD;
    uint32_t pad_mask = 0;
    int ld_row[LOADS], ld_dc[LOADS], qoff[LOADS], dooff[LOADS], soff[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int id = tid + i * BWD_THREADS;
        ld_row[i] = id / CPR;
        ld_dc[i] = id % CPR;
        const bool pad = ld_dc[i] * 8 >= p.D;
        pad_mask |= (pad ? 1u : 0u) << i;
        qoff[i] = ld_row[i] * (int)p.q.sn + (pad ? 0 : ld_dc[i] * 8);
        dooff[i] = ld_row[i] * (int)p.dout.sn + (pad ? 0 : ld_dc[i] * 8);
        soff[i] = ld_row[i] * ST + ld_dc[i] * 8;
    }
    const bool fast_tiles = vec;  // rows made of whole 16-byte chunks
    u32x4 qst[LOADS], dst[LOADS];
    float lse_st = 0.f, delta_st = 0.f;  // raw values as loaded; they are transformed when they are stored to LDS
    bool row_st = false;                 // the row exists
    // FAST (compile time): all BQ query rows of the tile exist and the 16-byte path applies.  The main loop runs on
    // FAST steps only (see the dQ kernel).
    auto issue_loads = [&](int tile, auto FAST) __attribute__((always_inline)) {
        constexpr bool F = decltype(FAST)::value != 0;
        const int q0 = tile * BQ;
        const T* qt = qbase + (int64_t)q0 * p.q.sn;
        const T* dot = dobase + (int64_t)q0 * p.dout.sn;
        if (F || (fast_tiles && q0 + BQ <= p.Tq)) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                if (TASKS % BWD_THREADS == 0 || tid + i * BWD_THREADS < TASKS) {
                    qst[i] = *reinterpret_cast<const u32x4*>(qt + qoff[i]);
                    dst[i] = *reinterpret_cast<const u32x4*>(dot + dooff[i]);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const bool ok = tid + i * BWD_THREADS < TASKS && q0 + ld_row[i] < p.Tq;
                qst[i] = load8<T>(qt + (int64_t)ld_row[i] * p.q.sn, ld_dc[i] * 8, p.D, ok, vec);
                dst[i] = load8<T>(dot + (int64_t)ld_row[i] * p.dout.sn, ld_dc[i] * 8, p.D, ok, vec);
            }
        }
        if (tid < BQ) {
            const int q = q0 + tid;
            const bool ok = F || q < p.Tq;
            // only the loads here: using the values now would make the wavefront wait for every load issued above
            lse_st = lsep[ok ? q : 0];
            delta_st = deltap[ok ? q : 0];
            row_st = ok;
        }
    };
    auto store_tiles = [&](int buf) __attribute__((always_inline)) {
        T* qs = reinterpret_cast<T*>(smem_raw + buf * BUFB);
        T* ds = qs + TILE;
        float* st = reinterpret_cast<float*>(smem_raw + buf * BUFB + 2 * TILE * 2);
        if (padded) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i)
                if (pad_mask >> i & 1u) qst[i] = dst[i] = u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            if (TASKS % BWD_THREADS == 0 || tid + i * BWD_THREADS < TASKS) {
                *reinterpret_cast<u32x4*>(qs + soff[i]) = qst[i];
                *reinterpret_cast<u32x4*>(ds + soff[i]) = dst[i];
            }
        }
        if (tid < BQ) {
            // rows that do not exist or have no finite logit get probability 0 (exp2(-inf)); delta is stored negated:
            // it is what the dP accumulator starts from
            st[tid] = (row_st && lse_st != -INFINITY) ? -lse_st * kLog2e : -INFINITY;
            st[BQ + tid] = row_st ? -delta_st : 0.f;
        }
    };
    const int a_off = mfma_row_perm(li) * ST + g * 8;
    const int tr_off = ((lane & 15) >> 2) * ST + mfma_row_perm(((lane >> 4) & 1) * 16 + (lane & 3) * 4) + g * 16 * ST;

    // A vector bias arrives with row stride 0, so it reads like a matrix whose rows are all the same.
    const TB* bias_base = nullptr;  // bias of this batch and head (wavefront-uniform)
    uint32_t bias_lane_off = 0;     // this lane's key column, 16*g rows down
    BiasColumn<TB> bias_cur[NSUB], bias_nxt[NSUB];  // fetched one tile ahead of use
    auto bias_load = [&](BiasColumn<TB> (&dst)[NSUB], int tile, auto FAST) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < NSUB; ++u) {
            const int q0 = tile * BQ + u * 32;
            // the ragged sub-tile clamps rows per lane half: its row base is that of the lane's own first row
            dst[u].load(bias_base + (int64_t)q0 * p.bias.sn, p.bias.sn, bias_lane_off, q0 + g * 16, p.Tq,
                        decltype(FAST)::value != 0 || q0 + 32 <= p.Tq);
        }
    };
    if constexpr (HAS_BIAS) {
        bias_base = static_cast<const TB*>(p.bias.ptr) + b * p.bias.sb + h * p.bias.sh;
        bias_lane_off = (uint32_t)k_ld + (uint32_t)(g * 16) * (uint32_t)p.bias.sn;
    }
    int run_end = ntiles;  // end of the run of steps that is being worked on

    // One tile of BQ query rows.  FAST: tile j+1 is a full tile on the 16-byte path.
    // NOMASK: every key of the workgroup exists and the launch is not causal, so no logit is masked (and the step
    // is one basic block for the instruction scheduler).
    // PING 0 / 1: one half of a pair of steps that swap the roles of the two bias register sets (0 uses bias_cur and
    // fills bias_nxt, 1 the other way round), so no step copies 16 registers per sub-tile; 2: a single step that
    // uses bias_cur and copies bias_nxt into it at its end.
    // WBIAS: the steps of the run have a bias (always, unless the tile classes say that they are ZERO).
    auto tile_step = [&](const int j, auto FAST, auto NOMASK, auto PING, auto WBIAS) __attribute__((always_inline)) {
        constexpr bool F = decltype(FAST)::value != 0;
        constexpr bool NM = decltype(NOMASK)::value != 0;
        constexpr int PP = decltype(PING)::value;
        BiasColumn<TB>(&b_fill)[NSUB] = pick_ref<PP == 1>(bias_nxt, bias_cur);
        const int buf = j & 1;
        if (F || j + 1 < run_end) {
            issue_loads(j + 1, FAST);
            if constexpr (BIAS_AHEAD) bias_load(b_fill, j + 1, FAST);
        }
        dq_phase(j - 1);  // one-pass form: dQ of the previous tile, beside this tile's first products
        const T* qs = reinterpret_cast<const T*>(smem_raw + buf * BUFB);
        const T* dos = qs + TILE;
        const float* st = reinterpret_cast<const float*>(smem_raw + buf * BUFB + 2 * TILE * 2);
        // The sub-tiles [U0, U1) of the step.  WB: they have a bias: the registers fetched a step ago, or (CLS) read here.
        auto body = [&](auto WB, auto UB, auto UE) __attribute__((always_inline)) {
        constexpr bool WITH_BIAS = decltype(WB)::value != 0;
        constexpr int U0 = decltype(UB)::value, U1 = decltype(UE)::value;
        BiasColumn<TB>(&b_use)[NSUB] = pick_ref<PP == 1>(bias_cur, bias_nxt);

        // the dP accumulators start from -delta of their query rows, so that product comes out as dP - delta
        f32x16 s[NSUB], dp[NSUB];
#pragma unroll
        for (int u = U0; u < U1; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f32x4 c = *reinterpret_cast<const f32x4*>(st + BQ + u * 32 + g * 16 + 4 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s[u][4 * i + e] = 0.f;
                    dp[u][4 * i + e] = c[e];
                }
            }
        // The operand reads run one step ahead of the matrix instructions that use them (the scheduling barriers keep
        // them there).  Left alone, the compiler issues each read right before its use, and with one wavefront per
        // SIMD (head dims above 64) nothing else covers the LDS round trip.  With two wavefronts it makes no difference.
        // (not with a bias: the 32 registers of the look-ahead push that variant into spills, and without them the
        // config-4-sized backward is 2.5 % shorter)
        constexpr bool READ_AHEAD = RGD_DKV_READ_AHEAD && DPAD > 64 && !HAS_BIAS;
        if constexpr (READ_AHEAD) {
            u32x4 qa[2][NSUB], da[2][NSUB];
            auto read_step = [&](int c) __attribute__((always_inline)) {
#pragma unroll
                for (int u = U0; u < U1; ++u) {
                    qa[c & 1][u] = *reinterpret_cast<const u32x4*>(qs + u * 32 * ST + a_off + c * 16);
                    da[c & 1][u] = *reinterpret_cast<const u32x4*>(dos + u * 32 * ST + a_off + c * 16);
                }
            };
            read_step(0);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (c + 1 < NC) read_step(c + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = U0; u < U1; ++u) {
                    s[u] = MM::run(as_v8<T>(qa[c & 1][u]), kreg[c], s[u]);
                    dp[u] = MM::run(as_v8<T>(da[c & 1][u]), vreg[c], dp[u]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int u = U0; u < U1; ++u) {
                    const u32x4 qa = *reinterpret_cast<const u32x4*>(qs + u * 32 * ST + a_off + c * 16);
                    s[u] = MM::run(as_v8<T>(qa), kreg[c], s[u]);
                    const u32x4 da = *reinterpret_cast<const u32x4*>(dos + u * 32 * ST + a_off + c * 16);
                    dp[u] = MM::run(as_v8<T>(da), vreg[c], dp[u]);
                }
        }
        // a step whose bias is -inf for every (query, key) pair of this wavefront has P = 0 and dS = 0: the rest of the step
        // is left out (tested where the bias is first needed, after the first two products have been issued).
        // The first value of every lane is looked at first, so a step with ordinary values costs a few instructions.
        bool masked_step = false;
        if constexpr (attn_skip_masked(DPAD, BIAS)) {
            bool first = true;
#pragma unroll
            for (int u = U0; u < U1; ++u) first = first && b_use[u].first_is_neg_inf();
            if (__builtin_amdgcn_ballot_w64(!first) == 0) {
                bool all = true;
#pragma unroll
                for (int u = U0; u < U1; ++u) all = all && b_use[u].lane_all_neg_inf();
                masked_step = __builtin_amdgcn_ballot_w64(!all) == 0;
            }
        }
        if (!masked_step) {
#pragma unroll
        for (int u = U0; u < U1; ++u) {
            const int q0 = j * BQ + u * 32;
            // t = logit - lse (log2 domain)
            float nlse[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f32x4 a = *reinterpret_cast<const f32x4*>(st + u * 32 + g * 16 + 4 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) nlse[4 * i + e] = a[e];
            }
            if constexpr (WITH_BIAS) {
                float bias_r[16];
                b_use[u].decode(bias_r);
#pragma unroll
                for (int v = 0; v < 16; ++v) s[u][v] = fmaf(s[u][v], p.scale_log2, fmaf(bias_r[v], kLog2e, nlse[v]));
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v) s[u][v] = fmaf(s[u][v], p.scale_log2, nlse[v]);
            }
            if constexpr (!NM) {
                const bool diag = p.causal && (q0 < kblk * BWD_BM + wave * 32 + 32);
                if (!k_valid || diag) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int q = q0 + g * 16 + v;
                        if (!k_valid || key > q) s[u][v] = -INFINITY;
                    }
                }
            }
            uint32_t pk[8], dsk[8];
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                const float p0 = __builtin_amdgcn_exp2f(s[u][v]);
                const float p1 = __builtin_amdgcn_exp2f(s[u][v + 1]);
                pk[v / 2] = pack2<T>(p0, p1);
                dsk[v / 2] = pack2<T>(p0 * dp[u][v], p1 * dp[u][v + 1]);
            }
            if constexpr (FUSED) {
                // dS of this lane's key for queries 16g .. 16g+15 of sub-tile u: one row piece of the [key][query] tile
                T* dsw = ds_base + ((j & 1) * NSUB + u) * DS_TILE + (wave * 32 + li) * DS_ST + 16 * g;
                *reinterpret_cast<u32x4*>(dsw) = u32x4{dsk[0], dsk[1], dsk[2], dsk[3]};
                *reinterpret_cast<u32x4*>(dsw + 8) = u32x4{dsk[4], dsk[5], dsk[6], dsk[7]};
            }
            // dV^T += dO^T . P ;  dK^T += Q^T . dS
            if constexpr (READ_AHEAD) {
                u32x4 dta[2], qta[2];  // transposed dO and Q operands, one (jj, d) step ahead
                auto read_t = [&](int t) __attribute__((always_inline)) {
                    const int jj = t / NDB, d = t % NDB;
                    const T* dsrc = dos + u * 32 * ST + tr_off + jj * 8 * ST + d * 32;
                    const u32x2 dlo = lds_read_tr<T>(dsrc);
                    const u32x2 dhi = lds_read_tr<T>(dsrc + 4 * ST);
                    dta[t & 1] = u32x4{dlo[0], dlo[1], dhi[0], dhi[1]};
                    const T* qsrc = qs + u * 32 * ST + tr_off + jj * 8 * ST + d * 32;
                    const u32x2 qlo = lds_read_tr<T>(qsrc);
                    const u32x2 qhi = lds_read_tr<T>(qsrc + 4 * ST);
                    qta[t & 1] = u32x4{qlo[0], qlo[1], qhi[0], qhi[1]};
                };
                read_t(0);
#pragma unroll
                for (int t = 0; t < 2 * NDB; ++t) {
                    const int jj = t / NDB, d = t % NDB;
                    if (t + 1 < 2 * NDB) read_t(t + 1);
                    __builtin_amdgcn_sched_barrier(0);
                    const u32x4 praw = {pk[jj * 4 + 0], pk[jj * 4 + 1], pk[jj * 4 + 2], pk[jj * 4 + 3]};
                    const u32x4 draw = {dsk[jj * 4 + 0], dsk[jj * 4 + 1], dsk[jj * 4 + 2], dsk[jj * 4 + 3]};
                    dv_acc[d] = MM::run(as_v8<T>(dta[t & 1]), as_v8<T>(praw), dv_acc[d]);
                    dk_acc[d] = MM::run(as_v8<T>(qta[t & 1]), as_v8<T>(draw), dk_acc[d]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    const u32x4 praw = {pk[jj * 4 + 0], pk[jj * 4 + 1], pk[jj * 4 + 2], pk[jj * 4 + 3]};
                    const u32x4 draw = {dsk[jj * 4 + 0], dsk[jj * 4 + 1], dsk[jj * 4 + 2], dsk[jj * 4 + 3]};
                    const typename MM::V8 pb = as_v8<T>(praw), db = as_v8<T>(draw);
#pragma unroll
                    for (int d = 0; d < NDB; ++d) {
                        const T* dsrc = dos + u * 32 * ST + tr_off + jj * 8 * ST + d * 32;
                        const u32x2 dlo = lds_read_tr<T>(dsrc);
                        const u32x2 dhi = lds_read_tr<T>(dsrc + 4 * ST);
                        const u32x4 da = {dlo[0], dlo[1], dhi[0], dhi[1]};
                        dv_acc[d] = MM::run(as_v8<T>(da), pb, dv_acc[d]);
                        const T* qsrc = qs + u * 32 * ST + tr_off + jj * 8 * ST + d * 32;
                        const u32x2 qlo = lds_read_tr<T>(qsrc);
                        const u32x2 qhi = lds_read_tr<T>(qsrc + 4 * ST);
                        const u32x4 qa = {qlo[0], qlo[1], qhi[0], qhi[1]};
                        dk_acc[d] = MM::run(as_v8<T>(qa), db, dk_acc[d]);
                    }
                }
            }
        }
        }  // !masked_step
        };  // body
        body(WBIAS, IntC<0>{}, IntC<NSUB>{});
        if (F || j + 1 < run_end) {
            store_tiles(buf ^ 1);
            if constexpr (BIAS_AHEAD && PP == 2) {
#pragma unroll
                for (int u = 0; u < NSUB; ++u) bias_cur[u] = bias_nxt[u];
            }
        }
        __syncthreads();
    };
    // The steps [rb, re), one after the other: the first tile is loaded and stored to LDS here, every step then fetches
    // the tile of the next.  A kernel without tile classes has one run, all its steps.
    auto run_steps = [&](const int rb, const int re, auto WBIAS) __attribute__((always_inline)) {
        run_end = re;
        if (rb < re) {
            issue_loads(rb, IntC<0>{});
            store_tiles(rb & 1);
            if constexpr (BIAS_AHEAD) bias_load(bias_cur, rb, IntC<0>{});
        }
        __syncthreads();
        // tiles below n_fast have all their query rows and take the 16-byte path; a FAST step prefetches tile j+1
        const int n_fast = fast_tiles ? min(re, p.Tq / BQ) : rb;
        int j = rb;
        if (!p.causal && (kblk + 1) * BWD_BM <= p.Tk && no_key_hidden) {
            if constexpr (BIAS_AHEAD) {
                for (; j + 2 < n_fast; j += 2) {
                    tile_step(j, IntC<1>{}, IntC<1>{}, IntC<0>{}, WBIAS);
                    tile_step(j + 1, IntC<1>{}, IntC<1>{}, IntC<1>{}, WBIAS);
                }
            }
            for (; j + 1 < n_fast; ++j) tile_step(j, IntC<1>{}, IntC<1>{}, IntC<2>{}, WBIAS);
        } else {
            for (; j + 1 < n_fast; ++j) tile_step(j, IntC<1>{}, IntC<0>{}, IntC<2>{}, WBIAS);
        }
        for (; j < re; ++j) tile_step(j, IntC<0>{}, IntC<0>{}, IntC<2>{}, WBIAS);
    };
    run_steps(tile_begin, ntiles, IntC<(BIAS_AHEAD ? 1 : 0)>{});
    if constexpr (FUSED) {
        if (tile_begin < ntiles) dq_phase(ntiles - 1);  // the last tile's dS is complete: the loop ended on a barrier
    }

    if (item.nparts > 1) {  // part of a split item: leave the unscaled fp32 sums, dK then dV
        float* row = p.part + (((int64_t)item.part_id * 2) * BWD_BM + wave * 32 + li) * DPAD;
#pragma unroll
        for (int d = 0; d < NDB; ++d) {
            store_part16(row, d * 32 + g * 16, dk_acc[d]);
            store_part16(row + (int64_t)BWD_BM * DPAD, d * 32 + g * 16, dv_acc[d]);
        }
        return;
    }
    if (key < p.Tk) {  // (a key hidden by the bias exists and gets its zeros)
        T* dkp = static_cast<T*>(const_cast<void*>(p.dk.ptr)) + b * p.dk.sb + h * p.dk.sh + (int64_t)key * p.dk.sn;
        T* dvp = static_cast<T*>(const_cast<void*>(p.dv.ptr)) + b * p.dv.sb + h * p.dv.sh + (int64_t)key * p.dv.sn;
#pragma unroll
        for (int d = 0; d < NDB; ++d) {
            store_row16<T>(dkp, d * 32 + g * 16, p.D, vec, dk_acc[d], p.scale);
            store_row16<T>(dvp, d * 32 + g * 16, p.D, vec, dv_acc[d], 1.0f);
        }
    }
}

// Adds the fp32 partial tiles of split items in part order and writes the rows in the tensor dtype.
// NT = tensors per item (1: dQ, 2: dK and dV).  One thread per (row, 4 consecutive columns);
// grid (split items, ceil(128 * DPAD/4 / 256), NT).
template <typename T, int DPAD> __global__ __launch_bounds__(256) void attn_bwd_merge_kernel(const AttnBwdParams p, int nt) {
    constexpr int CPR = DPAD / 4;
    const int id = blockIdx.y * 256 + threadIdx.x;
    if (id >= BWD_BM * CPR) return;
    const int row = id / CPR, col = (id - row * CPR) * 4;
    const int which = blockIdx.z;
    const int item = p.split_full + blockIdx.x;
    int blk, bh;
    if (nt == 2) dkv_block_of(item, p, blk, bh);
    else row_block_of(item, p.nblk, p.group_lg, p.causal != 0, blk, bh);
    const int b = bh / p.H, h = bh - b * p.H;
    const int t_row = blk * BWD_BM + row;
    const AttnTensor& out = nt == 1 ? p.dq : (which == 0 ? p.dk : p.dv);
    const int limit = nt == 1 ? p.Tq : p.Tk;
    const float mul = (nt == 2 && which == 1) ? 1.0f : p.scale;
    if (t_row >= limit) return;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < p.split_s; ++i) {
        const float* src = p.part + ((((int64_t)blockIdx.x * p.split_s + i) * nt + which) * BWD_BM + row) * DPAD + col;
        acc += *reinterpret_cast<const f32x4*>(src);
    }
    T* op = static_cast<T*>(const_cast<void*>(out.ptr)) + b * out.sb + h * out.sh + (int64_t)t_row * out.sn;
    if (p.vec && col + 4 <= p.D) {
        const uint32_t w0 = pack2<T>(acc[0] * mul, acc[1] * mul), w1 = pack2<T>(acc[2] * mul, acc[3] * mul);
        *reinterpret_cast<u32x2*>(op + col) = u32x2{w0, w1};
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (col + e < p.D) op[col + e] = static_cast<T>(acc[e] * mul);
    }
}

// ------------------------------------------------------------------------------------------------
// one-pass form: before and after the main kernel
// ------------------------------------------------------------------------------------------------
// delta[b, h, q] = rowsum(O * dO) for q < Tq (0 for the padding rows up to Tq_rounded) and dq_accum = 0.
// A row of DPAD channels is handled by DPAD/8 consecutive lanes (16-byte pieces); grid = rows / (256 / (DPAD/8)).
template <typename T, int DPAD> __global__ __launch_bounds__(256) void attn_bwd_prep_kernel(const AttnBwdParams p) {
    constexpr int CPR = DPAD / 8;
    static_assert((CPR & (CPR - 1)) == 0, "lane groups are powers of two");
    const int64_t row = (int64_t)blockIdx.x * (256 / CPR) + threadIdx.x / CPR;  // over (b, h, Tq_rounded)
    const int c = threadIdx.x % CPR;
    if (row >= (int64_t)p.B * p.H * p.Tq_rounded) return;  // whole lane groups leave together
    const int bh = (int)(row / p.Tq_rounded), q = (int)(row - (int64_t)bh * p.Tq_rounded);
    const int b = bh / p.H, h = bh - b * p.H;
    const bool valid = q < p.Tq;
    const int ql = valid ? q : 0;
    const T* op = static_cast<const T*>(p.o.ptr) + b * p.o.sb + h * p.o.sh + (int64_t)ql * p.o.sn;
    const T* dop = static_cast<const T*>(p.dout.ptr) + b * p.dout.sb + h * p.dout.sh + (int64_t)ql * p.dout.sn;
    const typename Mfma<T>::V8 ov = as_v8<T>(load8<T>(op, c * 8, p.D, valid, p.vec != 0));
    const typename Mfma<T>::V8 dv = as_v8<T>(load8<T>(dop, c * 8, p.D, valid, p.vec != 0));
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) sum += static_cast<float>(ov[e]) * static_cast<float>(dv[e]);
    sum = group_reduce<CPR>(sum);
    if (c == 0) p.delta[row] = sum;
    f32x4* acc = reinterpret_cast<f32x4*>(p.dq_accum + row * DPAD + c * 8);
    acc[0] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc[1] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// dq[b, q, h, :] = scale * dq_accum[b, h, q, :], rounded once to the tensor type; one thread per 8 channels
template <typename T, int DPAD> __global__ __launch_bounds__(256) void attn_bwd_dq_convert_kernel(const AttnBwdParams p) {
    constexpr int CPR = DPAD / 8;
    const int64_t row = (int64_t)blockIdx.x * (256 / CPR) + threadIdx.x / CPR;  // over (b, h, Tq)
    const int c = threadIdx.x % CPR;
    if (row >= (int64_t)p.B * p.H * p.Tq) return;
    const int bh = (int)(row / p.Tq), q = (int)(row - (int64_t)bh * p.Tq);
    const int b = bh / p.H, h = bh - b * p.H;
    const float* src = p.dq_accum + ((int64_t)bh * p.Tq_rounded + q) * DPAD + c * 8;
    const f32x4 lo = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src));
    const f32x4 hi = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src) + 1);
    T* dq = static_cast<T*>(const_cast<void*>(p.dq.ptr)) + b * p.dq.sb + h * p.dq.sh + (int64_t)q * p.dq.sn;
    const int col = c * 8;
    if (p.vec) {
        if (col < p.D) {
            Pack16 o;
            o.w[0] = pack2<T>(lo[0] * p.scale, lo[1] * p.scale);
            o.w[1] = pack2<T>(lo[2] * p.scale, lo[3] * p.scale);
            o.w[2] = pack2<T>(hi[0] * p.scale, hi[1] * p.scale);
            o.w[3] = pack2<T>(hi[2] * p.scale, hi[3] * p.scale);
            *reinterpret_cast<u32x4*>(dq + col) = o.v;
        }
    } else {
        const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (col + e < p.D) dq[col + e] = static_cast<T>(v[e] * p.scale);
    }
}
