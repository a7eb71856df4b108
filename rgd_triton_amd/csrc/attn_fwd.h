// Attention forward: O = softmax(scale * Q K^T + bias) V, LSE = logsumexp of the logits.
//
// One workgroup = 4 wavefronts = 128 query rows of one (batch, head); each wavefront owns 32 query
// rows and walks the keys in tiles of 64.  Everything is computed transposed so that a query row
// lives in ONE lane column (lane % 32) for both matrix products:
//     S^T (keys x queries) = K (keys x d) . Q^T (d x queries)      A = K tile from LDS, B = Q in registers
//     O^T (d x queries)   += V^T (d x keys) . P^T (keys x queries)  A = V^T from LDS,    B = P in registers
// The accumulator layout of S^T is exactly the B-operand layout of the second product, so the
// probabilities never leave registers, the softmax state (reference exponent, running sum) is one
// value per lane, and a row reduction is in-lane work plus one exchange with lane ^ 32.
//
// K and V tiles are stored row-major in double-buffered LDS exactly as they arrive from HBM (16-byte
// stores); V^T operands are fetched with transposing LDS reads.  Global loads of tile j+1 are in
// flight while tile j is in the matrix cores.  The bias tile is read straight from HBM as 16-element
// contiguous runs per lane and is touched once.
//
// Softmax arithmetic (log2 domain, c = scale*log2e): t = s*c + bias*log2e - m is formed with fused
// multiply-adds against the running reference exponent m; m only moves when some logit exceeds it by
// more than 2^8 (then the accumulators are rescaled), so the usual per-tile subtract/rescale pass is
// rare after the first tiles.  p = exp2(t) <= 256 is safe for fp16/bf16 operands and fp32 sums, and
// LSE = (m + log2(l)) * ln2 does not depend on where m sits.
#pragma once
// 1: the main loop of the forward at d <= 64 fetches its K/V tiles two tiles ahead
#ifndef RGD_FWD_PREFETCH2
#define RGD_FWD_PREFETCH2 1
#endif
// ... also with a bias (the bias itself stays one tile ahead).  The biased kernels run two wavefronts per SIMD either
// way, so the second staging set costs no occupancy; (2,4352,24,64) with a (B,1,Q,K) bias: forward 0.368 -> 0.357 ms.
#ifndef RGD_FWD_PREFETCH2_BIAS
#define RGD_FWD_PREFETCH2_BIAS 1
#endif
// 1: the forward (head dims above 64) looks for an all -inf half tile before its first product, 0: after it.  The bias
// was requested a step earlier; config 4 forward -2 %, a bias without -inf blocks unchanged.
#ifndef RGD_FWD_SKIP_EARLY
#define RGD_FWD_SKIP_EARLY 1
#endif
#ifndef RGD_FWD_TRIM
#define RGD_FWD_TRIM 1
#endif
#ifndef RGD_FWD_LAZY_MAX
#define RGD_FWD_LAZY_MAX 1
#endif

// the variant that reads tile classes (CLS): wavefronts per SIMD, and whether it fetches K/V two tiles ahead
#ifndef RGD_CLS_FWD_OCC
#define RGD_CLS_FWD_OCC 3
#endif
#ifndef RGD_CLS_FWD_PF2
#define RGD_CLS_FWD_PF2 0
#endif

#include "attn_common.h"
#include "attn_classes.h"

constexpr int ATTN_BM = 128;  // query rows per workgroup
constexpr int ATTN_BN = 64;   // keys per tile
constexpr int ATTN_THREADS = 256;
constexpr float ATTN_RESCALE_THRESHOLD = 8.0f;  // log2 units
constexpr float ATTN_LAZY_LIMIT = 16384.0f;     // partial row sum of one tile above which the maximum is looked at

struct AttnFwdParams {
    AttnTensor q, k, v, bias, o;
    float* lse;
    int B, H, Tq, Tk, D, Tq_rounded, nqb;
    int bias_kind, bias_dtype, bias_vec, causal, vec;
    float scale_log2;  // softmax_scale * log2(e)
    // Split of the last, partly filled round of workgroups (see AttnSplit): hardware blocks below split_full
    // are whole items; the others are part (id % split_s) of item split_full + id / split_s and leave
    // unnormalised partial results, which attn_fwd_merge_kernel combines.  split_s <= 1: no split.
    int split_full, split_s;
    int group_lg;  // see row_block_of
    int trim;      // look for trailing all -inf bias tiles first (see bias_trim_end)
    float* part_o;   // (parts, 128, DPAD) fp32 accumulators, relative to the part's reference exponent
    float* part_ml;  // (parts, 128, 2): reference exponent (log2 domain), sum of probabilities
    // Tile classes of a bias shared by the heads (or words == null), read by the CLS variant of the kernel.
    // cls_take: which workgroups this launch serves when the classes came with two launches (see cls_batch_dense):
    // 0 all, 1 only batch elements whose bias is mostly ZERO / NEG tiles, 2 only the others.
    BiasClasses cls;
    int cls_take;
};

template <int DPAD> struct AttnFwdSmem {
    static constexpr int ST = attn_lds_stride(DPAD);  // row stride of the K and V tiles (elements)
    static constexpr int TILE = ATTN_BN * ST;
    static constexpr size_t BYTES = 2 * 2 * TILE * 2;  // K and V, double buffered
};

// CLS: the bias comes with tile classes (attn_classes.h).  The kernel is then laid out like the one without bias (no
// bias registers carried from tile to tile, three wavefronts per SIMD): ZERO tiles run the instructions of a tile without
// bias, NEG tiles are left out, and a MIXED tile reads its bias at the start of its own step.
template <typename T, int DPAD, int BIAS, bool CLS = false>
__global__ __launch_bounds__(ATTN_THREADS, CLS ? RGD_CLS_FWD_OCC : ((DPAD <= 64 && BIAS == BIAS_OFF) ? 3 : 2)) void attn_fwd_kernel(const AttnFwdParams p) {
    constexpr bool HAS_BIAS = BIAS != BIAS_OFF;
    static_assert(!CLS || (HAS_BIAS && DPAD <= 64), "tile classes: head dims up to 64, with a bias");
    constexpr bool BIAS_AHEAD = HAS_BIAS && !CLS;  // bias registers fetched one tile ahead of use
    typedef typename BiasElem<T, BIAS>::type TB;
    typedef Mfma<T> MM;
    typedef AttnFwdSmem<DPAD> SM;
    constexpr int ST = SM::ST;
    constexpr int TILE = SM::TILE;
    constexpr int NC = DPAD / 16;   // d chunks of the first product
    constexpr int NDB = DPAD / 32;  // 32-row blocks of O^T
    constexpr int CPR = DPAD / 8;   // 16-byte chunks per K/V row
    // d > 64: a 32-key half is finished (S -> p -> PV) before the next starts, which keeps only 16 logits
    // live and lets two wavefronts share a SIMD; at d <= 64 three wavefronts fit either way and the joint
    // form measured faster
    constexpr bool SPLIT_HALVES = DPAD > 64;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T* const ks_base = reinterpret_cast<T*>(smem_raw);
    T* const vs_base = ks_base + 2 * TILE;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 31;
    const int g = lane >> 5;

    int bid, part = 0, nparts = 1, part_id = 0;
    if (p.split_s <= 1) {
        bid = xcd_remap(blockIdx.x, gridDim.x);
    } else if ((int)blockIdx.x < p.split_full) {
        bid = xcd_remap(blockIdx.x, p.split_full);
    } else {
        part_id = blockIdx.x - p.split_full;
        bid = p.split_full + part_id / p.split_s;
        part = part_id % p.split_s;
        nparts = p.split_s;
    }
    int qb, bh;
    row_block_of(bid, p.nqb, p.group_lg, p.causal != 0, qb, bh);
    const int b = bh / p.H;
    const int h = bh - b * p.H;
    if constexpr (HAS_BIAS && DPAD <= 64) {
        // classes came with two launches over the same grid: this one serves the batch elements of its kind
        if (p.cls_take != 0) {
            if (cls_batch_dense(p.cls, b) != (p.cls_take == 2)) return;
        }
    }

    const int q_row = qb * ATTN_BM + wave * 32 + li;  // this lane's query row
    const bool q_valid = q_row < p.Tq;
    const int q_ld = q_valid ? q_row : p.Tq - 1;

    const T* qp = static_cast<const T*>(p.q.ptr) + b * p.q.sb + h * p.q.sh + (int64_t)q_ld * p.q.sn;
    const bool vec = p.vec != 0;

    typename MM::V8 qreg[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) qreg[c] = as_v8<T>(load8<T>(qp, c * 16 + g * 8, p.D, true, vec));

    f32x16 oacc[NDB];
#pragma unroll
    for (int d = 0; d < NDB; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[d][v] = 0.f;
    float m_ref = -INFINITY;  // reference exponent of this row (log2 domain); -inf until a finite logit is seen
    float l_run = 0.f;        // sum of p over this lane's keys, relative to m_ref

    int ntiles = (p.Tk + ATTN_BN - 1) / ATTN_BN;
    if (p.causal) ntiles = min(ntiles, (min(p.Tq, (qb + 1) * ATTN_BM) + ATTN_BN - 1) / ATTN_BN);
    // this workgroup's share of the key tiles (all of them unless the item is split)
    const int t_begin = (int)((int64_t)ntiles * part / nparts);
    int t_end = (int)((int64_t)ntiles * (part + 1) / nparts);
    if constexpr (attn_skip_masked(DPAD, BIAS) && RGD_FWD_TRIM) {
        if (p.trim && p.bias_vec && !p.causal && p.Tk % ATTN_BN == 0 && t_begin < t_end) {
            const int row0 = qb * ATTN_BM + __builtin_amdgcn_readfirstlane(wave) * 32;
            const TB* bh_rows = static_cast<const TB*>(p.bias.ptr) + b * p.bias.sb + h * p.bias.sh;
            const TB* rows = bh_rows + (int64_t)min(row0, p.Tq - 1) * p.bias.sn;
            t_end = bias_trim_end<TB, ATTN_BN>(bh_rows + (int64_t)(qb * ATTN_BM) * p.bias.sn, min(ATTN_BM, p.Tq - qb * ATTN_BM), rows,
                                               p.bias.sn, min(32, p.Tq - row0), t_begin, t_end, lane, tid,
                                               reinterpret_cast<int*>(smem_raw));
        }
    }

    // global -> register staging of the next tile.  Thread t moves the 16-byte chunks t, t+256, ... of the
    // tile; its offsets inside a tile are fixed, the tile base is wavefront-uniform.
    constexpr int TASKS = ATTN_BN * CPR;
    static_assert(TASKS % ATTN_THREADS == 0, "tile chunks must divide evenly over the workgroup");
    constexpr int LOADS = TASKS / ATTN_THREADS;
    // scalars the loop works with: copies of their own (see own_scalar)
    struct {
        int64_t ksn, vsn;
        int Tk, Tq, D, causal;
        float scale_log2;
    } L = {own_scalar(p.k.sn), own_scalar(p.v.sn), own_scalar(p.Tk), own_scalar(p.Tq), own_scalar(p.D), own_scalar(p.causal),
           own_scalar(p.scale_log2)};
    const T* kbase = static_cast<const T*>(p.k.ptr) + b * p.k.sb + h * p.k.sh;
    const T* vbase = static_cast<const T*>(p.v.ptr) + b * p.v.sb + h * p.v.sh;
    // chunk i of this thread is row (ld_key0 + i*ROWS_PER_PASS) when the row length divides the
    // workgroup size (head dims 32/64/128); otherwise (96) every chunk has its own row and column
    constexpr bool REGULAR = ATTN_THREADS % CPR == 0;
    constexpr int ROWS_PER_PASS = ATTN_THREADS / CPR;
    const int ld_key0 = tid / CPR, ld_dc0 = tid % CPR;
    auto chunk_key = [&](int i) __attribute__((always_inline)) { return REGULAR ? ld_key0 + i * ROWS_PER_PASS : (tid + i * ATTN_THREADS) / CPR; };
    auto chunk_dc = [&](int i) __attribute__((always_inline)) { return REGULAR ? ld_dc0 : (tid + i * ATTN_THREADS) % CPR; };
    // element offsets of this thread's chunks inside a tile: one offset plus a uniform row step (REGULAR), or one
    // offset per chunk (head dim 96)
    // A head dim below the padded one (40, 80, 112, ...) leaves whole chunks past the end of a row: the fast
    // loader reads chunk 0 of the row in their place and store_tiles writes zeros.
    const bool padded = L.D != DPAD;
    auto chunk_pad = [&](int i) __attribute__((always_inline)) { return chunk_dc(i) * 8 >= L.D; };  // recomputed where used: no register held
    auto chunk_col = [&](int i) __attribute__((always_inline)) { return chunk_pad(i) ? 0 : chunk_dc(i) * 8; };
    const int koff0 = ld_key0 * (int)L.ksn + chunk_col(0);
    const int voff0 = ld_key0 * (int)L.vsn + chunk_col(0);
    int koff[REGULAR ? 1 : LOADS], voff[REGULAR ? 1 : LOADS];
    if constexpr (!REGULAR) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            koff[i] = chunk_key(i) * (int)L.ksn + chunk_col(i);
            voff[i] = chunk_key(i) * (int)L.vsn + chunk_col(i);
        }
    }
    // rows made of whole 16-byte chunks: straight-line loads, no masking except in the last tile
    const bool fast_tiles = vec && L.D % 8 == 0;
    // two staging register sets when the main loop fetches two tiles ahead (PF2), else one
    constexpr bool PF2 = RGD_FWD_PREFETCH2 && DPAD <= 64 && (!HAS_BIAS || RGD_FWD_PREFETCH2_BIAS) && (!CLS || RGD_CLS_FWD_PF2);
    u32x4 kst_[PF2 ? 2 : 1][LOADS], vst_[PF2 ? 2 : 1][LOADS];
    // FAST (compile time): the caller knows the tile is full and the 16-byte path applies, so the loads are
    // straight-line code.  The main loop below runs on FAST steps only: with the element-wise loader of ragged
    // tiles inside the same loop, the compiler has to wait for every outstanding load before a tile's first
    // matrix instruction (registers shared between the two loaders), and the prefetch hides nothing.
    auto issue_loads = [&](int tile, auto FAST, auto SET) __attribute__((always_inline)) {
        u32x4(&kst)[LOADS] = kst_[PF2 ? decltype(SET)::value : 0];
        u32x4(&vst)[LOADS] = vst_[PF2 ? decltype(SET)::value : 0];
        const int key0 = tile * ATTN_BN;
        const T* kt = kbase + (int64_t)key0 * L.ksn;
        const T* vt = vbase + (int64_t)key0 * L.vsn;
        if (decltype(FAST)::value || (fast_tiles && key0 + ATTN_BN <= L.Tk)) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {  // wavefront-uniform tile base + fixed per-thread offset
                if constexpr (REGULAR) {
                    kst[i] = *reinterpret_cast<const u32x4*>(kt + (int64_t)(i * ROWS_PER_PASS) * L.ksn + koff0);
                    vst[i] = *reinterpret_cast<const u32x4*>(vt + (int64_t)(i * ROWS_PER_PASS) * L.vsn + voff0);
                } else {
                    kst[i] = *reinterpret_cast<const u32x4*>(kt + koff[i]);
                    vst[i] = *reinterpret_cast<const u32x4*>(vt + voff[i]);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const int key = chunk_key(i), dc = chunk_dc(i);
                const bool ok = key0 + key < L.Tk;
                kst[i] = load8<T>(kt + (int64_t)key * L.ksn, dc * 8, L.D, ok, vec);
                vst[i] = load8<T>(vt + (int64_t)key * L.vsn, dc * 8, L.D, ok, vec);
            }
        }
    };
    auto store_tiles = [&](int buf, auto SET) __attribute__((always_inline)) {
        u32x4(&kst)[LOADS] = kst_[PF2 ? decltype(SET)::value : 0];
        u32x4(&vst)[LOADS] = vst_[PF2 ? decltype(SET)::value : 0];
        if (padded) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i)
                if (chunk_pad(i)) kst[i] = vst[i] = u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int so = chunk_key(i) * ST + chunk_dc(i) * 8;
            *reinterpret_cast<u32x4*>(ks_base + buf * TILE + so) = kst[i];
            *reinterpret_cast<u32x4*>(vs_base + buf * TILE + so) = vst[i];
        }
    };

    // per-lane LDS offsets (elements) of the operand reads; everything else is a compile-time offset
    const int a_off = mfma_row_perm(li) * ST + g * 8;  // K rows as A operand
    const int tr_off = ((lane & 15) >> 2) * ST + mfma_row_perm(((lane >> 4) & 1) * 16 + (lane & 3) * 4) +
                       g * 16 * ST;  // V^T via transposing reads: tile row (key) j, column quad

    // bias of this lane's query row, fetched one tile ahead of its use
    const TB* bias_row = nullptr;
    BiasRuns<TB> bias_cur, bias_nxt;
    const uint8_t* const cls_lds = smem_raw + SM::BYTES;  // CLS: class of every key tile for the workgroup's 128 rows
    if constexpr (HAS_BIAS && !CLS)
        bias_row = static_cast<const TB*>(p.bias.ptr) + b * p.bias.sb + h * p.bias.sh + (int64_t)q_ld * p.bias.sn;
    if constexpr (CLS)
        cls_tiles_to_lds(p.cls, b, qb * (ATTN_BM / CLS_ROWS), ATTN_BM / CLS_ROWS, (L.Tk + ATTN_BN - 1) / ATTN_BN, smem_raw + SM::BYTES, tid);
    int run_end = t_end;  // end of the run of tiles that is being worked on (all of them unless CLS)
    // CLS: class of the tile of the next step, read from the table in LDS a step ahead (in a register of every lane; the
    // step makes a scalar of it)
    int cls_ahead = CLS_ZERO;

    // One key tile.  FAST: tiles j and j+1 are full tiles on the 16-byte path (and the bias, if any, is aligned).
    // AHEAD 0: the step fetches tile j+1 and stores it at its end.  AHEAD 1 / 2 (j even / odd): it fetches tile j+2
    // into the staging set of j's parity and stores tile j+1, fetched by the step before, from the other set: the
    // store no longer waits for loads issued a step ago at most.
    // WBIAS: the tiles of the run have a bias (always, unless the tile classes say that they are ZERO).
    auto tile_step = [&](const int j, auto FAST, auto AHEAD, auto WBIAS, const int tc) __attribute__((always_inline)) {
        constexpr bool F = decltype(FAST)::value != 0;
        constexpr int AH = decltype(AHEAD)::value;
        const int buf = j & 1;
        const int key0 = j * ATTN_BN;
        const bool tail = !F && key0 + ATTN_BN > L.Tk;
        // the fetch of the next tile(s).  CLS, d <= 64: issued inside either arm of the class test below, so that each arm
        // is one block of loads, address arithmetic, product and the first use of its result, as in the kernel without bias
        auto fetch = [&]() __attribute__((always_inline)) {
            if (F || j + 1 < run_end) {
                if constexpr (AH == 0) issue_loads(j + 1, FAST, IntC<0>{});
                else issue_loads(j + 2, FAST, IntC<AH - 1>{});
                if constexpr (BIAS_AHEAD)
                    bias_nxt.load(bias_row, key0 + ATTN_BN, g, L.Tk, F || (p.bias_vec && key0 + 2 * ATTN_BN <= L.Tk));
            }
        };
        if constexpr (!(CLS && !SPLIT_HALVES)) fetch();
        if constexpr (!SPLIT_HALVES) {
            // d <= 64: both 32-key halves of the tile go through the softmax together.
            // WB: the tile has a bias: the registers fetched a step ago, or (CLS, a MIXED tile) read here.
            auto body = [&](auto WB) __attribute__((always_inline)) {
            constexpr bool WITH_BIAS = decltype(WB)::value != 0;
            const BiasRuns<TB>& bias_use = bias_cur;

            // ---- S^T = K . Q^T ----
            const T* ks = ks_base + buf * TILE + a_off;
            f32x16 s[2];
            // the two halves alternate, so consecutive matrix instructions never wait for each other's result
            auto products = [&]() __attribute__((always_inline)) {
#pragma unroll
                for (int c = 0; c < NC; ++c)
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb) {
                        const u32x4 a = *reinterpret_cast<const u32x4*>(ks + kb * 32 * ST + c * 16);
                        s[kb] = MM::run(as_v8<T>(a), qreg[c], s[kb]);
                    }
            };
            auto from_zero = [&]() __attribute__((always_inline)) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[kb][v] = 0.f;
                products();
            };
            // t = logit - m_ref (log2 domain), for tiles whose bias, if any, is already inside s
            const float m_off = m_ref == -INFINITY ? 0.f : m_ref;
            auto logits = [&]() __attribute__((always_inline)) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[kb][v] = fmaf(s[kb][v], L.scale_log2, -m_off);
            };
            if constexpr (CLS) {
                // A MIXED or COLUMN tile (few; tc is its class): the product starts from the bias, in units of the raw
                // scores, instead of from zero, and the tile goes on like every other tile.  The bias is read here, straight
                // into the accumulators: no register is held for it while other tiles run, and the row address is formed
                // here for the same reason.  COLUMN: every row of the tile is the first row of this wavefront's 32, which
                // all its lanes read.  The product is written out twice, so that the one that starts from zero keeps its
                // zero inside its first matrix instructions instead of in 32 registers that something has to clear.
                // (A copy of the whole step for these tiles, which would leave the step of the other tiles exactly that of
                // the kernel without bias, costs that step registers it does not have: spills.)
                if (__builtin_expect(tc == CLS_ZERO, 1)) {
                    fetch();
                    from_zero();
                    logits();
                } else {
                    // (the class as a value of its own: the compiler otherwise threads the choice of the row through the
                    // test above, which puts four branches in front of every tile)
                    int tcc = tc;
                    asm volatile("" : "+s"(tcc));
                    int row = tcc == CLS_COLUMN ? min(qb * ATTN_BM + wave * 32, L.Tq - 1) : q_ld;
                    asm volatile("" : "+v"(row));
                    // the bias tensor is read from the kernel's argument memory here, not kept in scalar registers through the loop
                    const AttnTensor& bt = cold_params<AttnFwdParams>().bias;
                    const TB* here = static_cast<const TB*>(bt.ptr) + b * bt.sb + h * bt.sh + (int64_t)row * bt.sn;
                    const float per_score = kLog2e / L.scale_log2;
                    fetch();
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb) {
                        BiasRuns<TB, 1> half;
                        half.load(here, key0 + kb * 32, g, L.Tk, key0 + ATTN_BN <= L.Tk);
                        float bias_v[16];
                        half.decode_run(0, bias_v);
#pragma unroll
                        for (int v = 0; v < 16; ++v) s[kb][v] = bias_v[v] * per_score;
                    }
                    products();
                    logits();
                    asm volatile("" ::: "memory");  // (keeps the two copies apart)
                }
            } else {
                from_zero();
            }

            // ---- t = logit - m_ref (log2 domain) ----
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                if constexpr (CLS) {
                    // (done in either arm above)
                } else if constexpr (WITH_BIAS) {
                    float bias_v[16];
                    bias_use.decode_run(kb, bias_v);
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[kb][v] = fmaf(s[kb][v], L.scale_log2, fmaf(bias_v[v], kLog2e, -m_off));
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[kb][v] = fmaf(s[kb][v], L.scale_log2, -m_off);
                }
            }
            const bool diag = L.causal && (key0 + ATTN_BN - 1 > qb * ATTN_BM + wave * 32);
            // running maximum of the tile and, if needed, a move of the reference exponent (first finite logit of
            // the row, or growth > 2^8): rescales the accumulators and shifts the logits
            auto max_and_move = [&]() __attribute__((always_inline)) {
                float tmax = -INFINITY;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int v = 0; v < 16; v += 2) tmax = fmaxf(fmaxf(tmax, s[kb][v]), s[kb][v + 1]);
                tmax = fmaxf(tmax, lane_xor32(tmax));
                const bool move = (m_ref == -INFINITY) ? (tmax != -INFINITY) : (tmax > ATTN_RESCALE_THRESHOLD);
                if (__builtin_amdgcn_ballot_w64(move) != 0) {
                    const float m_old = m_ref == -INFINITY ? 0.f : m_ref;
                    const float shift = move ? tmax : 0.f;
                    const float alpha = move ? __builtin_amdgcn_exp2f(m_ref - (m_old + shift)) : 1.f;  // 0 when m_ref was -inf
                    m_ref = move ? m_old + shift : m_ref;
                    l_run *= alpha;
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int v = 0; v < 16; ++v) s[kb][v] -= shift;
#pragma unroll
                    for (int d = 0; d < NDB; ++d)
#pragma unroll
                        for (int v = 0; v < 16; ++v) oacc[d][v] *= alpha;
                }
            };
            // p = exp2(t), packed to the operand type; the row sum uses the unrounded fp32 values (LSE keeps fp32
            // accuracy)
            uint32_t pk[2][8];
            float lsum0 = 0.f, lsum1 = 0.f;
            auto exp_pack = [&]() __attribute__((always_inline)) {
                lsum0 = 0.f;
                lsum1 = 0.f;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int v = 0; v < 16; v += 2) {
                        const float p0 = __builtin_amdgcn_exp2f(s[kb][v]);
                        const float p1 = __builtin_amdgcn_exp2f(s[kb][v + 1]);
                        pk[kb][v / 2] = pack2<T>(p0, p1);
                        lsum0 += p0;
                        lsum1 += p1;
                    }
            };
            bool done = false;
#if RGD_FWD_LAZY_MAX
            if constexpr (F) {
                // Full tile away from the causal diagonal: exponentiate against the current reference first and
                // look at the maximum only if that went wrong somewhere in the wavefront (row without a reference
                // yet, or a partial row sum beyond 2^14, i.e. some p that large: still far inside fp16/bf16 range).
                if (!diag) {
                    exp_pack();
                    const bool bad = (m_ref == -INFINITY) || !(lsum0 + lsum1 <= ATTN_LAZY_LIMIT);  // catches inf and NaN
                    if (__builtin_amdgcn_ballot_w64(bad) != 0) {
                        max_and_move();
                        exp_pack();
                    }
                    done = true;
                }
            }
#endif
            if (!done) {
                if (tail || diag) {
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int key = key0 + kb * 32 + g * 16 + v;
                            if (key >= L.Tk || (L.causal && key > q_row)) s[kb][v] = -INFINITY;
                        }
                }
                max_and_move();
                exp_pack();
            }
            l_run += lsum0 + lsum1;

            // ---- O^T += V^T . P^T ----
            const T* vs = vs_base + buf * TILE + tr_off;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int kb = t >> 1, jj = t & 1;
                const u32x4 praw = {pk[kb][jj * 4 + 0], pk[kb][jj * 4 + 1], pk[kb][jj * 4 + 2], pk[kb][jj * 4 + 3]};
                const typename MM::V8 pb = as_v8<T>(praw);
#pragma unroll
                for (int d = 0; d < NDB; ++d) {
                    const T* src = vs + (kb * 32 + jj * 8) * ST + d * 32;
                    const u32x2 lo = lds_read_tr<T>(src);
                    const u32x2 hi = lds_read_tr<T>(src + 4 * ST);
                    const u32x4 a = {lo[0], lo[1], hi[0], hi[1]};
                    oacc[d] = MM::run(as_v8<T>(a), pb, oacc[d]);
                }
            }
            };  // body
            body(WBIAS);
        } else {
            // Each 32-key half of the tile is a complete softmax step of its own (S -> p -> PV), so only 16
            // logits are live at a time; the register budget buys wavefronts per SIMD, and those hide the
            // LDS and matrix-pipe latencies of one another.
            const bool diag = L.causal && (key0 + ATTN_BN - 1 > qb * ATTN_BM + wave * 32);
            const T* ks = ks_base + buf * TILE + a_off;
            const T* vs = vs_base + buf * TILE + tr_off;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                // ---- S^T = K . Q^T ----
                // a half whose bias is -inf everywhere for this wavefront adds nothing and is left out
#if RGD_FWD_SKIP_EARLY
                if constexpr (attn_skip_masked(DPAD, BIAS)) {
                    if (bias_cur.all_neg_inf(kb, 1)) continue;
                }
#endif
                f32x16 s;
#pragma unroll
                for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const u32x4 a = *reinterpret_cast<const u32x4*>(ks + kb * 32 * ST + c * 16);
                    s = MM::run(as_v8<T>(a), qreg[c], s);
                }
#if !RGD_FWD_SKIP_EARLY
                if constexpr (attn_skip_masked(DPAD, BIAS)) {
                    if (bias_cur.all_neg_inf(kb, 1)) continue;
                }
#endif

                // ---- t = logit - m_ref (log2 domain) ----
                const float m_off = m_ref == -INFINITY ? 0.f : m_ref;
                if constexpr (HAS_BIAS) {
                    float bias_v[16];
                    bias_cur.decode_run(kb, bias_v);
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[v] = fmaf(s[v], L.scale_log2, fmaf(bias_v[v], kLog2e, -m_off));
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[v] = fmaf(s[v], L.scale_log2, -m_off);
                }
                if (tail || diag) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int key = key0 + kb * 32 + g * 16 + v;
                        if (key >= L.Tk || (L.causal && key > q_row)) s[v] = -INFINITY;
                    }
                }
                float tmax = -INFINITY;
#pragma unroll
                for (int v = 0; v < 16; v += 2) tmax = fmaxf(fmaxf(tmax, s[v]), s[v + 1]);
                tmax = fmaxf(tmax, lane_xor32(tmax));

                // move the reference exponent only when needed (first finite logit of the row, or growth > 2^8)
                const bool move = (m_ref == -INFINITY) ? (tmax != -INFINITY) : (tmax > ATTN_RESCALE_THRESHOLD);
                if (__builtin_amdgcn_ballot_w64(move) != 0) {
                    const float shift = move ? tmax : 0.f;
                    const float alpha = move ? __builtin_amdgcn_exp2f(m_ref - (m_off + shift)) : 1.f;  // 0 when m_ref was -inf
                    m_ref = move ? m_off + shift : m_ref;
                    l_run *= alpha;
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[v] -= shift;
#pragma unroll
                    for (int d = 0; d < NDB; ++d)
#pragma unroll
                        for (int v = 0; v < 16; ++v) oacc[d][v] *= alpha;
                }

                // ---- p = exp2(t), packed to the operand type; fp32 row sum of the unrounded values ----
                uint32_t pk[8];
                float lsum0 = 0.f, lsum1 = 0.f;
#pragma unroll
                for (int v = 0; v < 16; v += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(s[v]);
                    const float p1 = __builtin_amdgcn_exp2f(s[v + 1]);
                    pk[v / 2] = pack2<T>(p0, p1);
                    lsum0 += p0;
                    lsum1 += p1;
                }
                l_run += lsum0 + lsum1;

                // ---- O^T += V^T . P^T ----
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    const u32x4 praw = {pk[jj * 4 + 0], pk[jj * 4 + 1], pk[jj * 4 + 2], pk[jj * 4 + 3]};
                    const typename MM::V8 pb = as_v8<T>(praw);
#pragma unroll
                    for (int d = 0; d < NDB; ++d) {
                        const T* src = vs + (kb * 32 + jj * 8) * ST + d * 32;
                        const u32x2 lo = lds_read_tr<T>(src);
                        const u32x2 hi = lds_read_tr<T>(src + 4 * ST);
                        const u32x4 a = {lo[0], lo[1], hi[0], hi[1]};
                        oacc[d] = MM::run(as_v8<T>(a), pb, oacc[d]);
                    }
                }
            }
        }

        if (F || j + 1 < run_end) {
            store_tiles(buf ^ 1, IntC<(AH == 0 ? 0 : 2 - AH)>{});
            if constexpr (BIAS_AHEAD) bias_cur = bias_nxt;
        }
        __syncthreads();
    };
    // CLS: the class of the tile goes into the step as a scalar (read from LDS a step ahead)
    auto step = [&](const int j, auto FAST, auto AHEAD, auto WBIAS) __attribute__((always_inline)) {
        if constexpr (CLS) {
#ifdef RGD_CLS_DEBUG_NOCHECK  // timing-only build (wrong results unless every tile is ZERO): what the class test costs
            tile_step(j, FAST, AHEAD, IntC<0>{}, CLS_ZERO);
#else
            const int tc = __builtin_amdgcn_readfirstlane(cls_ahead);
            cls_ahead = cls_lds[min(j + 1, CLS_MAX_TILES - 1)];
            tile_step(j, FAST, AHEAD, IntC<0>{}, tc);
#endif
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
            if constexpr (BIAS_AHEAD) bias_cur.load(bias_row, rb * ATTN_BN, g, L.Tk, p.bias_vec && (rb + 1) * ATTN_BN <= L.Tk);
        }
        __syncthreads();
        // tiles below n_fast are full and take the 16-byte path; a FAST step also prefetches tile j+1
        const bool fast_ok = fast_tiles && (!HAS_BIAS || p.bias_vec);
        const int n_fast = fast_ok ? min(re, L.Tk / ATTN_BN) : rb;
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
                // tile j is in LDS and tile j+1 in flight (set of its parity); the steps below fetch it again
            }
        }
        for (; j + 1 < n_fast; ++j) step(j, IntC<1>{}, IntC<0>{}, WBIAS);
        for (; j < re; ++j) step(j, IntC<0>{}, IntC<0>{}, WBIAS);
    };
    if constexpr (CLS) {
        // Runs of tiles that are not NEG go through the loop (the loop of the kernel without bias, plus the addition of the
        // bias on MIXED tiles); NEG runs (every probability 0) are left out, K/V loads and all.
        int j = cls_next_tile(cls_lds, t_begin, t_end, false);
        while (j < t_end) {
            const int e = cls_next_tile(cls_lds, j + 1, t_end, true);
            run_tiles(j, e, IntC<0>{});
            j = cls_next_tile(cls_lds, e, t_end, false);
        }
    } else {
        run_tiles(t_begin, t_end, IntC<(HAS_BIAS ? 1 : 0)>{});
    }

    const float l_tot = l_run + lane_xor32(l_run);
    // CLS: what only the epilogue needs (output tensor, LSE, partial results) is read from the kernel's argument memory
    // here instead of sitting in scalar registers through the loop, which has none to spare (the loop would re-read them
    // from spill lanes in every step)
    const AttnFwdParams& pe = CLS ? cold_params<AttnFwdParams>() : p;
    if (nparts > 1) {
        // ---- part of a split item: leave the unnormalised accumulators, m_ref and the row sum ----
        const int row = wave * 32 + li;
        float* po = pe.part_o + ((int64_t)part_id * ATTN_BM + row) * DPAD;
#pragma unroll
        for (int d = 0; d < NDB; ++d)
#pragma unroll
            for (int e = 0; e < 16; e += 4)
                *reinterpret_cast<f32x4*>(po + d * 32 + g * 16 + e) =
                    f32x4{oacc[d][e], oacc[d][e + 1], oacc[d][e + 2], oacc[d][e + 3]};
        if (g == 0) {
            float* pm = pe.part_ml + ((int64_t)part_id * ATTN_BM + row) * 2;
            pm[0] = m_ref;
            pm[1] = l_tot;
        }
        return;
    }
    // ---- epilogue: normalise, write O and LSE ----
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    T* op = static_cast<T*>(const_cast<void*>(pe.o.ptr)) + b * pe.o.sb + h * pe.o.sh + (int64_t)q_row * pe.o.sn;
    if (q_valid) {
#pragma unroll
        for (int d = 0; d < NDB; ++d) {
            const int col = d * 32 + g * 16;
            if (vec) {
                if (col < pe.D) {
                    Pack16 lo, hi;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        lo.w[e] = pack2<T>(oacc[d][2 * e] * inv, oacc[d][2 * e + 1] * inv);
                        hi.w[e] = pack2<T>(oacc[d][8 + 2 * e] * inv, oacc[d][8 + 2 * e + 1] * inv);
                    }
                    *reinterpret_cast<u32x4*>(op + col) = lo.v;
                    if (col + 8 < pe.D) *reinterpret_cast<u32x4*>(op + col + 8) = hi.v;
                }
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (col + v < pe.D) op[col + v] = static_cast<T>(oacc[d][v] * inv);
            }
        }
    }
    if (g == 0 && q_row < pe.Tq_rounded) {
        // natural-log logsumexp; padding rows get a fixed value
        const float lse = q_valid ? (m_ref + __builtin_amdgcn_logf(l_tot)) * kLn2 : 0.f;
        pe.lse[(int64_t)bh * pe.Tq_rounded + q_row] = lse;
    }
}

// Combines the parts of split items: for every row, m = max m_i, O = sum_i 2^(m_i - m) O_i / sum_i 2^(m_i - m) l_i,
// in part order.  One thread per (row, 4 consecutive columns); grid (split items, ceil(128 * DPAD/4 / 256)).
template <typename T, int DPAD> __global__ __launch_bounds__(256) void attn_fwd_merge_kernel(const AttnFwdParams p) {
    constexpr int CPR = DPAD / 4;  // 4-column chunks per row
    const int id = blockIdx.y * 256 + threadIdx.x;
    if (id >= ATTN_BM * CPR) return;
    const int row = id / CPR, col = (id - row * CPR) * 4;
    const int item = p.split_full + blockIdx.x;
    int qb, bh;
    row_block_of(item, p.nqb, p.group_lg, p.causal != 0, qb, bh);
    const int b = bh / p.H, h = bh - b * p.H;
    const int q_row = qb * ATTN_BM + row;
    const int64_t part0 = (int64_t)blockIdx.x * p.split_s;
    float m = -INFINITY;
    for (int i = 0; i < p.split_s; ++i) m = fmaxf(m, p.part_ml[((part0 + i) * ATTN_BM + row) * 2]);
    float l = 0.f;
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < p.split_s; ++i) {
        const float* pm = p.part_ml + ((part0 + i) * ATTN_BM + row) * 2;
        const float w = pm[0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(pm[0] - m);
        l += w * pm[1];
        const f32x4 oi = *reinterpret_cast<const f32x4*>(p.part_o + ((part0 + i) * ATTN_BM + row) * DPAD + col);
        o += oi * w;
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    if (q_row < p.Tq) {
        T* op = static_cast<T*>(const_cast<void*>(p.o.ptr)) + b * p.o.sb + h * p.o.sh + (int64_t)q_row * p.o.sn;
        if (p.vec && col + 4 <= p.D) {
            const uint32_t w0 = pack2<T>(o[0] * inv, o[1] * inv), w1 = pack2<T>(o[2] * inv, o[3] * inv);
            *reinterpret_cast<u32x2*>(op + col) = u32x2{w0, w1};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col + e < p.D) op[col + e] = static_cast<T>(o[e] * inv);
        }
    }
    if (col == 0 && q_row < p.Tq_rounded)
        p.lse[(int64_t)bh * p.Tq_rounded + q_row] = q_row < p.Tq ? (m + __builtin_amdgcn_logf(l)) * kLn2 : 0.f;
}
