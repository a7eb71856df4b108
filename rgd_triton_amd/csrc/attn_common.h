// Pieces shared by the attention kernels: the 32x32x16 MFMA wrappers, the row permutation that makes a
// lane's 16 accumulator values contiguous, tile loaders and bias access.
//
// MFMA v_mfma_f32_32x32x16_{bf16,f16} on a 64-lane wavefront, D = A(32x16) * B(16x32) + C:
//   A operand: lane l holds A[l%32][8*(l/32) .. +7]        (8 contiguous K values of one row)
//   B operand: lane l holds B[8*(l/32) .. +7][l%32]        (8 contiguous K values of one column)
//   C / D:     lane l holds column l%32, rows 8*(v/4) + 4*(l/32) + v%4 for v = 0..15
// Which matrix row an MFMA row stands for is the kernel's choice (it only decides which address a
// lane reads its A operand from).  All kernels here read MFMA row r = 8a + 4g + c from matrix row
// perm(r) = 16g + 4a + c, so that lane (l%32, g = l/32) ends up holding the 16 CONTIGUOUS matrix rows
// 16g .. 16g+15 of its column, in register order v = 0..15.  That makes bias loads, probability
// operands and output stores 16-element contiguous runs per lane.
#pragma once

#include "common.h"

// Row stride (elements) of the 16-bit tiles staged in LDS.  Measured on gfx950: with these strides both the
// 16-byte row reads of the MFMA A operands and the transposing 8-byte reads run at the full LDS rate;
// DPAD + 8 does too except for DPAD = 128, where the transposing reads take two-way bank conflicts.
constexpr int attn_lds_stride(int dpad) { return dpad + (dpad == 128 ? 24 : 8); }

template <typename T> struct Mfma;
template <> struct Mfma<bf16_t> {
    typedef bf16x8 V8;
    static __device__ __forceinline__ f32x16 run(V8 a, V8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mfma<f16_t> {
    typedef f16x8 V8;
    static __device__ __forceinline__ f32x16 run(V8 a, V8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// matrix row read by MFMA row r (r = lane % 32 for an A operand)
__device__ __forceinline__ int mfma_row_perm(int r) { return ((r >> 2) & 1) * 16 + (r >> 3) * 4 + (r & 3); }

union Pack16 {  // 8 16-bit elements <-> one 16-byte vector
    u32x4 v;
    uint32_t w[4];
    uint16_t h[8];
};

// 8 elements of a row starting at column `col`; columns >= ncols and rows flagged invalid read as 0.
// `vec` = 16-byte access is legal for this tensor.
template <typename T>
__device__ __forceinline__ u32x4 load8(const T* __restrict__ row, int col, int ncols, bool valid, bool vec) {
    Pack16 p;
    p.v = u32x4{0u, 0u, 0u, 0u};
    if (valid) {
        if (vec) {
            if (col < ncols) p.v = *reinterpret_cast<const u32x4*>(row + col);
        } else {
            const uint16_t* r16 = reinterpret_cast<const uint16_t*>(row);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (col + e < ncols) p.h[e] = r16[col + e];
        }
    }
    return p.v;
}

template <typename T> __device__ __forceinline__ typename Mfma<T>::V8 as_v8(u32x4 raw) {
    return __builtin_bit_cast(typename Mfma<T>::V8, raw);
}

// two fp32 -> one dword of two T (round to nearest even)
template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef T T2 __attribute__((ext_vector_type(2)));
    T2 t;
    t[0] = static_cast<T>(lo);
    t[1] = static_cast<T>(hi);
    return __builtin_bit_cast(uint32_t, t);
}

template <int N> struct IntC { static constexpr int value = N; };

// first or second of two references, chosen at compile time
template <bool SECOND, typename X> __device__ __forceinline__ X& pick_ref(X& a, X& b) {
    if constexpr (SECOND) return b;
    else return a;
}  // compile-time flag passed by value

// Bias kinds of the kernel templates: no bias, bias stored in the tensor dtype T, bias stored in fp32.
enum { BIAS_OFF = 0, BIAS_SAME = 1, BIAS_F32 = 2 };
template <typename T, int BIAS> struct BiasElem { typedef T type; };
template <typename T> struct BiasElem<T, BIAS_F32> { typedef float type; };

// Bit pattern of a dword that holds nothing but -inf in the bias type (two values for a 16-bit type).
template <typename TB> struct NegInfBits;
template <> struct NegInfBits<f16_t> { static constexpr uint32_t value = 0xFC00FC00u; };
template <> struct NegInfBits<bf16_t> { static constexpr uint32_t value = 0xFF80FF80u; };
template <> struct NegInfBits<float> { static constexpr uint32_t value = 0xFF800000u; };

// Blocks of logits whose bias is -inf everywhere are detected in the kernels and left out only at head dims above 64.
// Measured on (2,4352,24,64) with a bias that has no such block: the test (three instructions, but a branch between the
// first product and the softmax) costs the forward 7 % and the backward 1.5 %; on (2,2048,16,128) with a block-causal
// bias it gains 5 % and 7 %.
constexpr bool attn_skip_masked(int dpad, int bias) { return bias != 0 && dpad > 64; }

// Raw bias of one lane for one tile of 32*NKB keys in the "query per lane" layout: NKB runs of 16
// contiguous keys (key0 + 32*kb + 16*g ...).  load() only issues the memory reads, so it can run a whole tile
// ahead of decode(); the registers hold the undecoded bits (8 VGPRs for a 16-bit bias).
template <typename TB, int NKB = 2> struct BiasRuns {
    static constexpr int NV = 16 * sizeof(TB) / 16;  // 16-byte vectors per run
    u32x4 raw[NKB][NV];

    // row: &bias[b, h, q, 0].  fast = the run is 16-byte aligned and all keys of the tile exist.
    __device__ __forceinline__ void load(const TB* __restrict__ row, int key0, int g, int Tk, bool fast) {
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb) {
            const int first = key0 + kb * 32 + g * 16;
            if (fast) {
                const u32x4* src = reinterpret_cast<const u32x4*>(row + first);
#pragma unroll
                for (int i = 0; i < NV; ++i) raw[kb][i] = src[i];
            } else {
                // element loads from clamped indices; keys >= Tk are masked by the caller
                TB tmp[16];
#pragma unroll
                for (int e = 0; e < 16; ++e) tmp[e] = row[min(first + e, Tk - 1)];
                __builtin_memcpy(&raw[kb][0], tmp, sizeof(tmp));
            }
        }
    }
    // True (for the whole wavefront) when every bias value the wavefront holds for runs [kb0, kb0 + n) is -inf:
    // such a block of logits has probability 0 everywhere and can be left out.  The first dword of every lane is
    // looked at first, so a block with ordinary values costs three instructions.
    __device__ __forceinline__ bool all_neg_inf(int kb0, int n) const {
        constexpr uint32_t PAT = NegInfBits<TB>::value;
        if (__builtin_amdgcn_ballot_w64(raw[kb0][0][0] != PAT) != 0) return false;
        uint32_t all_and = PAT, all_or = PAT;
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb) {
            if (kb < kb0 || kb >= kb0 + n) continue;
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    all_and &= raw[kb][i][e];
                    all_or |= raw[kb][i][e];
                }
        }
        return __builtin_amdgcn_ballot_w64(all_and != PAT || all_or != PAT) == 0;
    }
    __device__ __forceinline__ void decode_run(int kb, float (&out)[16]) const {
        TB tmp[16];
        __builtin_memcpy(tmp, &raw[kb][0], sizeof(tmp));
#pragma unroll
        for (int e = 0; e < 16; ++e) out[e] = static_cast<float>(tmp[e]);
    }
    __device__ __forceinline__ void decode(float (&out)[NKB][16]) const {
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb) {
            TB tmp[16];
            __builtin_memcpy(tmp, &raw[kb][0], sizeof(tmp));
#pragma unroll
            for (int e = 0; e < 16; ++e) out[kb][e] = static_cast<float>(tmp[e]);
        }
    }
};

// Forward and dQ kernel: trailing key tiles whose bias is -inf for every (query, key) pair of the workgroup give P = 0
// and add nothing (a block-causal bias: all keys after the query block).  Returns the end of [t_begin, t_end) without
// them, found before anything else is loaded: every wavefront reads its [32 rows][BN keys] bias blocks backwards from
// the last tile, four tiles at a time and 16 bytes per lane (whole rows by neighbouring lanes), until it meets a value
// above -inf; the workgroup keeps the tiles up to the latest such tile.  (Inside the loop such a tile still costs its
// K/V loads and a barrier.)  wave_rows: &bias[b, h, first row of the wavefront, 0]; rows: how many of its 32 rows exist;
// slot: an int in LDS that nothing else uses until the next barrier after the call.  All tiles must be full tiles.
// A first look that is the same in every wavefront keeps an ordinary bias cheap: the first four bytes of the last tile in
// each of the workgroup's rows (wg_rows: &bias[b, h, first row of the workgroup, 0], wg_nrows of them, at most 128); one
// value above -inf there and the last tile stays, with no search and no barrier.
template <typename TB, int BN>
__device__ __forceinline__ int bias_trim_end(const TB* __restrict__ wg_rows, int wg_nrows, const TB* __restrict__ wave_rows,
                                             int64_t sn, int rows, int t_begin, int t_end, int lane, int tid, int* slot) {
    constexpr int EPC = 16 / (int)sizeof(TB);
    constexpr int CPR = BN / EPC;   // 16-byte chunks per row of a tile
    constexpr int RPL = 64 / CPR;   // rows per load instruction
    constexpr int LPT = 32 / RPL;   // load instructions per tile
    constexpr int BATCH = 4;
    constexpr uint32_t PAT = NegInfBits<TB>::value;
    {
        const TB* last = wg_rows + (int64_t)(t_end - 1) * BN;
        const uint32_t a = *reinterpret_cast<const uint32_t*>(last + (int64_t)min(lane, wg_nrows - 1) * sn);
        const uint32_t c = *reinterpret_cast<const uint32_t*>(last + (int64_t)min(lane + 64, wg_nrows - 1) * sn);
        if (__builtin_amdgcn_ballot_w64(a != PAT || c != PAT) != 0) return t_end;  // the same answer in every wavefront
    }
    int last = t_begin;  // end of this wavefront's live tiles
    if (rows > 0) {
        const TB* col = wave_rows + (lane % CPR) * EPC;
        const int rsub = lane / CPR;
        for (int t1 = t_end; t1 > t_begin && last == t_begin; t1 -= BATCH) {
            u32x4 v[BATCH][LPT];
#pragma unroll
            for (int bi = 0; bi < BATCH; ++bi)
#pragma unroll
                for (int i = 0; i < LPT; ++i) {
                    const int tile = max(t1 - 1 - bi, t_begin);
                    const int row = min(i * RPL + rsub, rows - 1);
                    v[bi][i] = *reinterpret_cast<const u32x4*>(col + (int64_t)row * sn + tile * BN);
                }
#pragma unroll
            for (int bi = BATCH - 1; bi >= 0; --bi) {  // ends on the latest tile of the batch
                uint32_t all_and = PAT, all_or = PAT;
#pragma unroll
                for (int i = 0; i < LPT; ++i)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        all_and &= v[bi][i][e];
                        all_or |= v[bi][i][e];
                    }
                const bool some = __builtin_amdgcn_ballot_w64(all_and != PAT || all_or != PAT) != 0;
                if (some && t1 - 1 - bi >= t_begin) last = t1 - bi;
            }
        }
    }
    if (tid == 0) *slot = t_begin;
    __syncthreads();
    if (lane == 0) atomicMax(slot, last);
    __syncthreads();
    const int end = *slot;
    __syncthreads();  // the slot's memory is free again
    return end;
}

typedef short s16x4 __attribute__((ext_vector_type(4)));

// 4 elements for this lane out of a transposing read; `p` is this lane's own 8-byte source piece
template <typename T> __device__ __forceinline__ u32x2 lds_read_tr(const T* p) {
    s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p));
    return __builtin_bit_cast(u32x2, r);
}

// A operand (32 rows x 16 k) taken transposed from a row-major tile: MFMA row r = matrix COLUMN
// col0 + perm(r), k index = tile ROW.  `row0` is the first of this lane-half's 8 tile rows.
// lane decomposition: s = lane%16 -> (j = s/4 tile row within a group of 4, c = s%4 column quad),
// gi = (lane/16)%2 selects MFMA rows 16..31.
template <typename T>
__device__ __forceinline__ typename Mfma<T>::V8 load_a_transposed(const T* tile, int stride, int row0, int col0,
                                                                   int lane) {
    const int s = lane & 15;
    const int j = s >> 2;
    const int cq = mfma_row_perm(((lane >> 4) & 1) * 16 + (s & 3) * 4);
    const T* p = tile + (row0 + j) * stride + col0 + cq;
    const u32x2 lo = lds_read_tr<T>(p);
    const u32x2 hi = lds_read_tr<T>(p + 4 * stride);
    const u32x4 raw = {lo[0], lo[1], hi[0], hi[1]};
    return as_v8<T>(raw);
}

// Workgroup ids are handed to the 8 XCDs round-robin and every XCD has its own L2.  This maps the
// hardware id to a logical id so that each XCD works through a contiguous range of logical ids:
// workgroups that share K/V (same batch and head, neighbouring row blocks) then run on one XCD, one
// after the other, and find those tiles in that XCD's L2.
constexpr int kNumXcd = 8;
__device__ __forceinline__ int xcd_remap(int id, int n) {
    const int per = n / kNumXcd, rem = n % kNumXcd;
    const int x = id % kNumXcd, slot = id / kNumXcd;
    return x < rem ? x * (per + 1) + slot : rem * (per + 1) + (x - rem) * per + slot;
}

#ifndef RGD_CAUSAL_GROUP_LOG2
#define RGD_CAUSAL_GROUP_LOG2 2
#endif
// Forward and dQ kernel: item -> (row block, batch*head).  Causal launches: the last row blocks of a (batch, head) have
// the most key tiles.  Their items run through groups of 4 (batch, head) pairs row block by row block, last row block
// first (group_lg = 2, set by the host when batch*head is a multiple of 4), so a launch starts on the long workgroups of
// several heads and ends on short ones; (8,2048,16,64) causal: forward 115 -> 106 us, backward 294 -> 276 us.
// Otherwise (group_lg = 0) one (batch, head) after the other.  One code path for both: a second path costs the
// forward without bias registers it does not have (config-3 forward +4 %).
__device__ __forceinline__ void row_block_of(int item, int nblk, int group_lg, bool last_first, int& blk, int& bh) {
    const int per = nblk << group_lg;
    const int grp = item / per, local = item - grp * per;
    const int pos = local >> group_lg;
    blk = last_first ? nblk - 1 - pos : pos;
    bh = (grp << group_lg) + (local & ((1 << group_lg) - 1));
}
inline int causal_group_lg(bool causal, int64_t nbh) { return causal && nbh % (1 << RGD_CAUSAL_GROUP_LOG2) == 0 ? RGD_CAUSAL_GROUP_LOG2 : 0; }

struct AttnTensor {
    const void* ptr;
    int64_t sb, sh, sn;
};

// A launch of `items` equal workgroups runs in rounds of cus * per_cu resident workgroups and the last round
// may leave most of the chip idle.  The plan keeps the items of the whole rounds as they are and splits each
// item of the last round into `s` parts along its inner loop; a merge kernel combines the parts' partial
// results.  s == 1: no split.  Host side only.
//
// Cost model (measured on MI355X): a compute unit with n resident workgroups of these kernels delivers
// thr(n) times the throughput of one workgroup alone, far below n (MFMA and VALU work of the wavefronts of a
// SIMD add up); the last round's time is the work of its busiest compute unit divided by that throughput.
// A split is taken when the time it saves exceeds the cost of writing, re-reading and merging the parts.
struct AttnSplit {
    int full = 0, s = 1;
    int items_split(int64_t items) const { return s > 1 ? (int)(items - full) : 0; }
    int64_t blocks(int64_t items) const { return s > 1 ? full + (items - full) * s : items; }
};
struct AttnSplitModel {
    float thr2, thr3;  // throughput of a compute unit with 2 / 3 resident workgroups, relative to 1
    float tile_us;     // one inner-loop step of a workgroup alone on its compute unit
};
inline AttnSplit attn_split_plan(int64_t items, int cus, int per_cu, int inner_tiles, size_t part_bytes,
                                 size_t workspace_bytes, AttnSplitModel m) {
    AttnSplit plan;
    if (items <= 0 || cus <= 0 || per_cu <= 0 || items >= (1ll << 30)) return plan;
    const int64_t slots = (int64_t)cus * per_cu;
    const int64_t full = items / slots * slots, rest = items - full;
    if (rest == 0) return plan;
    auto round_time = [&](int64_t parts, int s) {  // in units of one whole item alone on a compute unit
        const int64_t n = (parts + cus - 1) / cus;  // parts the busiest compute unit works through
        const int64_t res = n < per_cu ? n : per_cu;
        const double thr = res >= 3 ? m.thr3 : (res == 2 ? m.thr2 : 1.0);
        return (double)n / thr / s;
    };
    const double item_us = (double)inner_tiles * m.tile_us, t1 = round_time(rest, 1);
    double best_gain = 3.0;  // microseconds a split must save to be taken
    for (int s = 2; s <= 8; ++s) {
        if (inner_tiles < 2 * s) break;                                 // parts of at least two steps
        if (rest * s > 2 * slots) break;                                // at most two rounds of parts
        if ((size_t)(rest * s) * part_bytes > workspace_bytes) break;   // what the caller's workspace holds
        const double overhead_us = 6.0 + (double)(rest * s) * part_bytes * 2.0 / 4.0e6;  // merge launch + traffic at 4 TB/s
        const double gain = (t1 - round_time(rest * s, s)) * item_us - overhead_us;
        if (gain > best_gain) {
            best_gain = gain;
            plan.s = s;
        }
    }
    plan.full = plan.s > 1 ? (int)full : 0;
    return plan;
}

// A copy of a scalar (wavefront-uniform) value that the compiler treats as a value of its own.  The kernels receive their
// parameters as one struct, which arrives in groups of 8 or 16 scalar registers; a field that a loop uses keeps its whole
// group alive, and when scalar registers run short the compiler parks and fetches whole groups (16 lane reads per step
// for one stride).  Loop code therefore works on copies made with this function before the loop.
template <typename X> __device__ __forceinline__ X own_scalar(X v) {
    // a real move into a new register: an empty statement with a tied operand would be folded back into the group
    static_assert(sizeof(X) == 4 || sizeof(X) == 8, "own_scalar: 32- or 64-bit values");
    X r;
    if constexpr (sizeof(X) == 4)
        asm volatile("s_mov_b32 %0, %1" : "=s"(r) : "s"(v));
    else
        asm volatile("s_mov_b64 %0, %1" : "=s"(r) : "s"(v));
    return r;
}

// The kernel's parameter struct as it lies in argument memory (the kernels take one struct, by value, as their first
// argument), for code that runs rarely: a field read through this reference is loaded where it is used, instead of
// sitting in a scalar register through every loop of the kernel.  (The empty asm keeps the compiler from moving the
// loads out of the rarely executed block they are written in.)
template <typename P> __device__ __forceinline__ const P& cold_params() {
    auto ka = __builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(ka));
    return *(const P*)ka;
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
