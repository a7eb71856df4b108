// Tile classes of an attention bias matrix that is shared by the heads of a batch element (head stride 0).
//
// Such a bias is usually a mask: 0 where a query may look at a key and -inf where it may not (padding keys, documents
// packed into one sequence).  Every head re-reads it, in each of the three attention kernels, although most of its
// tiles say nothing: a tile that is +0.0 everywhere leaves the logits as they are, a tile that is -inf everywhere
// removes them.  One pass over the matrix (attn_bias_classify_kernel) therefore leaves two bits per tile of 32 query
// rows x 64 keys; the kernels then treat a ZERO tile like a tile without bias (bit-identical: the logit
// fma(s, c, fma(+0, log2e, -m)) is fma(s, c, -m)), leave a NEG tile out, and read the bias only for MIXED tiles.
//
// Layout: one 64-bit word per 32 consecutive key tiles, tile t of the word in bits [2t, 2t+2):
//     words[(b * nrow32 + r) * nwords + w]      r = query row / 32, w = key tile / 32
// nrow32 covers whole workgroups of 128 rows (rows past Tq repeat the last row); key tiles that are not full tiles of
// existing keys are MIXED, so ragged ends take the general path.  The reference streams the bias tile by tile for
// every head (flash_attn/flash_attn_triton_cached.py:151-175).
#pragma once

#include "attn_common.h"

// COLUMN: every row of the tile equals its first row (a mask of hidden keys that is neither all 0 nor all -inf: the usual
// padding mask); the kernels then read one row of the tile, or one value per key, instead of the tile.
enum { CLS_MIXED = 0, CLS_ZERO = 1, CLS_NEG = 2, CLS_COLUMN = 3 };
constexpr int CLS_ROWS = 32;           // query rows per class
constexpr int CLS_KEYS = 64;           // keys per class
constexpr int CLS_TILES_PER_WORD = 32;
constexpr int CLS_MAX_WORDS = 64;      // up to 2048 key tiles (131072 keys): one byte each in LDS
constexpr int CLS_MAX_ROWS = 4096;     // up to 2048 steps of 64 query rows (131072 rows): one byte each in LDS

struct BiasClasses {
    const uint64_t* words;  // null: no classes for this call
    int nwords;             // words per row of 32 query rows
    int nrow32;             // rows of the map per batch element
    int64_t sb;             // words between batch elements (0: one map for every batch element)
};

// host: shape of the map for a (Tq, Tk) bias
inline int cls_nwords(int64_t Tk) { return (int)(((Tk + CLS_KEYS - 1) / CLS_KEYS + CLS_TILES_PER_WORD - 1) / CLS_TILES_PER_WORD); }
inline int cls_nrow32(int64_t Tq) { return (int)((Tq + 127) / 128 * 4); }
inline size_t cls_bytes(int64_t nb, int64_t Tq, int64_t Tk) { return (size_t)nb * cls_nrow32(Tq) * cls_nwords(Tk) * sizeof(uint64_t); }

constexpr int CLS_LDS_BYTES = 2048;  // forward and dQ kernel: one byte per key tile

// Forward and dQ kernel: the class of every key tile for the workgroup's `nrows` rows of the map (its 128 query rows),
// one byte per tile in LDS: ZERO / NEG when the tile is that in every one of the rows, MIXED otherwise.  What the
// workgroup does with a tile (which loop runs it, whether its K/V are loaded at all) is then decided alike in all its
// wavefronts, and nothing of the classes lives in registers while the loops run.  Ends with a barrier.
__device__ __forceinline__ void cls_tiles_to_lds(const BiasClasses& c, int b, int row0, int nrows, int ntiles, uint8_t* lds, int tid) {
    for (int t = tid; t < ntiles; t += 256) {
        bool zero = true, neg = true, col = true;
        for (int r = 0; r < nrows; ++r) {
            const uint64_t w = c.words[b * c.sb + (int64_t)min(row0 + r, c.nrow32 - 1) * c.nwords + (t >> 5)];
            const uint32_t f = (uint32_t)(w >> (2 * (t & 31))) & 3u;
            zero = zero && f == CLS_ZERO;
            neg = neg && f == CLS_NEG;
            col = col && f != CLS_MIXED;  // each wavefront reads the first of its own 32 rows
        }
        lds[t] = zero ? CLS_ZERO : (neg ? CLS_NEG : (col ? CLS_COLUMN : CLS_MIXED));
    }
    __syncthreads();
}
// dK/dV kernel.  A workgroup owns 128 keys and walks the query rows; what a padding mask does to it does not change along
// the way: a key is hidden from every query or from none.  Such a key block is a "key mask" block: no tile of its two key
// tiles is MIXED, and for each of its keys the bias is +0 in every row or -inf in every row.  It then runs the loop of the
// kernel without bias, with its hidden keys treated like keys that do not exist (their probabilities are 0), and is left
// alone by the ordinary biased kernel that is launched behind it; every other key block leaves at once and is served by
// that kernel.  Both kernels call this function, so both decide alike.
//   key_col: &bias[b, h, 0, this lane's key] (an existing key); rows32: rows of the map that hold query rows.
//   slot: two ints in LDS nothing else uses.  Returns (the same in every lane of the workgroup) whether the block is a key
//   mask block; hidden: this lane's key is hidden; any_hidden / all_hidden: some / every key of the workgroup is.
template <typename TB>
__device__ __forceinline__ bool cls_key_mask_block(const BiasClasses& c, const TB* __restrict__ key_col, int64_t sn, int b, int tile0, int rows32,
                                                   int Tq, int lane, int tid, int* slot, bool& hidden, bool& any_hidden, bool& all_hidden) {
    typedef typename std::conditional<sizeof(TB) == 2, uint16_t, uint32_t>::type Bits;
    constexpr Bits NEG = (Bits)(NegInfBits<TB>::value & (sizeof(TB) == 2 ? 0xFFFFu : 0xFFFFFFFFu));
    // no MIXED tile in the two columns of the map: every thread looks at some of the rows
    bool ok = true;
    for (int r = tid; r < rows32; r += 256) {
        const uint32_t v = (uint32_t)(c.words[b * c.sb + (int64_t)r * c.nwords + (tile0 >> 5)] >> (2 * (tile0 & 31)));
        ok = ok && (v & 3u) != CLS_MIXED && ((v >> 2) & 3u) != CLS_MIXED;
    }
    // every 32 rows of such a column are the same row: the first one stands for them
    Bits all_and = (Bits)~(Bits)0, all_or = 0;
    for (int r0 = 0; r0 < rows32; r0 += 8) {
        Bits v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = __builtin_bit_cast(Bits, key_col[(int64_t)min((r0 + i) * CLS_ROWS, Tq - 1) * sn]);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            all_and &= v[i];
            all_or |= v[i];
        }
    }
    hidden = all_and == NEG && all_or == NEG;
    const bool plain = all_or == 0;
    ok = ok && (hidden || plain);
    if (tid == 0) {
        slot[0] = 1;  // all ok
        slot[1] = 0;  // bit 0: some key hidden, bit 1: some key not hidden
    }
    __syncthreads();
    const bool wave_bad = __builtin_amdgcn_ballot_w64(!ok) != 0;
    const int wave_bits = (__builtin_amdgcn_ballot_w64(hidden) != 0 ? 1 : 0) | (__builtin_amdgcn_ballot_w64(!hidden) != 0 ? 2 : 0);
    if (lane == 0) {
        if (wave_bad) slot[0] = 0;
        atomicOr(&slot[1], wave_bits);
    }
    __syncthreads();
    const bool pure = slot[0] != 0;
    any_hidden = (slot[1] & 1) != 0;
    all_hidden = (slot[1] & 2) == 0;
    __syncthreads();  // the slot's memory is free again
    return pure;
}
// class of tile / step j, the same value in every lane (a scalar for the compiler)
__device__ __forceinline__ int cls_lds_at(const uint8_t* lds, int j) { return __builtin_amdgcn_readfirstlane((int)lds[j]); }

// number of MIXED tiles among the first n tiles of a word
__device__ __forceinline__ int cls_count_mixed(uint64_t w, int n) {
    const uint64_t any = (w | (w >> 1)) & 0x5555555555555555ull;  // bit 2t set: tile t is not MIXED
    const uint64_t keep = n >= 32 ? ~0ull : ((1ull << (2 * n)) - 1);
    return n - (int)__builtin_popcountll(any & keep);
}

// Which kernels serve a batch element.  A bias with classes is launched twice over the same grid: the CLS variant of
// the kernel (laid out like the kernel without bias; reads the bias only in the runs of MIXED tiles, at the start of each
// step) and the ordinary biased kernel (bias fetched a tile ahead in every step).  Every workgroup of both launches asks
// this function about its batch element and leaves at once if the other launch serves it: true (ordinary kernel) when more
// than half of a fixed sample of the map (64 of its words, evenly spaced) is MIXED, i.e. the bias is a dense one.  The
// same answer in every lane of every workgroup that asks: all items of a batch element run in one launch.
__device__ __forceinline__ bool cls_batch_dense(const BiasClasses& c, int b, int ntiles, int lane) {
    const int total = c.nrow32 * c.nwords;
    const int i = (int)((int64_t)lane * total / 64);  // 64 words, evenly spaced (all of them when the map has at most 64)
    const int w = i % c.nwords;
    const int n = min(32, ntiles - 32 * w);  // tiles of that word that exist
    int mixed = cls_count_mixed(c.words[b * c.sb + i], n), seen = n;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        mixed += __shfl_xor(mixed, off, 64);
        seen += __shfl_xor(seen, off, 64);
    }
    return 2 * mixed > seen;
}

// One wavefront classifies a strip of 32 query rows x 8 key tiles (512 keys): every load instruction reads whole rows
// of the strip (neighbouring lanes, 16 bytes each), and the strip is left as soon as every one of its tiles is known to
// be MIXED, so a dense bias costs a fraction of a pass.  grid (ceil(nrow32 * nstrips / 4), nb), 256 threads.
template <typename TB>
__global__ __launch_bounds__(256) void attn_bias_classify_kernel(const TB* __restrict__ bias, int64_t sb, int64_t sn, int Tq, int Tk,
                                                                 int nrow32, int nstrips, uint16_t* __restrict__ out) {
    constexpr int EPC = 16 / (int)sizeof(TB);      // elements per 16-byte chunk
    constexpr int NLD = 512 / (64 * EPC);          // load instructions per row of the strip (1 or 2)
    constexpr int LPT = CLS_KEYS / EPC;            // lanes per tile (8 or 16)
    constexpr uint32_t PAT = NegInfBits<TB>::value;
    const int lane = threadIdx.x & 63;
    const int w = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (w >= nrow32 * nstrips) return;
    const int row32 = w / nstrips, strip = w - row32 * nstrips;
    const int b = blockIdx.y;
    const int full_tiles = Tk / CLS_KEYS;
    const TB* base = bias + b * sb;
    int key[NLD];
    bool ok[NLD];
    u32x4 all_and[NLD], all_or[NLD];  // per dword: one or two columns of the tile over the rows seen so far
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        key[i] = strip * 512 + i * 64 * EPC + lane * EPC;
        ok[i] = key[i] / CLS_KEYS < full_tiles;
        if (!ok[i]) key[i] = 0;  // read something that exists; the tile is MIXED whatever it holds
        all_and[i] = u32x4{~0u, ~0u, ~0u, ~0u};
        all_or[i] = u32x4{0u, 0u, 0u, 0u};
    }
    // bit t*LPT of the result: all LPT lanes of tile t have their bit set in m
    auto fold = [](uint64_t m) {
        m &= m >> 4;
        m &= m >> 2;
        m &= m >> 1;
        if (LPT == 16) m &= m >> 8;
        return m & (LPT == 16 ? 0x0001000100010001ull : 0x0101010101010101ull);
    };
    uint64_t zero_t[NLD], neg_t[NLD], col_t[NLD];
    // rows [r0, r0 + N) of the strip, all their loads in flight at once; returns whether any tile may still be something
    // other than MIXED
    auto rows = [&](auto R0, auto N) __attribute__((always_inline)) {
        constexpr int r0 = decltype(R0)::value, n = decltype(N)::value;
        u32x4 v[n][NLD];
#pragma unroll
        for (int r = 0; r < n; ++r) {
            const int row = min(row32 * CLS_ROWS + r0 + r, Tq - 1);
#pragma unroll
            for (int i = 0; i < NLD; ++i) v[r][i] = *reinterpret_cast<const u32x4*>(base + (int64_t)row * sn + key[i]);
        }
#pragma unroll
        for (int r = 0; r < n; ++r)
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                all_and[i] &= v[r][i];
                all_or[i] |= v[r][i];
            }
        uint64_t open = 0;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const uint32_t a = all_and[i][0] & all_and[i][1] & all_and[i][2] & all_and[i][3];
            const uint32_t o = all_or[i][0] | all_or[i][1] | all_or[i][2] | all_or[i][3];
            const bool same = all_and[i][0] == all_or[i][0] && all_and[i][1] == all_or[i][1] && all_and[i][2] == all_or[i][2] &&
                              all_and[i][3] == all_or[i][3];  // every bit the same in all rows: every column constant
            zero_t[i] = fold(__builtin_amdgcn_ballot_w64(ok[i] && o == 0u));
            neg_t[i] = fold(__builtin_amdgcn_ballot_w64(ok[i] && a == PAT && o == PAT));
            col_t[i] = fold(__builtin_amdgcn_ballot_w64(ok[i] && same));
            open |= col_t[i];  // a ZERO or NEG tile is a COLUMN tile too
        }
        return open != 0;
    };
    // two rows tell a dense bias from a mask (two rows of a dense bias differ in every tile): the strip is left after
    // them; otherwise the other thirty rows follow, all their loads in flight at once
    if (rows(IntC<0>{}, IntC<2>{})) {
        if constexpr (NLD == 1) {
            rows(IntC<2>{}, IntC<CLS_ROWS - 2>{});
        } else {
            if (rows(IntC<2>{}, IntC<14>{})) rows(IntC<16>{}, IntC<16>{});
        }
    }
    if (lane == 0) {
        uint32_t code = 0;
#pragma unroll
        for (int i = 0; i < NLD; ++i)
#pragma unroll
            for (int t = 0; t < 8 / NLD; ++t) {
                const int tile = i * (8 / NLD) + t;
                uint32_t c = CLS_MIXED;
                if (col_t[i] >> (t * LPT) & 1ull) c = CLS_COLUMN;
                if (neg_t[i] >> (t * LPT) & 1ull) c = CLS_NEG;
                if (zero_t[i] >> (t * LPT) & 1ull) c = CLS_ZERO;
                code |= c << (2 * tile);
            }
        out[((int64_t)b * nrow32 + row32) * nstrips + strip] = (uint16_t)code;
    }
}
