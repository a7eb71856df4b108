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

constexpr int CLS_KEY_BLOCK = 128;     // keys per workgroup of the dK/dV kernel at head dims up to 64
constexpr int CLS_INFO_HEAD = 4;       // 32-bit words of a batch element's summary in front of its key block entries
constexpr int CLS_INFO_ENTRY = 8;      // 32-bit words per key block entry

// Behind the map lies a summary per batch element, written by a second launch (attn_bias_summary_kernel), so that no
// workgroup of the attention kernels has to derive it again:
//     info[b * info_sb + 0]                             1: most tiles have to be read, the ordinary biased kernels serve b
//     info[b * info_sb + CLS_INFO_HEAD + kb * 8 + 0..3]  key block kb (128 keys): bit k set = key k is hidden from every query
//     info[b * info_sb + CLS_INFO_HEAD + kb * 8 + 4]     bit 0: "key mask" block (see attn_bias_summary_kernel), bit 1: some key
//                                                       of it is hidden, bit 2: every key of it is
struct BiasClasses {
    const uint64_t* words;  // null: no classes for this call
    int nwords;             // words per row of 32 query rows
    int nrow32;             // rows of the map per batch element
    int64_t sb;             // words between batch elements (0: one map for every batch element)
    const uint32_t* info;   // summaries, behind the words
    int64_t info_sb;        // 32-bit words between the summaries of two batch elements (0: one for all)
};
enum { CLS_KB_PURE = 1, CLS_KB_ANY_HIDDEN = 2, CLS_KB_ALL_HIDDEN = 4 };

// host: shape of the map for a (Tq, Tk) bias
inline int cls_nwords(int64_t Tk) { return (int)(((Tk + CLS_KEYS - 1) / CLS_KEYS + CLS_TILES_PER_WORD - 1) / CLS_TILES_PER_WORD); }
inline int cls_nrow32(int64_t Tq) { return (int)((Tq + 127) / 128 * 4); }
inline int cls_nkb(int64_t Tk) { return (int)((Tk + CLS_KEY_BLOCK - 1) / CLS_KEY_BLOCK); }
inline size_t cls_words_bytes(int64_t nb, int64_t Tq, int64_t Tk) { return (size_t)nb * cls_nrow32(Tq) * cls_nwords(Tk) * sizeof(uint64_t); }
inline int64_t cls_info_words(int64_t Tk) { return CLS_INFO_HEAD + (int64_t)cls_nkb(Tk) * CLS_INFO_ENTRY; }
inline size_t cls_bytes(int64_t nb, int64_t Tq, int64_t Tk) {
    return cls_words_bytes(nb, Tq, Tk) + (size_t)nb * cls_info_words(Tk) * sizeof(uint32_t);
}

// host: the parts of a classes buffer written for nb batch elements (nb = 1: one map that every batch element uses)
// one_row: every row of the bias is the same row (row stride 0: a vector, or a matrix expanded from one); the map then
// has one row per batch element, which stands for all of them (the kernels clamp the row index to nrow32 - 1)
inline BiasClasses cls_layout(const void* buffer, int64_t nb, int64_t Tq, int64_t Tk, bool one_row) {
    BiasClasses c;
    c.words = static_cast<const uint64_t*>(buffer);
    c.nwords = cls_nwords(Tk);
    c.nrow32 = one_row ? 1 : cls_nrow32(Tq);
    c.sb = nb == 1 ? 0 : (int64_t)c.nrow32 * c.nwords;
    c.info = reinterpret_cast<const uint32_t*>(static_cast<const char*>(buffer) + cls_words_bytes(nb, Tq, Tk));
    c.info_sb = nb == 1 ? 0 : cls_info_words(Tk);
    return c;
}

constexpr int CLS_MAX_TILES = CLS_MAX_WORDS * CLS_TILES_PER_WORD;  // 2048
constexpr int CLS_NEG_WORDS = CLS_MAX_TILES / 64;
// forward and dQ kernel: one byte per key tile, then one bit per key tile (set: the tile is NEG)
constexpr int CLS_LDS_BYTES = CLS_MAX_TILES + CLS_NEG_WORDS * 8;

// Forward and dQ kernel: the class of every key tile for the workgroup's `nrows` rows of the map (its 128 query rows),
// one byte per tile in LDS: ZERO / NEG when the tile is that in every one of the rows, MIXED otherwise; behind the bytes,
// the NEG tiles as a bit mask (64 tiles per word), in which the loop driver finds the runs of tiles to work on with a
// few scalar instructions per run instead of one LDS round trip per tile.  What the workgroup does with a tile (which
// arm runs it, whether its K/V are loaded at all) is then decided alike in all its wavefronts, and nothing of the classes
// lives in registers while the loops run.  256 threads; ends with a barrier.
__device__ __forceinline__ void cls_tiles_to_lds(const BiasClasses& c, int b, int row0, int nrows, int ntiles, uint8_t* lds, int tid) {
    uint64_t* neg_mask = reinterpret_cast<uint64_t*>(lds + CLS_MAX_TILES);
    for (int base = 0; base < ntiles; base += 256) {  // (the same trip count in every wavefront: the ballot below)
        const int t = base + tid;
        bool zero = true, neg = true, col = true;
        if (t < ntiles) {
            for (int r = 0; r < nrows; ++r) {
                const uint64_t w = c.words[b * c.sb + (int64_t)min(row0 + r, c.nrow32 - 1) * c.nwords + (t >> 5)];
                const uint32_t f = (uint32_t)(w >> (2 * (t & 31))) & 3u;
                zero = zero && f == CLS_ZERO;
                neg = neg && f == CLS_NEG;
                col = col && f != CLS_MIXED;  // each wavefront reads the first of its own 32 rows
            }
            lds[t] = zero ? CLS_ZERO : (neg ? CLS_NEG : (col ? CLS_COLUMN : CLS_MIXED));
        }
        const uint64_t m = __builtin_amdgcn_ballot_w64(t < ntiles && neg);
        if ((tid & 63) == 0) neg_mask[t >> 6] = m;
    }
    __syncthreads();
}
// the first tile in [j, end) whose NEG bit equals `neg` (end if there is none); wavefront-uniform
__device__ __forceinline__ int cls_next_tile(const uint8_t* lds, int j, int end, bool neg) {
    const uint64_t* neg_mask = reinterpret_cast<const uint64_t*>(lds + CLS_MAX_TILES);
    while (j < end) {
        const uint64_t raw = neg_mask[j >> 6];
        uint64_t w = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(raw >> 32)) << 32) |
                     (uint32_t)__builtin_amdgcn_readfirstlane((int)raw);
        if (!neg) w = ~w;
        w &= ~0ull << (j & 63);
        if (w != 0) return min(end, (j & ~63) + (int)__builtin_ctzll(w));
        j = (j & ~63) + 64;
    }
    return end;
}
// class of tile / step j, the same value in every lane (a scalar for the compiler)
__device__ __forceinline__ int cls_lds_at(const uint8_t* lds, int j) { return __builtin_amdgcn_readfirstlane((int)lds[j]); }

// number of tiles among the first n of a word whose bias has to be read (MIXED or COLUMN: both bits alike)
__device__ __forceinline__ int cls_count_read(uint64_t w, int n) {
    const uint64_t alike = ~(w ^ (w >> 1)) & 0x5555555555555555ull;  // bit 2t set: tile t is MIXED (00) or COLUMN (11)
    const uint64_t keep = n >= 32 ? ~0ull : ((1ull << (2 * n)) - 1);
    return (int)__builtin_popcountll(alike & keep);
}

// Which kernels serve a batch element.  A bias with classes is launched twice over the same grid: the CLS variant of
// the kernel (laid out like the kernel without bias; reads the bias only for the tiles that are not ZERO, at the start of
// their step) and the ordinary biased kernel (bias fetched a tile ahead in every step).  Every workgroup of both launches
// reads this flag of its batch element and leaves at once if the other launch serves it.
__device__ __forceinline__ bool cls_batch_dense(const BiasClasses& c, int b) {
    return __builtin_amdgcn_readfirstlane((int)c.info[b * c.info_sb]) != 0;
}
// dK/dV kernel: the entry of key block kb (uniform address: the compiler reads it through the scalar cache)
__device__ __forceinline__ const uint32_t* cls_key_block(const BiasClasses& c, int b, int kb) {
    return c.info + b * c.info_sb + CLS_INFO_HEAD + (int64_t)kb * CLS_INFO_ENTRY;
}

// Second launch of the classification, grid (key blocks + 1, batch elements), 256 threads.
//
// Workgroup kb < nkb writes the entry of key block kb for the dK/dV kernel.  A workgroup of that kernel owns 128 keys and
// walks the query rows; what a padding mask does to it does not change along the way: a key is hidden from every query
// or from none.  Such a key block is a "key mask" block: no tile of its two key tiles is MIXED (so every 32 rows of it are
// the same row, and the first one stands for them), and for each of its keys the bias is +0 in every row or -inf in every
// row.  It then runs the loop of the kernel without bias, with its hidden keys treated like keys that do not exist (their
// probabilities are 0); every other key block runs in the ordinary biased kernel.
//
// The last workgroup writes whether the batch element is a dense one: in more than half of a fixed sample of the map (64
// of its words, evenly spaced; all of them when the map has at most 64) the bias has to be read (MIXED or COLUMN tiles).
template <typename TB>
__global__ __launch_bounds__(256) void attn_bias_summary_kernel(const TB* __restrict__ bias, int64_t sb, int64_t sn, int Tq, int Tk,
                                                                BiasClasses c, uint32_t* __restrict__ info) {
    typedef typename std::conditional<sizeof(TB) == 2, uint16_t, uint32_t>::type Bits;
    constexpr Bits NEG = (Bits)(NegInfBits<TB>::value & (sizeof(TB) == 2 ? 0xFFFFu : 0xFFFFFFFFu));
    __shared__ uint32_t s_and[256], s_or[256], s_any[2], s_open[2];
    __shared__ int s_ok;
    const int tid = threadIdx.x, lane = tid & 63, b = blockIdx.y;
    const int nkb = (Tk + CLS_KEY_BLOCK - 1) / CLS_KEY_BLOCK;
    uint32_t* out = info + b * c.info_sb;
    if ((int)blockIdx.x == nkb) {
        if (tid >= 64) return;
        const int ntiles = (Tk + CLS_KEYS - 1) / CLS_KEYS;
        const int total = c.nrow32 * c.nwords;
        const int i = (int)((int64_t)lane * total / 64);
        const int w = i % c.nwords;
        const int n = min(32, ntiles - 32 * w);  // tiles of that word that exist
        int mixed = cls_count_read(c.words[b * c.sb + i], n), seen = n;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            mixed += __shfl_xor(mixed, off, 64);
            seen += __shfl_xor(seen, off, 64);
        }
        if (lane == 0) out[0] = 2 * mixed > seen ? 1u : 0u;
        return;
    }
    const int kb = blockIdx.x;
    const int rows32 = min((Tq + CLS_ROWS - 1) / CLS_ROWS, c.nrow32);  // rows of the map that hold query rows
    const int tile0 = kb * (CLS_KEY_BLOCK / CLS_KEYS);
    if (tid == 0) s_ok = 1;
    // no MIXED tile in the two columns of the map: every thread looks at some of the rows
    bool ok = true;
    for (int r = tid; r < rows32; r += 256) {
        const uint32_t v = (uint32_t)(c.words[b * c.sb + (int64_t)r * c.nwords + (tile0 >> 5)] >> (2 * (tile0 & 31)));
        ok = ok && (v & 3u) != CLS_MIXED && ((v >> 2) & 3u) != CLS_MIXED;
    }
    // the first row of every 32, for this thread's key: the two halves of the workgroup take every other one
    const int key_local = tid & (CLS_KEY_BLOCK - 1), half = tid >> 7;
    const TB* key_col = bias + b * sb + min(kb * CLS_KEY_BLOCK + key_local, Tk - 1);
    Bits all_and = (Bits)~(Bits)0, all_or = 0;
    for (int r0 = half; r0 < rows32; r0 += 32) {
        Bits v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
            v[i] = __builtin_bit_cast(Bits, key_col[(int64_t)min(min(r0 + 2 * i, rows32 - 1) * CLS_ROWS, Tq - 1) * sn]);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            all_and &= v[i];
            all_or |= v[i];
        }
    }
    s_and[tid] = all_and;
    s_or[tid] = all_or;
    __syncthreads();
    if (!ok) atomicAnd(&s_ok, 0);
    bool hidden = false, good = true;
    if (tid < CLS_KEY_BLOCK) {
        const uint32_t a = s_and[tid] & s_and[tid + CLS_KEY_BLOCK], o = s_or[tid] | s_or[tid + CLS_KEY_BLOCK];
        hidden = a == NEG && o == NEG;
        good = hidden || o == 0;
    }
    const uint64_t hid = __builtin_amdgcn_ballot_w64(hidden);
    if (__builtin_amdgcn_ballot_w64(!good) != 0 && lane == 0) atomicAnd(&s_ok, 0);
    uint32_t* e = out + CLS_INFO_HEAD + kb * CLS_INFO_ENTRY;
    if (tid < CLS_KEY_BLOCK && lane == 0) {
        e[(tid >> 6) * 2] = (uint32_t)hid;
        e[(tid >> 6) * 2 + 1] = (uint32_t)(hid >> 32);
        s_any[tid >> 6] = hid != 0 ? 1u : 0u;        // some key of this half hidden
        s_open[tid >> 6] = hid != ~0ull ? 1u : 0u;   // some key of this half not hidden
    }
    __syncthreads();
    if (tid == 0) {
        const bool any_hidden = (s_any[0] | s_any[1]) != 0, any_open = (s_open[0] | s_open[1]) != 0;
        e[4] = (s_ok != 0 ? CLS_KB_PURE : 0u) | (any_hidden ? CLS_KB_ANY_HIDDEN : 0u) | (!any_open ? CLS_KB_ALL_HIDDEN : 0u);
    }
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
