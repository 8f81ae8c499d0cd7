// Matrix-core disentangled-attention forward for bf16 and fp16, head_dim 64 (gfx950, wave64, MFMA 32x32x16).
//
// One workgroup = one tile of 128 query rows of one (sequence, head), walked over the keys 64 at a
// time.  It has 8 waves in two roles, paired on the SIMDs so that their matrix and vector work
// interleave:
//   * 4 "score" waves, 32 query rows each: S^T = K.Q^T on top of the position terms, streaming
//     softmax, O^T += V^T.P^T.  Scores are kept transposed so that a lane owns ONE query row: row
//     max / row sum are in-lane reductions plus one exchange between the half-waves, and the S^T
//     accumulator registers are already the B operand of the P.V product, so probabilities never
//     touch LDS.  Wave w owns the query rows  row0 + 4n + w  (n = lane & 31): rows are dealt to the
//     waves round robin, which is what makes the c2p ring below addressable with aligned vectors.
//   * 4 "position" waves: they stage the relative-position rows from global memory into LDS and
//     compute, one key step ahead, the position products on the matrix cores.  (K and V are staged
//     by the score waves.)
//
// Position terms, in "position space" (relative position r = i - j; delta(r) comes from the
// host-built table, so log bucketing, saturation beyond max_relative_positions and the un-bucketed
// case are one code path with bit-exact indices).  Key step s covers keys 64s .. 64s+63 and touches
// the window r = B_s .. B_s + 190, B_s = row0 - 64s - 63; rows K_r[delta(r)] and Q_r[delta(r)] of the
// per-head tables for that window live in two 192-row LDS rings (each step fetches the 64 new rows).
//   c2p:  every relative position a query meets is met exactly once, so the products
//         C'[i][r] = Q_i . K_r[delta(r)] are computed once per (query, position): each step the
//         position wave of query block w contracts only the 64 positions that are new to the block
//         (2 MFMA tiles) and files the results, as bf16, under the KEY they belong to (j = i - r) in
//         a per-query ring of 192 key slots.  Because the rows of a wave are 4 apart, four consecutive
//         positions of the MFMA result land on four consecutive keys at a 4-aligned slot for every
//         lane: 8-byte stores going in, and the score wave reads the 8 consecutive keys an MFMA B
//         operand holds with one 16-byte load and adds them to the score accumulators with an MFMA
//         against an identity fragment -- no per-element gather, no unpacking.
//   p2c:  P'^T[r, j] = Q_r[delta(r)] . K_j for the window of the step (10 MFMA tiles: the corners
//         of the window that no (query, key) pair of the tile reaches are skipped), written to LDS
//         as bf16 P'[j][r - B_s] and read back skewed by the score waves: score (i, j) takes
//         P'[j][i - j - B_s], which becomes the initial value of the S^T accumulator.
// Together: S[i,j] = Q_i.K_j + Q_i.K_r[delta(i-j)] + K_j.Q_r[delta(i-j)], the Hugging Face eager
// definition (modeling_deberta_v2.py:317-324, :337-343).
//
// Callers of the reference's own signature hold the position products already, as strips
// c2p[i][x] = Q_i.K_r[x] and p2c[j][x] = K_j.Q_r[x] over all 2*span table rows x.  The strip instances
// keep the score waves as they are and give the position waves a different job: no tables, no
// products -- they gather c2p[i][delta(i-j)] and p2c[j][delta(i-j)] from global memory into the same
// ring and scratch layouts, one key step ahead, between the same barriers.
#include <atomic>
#include <mutex>
#include <type_traits>
#include <utility>

#include "tdb_internal.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define TDB_LDS(T, p) ((__attribute__((address_space(3))) T*)(p))

constexpr int BM = TDB_MFMA_TILE;   // query rows per workgroup
constexpr int BN = 64;              // keys per step
constexpr int D = 64;
constexpr int NTHREADS = 512;       // 4 score waves + 4 position waves
constexpr int WIN = BM + BN;        // ring of staged window rows (one more than the 191 positions in use)
constexpr int RS = 72;              // LDS row stride (elements) of 64-wide 16-bit rows: 144 B, conflict-free b128
constexpr int CRING = 192;          // key slots of the c2p ring of one query row
constexpr int CRS = 200;            // its row stride (elements): 400 B, so that 32 rows read 16 B or write 8 B on distinct banks
constexpr int PS = 196;             // row stride (elements) of the p2c scratch [64 keys][191 positions]
constexpr int RSRC_FLAGS = 0x00020000;   // raw buffer resource, 32-bit data format
// Query tiles that are neighbours along the query axis (they read the same K and V) are kept on ONE XCD at the same
// time, in groups of 2^XG tile ids: 4 in the plain instances (the four tiles of a 512-token sequence), 32 -- every CU
// of an XCD -- in the instances for long sequences, where a (sequence, head) has 12 tiles and more and its keys and
// values (up to megabytes) then stream through that XCD's L2 once instead of once per group of four
// (b4 x L4096: 0.512 -> 0.491 ms).
constexpr int XG_PLAIN = 2, XG_LONG = 5;

struct Smem {
    uint16_t k[2][BN * RS];             // keys of step s live in k[s & 1]
    uint16_t v[BN * RS];
    uint16_t kr[WIN * RS];
    uint16_t qr[WIN * RS];
    uint16_t c[BM * CRS];               // c2p ring: row 32w + n belongs to query row0 + 4n + w, slot = key mod 192
    uint16_t p[BN * PS];
    int seq_n[64], seq_lo[64];          // valid length and first token of the first 64 sequences
    int srt_seq[64];                    // packed: the sequences in order of decreasing length (ties: lower index first)
    int64_t seq_pre[64];                // packed: inclusive prefix sum, in that order, of the sequences' tile counts (all heads)
    int deal_round[NTHREADS / 64];      // packed: how many tiles this workgroup has taken so far, one copy per wave
};

// The two 16-bit element types the kernel is instantiated for: what differs is the MFMA and the float conversion.
// (No dot-product instructions anywhere: v_dot2 runs on the matrix pipe and would queue behind the other role's MFMAs,
// while plain vector instructions run beside them.)  (bf16: fp32's range, 8 significant bits; fp16: 11 bits, range 65504 --
// the position products are stored in the element type, the probabilities are at most 2^8.)
template <int DT>
struct Elem;
template <>
struct Elem<TDB_BF16> {
    using T = __bf16;
    using X2 = bf16x2;
    using X8 = bf16x8;
    static __device__ __forceinline__ f32x16 mfma(X8 a, X8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
    // One half of a dword as fp32 through a byte permute (the selector says which half): bf16 -> fp32 is a shift.
    static constexpr uint32_t PICK_LO = 0x05040c0cu, PICK_HI = 0x07060c0cu;
    static __device__ __forceinline__ float pick(uint32_t pair, uint32_t sel) {
        return __builtin_bit_cast(float, __builtin_amdgcn_perm(pair, 0u, sel));
    }
};
template <>
struct Elem<TDB_F16> {
    using T = _Float16;
    using X2 = f16x2;
    using X8 = f16x8;
    static __device__ __forceinline__ f32x16 mfma(X8 a, X8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
    static constexpr uint32_t PICK_LO = 0x0c0c0504u, PICK_HI = 0x0c0c0706u;
    static __device__ __forceinline__ float pick(uint32_t pair, uint32_t sel) {
        return (float)__builtin_bit_cast(X2, __builtin_amdgcn_perm(pair, 0u, sel))[0];
    }
};

template <typename X8>
__device__ __forceinline__ X8 lds_frag(const uint16_t* row_base, int row, int col) {
    return *reinterpret_cast<const X8*>(row_base + row * RS + col);
}

template <typename E>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typename E::X2 v = {(typename E::T)lo, (typename E::T)hi};
    return __builtin_bit_cast(uint32_t, v);
}

// Workgroup barrier that instruction scheduling may not move anything across either: register-only work (MFMAs,
// address arithmetic) stays in the pipeline half it was written in.
__device__ __forceinline__ void phase_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
}

// Template parameters: which position terms exist, the element type, whether far key steps are looked for, the
// layout (VARLEN: packed sequences) and the form of the position terms (STRIP: the caller's strips, not tables).  The layout is a compile-time fact because the tile bookkeeping of the two layouts
// has nothing in common: with both compiled into one instance, the unused one still cost scalar registers (spilled
// into vector lanes and reloaded in the step loops) and several hundred scalar instructions per tile.
template <bool HAS_C2P, bool HAS_P2C, int DT, bool FARZ, bool VARLEN, bool STRIP = false>
__global__ __launch_bounds__(NTHREADS) void attn_mfma_kernel(const TdbKernelParams p, const int nblocks) {
    static_assert(!(STRIP && FARZ), "the strip instances have no far steps");
    using E = Elem<DT>;
    using ET = typename E::T;
    using X2 = typename E::X2;
    using X8 = typename E::X8;
    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    Smem& sm = *reinterpret_cast<Smem*>(smem_raw);
    constexpr bool HAS_POS = HAS_C2P || HAS_P2C;
    // The packed instances also take right-padded batches of a fixed layout (lengths in p.seqlens, no cu_seqlens): the
    // tiles are dealt like those of packed sequences, the rows are addressed through the batch strides.
    const bool packed_rows = VARLEN && !p.seqlens;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool score_role = wave < 4;     // waves 0..3 score, 4..7 position; wave w and w+4 share query block w
    const int w = wave & 3, l = tid & 63;
    const int il = l & 31, hh = l >> 5;

    // ---- tiles --------------------------------------------------------------------------------------------------
    // The workgroup is persistent: the launch has one workgroup per CU (LDS admits no second one), and workgroup g
    // takes the virtual blocks g, g + gridDim.x, ...  While the last key step of a tile runs, the first LDS stage of
    // the next tile is already on its way from global memory, so that the chain of dependent global reads that
    // starts a tile (sequence length -> delta table -> rows) is only exposed once per workgroup.
    // Virtual block -> (tile, head): consecutive ids go round-robin over the 8 XCDs, each with its own L2; ids are
    // regrouped so that G tiles that are neighbours along the query axis -- the tiles that read the same K
    // and V -- run on one XCD and fetch K / V from HBM once instead of once each.
    const int tiles_x = VARLEN ? p.total / BM + p.B : p.B * ((p.L + BM - 1) / BM);
    const int lut_max = 2 * p.lut_half;
    auto delta_of = [&](int r) { return p.lut[min(max(r + p.lut_half, 0), lut_max)]; };

    struct Tile {
        int vb, head, b, row0, len;       // vb < 0: no tile
        int64_t tok0;
    };
    auto tile_index = [&](int vb, int& hd, int& tile_id) {   // false: the virtual block has no tile
        const int xcd = vb & 7, slot = vb >> 3;
        constexpr int G = 1 << (FARZ ? XG_LONG : XG_PLAIN);
        const int v = ((slot / G) * 8 + xcd) * G + slot % G;
        if (vb >= nblocks || v >= tiles_x * p.H) return false;
        hd = v / tiles_x;
        tile_id = v - hd * tiles_x;
        return true;
    };
    // The lengths (fixed layout) or boundaries (packed) of the first 64 sequences sit in LDS, so that looking a tile
    // up reads nothing from global memory for batches of up to 64 sequences and keeps no register between lookups.
    // Every wave writes the same values (lane l: sequence l) and reads them back itself: no barrier is needed.
    auto lds_int = [&](const int* q) { return __builtin_amdgcn_readfirstlane(*q); };
    auto lds_i64 = [&](const int64_t* q) {
        const int64_t v = *q;
        const int lo = __builtin_amdgcn_readfirstlane(int(uint32_t(uint64_t(v))));
        const int hi = __builtin_amdgcn_readfirstlane(int(uint32_t(uint64_t(v) >> 32)));
        return int64_t((uint64_t(uint32_t(hi)) << 32) | uint32_t(lo));
    };
    auto tiles_of = [](int n) { return (n + BM - 1) / BM; };
    // Packed launches (at most 64 sequences: the launcher splits larger batches) deal their tiles by cost instead of
    // the strided walk of the fixed layout: a tile costs about 3 key steps plus one per 64 keys of its sequence, so
    // tiles differ by up to 3x.  The tiles are listed by decreasing length of their sequence (then head, then query
    // tile) and dealt to the G workgroups back and forth: round j hands tiles j*G .. j*G+G-1 out in ascending order
    // of the workgroup number when j is even, in descending order when it is odd, so that whoever got the costlier
    // tile of one round gets the cheaper one of the next, and the last, incomplete round -- the cheapest tiles --
    // goes to the workgroups that have the least so far.  Every workgroup derives its own tiles from the sequence
    // boundaries alone (a rank per sequence, a prefix sum of tile counts in rank order, one search per tile); nothing
    // is shared between workgroups.  (64 sequences of 16..512 tokens: the most loaded workgroup carries 1.04-1.07x
    // the mean; contiguous cost-balanced ranges of the unsorted list, the earlier scheme, 1.11x and a 10 % longer
    // launch.)  Workgroups are numbered for the deal so that neighbours sit on ONE XCD (block ids go round-robin
    // over the 8 XCDs): the query tiles of one (sequence, head), neighbours in the list, then run at the same time
    // on CUs that share an L2 and read K and V from HBM once, not once per tile.  The round counter lives in LDS,
    // one copy per wave: it is touched once per tile and would otherwise occupy a register all through the key steps.
    constexpr bool balanced = VARLEN;
    {
        int n = p.L, lo = 0;
        if (VARLEN && p.seqlens) {
            // right-padded sequences of a fixed layout, dealt like packed ones (the launcher sends such calls here)
            n = l < p.B ? min(max(p.seqlens[min(l, p.B - 1)], 0), p.L) : 0;
        } else if (VARLEN) {
            lo = p.cu_seqlens[min(l, p.B)];
            const int hi = p.cu_seqlens[min(l + 1, p.B)];
            n = hi - lo;
            if (l >= p.B || lo < 0 || n < 0 || hi > p.total) n = 0;      // malformed entry: no tiles
            n = min(n, p.L);
        } else if (p.seqlens) {
            n = min(max(p.seqlens[min(l, p.B - 1)], 0), p.L);
        }
        sm.seq_n[l] = n;
        if (VARLEN) {                     // (the fixed layout's walk needs the lengths only)
            sm.seq_lo[l] = lo;
            // Rank of this lane's sequence by decreasing length (ties: lower index first); the sequence and the tile
            // count (all heads) that belong at rank l travel to lane l inside the wave, and the tile counts become an
            // inclusive prefix sum in that order.  (All eight waves write the same final values into the shared
            // arrays and each reads back what it wrote itself; nothing intermediate goes through them -- a second
            // wave could be anywhere in this sequence.)
            int rank = 0;
            for (int b2 = 0; b2 < 64; ++b2) {
                const int n2 = sm.seq_n[b2];
                rank += (n2 > n || (n2 == n && b2 < l)) ? 1 : 0;
            }
            const int seq_here = __builtin_amdgcn_ds_permute(rank * 4, l);
            int64_t cnt = int64_t(__builtin_amdgcn_ds_permute(rank * 4, tiles_of(n))) * p.H;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int64_t up = __shfl_up(cnt, d);
                if (l >= d) cnt += up;
            }
            sm.srt_seq[l] = seq_here;
            sm.seq_pre[l] = cnt;
        }
    }
    // fixed layout: tile_id -> (sequence, first row, valid length); same map as tdb_locate_tile
    auto locate = [&](int tile_id, int& bb, int& r0, int& ln, int64_t& t0) {
        const int tiles = (p.L + BM - 1) / BM;
        bb = tile_id / tiles;
        r0 = (tile_id - bb * tiles) * BM;
        ln = !p.seqlens ? p.L : bb < 64 ? lds_int(&sm.seq_n[bb]) : min(max(p.seqlens[bb], 0), p.L);
        t0 = 0;
        return true;
    };
    auto no_tile = []() {
        Tile t;
        t.vb = -1;
        t.head = t.b = t.row0 = t.len = 0;
        t.tok0 = 0;
        return t;
    };
    // Tile j of this workgroup in the back-and-forth deal (gridDim.x is a multiple of 8).
    auto dealt_tile = [&](int j) {
        const int64_t G = gridDim.x, g = int64_t(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
        const int64_t k = int64_t(j) * G + ((j & 1) ? G - 1 - g : g);
        Tile t = no_tile();
        if (k >= lds_i64(&sm.seq_pre[63])) return t;
        const unsigned long long owners = __builtin_amdgcn_ballot_w64(sm.seq_pre[l] > k);
        const int r = __builtin_amdgcn_readfirstlane(__builtin_ctzll(owners));
        t.b = lds_int(&sm.srt_seq[r]);
        t.len = lds_int(&sm.seq_n[t.b]);
        t.tok0 = lds_int(&sm.seq_lo[t.b]);
        const int per_head = tiles_of(t.len);
        if (owners == 0 || per_head <= 0) return no_tile();
        const int within = int(k - (lds_i64(&sm.seq_pre[r]) - int64_t(per_head) * p.H));
        t.head = within / per_head;
        t.row0 = (within - t.head * per_head) * BM;
        t.vb = (within >= 0 && t.head < p.H) ? 0 : -1;     // (always true for a consistent prefix: no tile rather than a stray address)
        return t;
    };
    auto take = [&]() {
        const int j = lds_int(&sm.deal_round[wave]) + 1;
        sm.deal_round[wave] = j;
        return dealt_tile(j);
    };
    auto first_balanced = [&]() {
        sm.deal_round[wave] = 0;
        return dealt_tile(0);
    };
    // First tile with live query rows among the virtual blocks vb, vb + gridDim.x, ...; vb = -1 if there is none.
    // Tiles that hold only padded query rows (fixed layout) get their zeros here, from whoever looks them up:
    // every wave of the workgroup walks the same list, each thread fills its share.
    auto find_tile = [&](int vb) {
        Tile t;
        t.vb = -1;
        t.head = t.b = t.row0 = t.len = 0;
        t.tok0 = 0;
        for (; vb < nblocks; vb += gridDim.x) {
            int hd, tile_id;
            if (!tile_index(vb, hd, tile_id)) continue;
            int bb, r0, ln;
            int64_t t0;
            if (!locate(tile_id, bb, r0, ln, t0)) continue;
            if (r0 >= ln) {
                uint16_t* Oz = static_cast<uint16_t*>(p.o) + (VARLEN ? t0 * p.os_l : int64_t(bb) * p.os_b) + int64_t(hd) * p.os_h;
                const int rows = min(BM, (VARLEN ? ln : p.L) - r0);
                for (int idx = tid; idx < rows * (D / 8); idx += NTHREADS)
                    *reinterpret_cast<u32x4*>(Oz + int64_t(r0 + (idx >> 3)) * p.os_l + (idx & 7) * 8) = u32x4{0, 0, 0, 0};
                continue;
            }
            t.vb = vb;
            t.head = hd;
            t.b = bb;
            t.row0 = r0;
            t.len = ln;
            t.tok0 = t0;
            break;
        }
        return t;
    };
    auto k_of = [&](const Tile& t) {
        return static_cast<const uint16_t*>(p.k) + (packed_rows ? t.tok0 * p.ks_l : int64_t(t.b) * p.ks_b) + int64_t(t.head) * p.ks_h;
    };
    auto pk_of = [&](const Tile& t) { return HAS_C2P && !STRIP ? static_cast<const uint16_t*>(p.pk) + int64_t(t.head) * p.pks_h : nullptr; };
    auto pq_of = [&](const Tile& t) { return HAS_P2C && !STRIP ? static_cast<const uint16_t*>(p.pq) + int64_t(t.head) * p.pqs_h : nullptr; };

    auto next_tile = [&](const Tile& t) {
        if constexpr (balanced) return take();
        else return find_tile(t.vb + gridDim.x);
    };
    // A key step is "far" when its whole window of relative positions maps to ONE table row (delta is monotone in r, so
    // its two ends decide): beyond max_relative_positions on either side, which is most of a long sequence.  Then the
    // c2p term is one value per query and the p2c term one value per key, and the step needs no window products, no
    // ring and no scratch.  Step t of the tile that starts at query row r0: window r0 - 64t - 63 .. + 190.
    auto far_at = [&](int r0, int t) {
        if (!HAS_POS || !FARZ) return false;
        const int b = r0 - BN * t - (BN - 1);
        return delta_of(b) == delta_of(b + WIN - 2);
    };

    if (VARLEN && p.seqlens) {
        // The deal only lists tiles with valid query rows; tiles that hold padded rows alone get their zeros here,
        // shared out over the workgroups (every thread fills its share of a tile's rows).
        const int per_seq = (p.L + BM - 1) / BM;
        for (int idx = blockIdx.x; idx < p.B * p.H * per_seq; idx += gridDim.x) {
            const int bb = idx / (p.H * per_seq), rem = idx - bb * (p.H * per_seq);
            const int hd = rem / per_seq, r0 = (rem - hd * per_seq) * BM;
            if (r0 < lds_int(&sm.seq_n[bb])) continue;
            uint16_t* Oz = static_cast<uint16_t*>(p.o) + int64_t(bb) * p.os_b + int64_t(hd) * p.os_h;
            const int rows = min(BM, p.L - r0);
            for (int i2 = tid; i2 < rows * (D / 8); i2 += NTHREADS)
                *reinterpret_cast<u32x4*>(Oz + int64_t(r0 + (i2 >> 3)) * p.os_l + (i2 & 7) * 8) = u32x4{0, 0, 0, 0};
        }
    }
    Tile cur;
    if constexpr (balanced) cur = first_balanced();
    else cur = find_tile(blockIdx.x);
    if (cur.vb < 0) return;

    // ---- pipeline of one tile -----------------------------------------------------------------------------------
    // Key step s covers keys 64s .. 64s+63 and needs relative positions B_s .. B_s+190, B_s = row0 - 64s - 63.
    // The rows K_r[delta(r)] / Q_r[delta(r)] of that window live in a 192-row ring: going to the next step the
    // window slides down by 64, so only its 64 lowest positions are fetched and they overwrite the 64 highest
    // of the previous step.  Window row x of step s sits in ring slot (x + off_s) mod 192, off_s = (128*s) mod 192.
    // The 64 + 3 lowest rows of the window are exactly the positions that are new to the four query blocks
    // (block w: window rows w .. w+63), i.e. what the c2p products of the step contract.
    //
    // A tile opens with its first stage in LDS (written during the last step of the tile before; for the first tile of
    // the workgroup by all threads) and two barriers: position products of step 0 in LDS; window of step 1
    // complete.  Then each step has two halves separated by workgroup barriers, arranged so that in either half one
    // role leans on the LDS and the other on the matrix cores:
    //   A  score waves read this step's position terms (c2p ring fragments, P' scratch), hand register-prefetched
    //      keys (step s+2) and values (step s) to LDS, run the S^T(s) MFMAs on top of the position terms and pick up
    //      the K fragments of step s+1; position waves run the position MFMAs of step s+1 on fragments they already
    //      hold, then store the 64 new window rows of step s+2 and request those of step s+3;
    //   B  score waves: softmax(s), P.V(s), and they request keys and values for the next half A; position waves:
    //      results of step s+1 into the ring and the now free scratch, LDS fragments of step s+2.
    // Both roles pass 2 + 2*nsteps barriers per tile (the barrier that ends the last step is also the one after which
    // the next tile's first stage is visible) and walk the same tile list.
    //
    // c2p ring bookkeeping.  "Batch" t is the set of positions new at step t: for block w, r = row0 + w - 64t - 63 + m,
    // m = 0..63; lane n of the block (query row0 + 4n + w) meets them at keys 64t + 63 + 4n - m.  A tile opens with
    // batches -2, -1, 0 (together the 188 positions step 0 needs; the part that falls on negative keys lands in slots
    // that their proper batch rewrites before anybody reads them).  Batch t+1 is written in half B of step t, after the
    // score waves have read the keys of step t; the slots it overwrites held keys below 64(t+1).
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    auto prev_off = [](int o) { return o >= BN ? o - BN : o + WIN - BN; };   // ring offset of the following step

    // state of the current tile, rebound when the workgroup moves on
    int row0 = 0, len = 0, nsteps = 0, nfull = 0, rows_here = 0;
    const uint16_t *Q = nullptr, *K = nullptr, *V = nullptr, *PK = nullptr, *PQ = nullptr;
    uint16_t* O = nullptr;
    auto bind = [&](const Tile& t) {
        row0 = t.row0;
        len = t.len;
        nsteps = (len + BN - 1) / BN;
        nfull = len / BN;                 // steps that need no key mask
        rows_here = min(BM, (packed_rows ? len : p.L) - row0);   // rows of this tile that exist in memory
        Q = static_cast<const uint16_t*>(p.q) + (packed_rows ? t.tok0 * p.qs_l : int64_t(t.b) * p.qs_b) + int64_t(t.head) * p.qs_h;
        K = k_of(t);
        V = static_cast<const uint16_t*>(p.v) + (packed_rows ? t.tok0 * p.vs_l : int64_t(t.b) * p.vs_b) + int64_t(t.head) * p.vs_h;
        O = static_cast<uint16_t*>(p.o) + (packed_rows ? t.tok0 * p.os_l : int64_t(t.b) * p.os_b) + int64_t(t.head) * p.os_h;
        PK = pk_of(t);
        PQ = pq_of(t);
    };
    bind(cur);

    // Q^T fragments of query block w: B operand of S^T = K.Q^T (score wave) and of C'^T = K_r'.Q^T (position wave)
    X8 qb[4];
    auto load_q = [&](X8 (&dst)[4], const Tile& t) {
        const uint16_t* Qt = static_cast<const uint16_t*>(p.q) + (packed_rows ? t.tok0 * p.qs_l : int64_t(t.b) * p.qs_b) + int64_t(t.head) * p.qs_h;
        const int qrow = t.row0 + 4 * il + w;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            u32x4 x = {0, 0, 0, 0};
            if (t.vb >= 0 && qrow < t.len) x = *reinterpret_cast<const u32x4*>(Qt + int64_t(qrow) * p.qs_l + 16 * c + 8 * hh);
            dst[c] = __builtin_bit_cast(X8, x);
        }
    };
    load_q(qb, cur);

    // First tile of the workgroup: nothing was requested ahead, so all 512 threads share its first LDS stage (keys of
    // steps 0 and 1, the whole window of step 0: 8 chunks of 16 B per thread) and the chain of dependent reads
    // (delta table -> rows) is as short as it can be.  Later tiles are staged by the position waves alone, with
    // reads issued a key step ahead.
    int dl_cold[3][2] = {{0, 0}, {0, 0}, {0, 0}};   // position waves: delta of the new window rows of steps 1 to 3
    {
        const int row = tid >> 3, ch = tid & 7;     // rows 0..63
        int dl[WIN / 64] = {0, 0, 0};
        if (HAS_POS && !STRIP) {
#pragma unroll
            for (int n = 0; n < WIN / 64; ++n) dl[n] = delta_of(row0 - (BN - 1) + row + 64 * n);
            if (!score_role) {
#pragma unroll
                for (int s1 = 0; s1 < 3; ++s1)
#pragma unroll
                    for (int n = 0; n < 2; ++n)
                        dl_cold[s1][n] = delta_of(row0 - BN * (s1 + 1) - (BN - 1) + ((tid - 256) >> 3) + 32 * n);
            }
        }
        const u32x4 k0 = *reinterpret_cast<const u32x4*>(K + int64_t(min(row, len - 1)) * p.ks_l + ch * 8);
        const u32x4 k1 = *reinterpret_cast<const u32x4*>(K + int64_t(min(BN + row, len - 1)) * p.ks_l + ch * 8);
        u32x4 wk[WIN / 64], wq[WIN / 64];
#pragma unroll
        for (int n = 0; n < WIN / 64; ++n) {
            if (HAS_C2P && !STRIP) wk[n] = *reinterpret_cast<const u32x4*>(PK + int64_t(dl[n]) * p.pks_r + ch * 8);
            if (HAS_P2C && !STRIP) wq[n] = *reinterpret_cast<const u32x4*>(PQ + int64_t(dl[n]) * p.pqs_r + ch * 8);
        }
        *reinterpret_cast<u32x4*>(&sm.k[0][row * RS + ch * 8]) = k0;
        *reinterpret_cast<u32x4*>(&sm.k[1][row * RS + ch * 8]) = k1;
#pragma unroll
        for (int n = 0; n < WIN / 64; ++n) {
            if (HAS_C2P && !STRIP) *reinterpret_cast<u32x4*>(&sm.kr[(row + 64 * n) * RS + ch * 8]) = wk[n];
            if (HAS_P2C && !STRIP) *reinterpret_cast<u32x4*>(&sm.qr[(row + 64 * n) * RS + ch * 8]) = wq[n];
        }
    }

    if constexpr (STRIP) {
        if (!score_role) {
            // ============================== position waves, strip instances =======================================
            // The caller has the position terms as strips: c2p[i][delta] = Q_i.K_r[delta] per query row, p2c[j][delta] =
            // K_j.Q_r[delta] per key row.  These waves only move them: for key step s they gather
            //   ring[query i][key j mod 192] = c2p[i][delta(i - j)]     (128 queries x 64 keys), and
            //   P'[key jl][x]               = p2c[j][delta(r_x)],  r_x = row0 - 64s + x - 63  (x = i - jl + 63, 128 per key)
            // into the same LDS layouts the score waves read in the table instances, with the same barriers.  A lane is
            // a key (c2p) or a window position x (p2c), so a load reads neighbouring columns of one strip row.  Rows
            // past the end of the sequence read as zeros (buffer range check); the column comes from the delta table,
            // whose values lie in [0, 2*span).
            const int stid = tid - 256, srow = stid >> 3, sch = stid & 7;
            const int c2s_bytes = int(p.c2s_l) * 2, p2s_bytes = int(p.p2s_l) * 2;
            __amdgpu_buffer_rsrc_t c_rsrc, p_rsrc;
            auto bind_strips = [&](const Tile& t) {
                const uint16_t* cbase = HAS_C2P ? static_cast<const uint16_t*>(p.c2p) + (packed_rows ? t.tok0 * p.c2s_l : int64_t(t.b) * p.c2s_b) + int64_t(t.head) * p.c2s_h
                                                : k_of(t);
                const uint16_t* pbase = HAS_P2C ? static_cast<const uint16_t*>(p.p2c) + (packed_rows ? t.tok0 * p.p2s_l : int64_t(t.b) * p.p2s_b) + int64_t(t.head) * p.p2s_h
                                                : k_of(t);
                const bool any = t.vb >= 0 && t.len > 0;
                c_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(cbase), 0, HAS_C2P && any ? (t.len - 1) * c2s_bytes + 4 * p.span : 0, RSRC_FLAGS);
                p_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(pbase), 0, HAS_P2C && any ? (t.len - 1) * p2s_bytes + 4 * p.span : 0, RSRC_FLAGS);
            };
            uint16_t cv[32], pv[32];
            // c2p of key step s of the tile at query row r0: this wave takes queries r0 + 32w + t, lane l is key 64s + l
            auto gather_c = [&](int r0, int s) {
                if (HAS_C2P) {
                    // Column of (query q0 + t, lane l): delta(q0 + t - 64s - l).  Going from one query to the next every
                    // lane takes over the column of its lower neighbour (a shift of the whole wave by one lane) and
                    // lane 0 takes delta(q0 + t + 1 - 64s), which lane t of `ahead` has held since before the loop: two
                    // reads of the delta table per step and wave instead of one per element.
                    const int q0 = r0 + 32 * w;
                    int d = delta_of(q0 - BN * s - l);
                    const int ahead = delta_of(q0 + 1 + l - BN * s);
#pragma unroll
                    for (int t = 0; t < 32; ++t) {
                        cv[t] = uint16_t(__builtin_amdgcn_raw_buffer_load_b16(c_rsrc, (q0 + t) * c2s_bytes + 2 * d, 0, 0));
                        if (t < 31) d = __builtin_amdgcn_update_dpp(__builtin_amdgcn_readlane(ahead, t), d, 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
                    }
                }
            };
            // ring row of tile row 4n + ws is 32 ws + n; the slots of step s start at (64 s) mod 192
            auto write_c = [&](int phase) {
                if (HAS_C2P) {
#pragma unroll
                    for (int t = 0; t < 32; ++t) sm.c[(32 * (t & 3) + 8 * w + (t >> 2)) * CRS + phase + l] = cv[t];
                }
            };
            // p2c of key step s: this wave takes keys 64s + 16w + u; per key one load for x = 64 + l and one for
            // x = l (lanes l >= 63 - jl) or x = 128 + l (the others) -- together the 128 positions the key is read at
            auto gather_p = [&](int r0, int s) {
                if (HAS_P2C) {
                    int dx[3];
#pragma unroll
                    for (int c = 0; c < 3; ++c) dx[c] = 2 * delta_of(r0 - BN * s - (BN - 1) + 64 * c + l);
#pragma unroll
                    for (int u = 0; u < 16; ++u) {
                        const int jl = 16 * w + u;
                        const int rowoff = (BN * s + jl) * p2s_bytes;
                        const int dsel = l + jl >= BN - 1 ? dx[0] : dx[2];
                        pv[2 * u] = uint16_t(__builtin_amdgcn_raw_buffer_load_b16(p_rsrc, rowoff + dsel, 0, 0));
                        pv[2 * u + 1] = uint16_t(__builtin_amdgcn_raw_buffer_load_b16(p_rsrc, rowoff + dx[1], 0, 0));
                    }
                }
            };
            auto write_p = [&]() {
                if (HAS_P2C) {
#pragma unroll
                    for (int u = 0; u < 16; ++u) {
                        const int jl = 16 * w + u;
                        sm.p[jl * PS + (l + jl >= BN - 1 ? l : 2 * BN + l)] = pv[2 * u];
                        sm.p[jl * PS + BN + l] = pv[2 * u + 1];
                    }
                }
            };
            auto next_phase = [](int ph) { return ph == 2 * BN ? 0 : ph + BN; };
            bind_strips(cur);
            gather_c(cur.row0, 0);
            gather_p(cur.row0, 0);
            phase_barrier();              // first stage of the first tile is in LDS
            while (true) {
                write_c(0);               // position terms of step 0 (gathered during the last step of the tile before)
                write_p();
                phase_barrier();          // the two opening barriers of the table instances
                phase_barrier();
                const Tile nxt = next_tile(cur);
                int phase = BN;
                for (int s = 0; s + 1 < nsteps; ++s) {
                    phase_barrier();      // position terms of step s complete
                    gather_c(row0, s + 1);
                    gather_p(row0, s + 1);
                    write_c(phase);       // (these ring slots were last read three steps ago)
                    phase_barrier();      // the score waves are done with the scratch
                    write_p();
                    phase = next_phase(phase);
                }
                // Last key step: the next tile moves in -- its keys of steps 0 and 1 into both key buffers, its first
                // position terms into registers (they go to LDS once the score waves have read this step's).
                phase_barrier();
                {
                    const uint16_t* Kt = k_of(nxt);
                    u32x4 st_k[4];
#pragma unroll
                    for (int n = 0; n < 4; ++n) {
                        st_k[n] = u32x4{0, 0, 0, 0};
                        if (nxt.vb >= 0) st_k[n] = *reinterpret_cast<const u32x4*>(Kt + int64_t(min(srow + 32 * n, nxt.len - 1)) * p.ks_l + sch * 8);
                    }
                    if (nxt.vb >= 0) {
                        bind_strips(nxt);
                        gather_c(nxt.row0, 0);
                        gather_p(nxt.row0, 0);
#pragma unroll
                        for (int n = 0; n < 4; ++n)
                            *reinterpret_cast<u32x4*>(&sm.k[n >> 1][(srow + 32 * (n & 1)) * RS + sch * 8]) = st_k[n];
                    }
                }
                phase_barrier();
                if (nxt.vb < 0) break;
                cur = nxt;
                bind(cur);
            }
            return;
        }
    }

    if (!STRIP && !score_role) {
        // ================================================= position waves ==========================================
        const int stid = tid - 256;
        const int srow = stid >> 3, sch = stid & 7;          // this thread stages rows srow + 32n (chunk sch)
        // (The instance with far steps has no registers left for address terms hoisted out of the step loop: there the
        // lane coordinates are taken through `fresh`, which the optimiser cannot see through, so that the few
        // instructions of an address are redone at each use instead of living in registers that end up in scratch
        // memory -- a reload inside the loop waits for every outstanding prefetch as well.)
        auto fresh = [](int x) {
            if (FARZ) asm volatile("" : "+v"(x));
            return x;
        };
        // global -> registers through buffer loads.  The buffer of a step starts at its first row and ends with the
        // last row of the sequence, so rows past the end come back as zeros (hardware range check) with no lane
        // predicated off, and the per-load address arithmetic is scalar.
        const int pks_b = int(p.pks_r) * 2, pqs_b = int(p.pqs_r) * 2;
        __amdgpu_buffer_rsrc_t pk_rsrc, pq_rsrc;
        auto bind_tables = [&]() {
            pk_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(HAS_C2P ? PK : K), 0,
                                                        HAS_C2P ? (2 * p.span - 1) * pks_b + 128 : 0, RSRC_FLAGS);
            pq_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(HAS_P2C ? PQ : K), 0,
                                                        HAS_P2C ? (2 * p.span - 1) * pqs_b + 128 : 0, RSRC_FLAGS);
        };
        u32x4 pre_kr[2], pre_qr[2];
        int dl_next[2] = {0, 0};
        auto fetch = [&]() {                   // the 64 new window rows of a step (dl_next)
#pragma unroll
            for (int n = 0; n < 2; ++n) {
                if (HAS_C2P) pre_kr[n] = __builtin_amdgcn_raw_buffer_load_b128(pk_rsrc, dl_next[n] * pks_b + sch * 16, 0, 0);
                if (HAS_P2C) pre_qr[n] = __builtin_amdgcn_raw_buffer_load_b128(pq_rsrc, dl_next[n] * pqs_b + sch * 16, 0, 0);
            }
        };
        // delta of the 64 new window rows of key step s: relative positions row0 - 64s - 63 + srow (+ 32).  Read through
        // a buffer over the table: positions outside it (they belong to keys or queries that do not exist) read as 0,
        // a valid row, with no clamping arithmetic.
        const __amdgpu_buffer_rsrc_t lut_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(p.lut), 0, (lut_max + 1) * 4, RSRC_FLAGS);
        const int srow4 = srow * 4;
        auto fetch_delta = [&](int s) {
            if (HAS_POS) {
                const int off = srow4 + (row0 - BN * s - (BN - 1) + p.lut_half) * 4;
                dl_next[0] = __builtin_amdgcn_raw_buffer_load_b32(lut_rsrc, off, 0, 0);
                dl_next[1] = __builtin_amdgcn_raw_buffer_load_b32(lut_rsrc, off + 128, 0, 0);
            }
        };
        const int stage_el = srow * RS + sch * 8;
        auto store = [&](int o) {              // registers -> LDS: window rows at ring offset o
            const int el = stage_el + o * RS;  // (o is wave-uniform: one vector add, the row inside the step is an immediate)
#pragma unroll
            for (int n = 0; n < 2; ++n) {
                const int at = el + 32 * n * RS;
                if (HAS_C2P) *reinterpret_cast<u32x4*>(&sm.kr[at]) = pre_kr[n];
                if (HAS_P2C) *reinterpret_cast<u32x4*>(&sm.qr[at]) = pre_qr[n];
            }
        };
        // Position products of one key step, in three stages that the pipeline places in different halves:
        //   load_frags   MFMA operands out of LDS: for c2p the K_r' rows of window rows xb + 32 rt + m (xb = w: the
        //                64 positions new to query block w; the tiles are not aligned to the 32-row ring tiles, so each
        //                lane wraps its own row); for p2c the Q_r' rows of window tile w + 1 and, for waves 0 and 1,
        //                of tiles 0 and 5, and both key tiles (kb);
        //   products     c2p  C'^T[r, i] = K_r'[r].Q_i  (2 tiles),  p2c  P'^T[r, j] = Q_r'[r].K_j  (wave w: tile w + 1
        //                against both key tiles; wave 0: tile 0 against keys 32..63; wave 1: tile 5 against keys
        //                0..31; the other two corners of the window are never read) -- results packed to 16 bits;
        //   put_results  c2p into the ring (8-byte stores at 4-aligned key slots), p2c as P'[j][r''] into the scratch.
        X8 fr[2][4], fq[2][4], kb[2][4];
        u32x2 cpk[2][4], ppk[3][4];
        const int lane_col = il * RS + 8 * hh;
        auto load_fr = [&](int o, int xb) {
            if (HAS_C2P) {
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) {
                    int slot = min(xb + 32 * rt + il, WIN - 1) + o;     // rows past the window: any row will do (negative keys)
                    slot = slot >= WIN ? slot - WIN : slot;
                    const uint16_t* base = sm.kr + slot * RS + 8 * hh;
#pragma unroll
                    for (int c = 0; c < 4; ++c) fr[rt][c] = *reinterpret_cast<const X8*>(base + 16 * c);
                }
            }
        };
        auto load_fp = [&](int o, int kbuf) {
            // Window tiles are 32 rows and the ring offset is a multiple of 32, so a tile never straddles the wrap: the
            // ring slot of a tile is scalar arithmetic, the lane only adds its row inside the tile.
            auto ring_tile = [&](int t) { const int u = t + (o >> 5); return 32 * (u >= WIN / 32 ? u - WIN / 32 : u); };
            if (HAS_P2C) {
                const uint16_t* base3 = sm.qr + ring_tile(w + 1) * RS;
                const uint16_t* base4 = sm.qr + ring_tile(w == 1 ? 5 : 0) * RS;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    fq[0][c] = *reinterpret_cast<const X8*>(base3 + lane_col + 16 * c);
                    if (w < 2) fq[1][c] = *reinterpret_cast<const X8*>(base4 + lane_col + 16 * c);
                    kb[0][c] = lds_frag<X8>(sm.k[kbuf], il, 16 * c + 8 * hh);
                    kb[1][c] = lds_frag<X8>(sm.k[kbuf], 32 + il, 16 * c + 8 * hh);
                }
            }
        };
        auto chain = [&](const X8 (&a)[4], const X8 (&bb)[4]) {
            f32x16 acc = E::mfma(a[0], bb[0], zero16);
#pragma unroll
            for (int c = 1; c < 4; ++c) acc = E::mfma(a[c], bb[c], acc);
            return acc;
        };
        // c2p results, key order: register 4a + t of a tile holds position row 8a + 4hh + t, i.e. key k0 - t; the four
        // keys k0-3 .. k0 of a group go out together, lowest key first.
        auto pack_c = [&](const f32x16& acc, u32x2 (&out)[4]) {
#pragma unroll
            for (int a = 0; a < 4; ++a)
                out[a] = u32x2{pack2<E>(acc[4 * a + 3], acc[4 * a + 2]), pack2<E>(acc[4 * a + 1], acc[4 * a])};
        };
        auto pack_p = [&](const f32x16& acc, u32x2 (&out)[4]) {
#pragma unroll
            for (int a = 0; a < 4; ++a)
                out[a] = u32x2{pack2<E>(acc[4 * a], acc[4 * a + 1]), pack2<E>(acc[4 * a + 2], acc[4 * a + 3])};
        };
        auto products_c = [&]() {
            if (HAS_C2P) {
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) pack_c(chain(fr[rt], qb), cpk[rt]);
            }
        };
        auto products_p = [&]() {
            if (HAS_P2C) {
                pack_p(chain(fq[0], kb[0]), ppk[0]);
                pack_p(chain(fq[0], kb[1]), ppk[1]);
                if (w == 0) pack_p(chain(fq[1], kb[1]), ppk[2]);        // wave-uniform branches, no register copies
                else if (w == 1) pack_p(chain(fq[1], kb[0]), ppk[2]);
            }
        };
        // Far step: every window row is the same table row, so any fragment tile will do.  Row 0 of K_r'.Q^T is the one
        // c2p value of each query and row 0 of Q_r'.K^T the one p2c value of each key (position waves 0 and 1 take one key
        // tile each); register 0 of the lower half-wave holds row 0.  Both go to the (idle) scratch as fp32: 64 key values,
        // then 128 query values.
        float far_c = 0.f, far_d = 0.f;
        auto far_products = [&]() {
            if (HAS_C2P) far_c = chain(fr[0], qb)[0];
            if (HAS_P2C) {
                if (w == 0) far_d = chain(fq[0], kb[0])[0];
                else if (w == 1) far_d = chain(fq[0], kb[1])[0];
            }
        };
        auto put_far = [&]() {
            float* const fv = reinterpret_cast<float*>(sm.p);
            const int il_ = fresh(il);
            if (fresh(hh) == 0) {
                if (HAS_C2P) fv[BN + 32 * w + il_] = far_c;
                if (HAS_P2C && w < 2) fv[32 * w + il_] = far_d;
            }
        };
        // Ring slot of the group (rt, a) of batch t: key 64t + ckey - 32rt - 8a with ckey = 60 + 4il - 4hh; `phase` is
        // 64t mod 192.
        uint16_t* const crow_fixed = sm.c + (32 * w + il) * CRS;
        const int ckey_fixed = 60 + 4 * il - 4 * hh;
        auto put_c = [&](int phase) {
            if (HAS_C2P) {
                const int il_ = fresh(il), hh_ = fresh(hh);
                uint16_t* const crow = FARZ ? sm.c + (32 * w + il_) * CRS : crow_fixed;
                const int ckey = FARZ ? 60 + 4 * il_ - 4 * hh_ : ckey_fixed;
                // slot of group (rt, a): y = cb - 32rt - 8a, minus 192 once y reaches 192 -- two base addresses per
                // step, one compare and one select per store, the distance inside the group as an immediate
                const int cb = phase + ckey;                    // 56 .. 312
                uint16_t* const flat = crow + cb - 56;
                uint16_t* const wrapped = flat - CRING;
#pragma unroll
                for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                    for (int a = 0; a < 4; ++a) {
                        const int d = 32 * rt + 8 * a;
                        uint16_t* const base = cb >= CRING + d ? wrapped : flat;
                        *reinterpret_cast<u32x2*>(base + 56 - d) = cpk[rt][a];
                    }
            }
        };
        auto put_p = [&]() {
            if (HAS_P2C) {
                const int il_ = fresh(il), hh_ = fresh(hh);
                auto put1 = [&](int xt, int jt, const u32x2 (&v)[4]) {
#pragma unroll
                    for (int a = 0; a < 4; ++a)
                        *reinterpret_cast<u32x2*>(&sm.p[(32 * jt + il_) * PS + 32 * xt + 8 * a + 4 * hh_]) = v[a];
                };
                put1(w + 1, 0, ppk[0]);
                put1(w + 1, 1, ppk[1]);
                if (w == 0) put1(0, 1, ppk[2]);
                else if (w == 1) put1(5, 0, ppk[2]);
            }
        };
        auto next_phase = [](int ph) { return ph == 2 * BN ? 0 : ph + BN; };

        // First LDS stage of a tile: keys of steps 0 and 1 and the whole window of step 0 (192 rows of either
        // table), 16 chunks of 16 B per thread.  The delta values come first (dl_win for the window, dl_step for
        // the 64 new rows of steps 1 to 3), the row reads depend on them.
        int dl_win[WIN / 32], dl_step[3][2];
        u32x4 st_k[4], st_wk[WIN / 32], st_wq[WIN / 32];
        // (Both readers assign every register also when there is no next tile: a conditional assignment would keep the
        // previous tile's values alive across the whole tile body.)
        auto read_deltas = [&](const Tile& t) {
#pragma unroll
            for (int n = 0; n < WIN / 32; ++n) dl_win[n] = 0;
#pragma unroll
            for (int s1 = 0; s1 < 3; ++s1) dl_step[s1][0] = dl_step[s1][1] = 0;
            if (HAS_POS && t.vb >= 0) {
                int sr = srow;            // opaque: keeps a dozen precomputed row offsets out of long-lived registers
                asm volatile("" : "+v"(sr));
#pragma unroll
                for (int n = 0; n < WIN / 32; ++n) dl_win[n] = delta_of(t.row0 - (BN - 1) + sr + 32 * n);
#pragma unroll
                for (int s1 = 0; s1 < 3; ++s1)
#pragma unroll
                    for (int n = 0; n < 2; ++n) dl_step[s1][n] = delta_of(t.row0 - BN * (s1 + 1) - (BN - 1) + sr + 32 * n);
            }
        };
        auto read_stage = [&](const Tile& t) {
            const uint16_t *Kt = k_of(t), *PKt = pk_of(t), *PQt = pq_of(t);
            const u32x4 none = {0, 0, 0, 0};
#pragma unroll
            for (int n = 0; n < 4; ++n) st_k[n] = none;
#pragma unroll
            for (int n = 0; n < WIN / 32; ++n) st_wk[n] = st_wq[n] = none;
            if (t.vb >= 0) {
#pragma unroll
                for (int n = 0; n < 4; ++n)
                    st_k[n] = *reinterpret_cast<const u32x4*>(Kt + int64_t(min(srow + 32 * n, t.len - 1)) * p.ks_l + sch * 8);
#pragma unroll
                for (int n = 0; n < WIN / 32; ++n) {
                    if (HAS_C2P) st_wk[n] = *reinterpret_cast<const u32x4*>(PKt + int64_t(dl_win[n]) * p.pks_r + sch * 8);
                    if (HAS_P2C) st_wq[n] = *reinterpret_cast<const u32x4*>(PQt + int64_t(dl_win[n]) * p.pqs_r + sch * 8);
                }
            }
        };
        auto write_stage = [&]() {
#pragma unroll
            for (int n = 0; n < 4; ++n)
                *reinterpret_cast<u32x4*>(&sm.k[n >> 1][(srow + 32 * (n & 1)) * RS + sch * 8]) = st_k[n];
#pragma unroll
            for (int n = 0; n < WIN / 32; ++n) {
                if (HAS_C2P) *reinterpret_cast<u32x4*>(&sm.kr[(srow + 32 * n) * RS + sch * 8]) = st_wk[n];
                if (HAS_P2C) *reinterpret_cast<u32x4*>(&sm.qr[(srow + 32 * n) * RS + sch * 8]) = st_wq[n];
            }
        };

#pragma unroll
        for (int s1 = 0; s1 < 3; ++s1) {
            dl_step[s1][0] = dl_cold[s1][0];
            dl_step[s1][1] = dl_cold[s1][1];
        }
        // near flags (not far) of steps 0, 1, 2 of the tile about to open; c2p batch t is needed when one of the steps
        // t, t+1, t+2 -- the steps its keys 64t + 4n .. 64t + 63 + 4n fall into -- is near
        bool near0 = !far_at(cur.row0, 0), near1 = !far_at(cur.row0, 1), near2 = !far_at(cur.row0, 2);
        phase_barrier();                  // first stage of the first tile is in LDS
        while (true) {
            bind_tables();
            // Opening: the c2p batches -2, -1, 0 (window rows w + 128.., w + 64.., w.. of step 0) and the p2c products
            // of step 0; window rows of step 1 (they overwrite rows step 0 is done with); fragments of step 1.
            const int off1 = prev_off(0);
            dl_next[0] = dl_step[0][0];
            dl_next[1] = dl_step[0][1];
            fetch();                      // window rows of step 1; they arrive under the products of step 0
            load_fp(0, 0);
            // (In the instances with far steps the c2p batches -2, -1, 0 are computed by the score waves, each for the
            // ring rows it reads itself: without them the position role of those instances, which carries two step
            // bodies, fits its registers.  The plain instances are 2-4 % faster with the batches here.)
            if (FARZ) {
                if (!near0) load_fr(0, w);    // a far step 0 takes its one c2p value from any window row
            } else if (near0 || near1 || near2) {
                load_fr(0, w + 2 * BN);
                products_c();
                put_c(BN);                // batch -2: phase (-128) mod 192
                load_fr(0, w + BN);
                products_c();
                put_c(2 * BN);            // batch -1
                load_fr(0, w);
                products_c();
                put_c(0);                 // batch 0
            } else {
                load_fr(0, w);
            }
            if (near0) {
                products_p();
                put_p();
            } else {
                far_products();
                put_far();
            }
            phase_barrier();              // every position wave has read its fragments of step 0
            store(off1);
            dl_next[0] = dl_step[1][0];
            dl_next[1] = dl_step[1][1];
            fetch();                      // window rows of step 2
            dl_next[0] = dl_step[2][0];
            dl_next[1] = dl_step[2][1];
            phase_barrier();              // window of step 1 complete
            load_fp(off1, 1);
            load_fr(off1, w);
            // The tile after this one.  Its delta values are read at the end of the last step but one (when the fragment
            // and result registers are no longer needed); its first LDS stage is read from global memory and written
            // to LDS in half A of the last step, where this role has nothing else to do: after the barrier that ends
            // that half, it is already at the next tile's first position products while the score waves finish the
            // last step.
            const Tile nxt = next_tile(cur);

            int off2 = prev_off(off1);    // ring offset of step s+2
            int phase = BN;               // ring phase of batch s+1
            bool n1 = near1, n2 = near2, n3 = !far_at(row0, 3);      // near flags of steps s+1, s+2, s+3
            auto pos_step = [&](int s, auto tail_tag) {
                constexpr bool TAIL = decltype(tail_tag)::value;   // step nsteps-2: no step s+2 to prepare
                const bool batch = n1 || n2 || n3;                 // c2p batch s+1 has a reader
                const bool n4 = !far_at(row0, s + 4);              // (a scalar read, used in the next step)
                phase_barrier();          // position terms of step s complete
                if (batch) products_c();  // of step s+1, into registers; issued first: the wait for the
                if (n1) products_p();
                else far_products();
                __builtin_amdgcn_sched_barrier(0);  // prefetched global data then passes under the MFMAs
                if (!TAIL) {
                    store(off2);          // new window rows of step s+2
                    fetch();              // window rows of step s+3: a full step ahead of their store
                    fetch_delta(s + 4);
                }
                phase_barrier();          // score waves are done with the ring slots and the scratch; the staged tiles are visible
                if (batch) put_c(phase);  // of step s+1
                if (n1) put_p();
                else put_far();
                if (!TAIL) {
                    load_fp(off2, s & 1); // of step s+2
                    load_fr(off2, w);
                } else {
                    read_deltas(nxt);
                }
                off2 = prev_off(off2);
                phase = next_phase(phase);
                n1 = n2;
                n2 = n3;
                n3 = n4;
            };
            if (nsteps >= 2) {
                for (int s = 0; s + 2 < nsteps; ++s) pos_step(s, std::false_type{});
                pos_step(nsteps - 2, std::true_type{});
            } else {
                read_deltas(nxt);
            }
            // Last key step: nothing left to prepare for this tile.  The rings, both key buffers and the Q fragment
            // registers are free, so the next tile moves in; the barrier that ends this half is also the barrier
            // after which the next tile's first stage is in LDS.
            phase_barrier();
            near0 = !far_at(nxt.row0, 0);
            near1 = !far_at(nxt.row0, 1);
            near2 = !far_at(nxt.row0, 2);
            read_stage(nxt);
            load_q(qb, nxt);              // (the last products of this tile have read the old fragments)
            if (nxt.vb >= 0) write_stage();
            phase_barrier();
            if (nxt.vb < 0) break;
            cur = nxt;
            bind(cur);
        }
        return;
    }

    // ===================================================== score waves ============================================
    const float c_exp = p.scale * 1.4426950408889634f;   // softmax in base 2
    f32x16 o_acc[2];
    float m_run, l_run;

    X8 kf[2][4];                      // K fragments: A operand of S^T = K.Q^T
    auto load_kf = [&](int kbuf) {
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
            for (int c = 0; c < 4; ++c) kf[jt][c] = lds_frag<X8>(sm.k[kbuf], 32 * jt + il, 16 * c + 8 * hh);
    };
    // Identity fragments: A operand that adds a B operand of 16 keys x 32 queries onto rows 16c2 .. 16c2+15 of a score
    // tile.  Lane (row il, half hh) of an A operand holds columns 8hh .. 8hh+7 of its row.
    X8 idf[2];
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2)
#pragma unroll
        for (int t = 0; t < 8; ++t) idf[c2][t] = il == 16 * c2 + 8 * hh + t ? (ET)1.0f : (ET)0.0f;
    // Keys and values travel global -> registers -> LDS through the score waves: thread tid stages chunk sch of rows
    // srow and srow + 32 of a 64-row step.  Buffer loads: the buffer of a step starts at its first row and ends with
    // the last row of the sequence, so rows past the end come back as zeros (hardware range check) with no lane
    // predicated off, and the per-load address arithmetic is scalar.
    const int srow = tid >> 3, sch = tid & 7;
    const int ks_b = int(p.ks_l) * 2, vs_b = int(p.vs_l) * 2;
    int kvoff[2], vvoff[2];
#pragma unroll
    for (int n = 0; n < 2; ++n) {
        kvoff[n] = (srow + 32 * n) * ks_b + sch * 16;
        vvoff[n] = (srow + 32 * n) * vs_b + sch * 16;
    }
    u32x4 pre_k[2], pre_v[2];
    auto fetch_kv_from = [&](const uint16_t* Kt, const uint16_t* Vt, int tlen, int sk, int sv) {
        const int kleft = tlen - BN * sk, vleft = tlen - BN * sv;
        const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t*>(Kt) + int64_t(BN * sk) * p.ks_l, 0, kleft > 0 ? (kleft - 1) * ks_b + 128 : 0, RSRC_FLAGS);
        const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t*>(Vt) + int64_t(BN * sv) * p.vs_l, 0, vleft > 0 ? (vleft - 1) * vs_b + 128 : 0, RSRC_FLAGS);
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            pre_k[n] = __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, kvoff[n], 0, 0);
            pre_v[n] = __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, vvoff[n], 0, 0);
        }
    };
    auto fetch_kv = [&](int sk, int sv) { fetch_kv_from(K, V, len, sk, sv); };   // key rows of step sk, value rows of step sv
    auto store_kv = [&](int kbuf, bool with_keys) {
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            if (with_keys) *reinterpret_cast<u32x4*>(&sm.k[kbuf][(srow + 32 * n) * RS + sch * 8]) = pre_k[n];
            *reinterpret_cast<u32x4*>(&sm.v[(srow + 32 * n) * RS + sch * 8]) = pre_v[n];
        }
    };
    Tile nxt;                             // the tile after the current one (looked up while a tile opens)
    nxt.vb = -1;
    nxt.head = nxt.b = nxt.row0 = nxt.len = 0;
    nxt.tok0 = 0;
    int cphase = 0;                       // ring slot of the first key of the step: 64s mod 192
    bool far_cur = false;                 // whether the step about to run is far; far_open: step 0 of the tile to open
    bool far_open = far_at(cur.row0, 0);
    const uint16_t* const crow = sm.c + (32 * w + il) * CRS + 8 * hh;
    // One key step.  MASKED: the step reaches past the end of the sequence (only the last step can).
    // The value lane ^ 32 holds.  A lane swap in the vector ALU: a shuffle would travel through the LDS queue, behind
    // the transposing reads of this wave and the result stores of the position waves, with the softmax waiting for it.
    // Swapping the upper half of one copy with the lower half of another leaves {own, partner} in the two results
    // (in an order that depends on the half, which a maximum or a sum does not care about).
    auto both_halves = [](float x, float& a, float& b) {
        const uint32_t u = __builtin_bit_cast(uint32_t, x);
        const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        a = __builtin_bit_cast(float, uint32_t(r[0]));
        b = __builtin_bit_cast(float, uint32_t(r[1]));
    };
    auto key_step = [&](int s, auto masked_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        phase_barrier();                  // position terms of step s complete

        // ---- half A: keys of step s+2 and values of step s go to LDS (prefetched registers, nothing waits);
        //      position terms of step s: c2p as four B operands of 16 keys each, straight out of the ring (keys
        //      64s .. 64s+63 never straddle its wrap), p2c element by element: (key jj, query n) takes
        //      P'[jj][w + 4n + 63 - jj], converted to fp32 into what becomes the initial score accumulator ----------
        const bool far_nxt = far_at(row0, s + 1);     // (two scalar reads, used at the end of the step)
        X8 cf[2][2];
        if (HAS_C2P && !far_cur) {
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
#pragma unroll
                for (int c2 = 0; c2 < 2; ++c2) cf[jt][c2] = *reinterpret_cast<const X8*>(crow + cphase + 32 * jt + 16 * c2);
        }
        f32x16 s_acc[2];
        float cadd = 0.f;                 // far step: the c2p value of this lane's query, added when the scores are scaled
        if (far_cur) {
            // one p2c value per key (fp32, the same for every query): the initial accumulator; one c2p value per query
            const float* const fv = reinterpret_cast<const float*>(sm.p);
            if (HAS_C2P) cadd = fv[BN + 32 * w + il];
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    float4 d = float4{0.f, 0.f, 0.f, 0.f};
                    if (HAS_P2C) d = *reinterpret_cast<const float4*>(fv + 32 * jt + 8 * a + 4 * hh);
                    s_acc[jt][4 * a] = d.x;
                    s_acc[jt][4 * a + 1] = d.y;
                    s_acc[jt][4 * a + 2] = d.z;
                    s_acc[jt][4 * a + 3] = d.w;
                }
        } else if (HAS_P2C) {
            // Element (key jc, query n) sits at 16-bit index X + jc * (PS - 1), X = w + 63 + 4n: from one key to the next
            // the index moves by an odd amount, so the element alternates between the low and the high half of its
            // dword with the parity of jc, starting from the parity of w + 1 -- the same for every lane, because the
            // rows of a wave are 4 apart.  The dwords of keys jc and jc + 2 are (PS - 1) dwords apart: one two-address
            // read fetches both; a byte permute with a wave-uniform selector moves the wanted half into an fp32.
            // The gathers are ordinary LDS loads; the compiler pairs them and places the waits.  (Loads issued from
            // inline assembly would be invisible to it: it may then copy a destination register before the data has arrived.)
            constexpr int PD = PS - 1;            // dwords between the elements of keys jc and jc + 2
            const int px = (w + 1) & 1;
            const auto* p_even = TDB_LDS(const uint32_t, sm.p) + ((w + 63 + 4 * il) >> 1) + 2 * hh * PD;    // key 4hh
            const auto* p_odd = p_even + PD / 2 + px;                                                          // key 4hh + 1
            const uint32_t sel_even = px ? E::PICK_HI : E::PICK_LO, sel_odd = px ? E::PICK_LO : E::PICK_HI;
            uint32_t g[2][16];
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int jc = 32 * jt + 8 * (e >> 2) + (e & 3);
                    g[jt][e] = (jc & 1) ? p_odd[(jc / 2) * PD] : p_even[(jc / 2) * PD];
                }
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
#pragma unroll
                for (int e = 0; e < 16; ++e) s_acc[jt][e] = E::pick(g[jt][e], (e & 1) ? sel_odd : sel_even);
        } else {
            s_acc[0] = zero16;
            s_acc[1] = zero16;
        }
        cphase = cphase == 2 * BN ? 0 : cphase + BN;
        // all LDS reads of the half in flight together, then the conversions, then the score MFMAs (they share the
        // matrix pipe of this half with the position wave of the SIMD)
        store_kv(s & 1, s + 2 < nsteps);  // (in the last step the key buffers already take the next tile's keys)
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int jt = 0; jt < 2; ++jt) s_acc[jt] = E::mfma(kf[jt][c], qb[c], s_acc[jt]);
        if (HAS_C2P && !far_cur) {
#pragma unroll
            for (int c2 = 0; c2 < 2; ++c2)
#pragma unroll
                for (int jt = 0; jt < 2; ++jt) s_acc[jt] = E::mfma(idf[c2], cf[jt][c2], s_acc[jt]);
        }
        if (s + 1 < nsteps) load_kf((s + 1) & 1);   // K fragments of step s+1 (the MFMAs above have read this step's)
        phase_barrier();                  // ring slots and scratch are free again; keys of step s+1 and values of step s are staged

        // ---- half B ---------------------------------------------------------------------------------------------
        if (s + 1 == nsteps) {            // last step: the Q fragments of the next tile travel from here on
            load_q(qb, nxt);
            far_open = far_at(nxt.row0, 0);
            // keys of step 2 and values of step 0 of the next tile: its first half A stores them, and a first touch of
            // a new sequence takes longer than the opening of a tile lasts
            if (nxt.vb >= 0)
                fetch_kv_from(k_of(nxt), static_cast<const uint16_t*>(p.v) + (packed_rows ? nxt.tok0 * p.vs_l : int64_t(nxt.b) * p.vs_b) + int64_t(nxt.head) * p.vs_h,
                              nxt.len, 2, 0);
        }
        if (s + 1 < nsteps) fetch_kv(s + 3, s + 1);   // for the next half A (nothing left to fetch in the last step)
        // V^T fragments through the transposing LDS read: the lane provides the address of 4 dims of one key
        X8 vf[2][2][2];               // [key tile][16-key chunk][dim tile]
        {
            const int g = l >> 4, ll = l & 15;
            const uint16_t* vbase = &sm.v[((ll >> 2) + 4 * (g >> 1)) * RS + 16 * (g & 1) + 4 * (ll & 3)];
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
#pragma unroll
                for (int c = 0; c < 2; ++c)
#pragma unroll
                    for (int dt = 0; dt < 2; ++dt) {
                        const uint16_t* src = vbase + (32 * jt + 16 * c) * RS + 32 * dt;
                        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(TDB_LDS(s16x4, src));
                        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(TDB_LDS(s16x4, src + 8 * RS));
                        const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                        vf[jt][c][dt] = __builtin_bit_cast(X8, both);
                    }
        }
        if (MASKED) {
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int j = BN * s + 32 * jt + 8 * (e >> 2) + 4 * hh + (e & 3);
                    if (j >= len) s_acc[jt][e] = -INFINITY;
                }
        }
        // streaming softmax: this lane holds 32 of the 64 keys of its query row, lane^32 the others
        float mx = s_acc[0][0];
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s_acc[jt][e]);
        {
            float own_or_partner, partner_or_own;
            both_halves(mx, own_or_partner, partner_or_own);
            mx = fmaxf(own_or_partner, partner_or_own) + cadd;
        }
        // The running maximum is only raised (and the accumulators rescaled) when some row of the wave exceeds it
        // by more than 2^8; until then probabilities of this step may be as large as 256, which bf16 and the fp32
        // sums carry exactly as well.  (First step: m_run = -inf always triggers, alpha = 0.)
        const float m_new = fmaxf(m_run, mx);          // finite: key 64s < len is never masked
        if (__builtin_amdgcn_ballot_w64((m_new - m_run) * c_exp > 8.f) != 0) {
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c_exp);
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) o_acc[t][e] *= alpha;
            m_run = m_new;
        }
        const float mc = (m_run - cadd) * c_exp;
        float psum = 0.f;
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                uint32_t pw[4];
#pragma unroll
                for (int h2 = 0; h2 < 4; ++h2) {
                    const float p0 = __builtin_amdgcn_exp2f(fmaf(s_acc[jt][8 * c + 2 * h2], c_exp, -mc));
                    const float p1 = __builtin_amdgcn_exp2f(fmaf(s_acc[jt][8 * c + 2 * h2 + 1], c_exp, -mc));
                    const X2 pr = {(ET)p0, (ET)p1};
                    psum += p0 + p1;
                    pw[h2] = __builtin_bit_cast(uint32_t, pr);
                }
                const X8 pb = __builtin_bit_cast(X8, u32x4{pw[0], pw[1], pw[2], pw[3]});
                // O^T += V^T.P^T
#pragma unroll
                for (int dt = 0; dt < 2; ++dt)
                    o_acc[dt] = E::mfma(vf[jt][c][dt], pb, o_acc[dt]);
            }
        l_run += psum;
        far_cur = far_nxt;
    };

    // Opening of a tile, after its first barrier (first stage in LDS).  Everything that reads global memory is
    // requested here and waited for much later: keys of step 2 / values of step 0 (stored in half A of step 0).  The output rows of the previous tile are written
    // last: stores count on the same in-order counter as loads, so a wait for any load issued after them would
    // also wait for them.
    u32x4 o_out[2][2];                    // packed output rows of the tile just finished, 16 B per store
    uint16_t* o_ptr = nullptr;
    bool o_write = false, first_open = true;
    auto open_tile = [&]() {
        load_kf(0);
        if (first_open) fetch_kv(2, 0);   // first tile of the workgroup; later ones: requested in the last step before
        first_open = false;
        if (o_write) {
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int a = 0; a < 2; ++a) *reinterpret_cast<u32x4*>(o_ptr + 32 * dt + 16 * a) = o_out[dt][a];
        }
        cphase = 0;
        far_cur = far_open;
        // Instances with far steps: the c2p batches -2, -1, 0 of the tile (window rows w + 128.., w + 64.., w.. of step 0; together the 188
        // positions step 0 needs): C'^T[r, i] = K_r'[r].Q_i for 64 positions each, filed under their keys in this
        // wave's own rows of the ring.  The window is complete (the position waves staged it before the barrier in the
        // middle of the previous tile's last step) and stays untouched until the first barrier below.
        if (FARZ && HAS_C2P && (!far_open || !far_at(row0, 1) || !far_at(row0, 2))) {
            uint16_t* const cput = sm.c + (32 * w + il) * CRS;
            auto batch = [&](int xb, int phase) {
                X8 fr[2][4];
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) {
                    const int slot = min(xb + 32 * rt + il, WIN - 1);     // rows past the window: any row will do (negative keys)
                    const uint16_t* base = sm.kr + slot * RS + 8 * hh;
#pragma unroll
                    for (int c = 0; c < 4; ++c) fr[rt][c] = *reinterpret_cast<const X8*>(base + 16 * c);
                }
                f32x16 acc[2] = {E::mfma(fr[0][0], qb[0], zero16), E::mfma(fr[1][0], qb[0], zero16)};
#pragma unroll
                for (int c = 1; c < 4; ++c)
#pragma unroll
                    for (int rt = 0; rt < 2; ++rt) acc[rt] = E::mfma(fr[rt][c], qb[c], acc[rt]);
                // ring slot of the group (rt, a): key 64t + ckey - 32rt - 8a with ckey = 60 + 4il - 4hh, phase = 64t mod 192;
                // register 4a + t of a tile holds key k0 - t: the four keys of a group go out together, lowest first
                const int cb = phase + 60 + 4 * il - 4 * hh;      // 56 .. 312
#pragma unroll
                for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                    for (int a = 0; a < 4; ++a) {
                        const int y = cb - 32 * rt - 8 * a;
                        *reinterpret_cast<u32x2*>(cput + (y >= CRING ? y - CRING : y)) =
                            u32x2{pack2<E>(acc[rt][4 * a + 3], acc[rt][4 * a + 2]), pack2<E>(acc[rt][4 * a + 1], acc[rt][4 * a])};
                    }
            };
            batch(w + 2 * BN, BN);        // batch -2: phase (-128) mod 192
            batch(w + BN, 2 * BN);        // batch -1
            batch(w, 0);                  // batch 0
        }
        phase_barrier();                  // the two opening barriers of the position waves
        phase_barrier();
        // the tile after this one is looked up while the position waves get step 1 ready
        nxt = next_tile(cur);
    };
    // Epilogue of a tile: normalised output rows, packed.  A lane holds d = 32*dt + 8*a + 4*hh + 0..3 of its query row,
    // its partner lane^32 the other four of every eight; one swap between the lane halves per dword gives each lane
    // eight consecutive d (lane half hh keeps the blocks a = 2*a2 + hh), so a row goes out in 16-byte stores.
    auto close_tile = [&]() {
        const int qi = row0 + 4 * il + w;
        float l_a, l_b;
        both_halves(l_run, l_a, l_b);
        const float l_tot = l_a + l_b;
        const float inv = 1.f / l_tot;
        const bool live = qi < len;
        o_write = qi < row0 + rows_here;
        o_ptr = O + int64_t(qi) * p.os_l + 8 * hh;
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2) {
                u32x2 r[2];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const int a = 2 * a2 + t;
                    r[t] = u32x2{0, 0};
                    if (live) r[t] = u32x2{pack2<E>(o_acc[dt][4 * a] * inv, o_acc[dt][4 * a + 1] * inv),
                                           pack2<E>(o_acc[dt][4 * a + 2] * inv, o_acc[dt][4 * a + 3] * inv)};
                }
                // lower half: (own block 2*a2, partner's block 2*a2); upper half: (partner's block 2*a2+1, own block 2*a2+1)
                const auto k0 = __builtin_amdgcn_permlane32_swap(r[0][0], r[1][0], false, false);
                const auto k1 = __builtin_amdgcn_permlane32_swap(r[0][1], r[1][1], false, false);
                o_out[dt][a2] = u32x4{k0[0], k1[0], k0[1], k1[1]};
            }
    };

    phase_barrier();                      // first stage of the first tile is in LDS
    open_tile();
    while (true) {
        o_acc[0] = zero16;
        o_acc[1] = zero16;
        m_run = -INFINITY;
        l_run = 0.f;
        for (int s = 0; s < nfull; ++s) key_step(s, std::false_type{});
        if (nfull < nsteps) key_step(nfull, std::true_type{});

        // The position waves put the first stage of the next tile into LDS during the last step and are at its
        // first position products by now; this tile is closed under those.
        close_tile();
        if (nxt.vb < 0) break;
        cur = nxt;
        bind(cur);
        open_tile();
    }
    if (o_write) {
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int a = 0; a < 2; ++a) *reinterpret_cast<u32x4*>(o_ptr + 32 * dt + 16 * a) = o_out[dt][a];
    }
}

}  // namespace

bool tdb_mfma_supported(const TdbKernelParams& p, int dtype) {
    // bf16 or fp16, head_dim 64, position terms as fused tables or as strips (or none); a call that mixes the two
    // forms goes to the generic kernel.  Buffer loads address rows with 32-bit byte offsets from the start of a
    // (sequence, head).
    if ((dtype != TDB_BF16 && dtype != TDB_F16) || p.D != 64) return false;
    if ((p.c2p || p.p2c) && (p.pk || p.pq)) return false;
    const int64_t lim = int64_t(1) << 31;
    const int64_t rows = p.L;
    if (p.c2p && (rows * p.c2s_l * 2 + int64_t(4) * p.span >= lim || p.c2s_l < 0)) return false;
    if (p.p2c && (rows * p.p2s_l * 2 + int64_t(4) * p.span >= lim || p.p2s_l < 0)) return false;
    if (rows * p.ks_l * 2 >= lim || rows * p.vs_l * 2 >= lim) return false;
    if (p.pk && int64_t(2) * p.span * p.pks_r * 2 >= lim) return false;
    if (p.pq && int64_t(2) * p.span * p.pqs_r * 2 >= lim) return false;
    return true;
}

namespace {

// Per-device launch facts, looked up once per device under a lock: CU count (rounded down to the 8 XCDs the block
// ids are dealt over) and, per kernel instance, whether its dynamic-LDS limit has been raised on that device.
constexpr int kMaxDevices = 64;
constexpr int FAR_MIN_LEN = 1536;
constexpr int kInstances = 64;      // 32 for tables (layout, far, type, c2p, p2c), the strip instances above them
std::mutex g_dev_mutex;
int g_cus[kMaxDevices] = {0};
bool g_attr_set[kMaxDevices][kInstances] = {{false}};
std::atomic<int> g_workgroup_limit{0};       // cap on the persistent workgroups of a launch (multiple of 8), 0 = none

}  // namespace

int tdb_mfma_set_workgroup_limit(int workgroups) {
    const int cap = workgroups <= 0 ? 0 : workgroups < 8 ? 8 : workgroups / 8 * 8;
    g_workgroup_limit.store(cap, std::memory_order_relaxed);
    return cap;
}

hipError_t tdb_launch_mfma(const TdbKernelParams& whole, int dtype, hipStream_t stream) {
    // Packed batches of more than 64 sequences go out as several launches of at most 64 (even parts): the kernel
    // balances a persistent launch from sequence boundaries held one per lane, which is worth ~20 % over handing
    // every tile to a workgroup of its own.  A part is the same call with fewer sequences: cu_seqlens holds
    // absolute token offsets, so only its start and the count move.
    if (whole.varlen && whole.B > 64) {
        const int parts = (whole.B + 63) / 64, per = (whole.B + parts - 1) / parts;
        for (int first = 0; first < whole.B; first += per) {
            TdbKernelParams part = whole;
            if (whole.cu_seqlens) {
                part.cu_seqlens = whole.cu_seqlens + first;
            } else {                      // a padded batch dealt like packed sequences (below): the part starts `first` sequences in
                auto at = [first](const void* base, int64_t stride_b) { return base ? static_cast<const uint16_t*>(base) + first * stride_b : nullptr; };
                part.seqlens = whole.seqlens + first;
                part.q = at(whole.q, whole.qs_b);
                part.k = at(whole.k, whole.ks_b);
                part.v = at(whole.v, whole.vs_b);
                part.o = const_cast<uint16_t*>(at(whole.o, whole.os_b));
                part.c2p = at(whole.c2p, whole.c2s_b);
                part.p2c = at(whole.p2c, whole.p2s_b);
            }
            part.B = whole.B - first < per ? whole.B - first : per;
            const hipError_t e = tdb_launch_mfma(part, dtype, stream);
            if (e != hipSuccess) return e;
        }
        return hipSuccess;
    }
    // A fixed-layout call with valid lengths is a batch of sequences of different cost, and the strided walk of the
    // fixed instances gives a workgroup the same (sequence, tile) in every head: the launch takes what its longest
    // sequence takes, however short the others are.  Such a call goes to the packed instances, whose deal balances
    // tiles of different cost (b32 x L512: lengths U[64,512] 0.092 -> 0.053 ms, U[384,512] 0.0934 -> 0.0915 ms); they
    // address its rows through the batch strides and padded rows still come back as zeros.  Calls without lengths
    // (every tile costs the same) keep the fixed instances.
    if (!whole.varlen && whole.seqlens && int64_t(whole.B) * whole.L < (int64_t(1) << 31)) {
        TdbKernelParams packed = whole;
        packed.varlen = 1;
        packed.cu_seqlens = nullptr;
        packed.total = whole.B * whole.L;        // (sizes the upper bound of the tile count)
        return tdb_launch_mfma(packed, dtype, stream);
    }
    const TdbKernelParams& p = whole;
    const int64_t tiles = int64_t(p.varlen ? p.total / BM + p.B : p.B * ((p.L + BM - 1) / BM)) * p.H;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    const bool strip = p.c2p != nullptr || p.p2c != nullptr;
    const bool c2p = strip ? p.c2p != nullptr : p.pk != nullptr, p2c = strip ? p.p2c != nullptr : p.pq != nullptr;
    // Far key steps only exist in sequences longer than the table's reach; the instance that looks for them carries
    // both step bodies and its near steps take 1.12x the time, a far step 0.65x.  At length 1024 a quarter of the steps
    // are far and the plain instance is 7 % faster; at 1536 the far instance wins by 2 %, at 4096 by 13 %.
    const bool farz = !strip && (c2p || p2c) && p.L >= FAR_MIN_LEN;
    const int64_t round = int64_t(8) << (farz ? XG_LONG : XG_PLAIN);     // the id regrouping is a bijection on multiples of this
    const int nblocks = int((tiles + round - 1) / round * round);
    const int instance = (p.varlen ? 16 : 0) + (farz ? 8 : 0) + (dtype == TDB_F16 ? 4 : 0) + (c2p ? 2 : 0) + (p2c ? 1 : 0) +
                         (strip ? 32 : 0);
    const size_t smem = sizeof(Smem);
    const void* fn = nullptr;
#define TDB_PICK(A, B, T)                                                                                        \
    fn = farz ? (p.varlen ? reinterpret_cast<const void*>(&attn_mfma_kernel<A, B, T, true, true>)                \
                          : reinterpret_cast<const void*>(&attn_mfma_kernel<A, B, T, true, false>))              \
              : (p.varlen ? reinterpret_cast<const void*>(&attn_mfma_kernel<A, B, T, false, true>)               \
                          : reinterpret_cast<const void*>(&attn_mfma_kernel<A, B, T, false, false>))
#define TDB_PICK_STRIP(A, B, T)                                                                                  \
    fn = p.varlen ? reinterpret_cast<const void*>(&attn_mfma_kernel<A, B, T, false, true, true>)                 \
                  : reinterpret_cast<const void*>(&attn_mfma_kernel<A, B, T, false, false, true>)
#define TDB_PICK_T(T)                                      \
    do {                                                   \
        if (strip) {                                       \
            if (c2p && p2c) TDB_PICK_STRIP(true, true, T); \
            else if (c2p) TDB_PICK_STRIP(true, false, T);  \
            else TDB_PICK_STRIP(false, true, T);           \
        } else if (c2p && p2c) TDB_PICK(true, true, T);    \
        else if (c2p) TDB_PICK(true, false, T);            \
        else if (p2c) TDB_PICK(false, true, T);            \
        else TDB_PICK(false, false, T);                    \
    } while (0)
    if (dtype == TDB_F16) TDB_PICK_T(TDB_F16);
    else TDB_PICK_T(TDB_BF16);
#undef TDB_PICK_T
#undef TDB_PICK_STRIP
#undef TDB_PICK
    int cus = 0;
    {
        std::lock_guard<std::mutex> lock(g_dev_mutex);
        if (g_cus[dev] == 0) {
            int n = 0;
            if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 8) n = 8;
            g_cus[dev] = n / 8 * 8;
        }
        cus = g_cus[dev];
        if (!g_attr_set[dev][instance]) {
            e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, int(smem));
            if (e != hipSuccess) return e;
            g_attr_set[dev][instance] = true;
        }
    }
    // Persistent workgroups, one per CU: fixed layout with a strided deal (tiles cost about the same), packed
    // batches with a cost-balanced deal computed in the kernel.
    const int limit = g_workgroup_limit.load(std::memory_order_relaxed);
    if (limit > 0 && limit < cus) cus = limit;
    const int persistent = nblocks < cus ? nblocks : cus;
    void* args[] = {const_cast<TdbKernelParams*>(&p), const_cast<int*>(&nblocks)};
    return hipLaunchKernel(fn, dim3(unsigned(persistent)), dim3(NTHREADS), args, smem, stream);
}
