// Matrix-core disentangled-attention forward for bf16, head_dim 64 (gfx950, wave64, MFMA 32x32x16).
//
// One workgroup = 4 waves = one tile of 128 query rows of one (sequence, head); each wave owns 32
// query rows and walks the keys 64 at a time with a streaming softmax.  Scores are kept
// transposed (S^T = K.Q^T) so that a lane owns ONE query row: row max / row sum are in-lane
// reductions plus one exchange between the two half-waves, and the S^T accumulator registers are
// already the B operand of the P.V product (O^T += V^T.P^T), so probabilities never touch LDS.
//
// Position terms, per key step (j0 .. j0+63), in "position space": the workgroup needs relative
// positions r = i - j in a window of 128+64-1 values.  Rows K_r[delta(r)] and Q_r[delta(r)] of the
// per-head tables are staged in LDS for that window (delta from the host-built table, so log
// bucketing, saturation beyond max_relative_positions and the un-bucketed case are one code path
// with bit-exact indices).  Then
//   c2p:  C'^T[r, i] = K_r'[r] . Q_i      per wave, over its own 96-position sub-window,
//   p2c:  P'^T[r, j] = Q_r'[r] . K_j      once per workgroup,
// both on MFMA, written to LDS (c2p as fp32, p2c as bf16) and read back skewed: score (i, j) takes C'[i][i-j] and
// P'[j][i-j].  Score position (i, j) therefore gets Q_i.K_r[delta(i-j)] + K_j.Q_r[delta(i-j)], the
// Hugging Face eager definition (modeling_deberta_v2.py:317-324, :337-343).
#include <type_traits>
#include <utility>

#include "tdb_internal.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define TDB_LDS(T, p) ((__attribute__((address_space(3))) T*)(p))

// Phase timing for development builds (-DTDB_TIMING): one wave accumulates cycle counts per phase.
#ifdef TDB_TIMING
__device__ long long tdb_timing[16];
#define TDB_T0() long long tdb_t = clock64(); const bool tdb_on = blockIdx.x == 7 && blockIdx.y == 3 && threadIdx.x == 64
#define TDB_TICK(k)                                        \
    do {                                                   \
        const long long n_ = clock64();                    \
        if (tdb_on) tdb_timing[k] += n_ - tdb_t;           \
        tdb_t = n_;                                        \
    } while (0)
#else
#define TDB_T0() do {} while (0)
#define TDB_TICK(k) do {} while (0)
#endif

constexpr int BM = TDB_MFMA_TILE;   // query rows per workgroup
constexpr int BN = 64;              // keys per step
constexpr int D = 64;
constexpr int WIN = BM + BN;        // ring of staged window rows (one more than the 191 positions in use)
constexpr int RS = 72;              // LDS row stride (elements) of 64-wide bf16 rows: 144 B, conflict-free b128
constexpr int CS = 100;             // row stride (floats) of the per-wave c2p scratch [32][96 used]
constexpr int PS = 196;             // row stride of the p2c scratch           [64][192 used]

struct Smem {
    uint16_t k[BN * RS];
    uint16_t v[BN * RS];
    uint16_t kr[WIN * RS];
    uint16_t qr[WIN * RS];
    float c[4][32 * CS];
    uint16_t p[BN * PS];
};

__device__ __forceinline__ bf16x8 lds_frag(const uint16_t* row_base, int row, int col) {
    return *reinterpret_cast<const bf16x8*>(row_base + row * RS + col);
}

__device__ __forceinline__ u32x2 pack4(float a, float b, float c, float d) {
    bf16x2 lo = {(__bf16)a, (__bf16)b};
    bf16x2 hi = {(__bf16)c, (__bf16)d};
    u32x2 r;
    r[0] = __builtin_bit_cast(uint32_t, lo);
    r[1] = __builtin_bit_cast(uint32_t, hi);
    return r;
}

template <int... Is, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f) {
    (f(std::integral_constant<int, Is>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): loop indices usable as immediates
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// Skewed LDS gathers, issued as inline asm with immediate offsets.  (Left to the compiler, runs of
// neighbouring narrow reads get fused into 64-bit reads at 2- or 4-byte alignment, which this LDS
// serialises lane by lane.)  Results are valid after lds_wait().
template <int OFF0, int OFF1>   // two dwords at dword offsets OFF0, OFF1 from a 4-byte aligned address
__device__ __forceinline__ float2 lds_read2_f32(uint32_t addr) {
    float2 r;
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(r) : "v"(addr), "n"(OFF0), "n"(OFF1) : "memory");
    return r;
}
template <int OFF>              // one zero-extended 16-bit value at byte offset OFF
__device__ __forceinline__ uint32_t lds_read_u16(uint32_t addr) {
    uint32_t r;
    asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
__device__ __forceinline__ void lds_wait(f32x16& a, f32x16& b) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b) : : "memory");
}
__device__ __forceinline__ void lds_wait(uint32_t (&g)[16]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(g[0]), "+v"(g[1]), "+v"(g[2]), "+v"(g[3]), "+v"(g[4]), "+v"(g[5]), "+v"(g[6]), "+v"(g[7]),
                   "+v"(g[8]), "+v"(g[9]), "+v"(g[10]), "+v"(g[11]), "+v"(g[12]), "+v"(g[13]), "+v"(g[14]), "+v"(g[15])
                 :
                 : "memory");
}
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return uint32_t(uintptr_t(TDB_LDS(const char, p)));
}

template <bool HAS_C2P, bool HAS_P2C>
__global__ __launch_bounds__(256) void attn_mfma_kernel(const TdbKernelParams p) {
    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    Smem& sm = *reinterpret_cast<Smem*>(smem_raw);

    const int tid = threadIdx.x;
    const int w = tid >> 6, l = tid & 63;
    const int il = l & 31, hh = l >> 5;
    const int head = blockIdx.y;

    int b, row0, len;
    int64_t tok0;
    if (!tdb_locate_tile(p, BM, blockIdx.x, b, row0, len, tok0)) return;

    const uint16_t* Q = static_cast<const uint16_t*>(p.q) + (p.varlen ? tok0 * p.qs_l : int64_t(b) * p.qs_b) + int64_t(head) * p.qs_h;
    const uint16_t* K = static_cast<const uint16_t*>(p.k) + (p.varlen ? tok0 * p.ks_l : int64_t(b) * p.ks_b) + int64_t(head) * p.ks_h;
    const uint16_t* V = static_cast<const uint16_t*>(p.v) + (p.varlen ? tok0 * p.vs_l : int64_t(b) * p.vs_b) + int64_t(head) * p.vs_h;
    uint16_t* O = static_cast<uint16_t*>(p.o) + (p.varlen ? tok0 * p.os_l : int64_t(b) * p.os_b) + int64_t(head) * p.os_h;
    const int rows_here = min(BM, (p.varlen ? len : p.L) - row0);   // rows of this tile that exist in memory

    if (row0 >= len) {   // only padded query rows (fixed layout): zeros
        for (int idx = tid; idx < rows_here * (D / 8); idx += 256)
            *reinterpret_cast<u32x4*>(O + int64_t(row0 + (idx >> 3)) * p.os_l + (idx & 7) * 8) = u32x4{0, 0, 0, 0};
        return;
    }

    const uint16_t* PK = HAS_C2P ? static_cast<const uint16_t*>(p.pk) + int64_t(head) * p.pks_h : nullptr;
    const uint16_t* PQ = HAS_P2C ? static_cast<const uint16_t*>(p.pq) + int64_t(head) * p.pqs_h : nullptr;

    // B operand of every product against this wave's queries: Q^T, k = d.
    const int qi = row0 + 32 * w + il;
    bf16x8 qb[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        u32x4 t = {0, 0, 0, 0};
        if (qi < len) t = *reinterpret_cast<const u32x4*>(Q + int64_t(qi) * p.qs_l + 16 * c + 8 * hh);
        qb[c] = __builtin_bit_cast(bf16x8, t);
    }

    f32x16 o_acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[t][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const float c_exp = p.scale * 1.4426950408889634f;   // softmax in base 2

    const int lut_max = 2 * p.lut_half;
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};

    // ---- staging ---------------------------------------------------------------------------------------------
    // Key step s covers keys 64s .. 64s+63 and needs relative positions B_s .. B_s+190, B_s = row0 - 64s - 63.
    // The rows K_r[delta(r)] / Q_r[delta(r)] of that window live in a 192-row ring: going to the next step the
    // window slides down by 64, so only its 64 lowest positions are fetched and they overwrite the 64 highest
    // of the previous step.  Window row x of step s sits in ring slot (x + off_s) mod 192, off_s = (128*s) mod 192.
    // Everything a step needs from global memory is fetched one step ahead into registers (delta values two
    // steps ahead) and written to LDS between two barriers.
    constexpr bool HAS_POS = HAS_C2P || HAS_P2C;
    const int nsteps = (len + BN - 1) / BN;
    const int srow = tid >> 3, sch = tid & 7;              // this thread stages rows srow, srow+32 (chunk sch)
    auto delta_of = [&](int r) { return p.lut[min(max(r + p.lut_half, 0), lut_max)]; };

    u32x4 pre_k[2], pre_v[2], pre_kr[2], pre_qr[2];
    int dl_next[2] = {0, 0};
    auto fetch_step = [&](int s) {       // global -> registers for key step s (its keys and its 64 new window rows)
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            const int j = BN * s + srow + 32 * n;
            pre_k[n] = u32x4{0, 0, 0, 0};
            pre_v[n] = u32x4{0, 0, 0, 0};
            if (j < len) {
                pre_k[n] = *reinterpret_cast<const u32x4*>(K + int64_t(j) * p.ks_l + sch * 8);
                pre_v[n] = *reinterpret_cast<const u32x4*>(V + int64_t(j) * p.vs_l + sch * 8);
            }
            if (HAS_C2P) pre_kr[n] = *reinterpret_cast<const u32x4*>(PK + int64_t(dl_next[n]) * p.pks_r + sch * 8);
            if (HAS_P2C) pre_qr[n] = *reinterpret_cast<const u32x4*>(PQ + int64_t(dl_next[n]) * p.pqs_r + sch * 8);
        }
    };
    auto fetch_delta = [&](int s) {      // delta of the 64 new window rows of key step s
        if (HAS_POS) {
#pragma unroll
            for (int n = 0; n < 2; ++n) dl_next[n] = delta_of(row0 - BN * s - (BN - 1) + srow + 32 * n);
        }
    };
    auto store_step = [&](int off) {     // registers -> LDS
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            const int r = srow + 32 * n;
            *reinterpret_cast<u32x4*>(&sm.k[r * RS + sch * 8]) = pre_k[n];
            *reinterpret_cast<u32x4*>(&sm.v[r * RS + sch * 8]) = pre_v[n];
            if (HAS_C2P) *reinterpret_cast<u32x4*>(&sm.kr[(off + r) * RS + sch * 8]) = pre_kr[n];
            if (HAS_P2C) *reinterpret_cast<u32x4*>(&sm.qr[(off + r) * RS + sch * 8]) = pre_qr[n];
        }
    };

    // prologue: whole window of step 0 (slots 0..191), keys of step 0
    if (HAS_POS) {
#pragma unroll
        for (int n = 0; n < WIN * 8 / 256; ++n) {
            const int x = srow + 32 * n;
            const int dl = delta_of(row0 - (BN - 1) + x);
            if (HAS_C2P)
                *reinterpret_cast<u32x4*>(&sm.kr[x * RS + sch * 8]) = *reinterpret_cast<const u32x4*>(PK + int64_t(dl) * p.pks_r + sch * 8);
            if (HAS_P2C)
                *reinterpret_cast<u32x4*>(&sm.qr[x * RS + sch * 8]) = *reinterpret_cast<const u32x4*>(PQ + int64_t(dl) * p.pqs_r + sch * 8);
        }
    }
#pragma unroll
    for (int n = 0; n < 2; ++n) {
        const int r = srow + 32 * n;
        u32x4 kk = {0, 0, 0, 0}, vv = {0, 0, 0, 0};
        if (r < len) {
            kk = *reinterpret_cast<const u32x4*>(K + int64_t(r) * p.ks_l + sch * 8);
            vv = *reinterpret_cast<const u32x4*>(V + int64_t(r) * p.vs_l + sch * 8);
        }
        *reinterpret_cast<u32x4*>(&sm.k[r * RS + sch * 8]) = kk;
        *reinterpret_cast<u32x4*>(&sm.v[r * RS + sch * 8]) = vv;
    }
    fetch_delta(1);
    __syncthreads();
    if (nsteps > 1) {
        fetch_step(1);
        fetch_delta(2);
    }

    int off = 0;                          // ring slot of window row 0 of the current step
    TDB_T0();
    for (int s = 0; s < nsteps; ++s) {
        const int j0 = BN * s;
        // ring rows of the position tiles this wave reads as MFMA A operands
        auto ring = [&](int x) { const int t = x + off; return t >= WIN ? t - WIN : t; };

        TDB_TICK(0);
        // ---- K fragments: A operand of S^T = K.Q^T and B operand of P'^T = Q_r'.K^T ---------------------
        bf16x8 kf[2][4];
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
            for (int c = 0; c < 4; ++c) kf[jt][c] = lds_frag(sm.k, 32 * jt + il, 16 * c + 8 * hh);

        // ---- c2p: C'^T[r, i] over this wave's 96-position sub-window, to LDS as C'[i][r'] --------------
        if (HAS_C2P) {
#pragma unroll
            for (int rt = 0; rt < 3; ++rt) {
                f32x16 acc;
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[e] = 0.f;
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(sm.kr, ring(32 * w + 32 * rt + il), 16 * c + 8 * hh),
                                                                  qb[c], acc, 0, 0, 0);
#pragma unroll
                for (int a = 0; a < 4; ++a)
                    *reinterpret_cast<float4*>(&sm.c[w][il * CS + 32 * rt + 8 * a + 4 * hh]) =
                        float4{acc[4 * a], acc[4 * a + 1], acc[4 * a + 2], acc[4 * a + 3]};
            }
        }
        TDB_TICK(1);
        // ---- p2c: P'^T[r, j] for the whole window (6 x 2 tiles): wave w takes position tile w against both
        //      key tiles, then one tile of position tiles 4..5; to LDS as P'[j][r''] -----------------------------
        if (HAS_P2C) {
            auto p2c_tile = [&](int rt, int jt, const bf16x8 (&kb)[4]) {
                f32x16 acc;
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[e] = 0.f;
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(sm.qr, ring(32 * rt + il), 16 * c + 8 * hh), kb[c], acc, 0, 0, 0);
#pragma unroll
                for (int a = 0; a < 4; ++a)
                    *reinterpret_cast<u32x2*>(&sm.p[(32 * jt + il) * PS + 32 * rt + 8 * a + 4 * hh]) =
                        pack4(acc[4 * a], acc[4 * a + 1], acc[4 * a + 2], acc[4 * a + 3]);
            };
            p2c_tile(w, 0, kf[0]);
            p2c_tile(w, 1, kf[1]);
            if (w & 1) p2c_tile(4 + (w >> 1), 1, kf[1]);
            else p2c_tile(4 + (w >> 1), 0, kf[0]);
        }
        TDB_TICK(2);
        __syncthreads();
        TDB_TICK(3);

        // ---- S^T = K.Q^T + position terms.  Element (jj, i) of the tile takes C'[i][i-jj+63] (fp32, gathered
        //      straight into the accumulator the MFMA then adds onto) and P'[jj][32w+i-jj+63] (bf16) ------------
        f32x16 s_acc[2];
        if (HAS_C2P) {
            // float index of element e of key tile jt:  il*CS + il + 63 - 4*hh - jc,  jc = 32*jt + 8*(e>>2) + (e&3) <= 59
            const uint32_t caddr = lds_addr(&sm.c[w][il * (CS + 1) + 4 - 4 * hh]);
            static_for<16>([&](auto pc) {
                constexpr int pr = decltype(pc)::value, jt = pr >> 3, e = 2 * (pr & 7);
                constexpr int jc = 32 * jt + 8 * (e >> 2) + (e & 3);
                const float2 t = lds_read2_f32<59 - jc, 59 - jc - 1>(caddr);
                s_acc[jt][e] = t.x;
                s_acc[jt][e + 1] = t.y;
            });
            lds_wait(s_acc[0], s_acc[1]);
        } else {
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
#pragma unroll
                for (int e = 0; e < 16; ++e) s_acc[jt][e] = 0.f;
        }
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
            for (int c = 0; c < 4; ++c) s_acc[jt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[jt][c], qb[c], s_acc[jt], 0, 0, 0);
        if (HAS_P2C) {
            const uint32_t paddr = lds_addr(&sm.p[32 * w + il + 63 + 4 * hh * (PS - 1)]);
#pragma unroll
            for (int jt = 0; jt < 2; ++jt) {
                uint32_t g[16];
                static_for<16>([&](auto ec) {
                    constexpr int e = decltype(ec)::value, jc0 = 8 * (e >> 2) + (e & 3);
                    g[e] = jt == 0 ? lds_read_u16<2 * jc0 * (PS - 1)>(paddr) : lds_read_u16<2 * (32 + jc0) * (PS - 1)>(paddr);
                });
                lds_wait(g);
#pragma unroll
                for (int e = 0; e < 16; ++e)   // bf16 pair (value, 0) . (1, 1) + acc
                    s_acc[jt][e] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, g[e]), ones, s_acc[jt][e], false);
            }
        }
        TDB_TICK(4);
        // ---- mask keys past the end of the sequence (last step only) ------------------------------------------
        if (j0 + BN > len) {
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int j = j0 + 32 * jt + 8 * (e >> 2) + 4 * hh + (e & 3);
                    if (j >= len) s_acc[jt][e] = -INFINITY;
                }
        }
        // ---- streaming softmax: this lane holds 32 of the 64 keys of query row il, lane^32 the others -------
        float mx = s_acc[0][0];
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s_acc[jt][e]);
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);          // finite: key j0 < len is never masked
        const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c_exp);
        const float mc = m_new * c_exp;
        m_run = m_new;
        float psum = 0.f;
        bf16x8 pb[2][2];   // B operand of P.V: [key tile][16-key chunk]
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                float pe[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    pe[e] = __builtin_amdgcn_exp2f(fmaf(s_acc[jt][8 * c + e], c_exp, -mc));
                    psum += pe[e];
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) pb[jt][c][e] = (__bf16)pe[e];
            }
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) o_acc[t][e] *= alpha;

        TDB_TICK(5);
        // ---- O^T += V^T.P^T; V^T fragments come from row-major V through the transposing LDS read ----------
        {
            const int g = l >> 4, ll = l & 15;
            // source address of this lane inside a 4-key x 16-dim block: row (ll>>2), 4 dims at 4*(ll&3)
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
                        const __attribute__((ext_vector_type(8))) short both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                        o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pb[jt][c], o_acc[dt], 0, 0, 0);
                    }
        }

        TDB_TICK(6);
        // ---- hand the prefetched next step to LDS and start fetching the one after -------------------------
        if (s + 1 < nsteps) {
            off = off >= BN ? off - BN : off + WIN - BN;
            __syncthreads();              // every wave is done with this step's tiles
            store_step(off);
            __syncthreads();
            if (s + 2 < nsteps) {
                fetch_step(s + 2);
                fetch_delta(s + 3);
            }
        }
        TDB_TICK(7);
    }

    // ---- epilogue: normalise and store O[i][d]; lane holds d = 32*dt + 8*a + 4*hh + 0..3 of query row il ------
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv = 1.f / l_tot;
    if (qi < row0 + rows_here) {
        const bool live = qi < len;
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                u32x2 r = {0, 0};
                if (live) r = pack4(o_acc[dt][4 * a] * inv, o_acc[dt][4 * a + 1] * inv, o_acc[dt][4 * a + 2] * inv, o_acc[dt][4 * a + 3] * inv);
                *reinterpret_cast<u32x2*>(O + int64_t(qi) * p.os_l + 32 * dt + 8 * a + 4 * hh) = r;
            }
    }
}

}  // namespace

bool tdb_mfma_supported(const TdbKernelParams& p, int dtype) {
    // bf16, head_dim 64, position terms as fused tables (or none); strips go to the generic kernel
    return dtype == TDB_BF16 && p.D == 64 && !p.c2p && !p.p2c;
}

hipError_t tdb_launch_mfma(const TdbKernelParams& p, int, hipStream_t stream) {
    const int tiles = p.varlen ? p.total / BM + p.B : p.B * ((p.L + BM - 1) / BM);
    const dim3 grid(tiles, p.H), block(256);
    const size_t smem = sizeof(Smem);
    const bool c2p = p.pk != nullptr, p2c = p.pq != nullptr;
#define TDB_LAUNCH(A, B)                                                                                        \
    do {                                                                                                        \
        static bool attr_set = false;                                                                           \
        if (!attr_set) {                                                                                        \
            hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_mfma_kernel<A, B>),                         \
                                hipFuncAttributeMaxDynamicSharedMemorySize, int(smem));                         \
            attr_set = true;                                                                                    \
        }                                                                                                       \
        hipLaunchKernelGGL((attn_mfma_kernel<A, B>), grid, block, smem, stream, p);                             \
    } while (0)
    if (c2p && p2c) TDB_LAUNCH(true, true);
    else if (c2p) TDB_LAUNCH(true, false);
    else if (p2c) TDB_LAUNCH(false, true);
    else TDB_LAUNCH(false, false);
#undef TDB_LAUNCH
    return hipGetLastError();
}
