// Internal declarations shared by the C-ABI front end and the HIP kernels of libtdb_attn.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tdb_attn.h"

// One flattened description of a launch; fixed-length and packed calls both reduce to it.
// A sequence b starts at element offset  b*stride_b  (fixed)  or  cu_seqlens[b]*stride_l  (packed)
// and its row l, head h lives at  + l*stride_l + h*stride_h.
struct TdbKernelParams {
    const void *q, *k, *v;
    void* o;
    int64_t qs_b, qs_h, qs_l;
    int64_t ks_b, ks_h, ks_l;
    int64_t vs_b, vs_h, vs_l;
    int64_t os_b, os_h, os_l;
    const int32_t* seqlens;     // fixed: [B] valid lengths or nullptr
    const int32_t* cu_seqlens;  // packed: [B+1] or nullptr
    int32_t B, H, D, L;         // L: padded length (fixed) / max_seqlen (packed)
    int32_t total;              // packed: token count
    int32_t varlen;
    float scale;
    // position terms
    int32_t span, lut_half;
    const int32_t* lut;
    const void *pk, *pq;        // fused tables [H, 2*span, D]
    int64_t pks_h, pks_r, pqs_h, pqs_r;
    const void *c2p, *p2c;      // strips
    int64_t c2s_b, c2s_h, c2s_l;
    int64_t p2s_b, p2s_h, p2s_l;
};

// tile heights (query rows per workgroup)
constexpr int TDB_GENERIC_TILE = 16;
constexpr int TDB_MFMA_TILE = 128;

// true when the matrix-core kernel can take this launch
bool tdb_mfma_supported(const TdbKernelParams& p, int dtype);

// launchers; return hipError_t of the launch
hipError_t tdb_launch_generic(const TdbKernelParams& p, int dtype, hipStream_t stream);
hipError_t tdb_launch_mfma(const TdbKernelParams& p, int dtype, hipStream_t stream);
// Cap on the persistent workgroups of a launch (multiple of 8, 0 = none); returns the cap in force.
int tdb_mfma_set_workgroup_limit(int workgroups);

// Maps blockIdx.x to (sequence, first row of the tile, valid length).  Returns false when the
// block has no tile (packed launches are sized by an upper bound on the tile count).  Must be
// called by whole waves with identical arguments.  For packed input the wave scans cu_seqlens 64
// sequences at a time: one load per lane, a prefix sum of the per-sequence tile counts across the
// wave, and a ballot to pick the sequence that owns tile `block` -- no serial chain of dependent
// loads, and no work list built on the host.
__device__ __forceinline__ bool tdb_locate_tile(const TdbKernelParams& p, int tile_rows, int block,
                                                int& b, int& row0, int& len, int64_t& tok0) {
    if (!p.varlen) {
        const int tiles = (p.L + tile_rows - 1) / tile_rows;
        b = block / tiles;
        row0 = (block - b * tiles) * tile_rows;
        len = p.seqlens ? min(max(p.seqlens[b], 0), p.L) : p.L;
        tok0 = 0;
        return true;
    }
    const int lane = threadIdx.x & 63;
    int t = block;
    for (int b0 = 0; b0 < p.B; b0 += 64) {
        const int bb = b0 + lane;
        int s = 0, n = 0;
        if (bb < p.B) {
            s = p.cu_seqlens[bb];
            const int e = p.cu_seqlens[bb + 1];
            n = e - s;
            if (s < 0 || n < 0 || e > p.total) n = 0;   // malformed entry: no tiles
            n = min(n, p.L);
        }
        const int nt = (n + tile_rows - 1) / tile_rows;
        int incl = nt;                                   // inclusive prefix sum over the wave
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        const int chunk_tiles = __builtin_amdgcn_readlane(incl, 63);
        if (t < chunk_tiles) {
            const unsigned long long owners = __builtin_amdgcn_ballot_w64(incl > t);
            const int ln = __builtin_amdgcn_readfirstlane(__builtin_ctzll(owners));
            const int before = __builtin_amdgcn_readlane(incl, ln) - __builtin_amdgcn_readlane(nt, ln);
            b = b0 + ln;
            row0 = (t - before) * tile_rows;
            len = __builtin_amdgcn_readlane(n, ln);
            tok0 = __builtin_amdgcn_readlane(s, ln);
            return true;
        }
        t -= chunk_tiles;
    }
    return false;
}
