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

// Maps blockIdx.x to (sequence, first row of the tile, valid length).  Returns false when the
// block has no tile (packed launches are sized by an upper bound on the tile count).
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
    int t = block;
    for (b = 0; b < p.B; ++b) {
        const int s = p.cu_seqlens[b], e = p.cu_seqlens[b + 1];
        int n = e - s;
        if (s < 0 || n < 0 || e > p.total) n = 0;       // malformed entry: no tiles
        n = min(n, p.L);
        const int nt = (n + tile_rows - 1) / tile_rows;
        if (t < nt) {
            row0 = t * tile_rows;
            len = n;
            tok0 = s;
            return true;
        }
        t -= nt;
    }
    return false;
}
