// Generic disentangled-attention forward: fp32 arithmetic on the vector ALUs for any element
// type, any head_dim that is a multiple of 8 up to 256, fused tables or precomputed strips.
// It is the path for fp32 inputs (the 1e-4 parity case) and for shapes the matrix-core kernel
// does not take.  One wave owns 4 query rows; lanes run over 64 keys at a time.
//
//   S[i,j] = scale * ( Q_i.K_j + Q_i.K_r[delta] + K_j.Q_r[delta] ),  delta = lut[i - j + lut_half]
// as in Hugging Face's DisentangledSelfAttention (modeling_deberta_v2.py:243, :317-324, :337-343),
// followed by a streaming softmax over the valid keys and P.V.
#include "tdb_internal.h"

namespace {

constexpr int ROWS = 4;     // query rows per wave
constexpr int WAVES = 4;    // waves per workgroup
constexpr int MAXC = 4;     // head_dim <= 64 * MAXC

template <typename T> struct Cvt;
template <> struct Cvt<float> {
    static __device__ __forceinline__ float to_f(float x) { return x; }
    static __device__ __forceinline__ float from_f(float x) { return x; }
};
template <> struct Cvt<uint16_t> {   // bfloat16 bits
    static __device__ __forceinline__ float to_f(uint16_t x) { return __uint_as_float(uint32_t(x) << 16); }
    static __device__ __forceinline__ uint16_t from_f(float f) {   // round to nearest even
        uint32_t u = __float_as_uint(f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x40);
        u += 0x7fffu + ((u >> 16) & 1u);
        return uint16_t(u >> 16);
    }
};
template <> struct Cvt<_Float16> {
    static __device__ __forceinline__ float to_f(_Float16 x) { return float(x); }
    static __device__ __forceinline__ _Float16 from_f(float f) { return _Float16(f); }
};

template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&out)[8]) {
    if constexpr (sizeof(T) == 4) {
        const float4 a = *reinterpret_cast<const float4*>(p);
        const float4 b = *reinterpret_cast<const float4*>(p + 4);
        out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
        out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
    } else {
        union { uint4 v; T e[8]; } u;
        u.v = *reinterpret_cast<const uint4*>(p);
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = Cvt<T>::to_f(u.e[i]);
    }
}

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o));
    return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
    return x;
}

template <typename T>
__global__ __launch_bounds__(WAVES * 64) void attn_generic_kernel(const TdbKernelParams p) {
    extern __shared__ float smem[];
    float* sQ = smem;                                  // [TILE][D]
    float* sP = smem + TDB_GENERIC_TILE * p.D;         // [WAVES][ROWS][64]

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int h = blockIdx.y;
    int b, row0, len;
    int64_t tok0;
    if (!tdb_locate_tile(p, TDB_GENERIC_TILE, blockIdx.x, b, row0, len, tok0)) return;

    const int D = p.D;
    const T* Q = static_cast<const T*>(p.q) + (p.varlen ? tok0 * p.qs_l : int64_t(b) * p.qs_b) + int64_t(h) * p.qs_h;
    const T* K = static_cast<const T*>(p.k) + (p.varlen ? tok0 * p.ks_l : int64_t(b) * p.ks_b) + int64_t(h) * p.ks_h;
    const T* V = static_cast<const T*>(p.v) + (p.varlen ? tok0 * p.vs_l : int64_t(b) * p.vs_b) + int64_t(h) * p.vs_h;
    T* O = static_cast<T*>(p.o) + (p.varlen ? tok0 * p.os_l : int64_t(b) * p.os_b) + int64_t(h) * p.os_h;

    const int tile_rows = p.varlen ? min(TDB_GENERIC_TILE, len - row0) : min(TDB_GENERIC_TILE, p.L - row0);
    const int nchunk = (D + 63) >> 6;

    if (row0 >= len) {   // tile of padded query rows only (fixed layout): zeros
        for (int idx = threadIdx.x; idx < tile_rows * D; idx += blockDim.x)
            O[int64_t(row0 + idx / D) * p.os_l + idx % D] = Cvt<T>::from_f(0.f);
        return;
    }

    for (int idx = threadIdx.x; idx < TDB_GENERIC_TILE * D; idx += blockDim.x) {
        const int r = idx / D, d = idx - r * D;
        const int row = row0 + r;
        sQ[idx] = row < len ? Cvt<T>::to_f(Q[int64_t(row) * p.qs_l + d]) : 0.f;
    }
    __syncthreads();

    const bool fused_c2p = p.pk != nullptr, fused_p2c = p.pq != nullptr;
    const bool strip_c2p = p.c2p != nullptr, strip_p2c = p.p2c != nullptr;
    const bool any_pos = fused_c2p || fused_p2c || strip_c2p || strip_p2c;
    const T* PK = fused_c2p ? static_cast<const T*>(p.pk) + int64_t(h) * p.pks_h : nullptr;
    const T* PQ = fused_p2c ? static_cast<const T*>(p.pq) + int64_t(h) * p.pqs_h : nullptr;
    const T* C2P = strip_c2p ? static_cast<const T*>(p.c2p) + (p.varlen ? tok0 * p.c2s_l : int64_t(b) * p.c2s_b) + int64_t(h) * p.c2s_h : nullptr;
    const T* P2C = strip_p2c ? static_cast<const T*>(p.p2c) + (p.varlen ? tok0 * p.p2s_l : int64_t(b) * p.p2s_b) + int64_t(h) * p.p2s_h : nullptr;

    const int wrow0 = row0 + wave * ROWS;
    float m[ROWS], l[ROWS], acc[ROWS][MAXC];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.f;
#pragma unroll
        for (int c = 0; c < MAXC; ++c) acc[r][c] = 0.f;
    }
    float* myP = sP + wave * ROWS * 64;

    for (int j0 = 0; j0 < len; j0 += 64) {
        const int j = j0 + lane;
        const bool valid = j < len;
        float s[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) s[r] = 0.f;
        if (valid) {
            int dl[ROWS];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const int row = min(wrow0 + r, len - 1);        // rows past the end only mirror the last row
                dl[r] = any_pos ? p.lut[row - j + p.lut_half] : 0;
            }
            const T* kj = K + int64_t(j) * p.ks_l;
            for (int d0 = 0; d0 < D; d0 += 8) {
                float kk[8];
                load8(kj + d0, kk);
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    const float* qq = sQ + (wave * ROWS + r) * D + d0;
                    float t = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) t = fmaf(qq[e], kk[e], t);
                    if (fused_c2p) {
                        float pr[8];
                        load8(PK + int64_t(dl[r]) * p.pks_r + d0, pr);
#pragma unroll
                        for (int e = 0; e < 8; ++e) t = fmaf(qq[e], pr[e], t);
                    }
                    if (fused_p2c) {
                        float pr[8];
                        load8(PQ + int64_t(dl[r]) * p.pqs_r + d0, pr);
#pragma unroll
                        for (int e = 0; e < 8; ++e) t = fmaf(kk[e], pr[e], t);
                    }
                    s[r] += t;
                }
            }
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const int row = min(wrow0 + r, len - 1);
                if (strip_c2p) s[r] += Cvt<T>::to_f(C2P[int64_t(row) * p.c2s_l + dl[r]]);
                if (strip_p2c) s[r] += Cvt<T>::to_f(P2C[int64_t(j) * p.p2s_l + dl[r]]);
                s[r] *= p.scale;
            }
        } else {
#pragma unroll
            for (int r = 0; r < ROWS; ++r) s[r] = -INFINITY;
        }

        __syncthreads();   // previous chunk's probabilities have been consumed
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const float mn = fmaxf(m[r], wave_max(s[r]));
            const float alpha = expf(m[r] - mn);        // m = -inf on the first chunk gives 0
            const float pr = valid ? expf(s[r] - mn) : 0.f;
            l[r] = l[r] * alpha + wave_sum(pr);
#pragma unroll
            for (int c = 0; c < MAXC; ++c) acc[r][c] *= alpha;
            m[r] = mn;
            myP[r * 64 + lane] = pr;
        }
        __syncthreads();

        const int nj = min(64, len - j0);
        for (int jj = 0; jj < nj; ++jj) {
            const T* vrow = V + int64_t(j0 + jj) * p.vs_l;
            float pj[ROWS];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) pj[r] = myP[r * 64 + jj];
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                const int d = lane + 64 * c;
                if (c < nchunk && d < D) {
                    const float vv = Cvt<T>::to_f(vrow[d]);
#pragma unroll
                    for (int r = 0; r < ROWS; ++r) acc[r][c] = fmaf(pj[r], vv, acc[r][c]);
                }
            }
        }
    }

#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int row = wrow0 + r;
        if (row >= row0 + tile_rows) continue;
        const float inv = row < len ? 1.f / l[r] : 0.f;
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            const int d = lane + 64 * c;
            if (c < nchunk && d < D) O[int64_t(row) * p.os_l + d] = Cvt<T>::from_f(row < len ? acc[r][c] * inv : 0.f);
        }
    }
}

}  // namespace

hipError_t tdb_launch_generic(const TdbKernelParams& p, int dtype, hipStream_t stream) {
    const int tiles = p.varlen ? p.total / TDB_GENERIC_TILE + p.B
                               : p.B * ((p.L + TDB_GENERIC_TILE - 1) / TDB_GENERIC_TILE);
    const dim3 grid(tiles, p.H), block(WAVES * 64);
    const size_t smem = sizeof(float) * (size_t(TDB_GENERIC_TILE) * p.D + WAVES * ROWS * 64);
    switch (dtype) {
        case TDB_F32: hipLaunchKernelGGL(attn_generic_kernel<float>, grid, block, smem, stream, p); break;
        case TDB_BF16: hipLaunchKernelGGL(attn_generic_kernel<uint16_t>, grid, block, smem, stream, p); break;
        default: hipLaunchKernelGGL(attn_generic_kernel<_Float16>, grid, block, smem, stream, p); break;
    }
    return hipGetLastError();
}
