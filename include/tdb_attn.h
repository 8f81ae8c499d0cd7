/*
 * tdb_attn.h -- C ABI of libtdb_attn.so: fused DeBERTa-v2/v3 disentangled-attention forward
 * for AMD MI355X (gfx950).
 *
 * The library is the device half of TurboDeBERTa's attention operators.  Every entry point
 * takes plain pointers and sizes; device buffers are owned by the caller, the library never
 * allocates, frees or synchronises, and every launch goes to the hipStream_t the caller passes
 * (as a void* so that this header needs no HIP include).  Functions return TDB_OK or a negative
 * TDB_ERR_* code and never throw; tdb_last_error() gives the thread's last message.
 *
 * Citations name the reference interface each entry point stands in for
 * (paths relative to the TurboDeBERTa source tree).
 */
#ifndef TDB_ATTN_H
#define TDB_ATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TDB_ABI_VERSION 2

/* status codes */
#define TDB_OK                 0
#define TDB_ERR_NULL          (-1)  /* a required pointer is NULL                                */
#define TDB_ERR_DTYPE         (-2)  /* dtype is not one of TDB_F32 / TDB_BF16 / TDB_F16          */
#define TDB_ERR_SHAPE         (-3)  /* a size is non-positive, too large, or head_dim unsupported */
#define TDB_ERR_STRIDE        (-4)  /* a stride is negative or breaks 16-byte row alignment      */
#define TDB_ERR_ALIGN         (-5)  /* a base pointer is not 16-byte aligned                     */
#define TDB_ERR_CAUSAL        (-6)  /* causal != 0 (the reference never enables it either)       */
#define TDB_ERR_CU_SEQLENS    (-7)  /* cu_seqlens not starting at 0, decreasing, or past total   */
#define TDB_ERR_POSITION      (-8)  /* inconsistent position inputs (span, table, LUT length)    */
#define TDB_ERR_BUCKET_MARGIN (-9)  /* log-bucket ceil() argument too close to an integer        */
#define TDB_ERR_LAUNCH        (-10) /* HIP reported an error at launch                           */

/* element types of q, k, v, o and of the position tables / strips */
#define TDB_F32  0
#define TDB_BF16 1
#define TDB_F16  2

/* bits of the `flags` field */
#define TDB_FLAG_FORCE_GENERIC 1  /* run the vector-ALU kernel even where the matrix-core kernel applies */

/*
 * Position inputs shared by both entry points.  Two modes, chosen per term:
 *
 *  fused   pos_key / pos_query point at the per-head projections of the first 2*span rows of the
 *          relative-embedding table, K_r = key_proj(rel) and Q_r = query_proj(rel), laid out
 *          [heads, 2*span, head_dim] with the element strides given.  The kernel contracts them
 *          with Q / K on the matrix cores; no [L, 2*span] strip ever exists in HBM.
 *  strip   c2p_strip / p2c_strip point at the strips the reference glue materialises
 *          (model.py:122-125, :146-148): Q.K_r^T and K.Q_r^T, [batch, heads, L, 2*span]
 *          (fixed) or [total, heads, 2*span] (varlen).  The kernel only gathers from them
 *          (on the matrix-core kernel when both terms are 16-bit strips and head_dim is 64).
 *
 * For score position (i, j) both terms use column delta(i - j) = delta_lut[i - j + lut_half],
 * the clamp(bucket(i - j) + span, 0, 2*span - 1) of Hugging Face's eager code
 * (modeling_deberta_v2.py:318 and :336-343).  A NULL pointer pair switches a term off.
 */
typedef struct tdb_pos_args {
    int32_t        span;          /* att_span: position_buckets if > 0 else max_relative_positions */
    int32_t        lut_half;      /* delta_lut covers r in [-lut_half, lut_half]; >= max len - 1    */
    const int32_t* delta_lut;     /* device, [2*lut_half + 1], from tdb_delta_table()               */
    const void*    pos_key;       /* device, K_r [heads, 2*span, head_dim]  (c2p, fused)            */
    const void*    pos_query;     /* device, Q_r [heads, 2*span, head_dim]  (p2c, fused)            */
    int64_t        pos_key_stride_h, pos_key_stride_r;      /* element strides: head, row           */
    int64_t        pos_query_stride_h, pos_query_stride_r;
    const void*    c2p_strip;     /* device, strip mode, see above                                  */
    const void*    p2c_strip;
    int64_t        c2p_stride_b, c2p_stride_h, c2p_stride_l; /* fixed: batch, head, row; varlen:    */
    int64_t        p2c_stride_b, p2c_stride_h, p2c_stride_l; /* stride_b ignored, stride_l = token  */
} tdb_pos_args;

/*
 * Fixed-length call.  Replaces the device side of flash_attention_with_disentangled
 * (ops/flash_attention.py:345-369) / flash_attn_v2_fwd_dise (:221-316).
 * q, k, v, o: [batch, heads, seqlen, head_dim] addressed by element strides (last dim
 * contiguous), so both [B,H,L,D] and the projection-native [B,L,H,D] work without a copy.
 * seqlens_k (optional, device int32 [batch]): valid length of each right-padded sequence; keys
 * j >= len are masked (what HF's m_i*m_j mask does for valid rows) and query rows i >= len are
 * written as zeros (what the reference's re-padding produces, padding.py:11-15).
 */
typedef struct tdb_fixed_args {
    int32_t dtype, batch, heads, head_dim, seqlen, causal, flags;
    float   sm_scale;
    const void *q, *k, *v;
    void*   o;
    int64_t q_stride_b, q_stride_h, q_stride_l;
    int64_t k_stride_b, k_stride_h, k_stride_l;
    int64_t v_stride_b, v_stride_h, v_stride_l;
    int64_t o_stride_b, o_stride_h, o_stride_l;
    const int32_t* seqlens_k;
    tdb_pos_args pos;
} tdb_fixed_args;

/*
 * Packed variable-length call.  Replaces the device side of
 * flash_attention_with_disentangled_varlen (ops/flash_attention_varlen.py:348-374) including the
 * host-built tile work list get_mid (:10-22): tiles are mapped to sequences on the device from
 * cu_seqlens, with no host synchronisation.
 * q, k, v, o: [total_tokens, heads, head_dim]; cu_seqlens: device int32 [batch + 1], starts at 0,
 * non-decreasing, last entry == total_tokens; every length <= max_seqlen.  Relative positions
 * are in-sequence offsets (ops/flash_attention_varlen.py:70,118).
 */
typedef struct tdb_varlen_args {
    int32_t dtype, batch, heads, head_dim, total_tokens, max_seqlen, causal, flags;
    float   sm_scale;
    const void *q, *k, *v;
    void*   o;
    int64_t q_stride_t, q_stride_h;
    int64_t k_stride_t, k_stride_h;
    int64_t v_stride_t, v_stride_h;
    int64_t o_stride_t, o_stride_h;
    const int32_t* cu_seqlens;
    tdb_pos_args pos;
} tdb_varlen_args;

/* ABI version of the loaded library (== TDB_ABI_VERSION of the header it was built from). */
int tdb_version(void);

/* Message of the calling thread's last failing call ("" if none).  Never NULL. */
const char* tdb_last_error(void);

/* Launch the fixed-length forward on `stream` (a hipStream_t; NULL = the null stream). */
int tdb_attn_fwd_fixed(const tdb_fixed_args* args, void* stream);

/* Launch the packed variable-length forward on `stream`. */
int tdb_attn_fwd_varlen(const tdb_varlen_args* args, void* stream);

/*
 * Host-only.  Signed log-bucket of every r in [-(max_len-1), max_len-1] into out[r + max_len-1]:
 * Hugging Face's make_log_bucket_position (modeling_deberta_v2.py:57-69), which the reference
 * kernel re-evaluates per score element (ops/flash_attention.py:100-115).  Identity when
 * position_buckets <= 0 or max_position <= 0 (modeling_deberta_v2.py:96).  Evaluated in float32
 * and cross-checked in float64; returns TDB_ERR_BUCKET_MARGIN if any ceil() argument that can
 * affect the clamped index lies within 3e-5 of an integer (ten times the float32 evaluation
 * error), because then the result would depend on the logf implementation; no table is produced.
 */
int tdb_bucket_table(int32_t* out, int32_t max_len, int32_t position_buckets, int32_t max_position);

/*
 * Host-only.  delta(r) = clamp(bucket(r) + span, 0, 2*span - 1), span = position_buckets if > 0
 * else max_position, for r in [-(max_len-1), max_len-1] into out[r + max_len - 1].
 * This is the table tdb_pos_args.delta_lut expects (copied to the device by the caller).
 */
int tdb_delta_table(int32_t* out, int32_t max_len, int32_t position_buckets, int32_t max_position);

/*
 * Host-only.  Checks a HOST copy of cu_seqlens the way the launchers assume it:
 * cu[0] == 0, non-decreasing, cu[batch] == total_tokens, every length <= max_seqlen.
 * Returns TDB_OK or TDB_ERR_CU_SEQLENS.  (The launchers cannot check device memory without a
 * synchronisation; on the device a malformed entry makes that sequence's tiles exit early.)
 */
int tdb_check_cu_seqlens(const int32_t* cu_seqlens_host, int32_t batch, int32_t total_tokens, int32_t max_seqlen);

/*
 * Process-wide cap on the persistent workgroups (one per compute unit) that a matrix-core launch
 * starts: `workgroups` is rounded down to a multiple of 8 (one per XCD at least: minimum 8);
 * 0 or a negative value lifts the cap (default: every compute unit of the device).  For callers
 * that share the GPU with other streams, and for tests of the packed tile deal at other grid
 * sizes than this device's.  Returns the cap now in force (0 = none).  No counterpart in the
 * reference, whose launch grid is one program per tile (ops/flash_attention.py:360,
 * ops/flash_attention_varlen.py:328).
 */
int tdb_set_workgroup_limit(int workgroups);

#ifdef __cplusplus
}
#endif
#endif /* TDB_ATTN_H */
