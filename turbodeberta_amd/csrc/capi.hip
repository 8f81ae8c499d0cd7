// C-ABI front end of libtdb_attn.so: argument validation (host only, testable without a GPU),
// the relative-position tables, and the two launch entry points.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "tdb_internal.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

size_t elem_size(int dtype) { return dtype == TDB_F32 ? 4 : 2; }

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// a stride (in elements) that keeps every row start 16-byte aligned
bool stride_ok(int64_t s, int dtype) { return s >= 0 && (s * int64_t(elem_size(dtype))) % 16 == 0; }

constexpr int32_t kMaxLen = 1 << 20;

// Smallest distance of a ceil() argument to an integer that is still trusted.  float32 evaluation
// of log(a/mid)/log((P-1)/mid)*(mid-1) is off by a few ulps of a value below 2^10, i.e. < 3e-6.
constexpr double kMargin = 3e-5;

int check_common(int dtype, int batch, int heads, int head_dim, int len, int causal, const void* q, const void* k,
                 const void* v, const void* o) {
    if (dtype != TDB_F32 && dtype != TDB_BF16 && dtype != TDB_F16) return fail(TDB_ERR_DTYPE, "unknown dtype %d", dtype);
    if (batch < 0 || heads < 1 || heads > 65535) return fail(TDB_ERR_SHAPE, "bad batch %d / heads %d", batch, heads);
    if (head_dim < 8 || head_dim > 256 || head_dim % 8) return fail(TDB_ERR_SHAPE, "head_dim %d: need a multiple of 8 in [8, 256]", head_dim);
    if (len < 1 || len > kMaxLen) return fail(TDB_ERR_SHAPE, "sequence length %d out of range [1, %d]", len, kMaxLen);
    if (causal) return fail(TDB_ERR_CAUSAL, "causal attention is not supported");
    if (!q || !k || !v || !o) return fail(TDB_ERR_NULL, "q, k, v and o must be non-NULL");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o)) return fail(TDB_ERR_ALIGN, "q, k, v, o must be 16-byte aligned");
    return TDB_OK;
}

int check_pos(const tdb_pos_args& ps, int dtype, int len, bool varlen) {
    const bool any = ps.pos_key || ps.pos_query || ps.c2p_strip || ps.p2c_strip;
    if (!any) return TDB_OK;
    if ((ps.pos_key && ps.c2p_strip) || (ps.pos_query && ps.p2c_strip))
        return fail(TDB_ERR_POSITION, "a term takes either a fused table or a strip, not both");
    if (ps.span < 1 || ps.span > (1 << 20)) return fail(TDB_ERR_POSITION, "span %d out of range", ps.span);
    if (!ps.delta_lut) return fail(TDB_ERR_POSITION, "delta_lut is required when a position term is on");
    if (ps.lut_half < len - 1) return fail(TDB_ERR_POSITION, "delta_lut covers |r| <= %d but sequences reach %d", ps.lut_half, len - 1);
    const void* ptrs[4] = {ps.pos_key, ps.pos_query, ps.c2p_strip, ps.p2c_strip};
    for (const void* p : ptrs)
        if (p && !aligned16(p)) return fail(TDB_ERR_ALIGN, "position inputs must be 16-byte aligned");
    if (ps.pos_key && !(stride_ok(ps.pos_key_stride_h, dtype) && stride_ok(ps.pos_key_stride_r, dtype)))
        return fail(TDB_ERR_STRIDE, "pos_key strides must be non-negative multiples of 16 bytes");
    if (ps.pos_query && !(stride_ok(ps.pos_query_stride_h, dtype) && stride_ok(ps.pos_query_stride_r, dtype)))
        return fail(TDB_ERR_STRIDE, "pos_query strides must be non-negative multiples of 16 bytes");
    if (ps.c2p_strip && (ps.c2p_stride_h < 0 || ps.c2p_stride_l < 0 || (!varlen && ps.c2p_stride_b < 0)))
        return fail(TDB_ERR_STRIDE, "negative c2p strip stride");
    if (ps.p2c_strip && (ps.p2c_stride_h < 0 || ps.p2c_stride_l < 0 || (!varlen && ps.p2c_stride_b < 0)))
        return fail(TDB_ERR_STRIDE, "negative p2c strip stride");
    return TDB_OK;
}

void fill_pos(TdbKernelParams& kp, const tdb_pos_args& ps) {
    kp.span = ps.span;
    kp.lut_half = ps.lut_half;
    kp.lut = ps.delta_lut;
    kp.pk = ps.pos_key;
    kp.pq = ps.pos_query;
    kp.pks_h = ps.pos_key_stride_h;
    kp.pks_r = ps.pos_key_stride_r;
    kp.pqs_h = ps.pos_query_stride_h;
    kp.pqs_r = ps.pos_query_stride_r;
    kp.c2p = ps.c2p_strip;
    kp.p2c = ps.p2c_strip;
    kp.c2s_b = ps.c2p_stride_b;
    kp.c2s_h = ps.c2p_stride_h;
    kp.c2s_l = ps.c2p_stride_l;
    kp.p2s_b = ps.p2c_stride_b;
    kp.p2s_h = ps.p2c_stride_h;
    kp.p2s_l = ps.p2c_stride_l;
}

int dispatch(const TdbKernelParams& kp, int dtype, int flags, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (!(flags & TDB_FLAG_FORCE_GENERIC) && tdb_mfma_supported(kp, dtype))
        e = tdb_launch_mfma(kp, dtype, s);
    else
        e = tdb_launch_generic(kp, dtype, s);
    if (e != hipSuccess) return fail(TDB_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return TDB_OK;
}

// One relative position through the log-bucket map.  `exact` is cleared when the float32 and the
// float64 evaluations could disagree on a value that survives the clamp to [-span, span-1].
int32_t bucket_one(int32_t r, int32_t buckets, int32_t max_pos, bool& exact) {
    if (buckets <= 0 || max_pos <= 0) return r;
    const int32_t mid = buckets / 2;
    const int32_t a = r < 0 ? -r : r;
    const int32_t abs_pos = (r < mid && r > -mid) ? mid - 1 : a;
    if (abs_pos <= mid) return r;
    const float den_f = logf(float(double(max_pos - 1) / double(mid)));
    const float num_f = logf(float(abs_pos) / float(mid));
    const float x_f = num_f / den_f * float(mid - 1);
    const int32_t b_f = int32_t(ceilf(x_f)) + mid;
    const double x_d = std::log(double(abs_pos) / mid) / std::log(double(max_pos - 1) / mid) * (mid - 1);
    if (x_d < double(buckets - mid) + 0.5) {          // the value can still land below the clamp
        if (abs_pos == max_pos - 1) {
            // log(x)/log(x) of the same float32 value is exactly 1: the result is mid - 1 by construction
            if (float(abs_pos) / float(mid) != float(double(max_pos - 1) / double(mid))) exact = false;
        } else {
            const double frac = std::fabs(x_d - std::nearbyint(x_d));
            if (frac < kMargin || b_f != int32_t(std::ceil(x_d)) + mid) exact = false;
        }
    }
    return r < 0 ? -b_f : b_f;
}

}  // namespace

extern "C" {

int tdb_version(void) { return TDB_ABI_VERSION; }

const char* tdb_last_error(void) { return g_err; }

int tdb_bucket_table(int32_t* out, int32_t max_len, int32_t position_buckets, int32_t max_position) {
    if (!out) return fail(TDB_ERR_NULL, "out is NULL");
    if (max_len < 1 || max_len > kMaxLen) return fail(TDB_ERR_SHAPE, "max_len %d out of range", max_len);
    bool exact = true;
    for (int32_t r = -(max_len - 1); r <= max_len - 1; ++r) out[r + max_len - 1] = bucket_one(r, position_buckets, max_position, exact);
    if (!exact)
        return fail(TDB_ERR_BUCKET_MARGIN, "bucket(%d, %d): a ceil() argument is within 3e-5 of an integer; table withheld",
                    position_buckets, max_position);
    return TDB_OK;
}

int tdb_delta_table(int32_t* out, int32_t max_len, int32_t position_buckets, int32_t max_position) {
    const int32_t span = position_buckets > 0 ? position_buckets : max_position;
    if (span < 1) return fail(TDB_ERR_POSITION, "span %d: need position_buckets > 0 or max_position > 0", span);
    const int rc = tdb_bucket_table(out, max_len, position_buckets, max_position);
    if (rc != TDB_OK) return rc;
    for (int32_t i = 0; i < 2 * max_len - 1; ++i) {
        const int64_t d = int64_t(out[i]) + span;
        out[i] = int32_t(d < 0 ? 0 : (d > 2 * int64_t(span) - 1 ? 2 * int64_t(span) - 1 : d));
    }
    return TDB_OK;
}

int tdb_check_cu_seqlens(const int32_t* cu, int32_t batch, int32_t total_tokens, int32_t max_seqlen) {
    if (!cu) return fail(TDB_ERR_NULL, "cu_seqlens is NULL");
    if (batch < 0) return fail(TDB_ERR_SHAPE, "negative batch");
    if (cu[0] != 0) return fail(TDB_ERR_CU_SEQLENS, "cu_seqlens[0] = %d, expected 0", cu[0]);
    for (int32_t b = 0; b < batch; ++b) {
        const int64_t n = int64_t(cu[b + 1]) - cu[b];
        if (n < 0) return fail(TDB_ERR_CU_SEQLENS, "cu_seqlens decreases at %d", b + 1);
        if (n > max_seqlen) return fail(TDB_ERR_CU_SEQLENS, "sequence %d has %lld tokens > max_seqlen %d", b, (long long)n, max_seqlen);
    }
    if (cu[batch] != total_tokens) return fail(TDB_ERR_CU_SEQLENS, "cu_seqlens[%d] = %d, expected total_tokens %d", batch, cu[batch], total_tokens);
    return TDB_OK;
}

int tdb_set_workgroup_limit(int workgroups) { return tdb_mfma_set_workgroup_limit(workgroups); }

int tdb_attn_fwd_fixed(const tdb_fixed_args* a, void* stream) {
    if (!a) return fail(TDB_ERR_NULL, "args is NULL");
    int rc = check_common(a->dtype, a->batch, a->heads, a->head_dim, a->seqlen, a->causal, a->q, a->k, a->v, a->o);
    if (rc != TDB_OK) return rc;
    const int64_t* st[4] = {&a->q_stride_b, &a->k_stride_b, &a->v_stride_b, &a->o_stride_b};
    for (auto s : st)
        if (!stride_ok(s[0], a->dtype) || !stride_ok(s[1], a->dtype) || !stride_ok(s[2], a->dtype) || s[2] < a->head_dim)
            return fail(TDB_ERR_STRIDE, "q/k/v/o strides must be multiples of 16 bytes with row stride >= head_dim");
    rc = check_pos(a->pos, a->dtype, a->seqlen, false);
    if (rc != TDB_OK) return rc;
    if (a->batch == 0) return TDB_OK;

    TdbKernelParams kp;
    memset(&kp, 0, sizeof(kp));
    kp.q = a->q; kp.k = a->k; kp.v = a->v; kp.o = a->o;
    kp.qs_b = a->q_stride_b; kp.qs_h = a->q_stride_h; kp.qs_l = a->q_stride_l;
    kp.ks_b = a->k_stride_b; kp.ks_h = a->k_stride_h; kp.ks_l = a->k_stride_l;
    kp.vs_b = a->v_stride_b; kp.vs_h = a->v_stride_h; kp.vs_l = a->v_stride_l;
    kp.os_b = a->o_stride_b; kp.os_h = a->o_stride_h; kp.os_l = a->o_stride_l;
    kp.seqlens = a->seqlens_k;
    kp.B = a->batch; kp.H = a->heads; kp.D = a->head_dim; kp.L = a->seqlen;
    kp.scale = a->sm_scale;
    fill_pos(kp, a->pos);
    return dispatch(kp, a->dtype, a->flags, stream);
}

int tdb_attn_fwd_varlen(const tdb_varlen_args* a, void* stream) {
    if (!a) return fail(TDB_ERR_NULL, "args is NULL");
    if (a->total_tokens < 0) return fail(TDB_ERR_SHAPE, "negative total_tokens");
    int rc = check_common(a->dtype, a->batch, a->heads, a->head_dim, a->max_seqlen, a->causal, a->q, a->k, a->v, a->o);
    if (rc != TDB_OK) return rc;
    if (!a->cu_seqlens) return fail(TDB_ERR_NULL, "cu_seqlens is NULL");
    const int64_t* st[4] = {&a->q_stride_t, &a->k_stride_t, &a->v_stride_t, &a->o_stride_t};
    for (auto s : st)
        if (!stride_ok(s[0], a->dtype) || !stride_ok(s[1], a->dtype) || s[0] < a->head_dim)
            return fail(TDB_ERR_STRIDE, "q/k/v/o strides must be multiples of 16 bytes with token stride >= head_dim");
    rc = check_pos(a->pos, a->dtype, a->max_seqlen, true);
    if (rc != TDB_OK) return rc;
    if (a->batch == 0 || a->total_tokens == 0) return TDB_OK;

    TdbKernelParams kp;
    memset(&kp, 0, sizeof(kp));
    kp.q = a->q; kp.k = a->k; kp.v = a->v; kp.o = a->o;
    kp.qs_h = a->q_stride_h; kp.qs_l = a->q_stride_t;
    kp.ks_h = a->k_stride_h; kp.ks_l = a->k_stride_t;
    kp.vs_h = a->v_stride_h; kp.vs_l = a->v_stride_t;
    kp.os_h = a->o_stride_h; kp.os_l = a->o_stride_t;
    kp.cu_seqlens = a->cu_seqlens;
    kp.B = a->batch; kp.H = a->heads; kp.D = a->head_dim; kp.L = a->max_seqlen;
    kp.total = a->total_tokens;
    kp.varlen = 1;
    kp.scale = a->sm_scale;
    fill_pos(kp, a->pos);
    return dispatch(kp, a->dtype, a->flags, stream);
}

}  // extern "C"
