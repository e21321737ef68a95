/*
 * CPU oracle for the loopback data plane -- see hccl_oracle.h.  TEST INFRASTRUCTURE ONLY:
 * nothing under hccl_amd/ may link, load or call this file.
 *
 * "wrapper.cc" below is the reference file
 *   src/ops/op_common/algorithm/template/wrapper/alg_data_trans_wrapper.cc
 * and "template_utils.cc" is
 *   src/ops/op_common/algorithm/template/template_utils.cc.
 *
 * Parity status per function group:
 *   pinned   : orc_fp16_to_fp32 / orc_fp32_to_fp16 (exhaustive numpy float16 tables + NaN /
 *              boundary known answers), orc_aicpu_reduce (closed forms: modular integer
 *              arithmetic, single IEEE operations, enumerated +-0 / NaN / tie cases), the RHD /
 *              NHR step geometry (hand tables and invariants of the reference's unit tests),
 *              every executor's association order (brute force on tiny inputs against the
 *              order written in the reference's templates and worked examples), copies and
 *              packs (index-map brute force).
 *   unpinned : int16 and bf16 pairwise arithmetic and fp16 SUM/MAX/MIN on the device path
 *              (the reference computes them in libhcomm / DMA hardware that is not in its
 *              tree and no reference test holds a numeric answer).  Rules used: int16 wraps
 *              like int8 / int32; bf16 follows the fp16 host pattern; ORC_ACC_FP32 is the
 *              fp32-accumulated result the kernels are compared against.
 */
#include "hccl_oracle.h"

#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------------------------------------
 * dtype table (reference src/ops/op_common/inc/alg_param.h:55-73)
 * ------------------------------------------------------------------------------------------- */
size_t orc_dtype_size(int dtype)
{
    static const size_t sizes[18] = {1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 2, 1, 1, 1, 1};
    if (dtype < 0 || dtype >= 18) {
        return 0;
    }
    return sizes[dtype];
}

static uint32_t f2u(float f)
{
    uint32_t u;
    memcpy(&u, &f, sizeof(u));
    return u;
}

static float u2f(uint32_t u)
{
    float f;
    memcpy(&f, &u, sizeof(f));
    return f;
}

/* ---------------------------------------------------------------------------------------------
 * a2: fp16 <-> fp32 (wrapper.cc:1082-1235)
 * ------------------------------------------------------------------------------------------- */

/* wrapper.cc:1082-1152.  Zero keeps its sign; subnormals are renormalised; Inf / NaN keep the
 * 10 mantissa bits in the top of the fp32 mantissa. */
float orc_fp16_to_fp32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h >> 15) & 1u;
    uint32_t exponent = ((uint32_t)h >> 10) & 0x1Fu;
    uint32_t mantissa = (uint32_t)h & 0x3FFu;
    if (exponent == 0) {
        if (mantissa == 0) {
            return u2f(sign << 31);
        }
        int shift = 0;
        while ((mantissa & 0x400u) == 0) {
            mantissa <<= 1;
            shift++;
        }
        mantissa &= 0x3FFu;
        int32_t e32 = 127 - 15 + 1 - shift;
        if (e32 <= 0) {
            return u2f(sign << 31);
        }
        return u2f((sign << 31) | ((uint32_t)e32 << 23) | (mantissa << 13));
    }
    if (exponent == 0x1Fu) {
        return u2f((sign << 31) | (0xFFu << 23) | (mantissa << 13));
    }
    return u2f((sign << 31) | ((exponent + 112u) << 23) | (mantissa << 13));
}

/* wrapper.cc:1158-1179: fp32 normal that lands in the fp16 subnormal range; round to nearest
 * even on the shifted-out bits; a carry out of the mantissa becomes the smallest normal. */
static uint16_t fp32_denorm_to_fp16(uint32_t sign, uint32_t mantissa, int32_t e16)
{
    if (e16 < -10) {
        return (uint16_t)(sign << 15);
    }
    mantissa |= 0x800000u;
    int32_t shift = 14 - e16;
    uint32_t roundBit = (mantissa >> (shift - 1)) & 1u;
    uint32_t sticky = (mantissa & ((1u << (shift - 1)) - 1u)) != 0;
    uint16_t m16 = (uint16_t)(mantissa >> shift);
    m16 = (uint16_t)(m16 + (roundBit && (sticky || (m16 & 1u))));
    if (m16 & 0x400u) {
        return (uint16_t)((sign << 15) | (1u << 10));
    }
    return (uint16_t)((sign << 15) | m16);
}

/* wrapper.cc:1181-1235.  fp32 zero / subnormal -> signed zero; Inf -> Inf; NaN keeps the top
 * 10 mantissa bits, forced to 1 if they are all zero; overflow saturates to Inf; otherwise
 * round to nearest even with carry into the exponent. */
uint16_t orc_fp32_to_fp16(float f)
{
    uint32_t bits = f2u(f);
    uint32_t sign = (bits >> 31) & 1u;
    uint32_t exponent = (bits >> 23) & 0xFFu;
    uint32_t mantissa = bits & 0x7FFFFFu;
    if (exponent == 0) {
        return (uint16_t)(sign << 15);
    }
    if (exponent == 0xFFu) {
        if (mantissa == 0) {
            return (uint16_t)((sign << 15) | 0x7C00u);
        }
        uint16_t m16 = (uint16_t)(mantissa >> 13);
        if (m16 == 0) {
            m16 = 1;
        }
        return (uint16_t)((sign << 15) | 0x7C00u | m16);
    }
    int32_t e16 = (int32_t)exponent - 127 + 15;
    if (e16 >= 31) {
        return (uint16_t)((sign << 15) | 0x7C00u);
    }
    if (e16 <= 0) {
        return fp32_denorm_to_fp16(sign, mantissa, e16);
    }
    uint32_t discarded = mantissa & 0x1FFFu;
    uint16_t m16 = (uint16_t)(mantissa >> 13);
    uint32_t roundBit = (discarded >> 12) & 1u;
    uint32_t sticky = (discarded & 0xFFFu) != 0;
    m16 = (uint16_t)(m16 + (roundBit && (sticky || (m16 & 1u))));
    if (m16 == 0x400u) {
        m16 = 0;
        e16++;
    }
    if (e16 >= 31) {
        return (uint16_t)((sign << 15) | 0x7C00u);
    }
    return (uint16_t)((sign << 15) | ((uint32_t)e16 << 10) | m16);
}

/* bf16: no reference host path (parity unpinned). */
float orc_bf16_to_fp32(uint16_t h) { return u2f((uint32_t)h << 16); }

uint16_t orc_fp32_to_bf16(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu) != 0) {
        uint16_t hi = (uint16_t)(u >> 16);
        return (hi & 0x7Fu) ? hi : (uint16_t)(hi | 1u);
    }
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

void orc_fp16_to_fp32_n(const uint16_t* in, float* out, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) out[i] = orc_fp16_to_fp32(in[i]);
}

void orc_fp32_to_fp16_n(const float* in, uint16_t* out, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) out[i] = orc_fp32_to_fp16(in[i]);
}

void orc_bf16_to_fp32_n(const uint16_t* in, float* out, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) out[i] = orc_bf16_to_fp32(in[i]);
}

void orc_fp32_to_bf16_n(const float* in, uint16_t* out, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) out[i] = orc_fp32_to_bf16(in[i]);
}

/* ---------------------------------------------------------------------------------------------
 * a1: AicpuReduceTemplate<T> (wrapper.cc:1319-1358): dst[i] = src[i] (+) dst[i]
 *   SUM  : src + dst            (integers wrap; written with unsigned arithmetic)
 *   PROD : int8 via uint8 multiply, int32 via uint32 multiply, otherwise src * dst (wraps)
 *   MAX  : std::max(src, dst) == (src < dst) ? dst : src   -> ties / unordered return src
 *   MIN  : std::min(src, dst) == (dst < src) ? dst : src   -> ties / unordered return src
 * ------------------------------------------------------------------------------------------- */
#define DEFINE_INT_PAIR(NAME, T, UT)                                                      \
    static void NAME(T* dst, const T* src, uint64_t n, int op)                            \
    {                                                                                     \
        uint64_t i;                                                                       \
        switch (op) {                                                                     \
            case ORC_SUM:                                                                 \
                for (i = 0; i < n; ++i) dst[i] = (T)(UT)((UT)src[i] + (UT)dst[i]);        \
                break;                                                                    \
            case ORC_PROD:                                                                \
                for (i = 0; i < n; ++i) dst[i] = (T)(UT)((UT)src[i] * (UT)dst[i]);        \
                break;                                                                    \
            case ORC_MAX:                                                                 \
                for (i = 0; i < n; ++i) dst[i] = (src[i] < dst[i]) ? dst[i] : src[i];     \
                break;                                                                    \
            default:                                                                      \
                for (i = 0; i < n; ++i) dst[i] = (dst[i] < src[i]) ? dst[i] : src[i];     \
                break;                                                                    \
        }                                                                                 \
    }

#define DEFINE_FP_PAIR(NAME, T)                                                           \
    static void NAME(T* dst, const T* src, uint64_t n, int op)                            \
    {                                                                                     \
        uint64_t i;                                                                       \
        switch (op) {                                                                     \
            case ORC_SUM:                                                                 \
                for (i = 0; i < n; ++i) dst[i] = src[i] + dst[i];                         \
                break;                                                                    \
            case ORC_PROD:                                                                \
                for (i = 0; i < n; ++i) dst[i] = src[i] * dst[i];                         \
                break;                                                                    \
            case ORC_MAX:                                                                 \
                for (i = 0; i < n; ++i) dst[i] = (src[i] < dst[i]) ? dst[i] : src[i];     \
                break;                                                                    \
            default:                                                                      \
                for (i = 0; i < n; ++i) dst[i] = (dst[i] < src[i]) ? dst[i] : src[i];     \
                break;                                                                    \
        }                                                                                 \
    }

DEFINE_INT_PAIR(pair_i8, int8_t, uint8_t)
DEFINE_INT_PAIR(pair_i16, int16_t, uint16_t)
DEFINE_INT_PAIR(pair_i32, int32_t, uint32_t)
DEFINE_INT_PAIR(pair_i64, int64_t, uint64_t)
DEFINE_INT_PAIR(pair_u64, uint64_t, uint64_t)
DEFINE_FP_PAIR(pair_f32, float)
DEFINE_FP_PAIR(pair_f64, double)

static float fp32_op(float s, float d, int op)
{
    switch (op) {
        case ORC_SUM:
            return s + d;
        case ORC_PROD:
            return s * d;
        case ORC_MAX:
            return (s < d) ? d : s;
        default:
            return (d < s) ? d : s;
    }
}

/* AicpuReduceFp16 (wrapper.cc:1237-1257): widen both, fp32 op, narrow the result. */
static void pair_f16(uint16_t* dst, const uint16_t* src, uint64_t n, int op)
{
    for (uint64_t i = 0; i < n; ++i) {
        dst[i] = orc_fp32_to_fp16(fp32_op(orc_fp16_to_fp32(src[i]), orc_fp16_to_fp32(dst[i]), op));
    }
}

/* bf16 by analogy with the fp16 host pattern (parity unpinned). */
static void pair_bf16(uint16_t* dst, const uint16_t* src, uint64_t n, int op)
{
    for (uint64_t i = 0; i < n; ++i) {
        dst[i] = orc_fp32_to_bf16(fp32_op(orc_bf16_to_fp32(src[i]), orc_bf16_to_fp32(dst[i]), op));
    }
}

int orc_pair_reduce(void* dst, const void* src, uint64_t count, int dtype, int op)
{
    if (op < ORC_SUM || op > ORC_MIN) {
        return ORC_E_INTERNAL;
    }
    switch (dtype) {
        case ORC_INT8:
            pair_i8((int8_t*)dst, (const int8_t*)src, count, op);
            return ORC_OK;
        case ORC_INT16:
            pair_i16((int16_t*)dst, (const int16_t*)src, count, op);
            return ORC_OK;
        case ORC_INT32:
            pair_i32((int32_t*)dst, (const int32_t*)src, count, op);
            return ORC_OK;
        case ORC_INT64:
            pair_i64((int64_t*)dst, (const int64_t*)src, count, op);
            return ORC_OK;
        case ORC_UINT64:
            pair_u64((uint64_t*)dst, (const uint64_t*)src, count, op);
            return ORC_OK;
        case ORC_FP16:
            pair_f16((uint16_t*)dst, (const uint16_t*)src, count, op);
            return ORC_OK;
        case ORC_BF16:
            pair_bf16((uint16_t*)dst, (const uint16_t*)src, count, op);
            return ORC_OK;
        case ORC_FP32:
            pair_f32((float*)dst, (const float*)src, count, op);
            return ORC_OK;
        case ORC_FP64:
            pair_f64((double*)dst, (const double*)src, count, op);
            return ORC_OK;
        default:
            return ORC_E_INTERNAL;
    }
}

/* AicpuReduce (wrapper.cc:1259-1316). */
int orc_aicpu_reduce(void* dst, uint64_t dstBytes, const void* src, uint64_t srcBytes, int dtype, int op)
{
    if (dstBytes != srcBytes) {
        return ORC_E_INTERNAL;
    }
    switch (dtype) {
        case ORC_INT8:
        case ORC_INT32:
        case ORC_FP16:
        case ORC_FP32:
        case ORC_INT64:
        case ORC_UINT64:
        case ORC_FP64:
            return orc_pair_reduce(dst, src, dstBytes / orc_dtype_size(dtype), dtype, op);
        default:
            return ORC_E_INTERNAL;
    }
}

/* ---------------------------------------------------------------------------------------------
 * Accumulation domain shared by the executors
 * ------------------------------------------------------------------------------------------- */
typedef struct {
    int dtype, op, accF32;
    size_t esz, asz;
} red_t;

/* Admission follows reference op_common.cc:4323-4413 (CheckDataType / CheckReduceOp). */
static int red_init(red_t* r, int dtype, int op, int accMode)
{
    switch (dtype) {
        case ORC_INT8:
        case ORC_INT16:
        case ORC_INT32:
        case ORC_INT64:
        case ORC_UINT64:
        case ORC_FP16:
        case ORC_FP32:
        case ORC_FP64:
        case ORC_BF16:
            break;
        default:
            return ORC_E_NOT_SUPPORT;
    }
    if (op < ORC_SUM || op > ORC_MIN) {
        return ORC_E_PARA;
    }
    if (op == ORC_PROD && (dtype == ORC_INT16 || dtype == ORC_BF16)) {
        return ORC_E_NOT_SUPPORT;
    }
    r->dtype = dtype;
    r->op = op;
    r->esz = orc_dtype_size(dtype);
    r->accF32 = (accMode == ORC_ACC_FP32) && (dtype == ORC_FP16 || dtype == ORC_BF16) && op == ORC_SUM;
    r->asz = r->accF32 ? sizeof(float) : r->esz;
    return ORC_OK;
}

static void red_widen(const red_t* r, const void* in, void* acc, uint64_t n)
{
    if (!r->accF32) {
        memcpy(acc, in, n * r->esz);
        return;
    }
    const uint16_t* h = (const uint16_t*)in;
    float* a = (float*)acc;
    if (r->dtype == ORC_FP16) {
        for (uint64_t i = 0; i < n; ++i) a[i] = orc_fp16_to_fp32(h[i]);
    } else {
        for (uint64_t i = 0; i < n; ++i) a[i] = orc_bf16_to_fp32(h[i]);
    }
}

static void red_narrow(const red_t* r, const void* acc, void* out, uint64_t n)
{
    if (!r->accF32) {
        memcpy(out, acc, n * r->esz);
        return;
    }
    const float* a = (const float*)acc;
    uint16_t* h = (uint16_t*)out;
    if (r->dtype == ORC_FP16) {
        for (uint64_t i = 0; i < n; ++i) h[i] = orc_fp32_to_fp16(a[i]);
    } else {
        for (uint64_t i = 0; i < n; ++i) h[i] = orc_fp32_to_bf16(a[i]);
    }
}

/* dst = src (+) dst, both in the accumulation domain. */
static void red_pair(const red_t* r, void* dst, const void* src, uint64_t n)
{
    if (r->accF32) {
        pair_f32((float*)dst, (const float*)src, n, ORC_SUM);
    } else {
        orc_pair_reduce(dst, src, n, r->dtype, r->op);
    }
}

/* dst (accumulation domain) = widen(src in storage) (+) dst, without a staging copy. */
static void red_pair_from_storage(const red_t* r, void* dst, const void* src, uint64_t n, void* tmp)
{
    if (r->accF32) {
        red_widen(r, src, tmp, n);
        red_pair(r, dst, tmp, n);
    } else {
        orc_pair_reduce(dst, src, n, r->dtype, r->op);
    }
}

static const uint8_t* cbytes(const void* p) { return (const uint8_t*)p; }
static uint8_t* bytes(void* p) { return (uint8_t*)p; }

/* ---------------------------------------------------------------------------------------------
 * a16: slice geometry
 * ------------------------------------------------------------------------------------------- */
uint64_t orc_round_up(uint64_t dividend, uint64_t divisor)
{
    if (divisor == 0) {
        return dividend;
    }
    return dividend / divisor + ((dividend % divisor != 0) ? 1 : 0);
}

uint32_t orc_nhr_step_num(uint32_t rankSize)
{
    uint32_t n = 0;
    for (uint32_t t = rankSize - 1; t != 0; t >>= 1) n++;
    return n;
}

uint32_t orc_rhd_step_num(uint32_t rankSize)
{
    uint32_t n = 0;
    for (uint32_t t = rankSize; t > 1; t >>= 1) n++;
    return n;
}

/* r = p - 2^floor(log2 p) (template_utils.cc:53-63). */
static uint32_t rhd_pair_num(uint32_t p)
{
    if (p == 0) {
        return 0;
    }
    uint32_t hp = 1;
    while (hp <= p / 2) hp *= 2;
    return p - hp;
}

static int rhd_rep_is_low(uint32_t r, uint32_t root)
{
    return (root == ORC_INVALID_RANK || root >= 2 * r) ? 1 : (root < r);
}

static uint32_t rhd_unit_start_impl(uint32_t r, uint32_t j)
{
    if (j < r) {
        return 2 * j;
    }
    if (j < 2 * r) {
        return 2 * (j - r) + 1;
    }
    return j;
}

uint32_t orc_rhd_unit_start_of_rank(uint32_t p, uint32_t j)
{
    if (p == 0 || j >= p) {
        return ORC_INVALID_RANK;
    }
    return rhd_unit_start_impl(rhd_pair_num(p), j);
}

uint32_t orc_rhd_alg_rank_of_virtual(uint32_t p, uint32_t root, uint32_t v)
{
    if (p == 0) {
        return ORC_INVALID_RANK;
    }
    uint32_t r = rhd_pair_num(p);
    uint32_t P = p - r;
    if (v >= P) {
        return ORC_INVALID_RANK;
    }
    if (v >= r) {
        return v + r;
    }
    return rhd_rep_is_low(r, root) ? v : v + r;
}

uint32_t orc_rhd_owner_of_unit(uint32_t p, uint32_t unit)
{
    uint32_t r = rhd_pair_num(p);
    if (unit >= 2 * r) {
        return unit;
    }
    return unit / 2 + ((unit % 2 == 0) ? 0 : r);
}

int orc_rhd_part1(uint32_t p, uint32_t j, uint32_t root, orc_rhd_part1_t* info)
{
    if (p == 0 || j >= p) {
        return ORC_E_PARA;
    }
    if (root != ORC_INVALID_RANK && root >= p) {
        return ORC_E_PARA;
    }
    memset(info, 0, sizeof(*info));
    uint32_t r = rhd_pair_num(p);
    info->r = r;
    info->isPowerOfTwo = (r == 0);
    info->effectiveRankSize = p - r;
    info->virtualRank = (j < 2 * r) ? (j % r) : (j - r);
    info->inPart1 = (j < 2 * r);
    if (info->inPart1) {
        uint32_t t = j % r;
        int low = j < r;
        info->pairedAlgRank = low ? (t + r) : t;
        int repLow = rhd_rep_is_low(r, root);
        info->isRepresentative = repLow ? low : !low;
        if (info->isRepresentative) {
            info->unitStart = 2 * t;
            info->unitCount = 2;
        } else {
            info->unitStart = orc_rhd_unit_start_of_rank(p, j);
            info->unitCount = 1;
        }
    } else {
        info->pairedAlgRank = ORC_INVALID_RANK;
        info->isRepresentative = 0;
        info->unitStart = j;
        info->unitCount = 1;
    }
    return ORC_OK;
}

static uint32_t unit_start_of_virtual(uint32_t r, uint32_t a) { return (a < r) ? 2 * a : a + r; }
static uint32_t unit_end_of_virtual(uint32_t r, uint32_t b) { return (b <= r) ? 2 * b : b + r; }

static int rhd_info_ok(const orc_rhd_part1_t* info)
{
    uint32_t P = info->effectiveRankSize;
    if (P == 0 || info->virtualRank >= P) {
        return 0;
    }
    if ((P & (P - 1)) != 0 || info->r >= P) {
        return 0;
    }
    return 1;
}

int orc_rhd_rs_steps(const orc_rhd_part1_t* info, orc_rhd_step_t* steps, uint32_t* nSteps)
{
    *nSteps = 0;
    if (!rhd_info_ok(info)) {
        return ORC_E_PARA;
    }
    uint32_t v = info->virtualRank, P = info->effectiveRankSize, r = info->r;
    uint32_t n = orc_rhd_step_num(P);
    for (uint32_t k = 0; k < n; ++k) {
        uint32_t dist = P >> (k + 1);
        uint32_t peer = v ^ dist;
        uint32_t peerBase = peer & ~(dist - 1);
        uint32_t myBase = v & ~(dist - 1);
        orc_rhd_step_t* s = &steps[k];
        s->step = k;
        s->peer = peer;
        s->nSlices = dist;
        s->txSegStart = unit_start_of_virtual(r, peerBase);
        s->txSegEnd = unit_end_of_virtual(r, peerBase + dist);
        s->rxSegStart = unit_start_of_virtual(r, myBase);
        s->rxSegEnd = unit_end_of_virtual(r, myBase + dist);
    }
    *nSteps = n;
    return ORC_OK;
}

int orc_rhd_ag_steps(const orc_rhd_part1_t* info, orc_rhd_step_t* steps, uint32_t* nSteps)
{
    *nSteps = 0;
    if (!rhd_info_ok(info)) {
        return ORC_E_PARA;
    }
    uint32_t v = info->virtualRank, P = info->effectiveRankSize, r = info->r;
    uint32_t n = orc_rhd_step_num(P);
    for (uint32_t k = 0; k < n; ++k) {
        uint32_t dist = 1u << k;
        uint32_t held = v & ~(dist - 1);
        uint32_t rx = held ^ dist;
        orc_rhd_step_t* s = &steps[k];
        s->step = k;
        s->peer = v ^ dist;
        s->nSlices = dist;
        s->txSegStart = unit_start_of_virtual(r, held);
        s->txSegEnd = unit_end_of_virtual(r, held + dist);
        s->rxSegStart = unit_start_of_virtual(r, rx);
        s->rxSegEnd = unit_end_of_virtual(r, rx + dist);
    }
    *nSteps = n;
    return ORC_OK;
}

int orc_rhd_prepost(const orc_rhd_part1_t* info, orc_rhd_step_t* pre, orc_rhd_step_t* post, int preFull,
                    int postFull)
{
    memset(pre, 0, sizeof(*pre));
    memset(post, 0, sizeof(*post));
    uint32_t P = info->effectiveRankSize;
    if ((P & (P - 1)) != 0 || info->r >= P) {
        return ORC_E_PARA;
    }
    if (!info->inPart1) {
        pre->peer = ORC_INVALID_RANK;
        post->peer = ORC_INVALID_RANK;
        return ORC_OK;
    }
    uint32_t p = P + info->r;
    if (info->pairedAlgRank >= p || (!info->isRepresentative && info->unitStart >= p)) {
        return ORC_E_PARA;
    }
    uint32_t segStart = info->isRepresentative ? orc_rhd_unit_start_of_rank(p, info->pairedAlgRank) : info->unitStart;
    uint32_t segEnd = segStart + 1;
    uint32_t preS = preFull ? 0 : segStart, preE = preFull ? p : segEnd, preN = preFull ? p : 1;
    uint32_t postS = postFull ? 0 : segStart, postE = postFull ? p : segEnd, postN = postFull ? p : 1;
    pre->peer = info->pairedAlgRank;
    post->peer = info->pairedAlgRank;
    pre->nSlices = preN;
    post->nSlices = postN;
    if (info->isRepresentative) {
        pre->rxSegStart = preS;
        pre->rxSegEnd = preE;
        post->txSegStart = postS;
        post->txSegEnd = postE;
    } else {
        pre->txSegStart = preS;
        pre->txSegEnd = preE;
        post->rxSegStart = postS;
        post->rxSegEnd = postE;
    }
    return ORC_OK;
}

void orc_rhd_seg_bytes_uniform(uint32_t us, uint32_t ue, uint64_t sliceSize, uint64_t tailSize, uint32_t tailUnit,
                               uint64_t* offset, uint64_t* len)
{
    *offset = 0;
    *len = 0;
    if (us >= ue) {
        return;
    }
    *offset = (uint64_t)us * sliceSize;
    uint64_t tailLen = (tailSize == 0) ? sliceSize : tailSize;
    int includesTail = ue > tailUnit;
    uint32_t normal = ue - us - (includesTail ? 1 : 0);
    *len = (uint64_t)normal * sliceSize + (includesTail ? tailLen : 0);
}

uint64_t orc_rhd_select_loop_count(uint64_t remaining, uint64_t maxCountPerLoop, uint64_t rankAlign)
{
    uint64_t count = remaining < maxCountPerLoop ? remaining : maxCountPerLoop;
    return count >= rankAlign ? count / rankAlign * rankAlign : count;
}

int orc_nhr_step_info(uint32_t n, uint32_t me, uint32_t step, uint32_t* toRank, uint32_t* fromRank,
                      uint32_t* nSlices, uint32_t* tx, uint32_t* rx)
{
    if (n == 0 || me >= n || step >= orc_nhr_step_num(n)) {
        return ORC_E_PARA;
    }
    uint32_t delta = 1u << step;
    uint32_t sendTo = (me + n - delta % n) % n;
    uint32_t recvFrom = (me + delta) % n;
    uint32_t cnt = (n - 1 + (1u << step)) / (1u << (step + 1));
    uint32_t dIdx = (1u << (step + 1)) % n;
    uint32_t t = sendTo, x = me;
    for (uint32_t i = 0; i < cnt; ++i) {
        tx[i] = t;
        rx[i] = x;
        t = (t + n - dIdx) % n;
        x = (x + n - dIdx) % n;
    }
    *toRank = sendTo;
    *fromRank = recvFrom;
    *nSlices = cnt;
    return ORC_OK;
}

/* ---------------------------------------------------------------------------------------------
 * a6 / a7: AllReduce in rank order.  Scratch slot r holds rank r's input; slot 0 accumulates
 * slots 1..N-1 ascending; slot 0 is copied to every output (one_shot.cc:223-239,
 * aicpu_reduce_nhr.cc:272-285).
 * ------------------------------------------------------------------------------------------- */
static int all_reduce_mesh_range(uint32_t n, const void* const* in, void* const* out, uint64_t first, uint64_t count,
                                 const red_t* r)
{
    if (count == 0) {
        return ORC_OK;
    }
    void* acc = malloc(count * r->asz);
    void* tmp = r->accF32 ? malloc(count * r->asz) : NULL;
    if (!acc || (r->accF32 && !tmp)) {
        free(acc);
        free(tmp);
        return ORC_E_INTERNAL;
    }
    red_widen(r, cbytes(in[0]) + first * r->esz, acc, count);
    for (uint32_t k = 1; k < n; ++k) {
        red_pair_from_storage(r, acc, cbytes(in[k]) + first * r->esz, count, tmp);
    }
    for (uint32_t k = 0; k < n; ++k) {
        red_narrow(r, acc, bytes(out[k]) + first * r->esz, count);
    }
    free(acc);
    free(tmp);
    return ORC_OK;
}

int orc_all_reduce_mesh(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                        int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    return all_reduce_mesh_range(n, in, out, 0, count, &r);
}

/* a8: slice k = [k*ceil(count/n), min(count, (k+1)*ceil(count/n))) is reduced by rank k in rank
 * order, then gathered (two_shot.cc:178-210, 326-360). */
int orc_all_reduce_two_shot(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                            int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    uint64_t sliceCount = orc_round_up(count, n);
    uint64_t off = 0;
    for (uint32_t k = 0; k < n; ++k) {
        uint64_t cur = (count - off > sliceCount) ? sliceCount : count - off;
        rc = all_reduce_mesh_range(n, in, out, off, cur, &r);
        if (rc != ORC_OK) {
            return rc;
        }
        off += cur;
    }
    return ORC_OK;
}

/* AllReduce of the two-shot executor over one mesh (ins_v2_all_reduce_two_shot_sole_executor.cc; registered as
 * Aicpu AllReduce Sole MeshConcur, :395-398): per loop a mesh ReduceScatter on n slices of floor(len / n) elements,
 * the last slice taking the rest (:236-237), slice k folded by rank k, its own input first and the other ranks
 * ascending (reduce_scatter_mesh_1D.cc:203-237), then the AllGather.  Loops of maxCountPerLoop elements floored to
 * a multiple of n (:335-336), the last one taking what is left (:354); 0 = one loop. */
int orc_all_reduce_mesh_concur(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                               int accMode, uint64_t maxCountPerLoop)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (count == 0) {
        return ORC_OK;
    }
    if (maxCountPerLoop == 0) {
        maxCountPerLoop = UINT64_MAX / 2;
    }
    maxCountPerLoop = maxCountPerLoop / n * n;
    if (maxCountPerLoop == 0) {
        return ORC_E_INTERNAL;
    }
    void* acc = malloc(count * r.asz);
    void* tmp = malloc(count * r.asz);
    uint8_t* res = (uint8_t*)malloc(count * r.esz);
    if (!acc || !tmp || !res) {
        free(acc);
        free(tmp);
        free(res);
        return ORC_E_INTERNAL;
    }
    for (uint64_t done = 0; done < count;) {
        uint64_t len = count - done < maxCountPerLoop ? count - done : maxCountPerLoop;
        uint64_t slice = len / n;
        for (uint32_t k = 0; k < n; ++k) {
            uint64_t off = done + (uint64_t)k * slice;
            uint64_t cur = k == n - 1 ? len - slice * (n - 1) : slice;
            if (cur == 0) {
                continue;
            }
            red_widen(&r, cbytes(in[k]) + off * r.esz, acc, cur);
            for (uint32_t t = 0; t < n; ++t) {
                if (t != k) {
                    red_pair_from_storage(&r, acc, cbytes(in[t]) + off * r.esz, cur, tmp);
                }
            }
            red_narrow(&r, acc, res + off * r.esz, cur);
        }
        done += len;
    }
    for (uint32_t d = 0; d < n; ++d) {
        memcpy(out[d], res, count * r.esz);
    }
    free(acc);
    free(tmp);
    free(res);
    return ORC_OK;
}

/* Two-shot, symmetric-memory variant (two_shot.cc:341-357 with supportSymmetricMemAccess_): slice k starts
 * from rank k's own input slice, then the other ranks ascending; every rank gets every slice. */
int orc_all_reduce_two_shot_symmetric(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype,
                                      int op, int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    uint64_t sliceCount = orc_round_up(count, n);   /* two_shot.cc:184 */
    void* acc = malloc((sliceCount ? sliceCount : 1) * r.asz);
    void* tmp = malloc((sliceCount ? sliceCount : 1) * r.asz);
    uint8_t* res = (uint8_t*)malloc((count ? count : 1) * r.esz);
    if (!acc || !tmp || !res) {
        free(acc);
        free(tmp);
        free(res);
        return ORC_E_INTERNAL;
    }
    uint64_t off = 0;
    for (uint32_t k = 0; k < n; ++k) {
        uint64_t cur = (count - off > sliceCount) ? sliceCount : count - off;
        if (cur != 0) {
            red_widen(&r, cbytes(in[k]) + off * r.esz, acc, cur);
            for (uint32_t t = 0; t < n; ++t) {
                if (t != k) {
                    red_pair_from_storage(&r, acc, cbytes(in[t]) + off * r.esz, cur, tmp);
                }
            }
            red_narrow(&r, acc, res + off * r.esz, cur);
        }
        off += cur;
    }
    for (uint32_t d = 0; d < n; ++d) {
        memcpy(out[d], res, count * r.esz);
    }
    free(acc);
    free(tmp);
    free(res);
    return ORC_OK;
}

/* a9: rank k: out = in_k[k]; for t = 0..N-1, t != k: out = in_t[k] (+) out. */
static int reduce_scatter_mesh_range(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount,
                                     uint64_t first, uint64_t count, const red_t* r)
{
    if (count == 0) {
        return ORC_OK;
    }
    void* acc = malloc(count * r->asz);
    void* tmp = r->accF32 ? malloc(count * r->asz) : NULL;
    if (!acc || (r->accF32 && !tmp)) {
        free(acc);
        free(tmp);
        return ORC_E_INTERNAL;
    }
    for (uint32_t k = 0; k < n; ++k) {
        uint64_t base = ((uint64_t)k * recvCount + first) * r->esz;
        red_widen(r, cbytes(in[k]) + base, acc, count);
        for (uint32_t t = 0; t < n; ++t) {
            if (t != k) {
                red_pair_from_storage(r, acc, cbytes(in[t]) + base, count, tmp);
            }
        }
        red_narrow(r, acc, bytes(out[k]) + first * r->esz, count);
    }
    free(acc);
    free(tmp);
    return ORC_OK;
}

int orc_reduce_scatter_mesh(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                            int op, int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    return reduce_scatter_mesh_range(n, in, out, recvCount, 0, recvCount, &r);
}

/* ---------------------------------------------------------------------------------------------
 * Per-rank scratch used by the step-driven executors: scratch[rank][slot][elem].
 * ------------------------------------------------------------------------------------------- */
typedef struct {
    uint32_t n;
    uint64_t slotElems;
    size_t asz;
    uint8_t* mem;
} scratch_t;

static int scratch_alloc(scratch_t* s, uint32_t n, uint64_t slotElems, size_t asz)
{
    s->n = n;
    s->slotElems = slotElems;
    s->asz = asz;
    uint64_t total = (uint64_t)n * n * slotElems * asz;
    s->mem = (uint8_t*)malloc(total ? total : 1);
    return s->mem ? ORC_OK : ORC_E_INTERNAL;
}

static uint8_t* scratch_at(const scratch_t* s, uint32_t rank, uint32_t slot)
{
    return s->mem + ((uint64_t)rank * s->n + slot) * s->slotElems * s->asz;
}

/* a10: NHR reduce-scatter.  Slot i of a rank's scratch starts as its input slice i; in step s
 * rank m write-reduces its slots txSliceIdxs into the same slots of rank (m - 2^s) mod N
 * (receiver's value is dst, incoming is src; reduce_scatter_nhr.cc:316-447).  After the last
 * step rank m's slot m is its output (:268-312). */
static int nhr_reduce_scatter_scratch(const red_t* r, scratch_t* sc)
{
    uint32_t n = sc->n;
    uint32_t steps = orc_nhr_step_num(n);
    uint32_t* tx = (uint32_t*)malloc(sizeof(uint32_t) * n * 2);
    uint32_t* rx = tx + n;
    uint8_t* dirty = (uint8_t*)malloc((size_t)n * n);
    if (!tx || !dirty) {
        free(tx);
        free(dirty);
        return ORC_E_INTERNAL;
    }
    int rc = ORC_OK;
    for (uint32_t s = 0; s < steps && rc == ORC_OK; ++s) {
        /* A slot written in this step must not also be read in it (sends and receives of one step run
         * concurrently in the reference). */
        memset(dirty, 0, (size_t)n * n);
        for (uint32_t m = 0; m < n; ++m) {
            uint32_t to, from, cnt;
            orc_nhr_step_info(n, m, s, &to, &from, &cnt, tx, rx);
            for (uint32_t i = 0; i < cnt; ++i) dirty[to * n + tx[i]] = 1;
        }
        for (uint32_t m = 0; m < n && rc == ORC_OK; ++m) {
            uint32_t to, from, cnt;
            orc_nhr_step_info(n, m, s, &to, &from, &cnt, tx, rx);
            for (uint32_t i = 0; i < cnt; ++i) {
                if (dirty[m * n + tx[i]]) {
                    rc = ORC_E_INTERNAL;
                    break;
                }
                red_pair(r, scratch_at(sc, to, tx[i]), scratch_at(sc, m, tx[i]), sc->slotElems);
            }
        }
    }
    free(tx);
    free(dirty);
    return rc;
}

int orc_reduce_scatter_nhr(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                           int op, int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (recvCount == 0) {
        return ORC_OK;
    }
    scratch_t sc;
    if (scratch_alloc(&sc, n, recvCount, r.asz) != ORC_OK) {
        return ORC_E_INTERNAL;
    }
    for (uint32_t m = 0; m < n; ++m) {
        for (uint32_t i = 0; i < n; ++i) {
            red_widen(&r, cbytes(in[m]) + (uint64_t)i * recvCount * r.esz, scratch_at(&sc, m, i), recvCount);
        }
    }
    rc = nhr_reduce_scatter_scratch(&r, &sc);
    if (rc == ORC_OK) {
        for (uint32_t m = 0; m < n; ++m) red_narrow(&r, scratch_at(&sc, m, m), out[m], recvCount);
    }
    free(sc.mem);
    return rc;
}

/* One KernelRun of InsTempAllReduceNHR (ins_temp_all_reduce_nhr.cc:214-216): the first n - 1 slices hold
 * floor(count / n) elements, the last one takes the rest; slice k is folded by the NHR step tree. */
static int nhr_all_reduce_once(red_t* r, uint32_t n, const void* const* in, void* const* out, uint64_t first,
                               uint64_t count)
{
    uint64_t slice = count / n;
    uint64_t tail = count - slice * (n - 1);
    scratch_t sc;
    if (scratch_alloc(&sc, n, tail, r->asz) != ORC_OK) {
        return ORC_E_INTERNAL;
    }
    memset(sc.mem, 0, (uint64_t)n * n * tail * r->asz);
    for (uint32_t m = 0; m < n; ++m) {
        for (uint32_t i = 0; i < n; ++i) {
            uint64_t cur = i == n - 1 ? tail : slice;
            red_widen(r, cbytes(in[m]) + (first + (uint64_t)i * slice) * r->esz, scratch_at(&sc, m, i), cur);
        }
    }
    int rc = nhr_reduce_scatter_scratch(r, &sc);
    if (rc == ORC_OK) {
        for (uint32_t i = 0; i < n; ++i) {
            uint64_t cur = i == n - 1 ? tail : slice;
            for (uint32_t m = 0; m < n; ++m) {
                red_narrow(r, scratch_at(&sc, i, i), bytes(out[m]) + (first + (uint64_t)i * slice) * r->esz, cur);
            }
        }
    }
    free(sc.mem);
    return rc;
}

int orc_all_reduce_nhr_looped(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                              int accMode, uint64_t maxCountPerLoop)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (maxCountPerLoop == 0) {
        maxCountPerLoop = count;
    }
    /* ins_v2_all_reduce_sole_executor.cc:266-300: full loops, the last one takes what is left */
    for (uint64_t done = 0; done < count && rc == ORC_OK;) {
        uint64_t cur = count - done < maxCountPerLoop ? count - done : maxCountPerLoop;
        rc = nhr_all_reduce_once(&r, n, in, out, done, cur);
        done += cur;
    }
    return rc;
}

int orc_all_reduce_nhr(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                       int accMode)
{
    return orc_all_reduce_nhr_looped(n, in, out, count, dtype, op, accMode, 0);
}

/* Reduce under ReduceNHR (src/ops/reduce/algorithm/template/aicpu/reduce_nhr.cc): slices of ceil(len / n)
 * elements, short or empty towards the end (CalcSlice :202-226), each folded along the NHR ReduceScatter step tree
 * (GetStepInfoList :481-519, RunReduce :263-339) and gathered at the root (:341-414); one staging slot
 * (CalcScratchMultiple :131-136), so the executor's loops hold maxCountPerLoop elements (reduce_sole_executor.cc:
 * 178-232; 0 = one loop).  Only out[root] is written. */
int orc_reduce_nhr(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op, int accMode,
                   uint32_t root, uint64_t maxCountPerLoop)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (root >= n) {
        return ORC_E_PARA;
    }
    if (maxCountPerLoop == 0) {
        maxCountPerLoop = count;
    }
    for (uint64_t done = 0; done < count && rc == ORC_OK;) {
        uint64_t len = count - done < maxCountPerLoop ? count - done : maxCountPerLoop;
        uint64_t slice = (len + n - 1) / n;
        scratch_t sc;
        if (scratch_alloc(&sc, n, slice, r.asz) != ORC_OK) {
            return ORC_E_INTERNAL;
        }
        memset(sc.mem, 0, (uint64_t)n * n * slice * r.asz);
        for (uint32_t m = 0; m < n; ++m) {
            uint64_t off = 0;
            for (uint32_t i = 0; i < n; ++i) {
                uint64_t cur = len - off < slice ? len - off : slice;
                red_widen(&r, cbytes(in[m]) + (done + off) * r.esz, scratch_at(&sc, m, i), cur);
                off += cur;
            }
        }
        rc = nhr_reduce_scatter_scratch(&r, &sc);
        uint64_t off = 0;
        for (uint32_t i = 0; i < n && rc == ORC_OK; ++i) {
            uint64_t cur = len - off < slice ? len - off : slice;
            red_narrow(&r, scratch_at(&sc, i, i), bytes(out[root]) + (done + off) * r.esz, cur);
            off += cur;
        }
        free(sc.mem);
        done += len;
    }
    return rc;
}

/* ---- staging-buffer loop limits ----------------------------------------------------------------
 * hccl_op_utils.cc:204-225: HCCL_BUFFSIZE in MB (default 200, at least 2, at most UINT32_MAX, digits only),
 * less 1 MiB that is kept back. */
int orc_ccl_buffer_available_size(const char* envValue, uint64_t* bytes)
{
    uint64_t mb = 200;
    if (envValue != NULL) {
        char* end = NULL;
        unsigned long long v = strtoull(envValue, &end, 10);
        if (end == envValue || *end != '\0' || v < 2 || v > 0xFFFFFFFFull) {
            return ORC_E_PARA;
        }
        mb = v;
    }
    *bytes = mb * 1024 * 1024 - 1024 * 1024;
    return ORC_OK;
}

/* ins_v2_all_reduce_sole_executor.cc:241-262: elements one loop of a single-template executor may take. */
uint64_t orc_sole_max_count_per_loop(uint64_t cclBytes, uint64_t scratchMultiple, uint64_t elemSize)
{
    uint64_t bytes = cclBytes;
    if (scratchMultiple != 0) {
        uint64_t bound = cclBytes / scratchMultiple / 128 * 128;
        bytes = bound < cclBytes ? bound : cclBytes;
    }
    return elemSize ? bytes / elemSize : 0;
}

/* ins_v2_all_reduce_sequence_rhd_tail.h:64-92: two 128-byte-rounded tiles of rankAlign elements are taken
 * from the end of the workspace when count is not a multiple of rankAlign. */
int orc_rhd_prepare_tail_workspace(uint64_t count, uint64_t rankAlign, uint64_t elemSize, uint64_t* workspaceBytes,
                                   uint64_t* inputOffset, uint64_t* outputOffset)
{
    if (rankAlign == 0 || elemSize == 0) {
        return ORC_E_PARA;
    }
    if (count % rankAlign == 0) {
        return ORC_OK;
    }
    uint64_t size = *workspaceBytes;
    if (rankAlign > size / elemSize / 2) {
        return ORC_E_INTERNAL;
    }
    uint64_t tile = rankAlign * elemSize;
    uint64_t slot = (tile / 128 + (tile % 128 != 0)) * 128;
    if (slot >= size / 2) {
        return ORC_E_INTERNAL;
    }
    *inputOffset = size - 2 * slot;
    *outputOffset = size - slot;
    *workspaceBytes = *inputOffset;
    return ORC_OK;
}

/* ins_v2_all_reduce_sequence_executor_aicpu.cc:592-600, 645-662, 668-675 with one rank per level-0 group:
 * the tail tiles come off first, half of what remains is the receive area, floored to 128 bytes, to whole
 * elements and to a multiple of p. */
int orc_rhd_max_count_per_loop(uint64_t cclBytes, uint64_t count, uint32_t p, uint64_t elemSize, uint64_t* maxCount)
{
    uint64_t size = cclBytes;
    uint64_t inOff = 0;
    uint64_t outOff = 0;
    int rc = orc_rhd_prepare_tail_workspace(count, p, elemSize, &size, &inOff, &outOff);
    if (rc != ORC_OK) {
        return rc;
    }
    uint64_t outHalf = size / 2;
    *maxCount = outHalf / 128 * 128 / elemSize / p * p;
    return *maxCount == 0 ? ORC_E_INTERNAL : ORC_OK;
}

/* ---------------------------------------------------------------------------------------------
 * a11: RHD.  One "frame" = p units of `unit` elements per rank.
 *   mirror : input slice i of every rank goes to slot sigma(i)            (rhd.cc:365-410)
 *   PRE    : merged rank t+r write-reduces all p slots into representative t (:412-476)
 *   MAIN   : step k, dist = P>>(k+1): virtual rank v write-reduces its tx segment into the
 *            same slots of v^dist; receiver's value is dst                (:478-564)
 *   POST   : representative writes the merged rank's slot back             (:566-629)
 * ------------------------------------------------------------------------------------------- */
static int rhd_rs_frame(const red_t* r, scratch_t* sc, int skipPost)
{
    uint32_t p = sc->n;
    orc_rhd_part1_t info;
    orc_rhd_step_t steps[32];
    uint32_t nSteps;
    /* PRE (FULL segment [0,p)) */
    for (uint32_t j = 0; j < p; ++j) {
        orc_rhd_part1(p, j, ORC_INVALID_RANK, &info);
        if (info.inPart1 && !info.isRepresentative) {
            orc_rhd_step_t pre, post;
            if (orc_rhd_prepost(&info, &pre, &post, 1, 0) != ORC_OK) {
                return ORC_E_INTERNAL;
            }
            for (uint32_t u = pre.txSegStart; u < pre.txSegEnd; ++u) {
                red_pair(r, scratch_at(sc, pre.peer, u), scratch_at(sc, j, u), sc->slotElems);
            }
        }
    }
    /* MAIN: tx and rx segments of a step are disjoint, so in-place per step is exact. */
    uint32_t P = p - rhd_pair_num(p);
    uint32_t total = orc_rhd_step_num(P);
    for (uint32_t k = 0; k < total; ++k) {
        for (uint32_t v = 0; v < P; ++v) {
            uint32_t phys = orc_rhd_alg_rank_of_virtual(p, ORC_INVALID_RANK, v);
            orc_rhd_part1(p, phys, ORC_INVALID_RANK, &info);
            if (orc_rhd_rs_steps(&info, steps, &nSteps) != ORC_OK) {
                return ORC_E_INTERNAL;
            }
            uint32_t peerPhys = orc_rhd_alg_rank_of_virtual(p, ORC_INVALID_RANK, steps[k].peer);
            for (uint32_t u = steps[k].txSegStart; u < steps[k].txSegEnd; ++u) {
                red_pair(r, scratch_at(sc, peerPhys, u), scratch_at(sc, phys, u), sc->slotElems);
            }
        }
    }
    /* POST (SHARE segment) */
    if (!skipPost) {
        for (uint32_t j = 0; j < p; ++j) {
            orc_rhd_part1(p, j, ORC_INVALID_RANK, &info);
            if (info.inPart1 && info.isRepresentative) {
                orc_rhd_step_t pre, post;
                if (orc_rhd_prepost(&info, &pre, &post, 1, 0) != ORC_OK) {
                    return ORC_E_INTERNAL;
                }
                for (uint32_t u = post.txSegStart; u < post.txSegEnd; ++u) {
                    memcpy(scratch_at(sc, post.peer, u), scratch_at(sc, j, u), sc->slotElems * sc->asz);
                }
            }
        }
    }
    return ORC_OK;
}

int orc_reduce_scatter_rhd(uint32_t p, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                           int op, int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (recvCount == 0) {
        return ORC_OK;
    }
    scratch_t sc;
    if (scratch_alloc(&sc, p, recvCount, r.asz) != ORC_OK) {
        return ORC_E_INTERNAL;
    }
    for (uint32_t j = 0; j < p; ++j) {
        for (uint32_t i = 0; i < p; ++i) {
            red_widen(&r, cbytes(in[j]) + (uint64_t)i * recvCount * r.esz,
                      scratch_at(&sc, j, orc_rhd_unit_start_of_rank(p, i)), recvCount);
        }
    }
    rc = rhd_rs_frame(&r, &sc, 0);
    if (rc == ORC_OK) {
        for (uint32_t j = 0; j < p; ++j) {
            red_narrow(&r, scratch_at(&sc, j, orc_rhd_unit_start_of_rank(p, j)), out[j], recvCount);
        }
    }
    free(sc.mem);
    return rc;
}

/* AG-RHD with PRE skipped and POST = FULL over a grid indexed by owner rank
 * (all_gather_rhd.cc:355-365 owner map; template_utils.cc:211-249 steps). */
static int rhd_ag_frame(scratch_t* grid)
{
    uint32_t p = grid->n;
    uint32_t P = p - rhd_pair_num(p);
    uint32_t total = orc_rhd_step_num(P);
    orc_rhd_part1_t info;
    orc_rhd_step_t steps[32];
    uint32_t nSteps;
    size_t slotBytes = grid->slotElems * grid->asz;
    for (uint32_t k = 0; k < total; ++k) {
        for (uint32_t v = 0; v < P; ++v) {
            uint32_t phys = orc_rhd_alg_rank_of_virtual(p, ORC_INVALID_RANK, v);
            orc_rhd_part1(p, phys, ORC_INVALID_RANK, &info);
            if (orc_rhd_ag_steps(&info, steps, &nSteps) != ORC_OK) {
                return ORC_E_INTERNAL;
            }
            uint32_t peerPhys = orc_rhd_alg_rank_of_virtual(p, ORC_INVALID_RANK, steps[k].peer);
            for (uint32_t u = steps[k].txSegStart; u < steps[k].txSegEnd; ++u) {
                uint32_t owner = orc_rhd_owner_of_unit(p, u);
                memcpy(scratch_at(grid, peerPhys, owner), scratch_at(grid, phys, owner), slotBytes);
            }
        }
    }
    for (uint32_t j = 0; j < p; ++j) {
        orc_rhd_part1(p, j, ORC_INVALID_RANK, &info);
        if (info.inPart1 && info.isRepresentative) {
            orc_rhd_step_t pre, post;
            if (orc_rhd_prepost(&info, &pre, &post, 0, 1) != ORC_OK) {
                return ORC_E_INTERNAL;
            }
            for (uint32_t u = post.txSegStart; u < post.txSegEnd; ++u) {
                uint32_t owner = orc_rhd_owner_of_unit(p, u);
                memcpy(scratch_at(grid, post.peer, owner), scratch_at(grid, j, owner), slotBytes);
            }
        }
    }
    return ORC_OK;
}

/* AllReduce over a flat p-rank RHD level: per loop the aligned prefix is split into p uniform
 * units; a final remainder shorter than p is staged into a p-element tile whose unused lanes
 * duplicate valid input (rhd_tail.h:98-165; executor_aicpu.cc:684-759). */
int orc_all_reduce_rhd(uint32_t p, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                       int accMode, uint64_t maxCountPerLoop)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (maxCountPerLoop == 0) {
        maxCountPerLoop = UINT64_MAX / 2;
    }
    maxCountPerLoop = maxCountPerLoop / p * p;
    if (maxCountPerLoop == 0) {
        return ORC_E_INTERNAL;
    }
    uint8_t* tile = (uint8_t*)malloc((size_t)p * p * r.esz);
    uint8_t* result = (uint8_t*)malloc((count ? count : 1) * r.esz * p);
    if (!tile || !result) {
        free(tile);
        free(result);
        return ORC_E_INTERNAL;
    }
    uint64_t processed = 0;
    while (processed < count && rc == ORC_OK) {
        uint64_t valid = orc_rhd_select_loop_count(count - processed, maxCountPerLoop, p);
        uint64_t curr = valid > p ? valid : p;
        int padded = valid != curr;
        uint64_t unit = curr / p;
        scratch_t sc, grid;
        if (scratch_alloc(&sc, p, unit, r.asz) != ORC_OK) {
            rc = ORC_E_INTERNAL;
            break;
        }
        if (scratch_alloc(&grid, p, unit, r.asz) != ORC_OK) {
            free(sc.mem);
            rc = ORC_E_INTERNAL;
            break;
        }
        for (uint32_t j = 0; j < p; ++j) {
            const uint8_t* src = cbytes(in[j]) + processed * r.esz;
            if (padded) {
                uint8_t* t = tile + (size_t)j * p * r.esz;
                memcpy(t, src, valid * r.esz);
                uint64_t filled = valid;
                while (filled < p) {
                    uint64_t c = filled < p - filled ? filled : p - filled;
                    memcpy(t + filled * r.esz, t, c * r.esz);
                    filled += c;
                }
                src = t;
            }
            for (uint32_t i = 0; i < p; ++i) {
                red_widen(&r, src + (uint64_t)i * unit * r.esz, scratch_at(&sc, j, orc_rhd_unit_start_of_rank(p, i)),
                          unit);
            }
        }
        rc = rhd_rs_frame(&r, &sc, 1);
        if (rc == ORC_OK) {
            size_t slotBytes = unit * r.asz;
            memset(grid.mem, 0, (uint64_t)p * p * slotBytes);
            for (uint32_t j = 0; j < p; ++j) {
                orc_rhd_part1_t info;
                orc_rhd_part1(p, j, ORC_INVALID_RANK, &info);
                if (info.inPart1 && !info.isRepresentative) {
                    continue; /* merged ranks skip the final copy when POST is skipped */
                }
                memcpy(scratch_at(&grid, j, j), scratch_at(&sc, j, orc_rhd_unit_start_of_rank(p, j)), slotBytes);
                if (info.inPart1 && info.isRepresentative) {
                    /* bridge: merged party's final slot 2t+1 -> owner slot t+r (rhd_tail.h:33-53) */
                    memcpy(scratch_at(&grid, j, info.pairedAlgRank), scratch_at(&sc, j, info.unitStart + 1),
                           slotBytes);
                }
            }
            rc = rhd_ag_frame(&grid);
        }
        if (rc == ORC_OK) {
            for (uint32_t j = 0; j < p; ++j) {
                uint8_t* dst = result + ((uint64_t)j * count + processed) * r.esz;
                if (padded) {
                    uint8_t* t = tile + (size_t)j * p * r.esz;
                    for (uint32_t i = 0; i < p; ++i) red_narrow(&r, scratch_at(&grid, j, i), t + (size_t)i * r.esz, 1);
                    memcpy(dst, t, valid * r.esz);
                } else {
                    for (uint32_t i = 0; i < p; ++i) {
                        red_narrow(&r, scratch_at(&grid, j, i), dst + (uint64_t)i * unit * r.esz, unit);
                    }
                }
            }
        }
        free(sc.mem);
        free(grid.mem);
        processed += valid;
    }
    if (rc == ORC_OK) {
        for (uint32_t j = 0; j < p; ++j) memcpy(out[j], result + (uint64_t)j * count * r.esz, count * r.esz);
    }
    free(tile);
    free(result);
    return rc;
}

/* ---------------------------------------------------------------------------------------------
 * Two-level AllReduce (ins_v2_all_reduce_sequence_executor_aicpu.cc:592-852, "executor.cc" below).
 * l0 consecutive ranks form a level-0 group ("box"), l1 = n / l0 boxes; rank b * l0 + i is member i of box b
 * and talks, between the boxes, to the members i of the other boxes.  Per loop:
 *   step 1  mesh ReduceScatter inside every box: member i ends with chunk i of the loop, its own input
 *           first, the other members ascending (reduce_scatter_mesh_1D.cc:203-237; the level-0 template
 *           ..._Z_axis_detour derives from it)
 *   step 2  the level-1 template between the members i of all boxes, on chunk i cut into l1 sub-slices
 *   steps 3, 4  the two AllGathers back: every rank ends with every sub-slice.
 * Level 1 (registrations executor.cc:974-1023):
 *   ORC_L1_RHD   RHD with POST skipped, the merged share bridged, AllGather with PRE skipped (:684-759); the
 *                loop is cut like the flat form with the rank alignment l0 * l1: aligned prefix in uniform
 *                units, a remainder shorter than that staged into a padded tile (rhd_tail.h:94-165)
 *   ORC_L1_NHR   NHR ReduceScatter (:784-789); chunks of floor(len / l0), the last member's chunk takes the rest
 *                (:413-415); sub-slices of floor(chunk / l1), the last box's takes the rest (:445-455)
 *   ORC_L1_MESH  the host-reduce template of PROD and the 64-bit types, own share first, the other boxes
 *                ascending (reduce_scatter_aicpu_reduce_nhr.cc:214-250), same cuts as NHR.
 * Everything is folded in the accumulation domain and narrowed once per output (see red_t).
 * ------------------------------------------------------------------------------------------- */
static void level0_fold(const red_t* r, uint32_t l0, uint32_t box, uint32_t member, const uint8_t* const* src,
                        uint64_t elemOff, uint64_t len, void* acc, void* tmp)
{
    red_widen(r, src[box * l0 + member] + elemOff * r->esz, acc, len);
    for (uint32_t t = 0; t < l0; ++t) {
        if (t != member) {
            red_pair_from_storage(r, acc, src[box * l0 + t] + elemOff * r->esz, len, tmp);
        }
    }
}

/* Level 1 over chunk `member` of one loop, cut into l1 units of `unit` elements (the last holds `last`);
 * writes unit j of every box's view to result[box] + (chunkOff + j * unit). */
static int level1_exchange(const red_t* r, uint32_t l0, uint32_t l1, int l1Algo, uint32_t member,
                           const uint8_t* const* src, uint64_t chunkOff, uint64_t unit, uint64_t last,
                           uint8_t* const* result, uint64_t resultOff)
{
    uint64_t slot = last > unit ? last : unit;
    if (slot == 0) {
        return ORC_OK;
    }
    scratch_t sc, grid;
    void* tmp = malloc(slot * r->asz);
    if (!tmp || scratch_alloc(&sc, l1, slot, r->asz) != ORC_OK) {
        free(tmp);
        return ORC_E_INTERNAL;
    }
    memset(sc.mem, 0, (uint64_t)l1 * l1 * slot * r->asz);
    int rc = ORC_OK;
    for (uint32_t b = 0; b < l1; ++b) {
        for (uint32_t j = 0; j < l1; ++j) {
            uint64_t cur = j == l1 - 1 ? last : unit;
            uint32_t at = l1Algo == ORC_L1_RHD ? orc_rhd_unit_start_of_rank(l1, j) : j;
            level0_fold(r, l0, b, member, src, chunkOff + (uint64_t)j * unit, cur, scratch_at(&sc, b, at), tmp);
        }
    }
    if (l1Algo == ORC_L1_RHD) {
        rc = rhd_rs_frame(r, &sc, 1);
        if (rc == ORC_OK && scratch_alloc(&grid, l1, slot, r->asz) != ORC_OK) {
            rc = ORC_E_INTERNAL;
        }
        if (rc == ORC_OK) {
            size_t slotBytes = slot * r->asz;
            memset(grid.mem, 0, (uint64_t)l1 * l1 * slotBytes);
            for (uint32_t b = 0; b < l1; ++b) {
                orc_rhd_part1_t info;
                orc_rhd_part1(l1, b, ORC_INVALID_RANK, &info);
                if (info.inPart1 && !info.isRepresentative) {
                    continue;
                }
                memcpy(scratch_at(&grid, b, b), scratch_at(&sc, b, orc_rhd_unit_start_of_rank(l1, b)), slotBytes);
                if (info.inPart1 && info.isRepresentative) {
                    memcpy(scratch_at(&grid, b, info.pairedAlgRank), scratch_at(&sc, b, info.unitStart + 1), slotBytes);
                }
            }
            rc = rhd_ag_frame(&grid);
            for (uint32_t b = 0; b < l1 && rc == ORC_OK; ++b) {
                for (uint32_t j = 0; j < l1; ++j) {
                    red_narrow(r, scratch_at(&grid, b, j), result[b] + (resultOff + (uint64_t)j * unit) * r->esz, unit);
                }
            }
            free(grid.mem);
        }
    } else {
        if (l1Algo == ORC_L1_NHR) {
            rc = nhr_reduce_scatter_scratch(r, &sc);
        } else {
            /* own share first: box j folds the other boxes' shares of unit j ascending into its own */
            for (uint32_t j = 0; j < l1; ++j) {
                uint64_t cur = j == l1 - 1 ? last : unit;
                for (uint32_t b = 0; b < l1; ++b) {
                    if (b != j) {
                        red_pair(r, scratch_at(&sc, j, j), scratch_at(&sc, b, j), cur);
                    }
                }
            }
        }
        for (uint32_t j = 0; j < l1 && rc == ORC_OK; ++j) {
            uint64_t cur = j == l1 - 1 ? last : unit;
            for (uint32_t b = 0; b < l1; ++b) {   /* AllGather: every box receives box j's unit j */
                red_narrow(r, scratch_at(&sc, j, j), result[b] + (resultOff + (uint64_t)j * unit) * r->esz, cur);
            }
        }
    }
    free(sc.mem);
    free(tmp);
    return rc;
}

/* ---------------------------------------------------------------------------------------------
 * Two-level ReduceScatter (ins_v2_reduce_scatter_sequence_executor_aicpu.cc:298-372, 388-500).  Boxes as
 * above; the input of every rank holds n slices of recvCount elements, slice b * l0 + i belongs to member i
 * of box b.  Per loop (a loop covers the same range of every slice, so the loops do not show in the result):
 *   step 1  l1 repeats of the mesh ReduceScatter inside every box (:311-319, repeatNum = l1, input stride
 *           l0 slices): in repeat q member i folds slice q * l0 + i of its box, its own input first
 *   step 2  the level-1 ReduceScatter between the members i of all boxes (:338-353): unit q of member i is
 *           what step 1 left for slice q * l0 + i; box j ends with unit j, which is rank j * l0 + i's output.
 * Level 1 (registrations :567-640): ORC_L1_RHD (reduce_scatter_rhd with its POST), ORC_L1_NHR, and ORC_L1_MESH
 * for the host-reduce template of PROD and the 64-bit types, own share first and the other boxes ascending
 * (reduce_scatter_aicpu_reduce_nhr_pcie.cc:212-280).
 * ------------------------------------------------------------------------------------------- */
int orc_reduce_scatter_two_level(uint32_t n, uint32_t l0, int l1Algo, const void* const* in, void* const* out,
                                 uint64_t recvCount, int dtype, int op, int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (l0 == 0 || n % l0 != 0 || l1Algo < ORC_L1_RHD || l1Algo > ORC_L1_MESH) {
        return ORC_E_PARA;
    }
    if (recvCount == 0) {
        return ORC_OK;
    }
    uint32_t l1 = n / l0;
    const uint8_t** src = (const uint8_t**)malloc(sizeof(uint8_t*) * n);
    void* tmp = malloc(recvCount * r.asz);
    scratch_t sc;
    if (!src || !tmp || scratch_alloc(&sc, l1, recvCount, r.asz) != ORC_OK) {
        free(src);
        free(tmp);
        return ORC_E_INTERNAL;
    }
    for (uint32_t j = 0; j < n; ++j) {
        src[j] = cbytes(in[j]);
    }
    for (uint32_t i = 0; i < l0 && rc == ORC_OK; ++i) {
        for (uint32_t b = 0; b < l1; ++b) {
            for (uint32_t q = 0; q < l1; ++q) {
                uint32_t at = l1Algo == ORC_L1_RHD ? orc_rhd_unit_start_of_rank(l1, q) : q;
                level0_fold(&r, l0, b, i, src, (uint64_t)(q * l0 + i) * recvCount, recvCount, scratch_at(&sc, b, at), tmp);
            }
        }
        if (l1Algo == ORC_L1_RHD) {
            rc = rhd_rs_frame(&r, &sc, 0);
        } else if (l1Algo == ORC_L1_NHR) {
            rc = nhr_reduce_scatter_scratch(&r, &sc);
        } else {
            for (uint32_t j = 0; j < l1; ++j) {
                for (uint32_t b = 0; b < l1; ++b) {
                    if (b != j) {
                        red_pair(&r, scratch_at(&sc, j, j), scratch_at(&sc, b, j), recvCount);
                    }
                }
            }
        }
        for (uint32_t j = 0; j < l1 && rc == ORC_OK; ++j) {
            uint32_t at = l1Algo == ORC_L1_RHD ? orc_rhd_unit_start_of_rank(l1, j) : j;
            red_narrow(&r, scratch_at(&sc, j, at), out[j * l0 + i], recvCount);
        }
    }
    free(sc.mem);
    free(src);
    free(tmp);
    return rc;
}

int orc_all_reduce_two_level(uint32_t n, uint32_t l0, int l1Algo, const void* const* in, void* const* out,
                             uint64_t count, int dtype, int op, int accMode, uint64_t maxCountPerLoop)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (l0 == 0 || n % l0 != 0 || l1Algo < ORC_L1_RHD || l1Algo > ORC_L1_MESH) {
        return ORC_E_PARA;
    }
    uint32_t l1 = n / l0;
    if (maxCountPerLoop == 0) {
        maxCountPerLoop = UINT64_MAX / 2;
    }
    maxCountPerLoop = maxCountPerLoop / n * n;   /* executor.cc:653-656 */
    if (maxCountPerLoop == 0) {
        return ORC_E_INTERNAL;
    }
    /* per-box result (the members of a box end with the same bytes), and the padded tiles of the RHD tail */
    uint8_t** result = (uint8_t**)calloc(l1, sizeof(uint8_t*));
    uint8_t* tiles = (uint8_t*)malloc((size_t)n * n * r.esz);
    uint8_t* tileOut = (uint8_t*)malloc((size_t)l1 * n * r.esz);
    const uint8_t** src = (const uint8_t**)malloc(sizeof(uint8_t*) * n);
    uint8_t** dst = (uint8_t**)malloc(sizeof(uint8_t*) * l1);
    if (!result || !tiles || !tileOut || !src || !dst) {
        rc = ORC_E_INTERNAL;
    }
    for (uint32_t b = 0; b < l1 && rc == ORC_OK; ++b) {
        result[b] = (uint8_t*)malloc((count ? count : 1) * r.esz);
        if (!result[b]) {
            rc = ORC_E_INTERNAL;
        }
    }
    uint64_t processed = 0;
    while (processed < count && rc == ORC_OK) {
        uint64_t remaining = count - processed;
        uint64_t valid, curr;
        int padded = 0;
        if (l1Algo == ORC_L1_RHD) {
            valid = orc_rhd_select_loop_count(remaining, maxCountPerLoop, n);
            curr = valid > n ? valid : n;
            padded = valid != curr;
        } else {
            valid = curr = remaining < maxCountPerLoop ? remaining : maxCountPerLoop;
        }
        uint64_t srcOff = processed;
        uint64_t dstOff = processed;
        for (uint32_t j = 0; j < n; ++j) {
            src[j] = cbytes(in[j]);
        }
        for (uint32_t b = 0; b < l1; ++b) {
            dst[b] = result[b];
        }
        if (padded) {
            /* rhd_tail.h:115-146: every rank stages its valid elements and doubles them up to the tile */
            for (uint32_t j = 0; j < n; ++j) {
                uint8_t* t = tiles + (size_t)j * n * r.esz;
                memcpy(t, cbytes(in[j]) + processed * r.esz, valid * r.esz);
                uint64_t filled = valid;
                while (filled < n) {
                    uint64_t c = filled < n - filled ? filled : n - filled;
                    memcpy(t + filled * r.esz, t, c * r.esz);
                    filled += c;
                }
                src[j] = t;
            }
            for (uint32_t b = 0; b < l1; ++b) {
                dst[b] = tileOut + (size_t)b * n * r.esz;
            }
            srcOff = 0;
            dstOff = 0;
        }
        uint64_t chunk = curr / l0;
        for (uint32_t i = 0; i < l0 && rc == ORC_OK; ++i) {
            uint64_t cur = (i == l0 - 1 && l1Algo != ORC_L1_RHD) ? curr - (uint64_t)i * chunk : chunk;
            uint64_t unit = cur / l1;
            uint64_t last = l1Algo == ORC_L1_RHD ? unit : cur - unit * (l1 - 1);
            rc = level1_exchange(&r, l0, l1, l1Algo, i, src, srcOff + (uint64_t)i * chunk, unit, last, dst,
                                 dstOff + (uint64_t)i * chunk);
        }
        if (padded && rc == ORC_OK) {
            for (uint32_t b = 0; b < l1; ++b) {
                memcpy(result[b] + processed * r.esz, tileOut + (size_t)b * n * r.esz, valid * r.esz);
            }
        }
        processed += valid;
    }
    if (rc == ORC_OK) {
        for (uint32_t j = 0; j < n; ++j) {
            memcpy(out[j], result[j / l0], count * r.esz);
        }
    }
    for (uint32_t b = 0; result && b < l1; ++b) {
        free(result[b]);
    }
    free(result);
    free(tiles);
    free(tileOut);
    free(src);
    free(dst);
    return rc;
}

/* ---------------------------------------------------------------------------------------------
 * Three levels (ins_v2_all_reduce_sequence_executor_aicpu_3level.cc, "3level.cc" below;
 * ins_v2_reduce_scatter_sequence_executor_3level.cc; reduce_sequence_executor_aicpu_3level.cc).  l0 consecutive
 * ranks form a box, l1 consecutive boxes a pod, l2 = n / (l0 * l1) pods: rank (g * l1 + b) * l0 + i is member i
 * of box b of pod g; between the boxes it talks to the members i of the boxes of its pod (3level.cc:209-216,
 * infos[1]), between the pods to the members i of the boxes b of the other pods (infos[2]).  Per loop of AllReduce
 * (3level.cc:586-693, 733-795):
 *   RSL0  mesh ReduceScatter inside every box: member i ends with chunk i, its own input first
 *   RSL1  the template between the boxes of a pod on chunk i cut into l1 sub-slices: box b ends with sub-slice b
 *   RSL2  the template between the pods on that sub-slice cut into l2 parts: pod g ends with part g
 *   AGL2, AGL1, AGL0  the AllGathers back.
 * Templates (registrations 3level.cc:806-838): NHR at both levels, or RHD at both; RSL1 keeps its POST (which
 * moves shares and folds nothing), RSL2 skips it and the representative's merged share is bridged (:622-660).
 * Cuts: NHR floor(len / d) with the rest in the last chunk / sub-slice / part (3level_utils.h:124-126, 150-160,
 * 3level.cc:361-370); RHD uniform units on the prefix aligned to n, the remainder staged into a padded tile
 * (rhd_tail.h:94-165).
 * The folds of a level run in the accumulation domain; a value is narrowed once, at the end.
 * ------------------------------------------------------------------------------------------- */
typedef struct {
    const red_t* r;
    uint32_t l0, l1, l2;
    int algo;                  /* ORC_L1_RHD or ORC_L1_NHR; ORC_L1_MESH with one pod */
    const uint8_t* const* src; /* n inputs (or staged tiles) */
    void* tmp;
} levels_t;

/* RSL0 + RSL1 for member i inside pod g on elements [off, off + (l1 - 1) * unit + last): vals[b] receives the
 * value box b ends with for sub-slice b (unit elements, `last` for the last box), in the accumulation domain. */
static int pod_reduce_scatter(const levels_t* lv, uint32_t g, uint32_t i, uint64_t off, uint64_t unit,
                              uint64_t last, uint8_t* const* vals)
{
    const red_t* r = lv->r;
    uint32_t l1 = lv->l1;
    uint64_t slot = last > unit ? last : unit;
    if (slot == 0) {
        return ORC_OK;
    }
    scratch_t sc;
    if (scratch_alloc(&sc, l1, slot, r->asz) != ORC_OK) {
        return ORC_E_INTERNAL;
    }
    memset(sc.mem, 0, (uint64_t)l1 * l1 * slot * r->asz);
    for (uint32_t b = 0; b < l1; ++b) {
        for (uint32_t j = 0; j < l1; ++j) {
            uint64_t cur = j == l1 - 1 ? last : unit;
            uint32_t at = lv->algo == ORC_L1_RHD ? orc_rhd_unit_start_of_rank(l1, j) : j;
            level0_fold(r, lv->l0, g * l1 + b, i, lv->src, off + (uint64_t)j * unit, cur, scratch_at(&sc, b, at), lv->tmp);
        }
    }
    int rc = ORC_OK;
    if (lv->algo == ORC_L1_MESH) {
        /* the host-reduce template: box j folds the other boxes' shares of unit j ascending into its own
         * (reduce_scatter_aicpu_reduce_nhr_pcie.cc:212-280) */
        for (uint32_t j = 0; j < l1; ++j) {
            for (uint32_t b = 0; b < l1; ++b) {
                if (b != j) {
                    red_pair(r, scratch_at(&sc, j, j), scratch_at(&sc, b, j), j == l1 - 1 ? last : unit);
                }
            }
        }
    } else {
        rc = lv->algo == ORC_L1_RHD ? rhd_rs_frame(r, &sc, 0) : nhr_reduce_scatter_scratch(r, &sc);
    }
    for (uint32_t j = 0; j < l1 && rc == ORC_OK; ++j) {
        uint64_t cur = j == l1 - 1 ? last : unit;
        uint32_t at = lv->algo == ORC_L1_RHD ? orc_rhd_unit_start_of_rank(l1, j) : j;
        memcpy(vals[j], scratch_at(&sc, j, at), cur * r->asz);
    }
    free(sc.mem);
    return rc;
}

/* RSL2 between the pods on one sub-slice: share[g] is what pod g holds for it (accumulation domain), cut into
 * l2 parts of `unit` elements (`last` for the last pod's); part k's final value goes, narrowed, to out + k * unit. */
static int pods_reduce_scatter(const levels_t* lv, uint8_t* const* share, uint64_t unit, uint64_t last, uint8_t* out)
{
    const red_t* r = lv->r;
    uint32_t l2 = lv->l2;
    uint64_t slot = last > unit ? last : unit;
    if (slot == 0) {
        return ORC_OK;
    }
    scratch_t sc;
    if (scratch_alloc(&sc, l2, slot, r->asz) != ORC_OK) {
        return ORC_E_INTERNAL;
    }
    memset(sc.mem, 0, (uint64_t)l2 * l2 * slot * r->asz);
    for (uint32_t g = 0; g < l2; ++g) {
        for (uint32_t k = 0; k < l2; ++k) {
            uint64_t cur = k == l2 - 1 ? last : unit;
            uint32_t at = lv->algo == ORC_L1_RHD ? orc_rhd_unit_start_of_rank(l2, k) : k;
            memcpy(scratch_at(&sc, g, at), share[g] + (uint64_t)k * unit * r->asz, cur * r->asz);
        }
    }
    int rc;
    if (lv->algo == ORC_L1_RHD) {
        /* POST skipped: a merged pod's share stays in its representative's slot 2t + 1 and is bridged to the
         * owner slot of the AllGather grid (rhd_tail.h:33-53); the AllGather only moves data */
        rc = rhd_rs_frame(r, &sc, 1);
        for (uint32_t k = 0; k < l2 && rc == ORC_OK; ++k) {
            orc_rhd_part1_t info;
            orc_rhd_part1(l2, k, ORC_INVALID_RANK, &info);
            const uint8_t* from;
            if (info.inPart1 && !info.isRepresentative) {
                orc_rhd_part1_t rep;
                orc_rhd_part1(l2, info.pairedAlgRank, ORC_INVALID_RANK, &rep);
                from = scratch_at(&sc, info.pairedAlgRank, rep.unitStart + 1);
            } else {
                from = scratch_at(&sc, k, orc_rhd_unit_start_of_rank(l2, k));
            }
            red_narrow(r, from, out + (uint64_t)k * unit * r->esz, k == l2 - 1 ? last : unit);
        }
    } else {
        rc = nhr_reduce_scatter_scratch(r, &sc);
        for (uint32_t k = 0; k < l2 && rc == ORC_OK; ++k) {
            red_narrow(r, scratch_at(&sc, k, k), out + (uint64_t)k * unit * r->esz, k == l2 - 1 ? last : unit);
        }
    }
    free(sc.mem);
    return rc;
}

/* One loop of `cur` elements from element `off` of lv->src into out + off (every rank ends with the same bytes);
 * uniform: every cut is exact (RHD), else floor with the rest in the last. */
static int levels_all_reduce_loop(const levels_t* lv, uint64_t off, uint64_t cur, int uniform, uint8_t* out,
                                  uint64_t outOff)
{
    const red_t* r = lv->r;
    uint32_t l0 = lv->l0, l1 = lv->l1, l2 = lv->l2;
    uint64_t chunk = cur / l0;
    uint64_t longest = cur - chunk * (l0 - 1);
    uint8_t** vals = (uint8_t**)calloc((size_t)l1 * l2, sizeof(uint8_t*));
    uint8_t** share = (uint8_t**)calloc(l2, sizeof(uint8_t*));
    int rc = vals && share ? ORC_OK : ORC_E_INTERNAL;
    for (uint32_t x = 0; x < l1 * l2 && rc == ORC_OK; ++x) {
        vals[x] = (uint8_t*)malloc((longest ? longest : 1) * r->asz);
        if (!vals[x]) {
            rc = ORC_E_INTERNAL;
        }
    }
    for (uint32_t i = 0; i < l0 && rc == ORC_OK; ++i) {
        uint64_t cLen = (i == l0 - 1 && !uniform) ? cur - (uint64_t)i * chunk : chunk;
        uint64_t cOff = (uint64_t)i * chunk;
        uint64_t sub = cLen / l1;
        uint64_t subLast = uniform ? sub : cLen - sub * (l1 - 1);
        for (uint32_t g = 0; g < l2 && rc == ORC_OK; ++g) {
            rc = pod_reduce_scatter(lv, g, i, off + cOff, sub, subLast, vals + (size_t)g * l1);
        }
        for (uint32_t j = 0; j < l1 && rc == ORC_OK; ++j) {
            uint64_t sLen = j == l1 - 1 ? subLast : sub;
            uint64_t part = sLen / l2;
            uint64_t partLast = uniform ? part : sLen - part * (l2 - 1);
            for (uint32_t g = 0; g < l2; ++g) {
                share[g] = vals[(size_t)g * l1 + j];
            }
            rc = pods_reduce_scatter(lv, share, part, partLast, out + (outOff + cOff + (uint64_t)j * sub) * r->esz);
        }
    }
    for (uint32_t x = 0; vals && x < l1 * l2; ++x) {
        free(vals[x]);
    }
    free(vals);
    free(share);
    return rc;
}

static int levels_check(uint32_t n, uint32_t l0, uint32_t l1, int algo)
{
    if (l0 == 0 || l1 == 0 || n % l0 != 0 || (n / l0) % l1 != 0 || algo < ORC_L1_RHD || algo > ORC_L1_MESH) {
        return ORC_E_PARA;
    }
    /* the host-reduce executors know two levels */
    return algo == ORC_L1_MESH && l1 != n / l0 ? ORC_E_PARA : ORC_OK;
}

int orc_all_reduce_three_level(uint32_t n, uint32_t l0, uint32_t l1, int algo, const void* const* in,
                               void* const* out, uint64_t count, int dtype, int op, int accMode, uint64_t cclBytes)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (levels_check(n, l0, l1, algo) != ORC_OK || algo == ORC_L1_MESH) {
        return ORC_E_PARA;
    }
    if (count == 0) {
        return ORC_OK;
    }
    uint64_t maxPerLoop = UINT64_MAX / 2 / n * n, resultElems = UINT64_MAX;
    if (cclBytes != 0) {
        rc = orc_sequence_max_count_per_loop(cclBytes, count, l0, n, r.esz, 128, algo == ORC_L1_RHD, &maxPerLoop,
                                             &resultElems);
        if (rc != ORC_OK) {
            return rc;
        }
    }
    levels_t lv = {&r, l0, l1, n / l0 / l1, algo, NULL, NULL};
    const uint8_t** src = (const uint8_t**)malloc(sizeof(uint8_t*) * n);
    uint8_t* tiles = (uint8_t*)malloc((size_t)n * n * r.esz);
    uint8_t* tileOut = (uint8_t*)malloc((size_t)n * r.esz);
    uint8_t* result = (uint8_t*)malloc(count * r.esz);
    lv.tmp = malloc(count * r.asz);
    lv.src = src;
    if (!src || !tiles || !tileOut || !result || !lv.tmp) {
        rc = ORC_E_INTERNAL;
    }
    uint64_t processed = 0;
    while (processed < count && rc == ORC_OK) {
        uint64_t remaining = count - processed;
        for (uint32_t j = 0; j < n; ++j) {
            src[j] = cbytes(in[j]);
        }
        if (algo == ORC_L1_RHD) {
            uint64_t valid = orc_rhd_select_loop_count(remaining, maxPerLoop, n);
            if (valid >= n) {
                rc = levels_all_reduce_loop(&lv, processed, valid, 1, result, processed);
            } else {
                /* rhd_tail.h:115-146: the valid elements staged and doubled up to a tile of n; only they come back */
                for (uint32_t j = 0; j < n; ++j) {
                    uint8_t* t = tiles + (size_t)j * n * r.esz;
                    memcpy(t, cbytes(in[j]) + processed * r.esz, valid * r.esz);
                    uint64_t filled = valid;
                    while (filled < n) {
                        uint64_t c = filled < n - filled ? filled : n - filled;
                        memcpy(t + filled * r.esz, t, c * r.esz);
                        filled += c;
                    }
                    src[j] = t;
                }
                rc = levels_all_reduce_loop(&lv, 0, n, 1, tileOut, 0);
                memcpy(result + processed * r.esz, tileOut, valid * r.esz);
            }
            processed += valid;
        } else {
            uint64_t cur = orc_sequence_select_loop_count(remaining, maxPerLoop, l0, resultElems);
            if (cur == 0) {
                rc = ORC_E_INTERNAL;
                break;
            }
            rc = levels_all_reduce_loop(&lv, processed, cur, 0, result, processed);
            processed += cur;
        }
    }
    for (uint32_t j = 0; j < n && rc == ORC_OK; ++j) {
        memcpy(out[j], result, count * r.esz);
    }
    free(src);
    free(tiles);
    free(tileOut);
    free(result);
    free(lv.tmp);
    return rc;
}

/* Reduce over two or three levels (reduce_sequence_executor_aicpu_3level.cc:744-990): the steps of the AllReduce
 * with the root's output as the only destination of the last AllGather, the cuts floor(len / d) with the rest in
 * the last for both templates (GenTempAlgParamsRSL0 / RSL1 / RSL2, :444-560), loops of
 * orc_sequence_max_count_per_loop with 4096-byte alignment (:877-889).  l1 = n / l0 makes it the two-level form. */
int orc_reduce_levels(uint32_t n, uint32_t l0, uint32_t l1, int algo, const void* const* in, void* const* out,
                      uint64_t count, int dtype, int op, uint32_t root, int accMode, uint64_t cclBytes)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (levels_check(n, l0, l1, algo) != ORC_OK || root >= n) {
        return ORC_E_PARA;
    }
    if (count == 0) {
        return ORC_OK;
    }
    uint64_t maxPerLoop = UINT64_MAX / 2 / n * n, resultElems = UINT64_MAX;
    if (cclBytes != 0) {
        rc = orc_sequence_max_count_per_loop(cclBytes, count, l0, n, r.esz, 4096, 0, &maxPerLoop, &resultElems);
        if (rc != ORC_OK) {
            return rc;
        }
    }
    levels_t lv = {&r, l0, l1, n / l0 / l1, algo, NULL, NULL};
    const uint8_t** src = (const uint8_t**)malloc(sizeof(uint8_t*) * n);
    lv.tmp = malloc(count * r.asz);
    lv.src = src;
    if (!src || !lv.tmp) {
        rc = ORC_E_INTERNAL;
    }
    for (uint32_t j = 0; j < n && rc == ORC_OK; ++j) {
        src[j] = cbytes(in[j]);
    }
    uint64_t processed = 0;
    while (processed < count && rc == ORC_OK) {
        uint64_t cur = orc_sequence_select_loop_count(count - processed, maxPerLoop, l0, resultElems);
        if (cur == 0) {
            rc = ORC_E_INTERNAL;
            break;
        }
        rc = levels_all_reduce_loop(&lv, processed, cur, 0, bytes(out[root]), processed);
        processed += cur;
    }
    free(src);
    free(lv.tmp);
    return rc;
}

/* ReduceScatter over three levels (ins_v2_reduce_scatter_sequence_executor_3level.cc:243-256): the mesh
 * ReduceScatter inside every box for the slices of every box of the world, the template between the boxes of a
 * pod for the slices of every pod, the template between the pods; rank (g * l1 + b) * l0 + i ends with its slice. */
int orc_reduce_scatter_three_level(uint32_t n, uint32_t l0, uint32_t l1, int algo, const void* const* in,
                                   void* const* out, uint64_t recvCount, int dtype, int op, int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (levels_check(n, l0, l1, algo) != ORC_OK || algo == ORC_L1_MESH) {
        return ORC_E_PARA;
    }
    if (recvCount == 0) {
        return ORC_OK;
    }
    uint32_t l2 = n / l0 / l1;
    const uint8_t** src = (const uint8_t**)malloc(sizeof(uint8_t*) * n);
    void* tmp = malloc(recvCount * r.asz);
    scratch_t sc1, sc2;
    sc1.mem = sc2.mem = NULL;
    if (!src || !tmp || scratch_alloc(&sc1, l1, recvCount, r.asz) != ORC_OK ||
        scratch_alloc(&sc2, l2, recvCount, r.asz) != ORC_OK) {
        rc = ORC_E_INTERNAL;
    }
    for (uint32_t j = 0; j < n && rc == ORC_OK; ++j) {
        src[j] = cbytes(in[j]);
    }
    for (uint32_t i = 0; i < l0 && rc == ORC_OK; ++i) {
        for (uint32_t b = 0; b < l1 && rc == ORC_OK; ++b) {
            /* the slices (q, b, i) of all pods q, as the pods hold them after RSL1: pod g's boxes fold their
             * level-0 results for the slices (q, b', i); box b ends with the units b */
            for (uint32_t q = 0; q < l2 && rc == ORC_OK; ++q) {
                for (uint32_t g = 0; g < l2 && rc == ORC_OK; ++g) {
                    for (uint32_t bb = 0; bb < l1; ++bb) {
                        for (uint32_t u = 0; u < l1; ++u) {
                            uint32_t at = algo == ORC_L1_RHD ? orc_rhd_unit_start_of_rank(l1, u) : u;
                            level0_fold(&r, l0, g * l1 + bb, i, src, (uint64_t)((q * l1 + u) * l0 + i) * recvCount,
                                        recvCount, scratch_at(&sc1, bb, at), tmp);
                        }
                    }
                    rc = algo == ORC_L1_RHD ? rhd_rs_frame(&r, &sc1, 0) : nhr_reduce_scatter_scratch(&r, &sc1);
                    uint32_t at1 = algo == ORC_L1_RHD ? orc_rhd_unit_start_of_rank(l1, b) : b;
                    uint32_t at2 = algo == ORC_L1_RHD ? orc_rhd_unit_start_of_rank(l2, q) : q;
                    memcpy(scratch_at(&sc2, g, at2), scratch_at(&sc1, b, at1), recvCount * r.asz);
                }
            }
            if (rc == ORC_OK) {
                rc = algo == ORC_L1_RHD ? rhd_rs_frame(&r, &sc2, 0) : nhr_reduce_scatter_scratch(&r, &sc2);
            }
            for (uint32_t g = 0; g < l2 && rc == ORC_OK; ++g) {
                uint32_t at2 = algo == ORC_L1_RHD ? orc_rhd_unit_start_of_rank(l2, g) : g;
                red_narrow(&r, scratch_at(&sc2, g, at2), out[(g * l1 + b) * l0 + i], recvCount);
            }
        }
    }
    free(sc1.mem);
    free(sc2.mem);
    free(src);
    free(tmp);
    return rc;
}

/* Loop rule of the three-level sequence executors (3level.cc:524-534; reduce_sequence_executor_aicpu_3level.cc:
 * 877-889): the buffer, less the two tail tiles of rhd_tail.h:64-92 when they are needed, is cut into l0 + 1
 * slices of whole elements; a loop holds what l0 of them take, floored to `align` bytes, whole elements and a
 * multiple of `total`.  resultElems: the elements of one slice. */
int orc_sequence_max_count_per_loop(uint64_t cclBytes, uint64_t count, uint32_t l0, uint32_t total, uint64_t esz,
                                    uint64_t align, int rhdTail, uint64_t* maxCount, uint64_t* resultElems)
{
    if (l0 == 0 || total == 0 || esz == 0 || align == 0) {
        return ORC_E_PARA;
    }
    uint64_t ws = cclBytes;
    if (rhdTail && count % total != 0) {
        if (total > ws / esz / 2) {
            return ORC_E_INTERNAL;
        }
        uint64_t tile = (uint64_t)total * esz;
        uint64_t slot = (tile / 128 + (tile % 128 != 0)) * 128;
        if (slot >= ws / 2) {
            return ORC_E_INTERNAL;
        }
        ws -= 2 * slot;
    }
    uint64_t slice = ws / (l0 + 1) / esz * esz;
    uint64_t comm = (uint64_t)l0 * slice;
    *resultElems = slice / esz;
    *maxCount = comm / align * align / esz / total * total;
    return *maxCount == 0 ? ORC_E_INTERNAL : ORC_OK;
}

/* 3level.cc:704-731: a last loop whose last chunk, floor(cur / l0) + cur mod l0 elements, would not fit the
 * result slice is shortened; what it leaves runs as one more loop. */
uint64_t orc_sequence_select_loop_count(uint64_t remaining, uint64_t maxCountPerLoop, uint32_t l0, uint64_t resultElems)
{
    if (remaining > maxCountPerLoop) {
        return maxCountPerLoop;
    }
    uint64_t cur = remaining;
    uint64_t q = cur / l0;
    uint64_t rem = cur % l0;
    if (q + rem > resultElems && q > 0) {
        if (resultElems == 0) {
            return 0;
        }
        uint64_t newQ = q - 1;
        uint64_t newR;
        if (newQ >= resultElems) {
            newQ = resultElems;
            newR = 0;
        } else {
            newR = l0 - 1 < resultElems - newQ ? l0 - 1 : resultElems - newQ;
        }
        cur = newQ * l0 + newR;
    }
    return cur;
}

/* a12: while blocks > 1: M = largest power of two < blocks; for src = M..blocks-1:
 * slot[src % M] = slot[src] (+) slot[src % M]; blocks = M.  Block v is rank v's contribution. */
static uint32_t largest_pow2_less_than(uint32_t v)
{
    if (v <= 1) {
        return 0;
    }
    uint32_t p = 1;
    while (p * 2 < v) p *= 2;
    return p;
}

static int order_preserved_fold(const red_t* r, uint32_t n, const void* const* in, uint64_t srcElemOff,
                                uint64_t count, void* accOut /* count * asz */)
{
    uint8_t* slots = (uint8_t*)malloc((uint64_t)n * count * r->asz);
    if (!slots) {
        return ORC_E_INTERNAL;
    }
    for (uint32_t v = 0; v < n; ++v) {
        red_widen(r, cbytes(in[v]) + srcElemOff * r->esz, slots + (uint64_t)v * count * r->asz, count);
    }
    uint32_t remaining = n;
    while (remaining > 1) {
        uint32_t M = largest_pow2_less_than(remaining);
        if (M == 0) {
            break;
        }
        for (uint32_t src = M; src < remaining; ++src) {
            red_pair(r, slots + (uint64_t)(src % M) * count * r->asz, slots + (uint64_t)src * count * r->asz, count);
        }
        remaining = M;
    }
    memcpy(accOut, slots, count * r->asz);
    free(slots);
    return ORC_OK;
}

int orc_reduce_scatter_order_preserved(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount,
                                       int dtype, int op, int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK || recvCount == 0) {
        return rc;
    }
    void* acc = malloc(recvCount * r.asz);
    if (!acc) {
        return ORC_E_INTERNAL;
    }
    for (uint32_t k = 0; k < n && rc == ORC_OK; ++k) {
        rc = order_preserved_fold(&r, n, in, (uint64_t)k * recvCount, recvCount, acc);
        if (rc == ORC_OK) {
            red_narrow(&r, acc, out[k], recvCount);
        }
    }
    free(acc);
    return rc;
}

int orc_all_reduce_order_preserved(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype,
                                   int op, int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK || count == 0) {
        return rc;
    }
    void* acc = malloc(count * r.asz);
    if (!acc) {
        return ORC_E_INTERNAL;
    }
    rc = order_preserved_fold(&r, n, in, 0, count, acc);
    if (rc == ORC_OK) {
        for (uint32_t k = 0; k < n; ++k) red_narrow(&r, acc, out[k], count);
    }
    free(acc);
    return rc;
}

/* Vector-core mesh: rank k's output is cut into N chunks of recvCount / N elements (the last takes
 * the remainder); chunk c = copy of peer c's slice, then peers c+1, c+2, ... (mod N) folded in. */
int orc_reduce_scatter_aiv_mesh(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                                int op, int accMode)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK || recvCount == 0) {
        return rc;
    }
    uint64_t per = recvCount / n;
    void* acc = malloc(recvCount * r.asz);
    void* tmp = malloc(recvCount * r.asz);
    if (!acc || !tmp) {
        free(acc);
        free(tmp);
        return ORC_E_INTERNAL;
    }
    for (uint32_t k = 0; k < n; ++k) {
        for (uint32_t c = 0; c < n; ++c) {
            uint64_t off = (uint64_t)c * per;
            uint64_t cnt = (c == n - 1) ? recvCount - per * (n - 1) : per;
            if (cnt == 0) {
                continue;
            }
            for (uint32_t i = 0; i < n; ++i) {
                uint32_t peer = (i + c) % n;
                const uint8_t* src = cbytes(in[peer]) + ((uint64_t)k * recvCount + off) * r.esz;
                if (i == 0) {
                    red_widen(&r, src, acc, cnt);
                } else {
                    red_pair_from_storage(&r, acc, src, cnt, tmp);
                }
            }
            red_narrow(&r, acc, bytes(out[k]) + off * r.esz, cnt);
        }
    }
    free(acc);
    free(tmp);
    return ORC_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Mesh-chunk order (reduce_scatter_mesh_1D_meshchunk.cc, reduce_scatter_v_mesh_1D_meshchunk.cc,
 * all_reduce_mesh_1D_two_shot_mesh_chunk.cc)
 * ------------------------------------------------------------------------------------------- */
/* Sizes in elements of the n - 1 segments of a slice of len elements.  align4k: the ReduceScatter(V) rule
 * (meshchunk.cc:233-258, v_meshchunk.cc:147-191): floor(bytes / (n-1)) rounded down to 4096 bytes for all but
 * the last segment, which takes the rest; when that is zero or n - 1 < 2, and always for AllReduce
 * (two_shot_mesh_chunk.cc:181-199), element-wise with the first len mod (n-1) segments one longer. */
#define ORC_MAX_RANKS 1024u   /* bound of the stack tables below */

void orc_mesh_chunk_segments(uint64_t len, uint32_t n, uint32_t elemSize, int align4k, uint64_t* segLen)
{
    if (n < 2) {
        return;
    }
    uint64_t segs = n - 1;
    uint64_t aligned = align4k ? (len * elemSize / segs) / 4096 * 4096 : 0;
    if (align4k && segs >= 2 && aligned > 0) {
        for (uint64_t i = 0; i + 1 < segs; ++i) segLen[i] = aligned / elemSize;
        segLen[segs - 1] = len - (aligned / elemSize) * (segs - 1);
        return;
    }
    uint64_t big = len % segs;
    for (uint64_t i = 0; i < segs; ++i) segLen[i] = len / segs + (i < big ? 1 : 0);
}

/* The exchange itself: slice k (sliceLen[k] elements, sliceOff[k] elements into every input) starts as rank
 * k's own input (PreCopy / LocalDataCopy); in step s every sender pushes, for i = 0 .. n-2, segment i of the
 * slice of the rank num = s + i + 1 (+1 from n on) places below it, and the owner write-reduces it
 * (DoMeshChunk, meshchunk.cc:277-375; v_meshchunk.cc:202-265; two_shot_mesh_chunk.cc:220-295).
 * acc[k] receives the widened result of slice k. */
static int mesh_chunk_exchange(const red_t* r, uint32_t n, const void* const* in, const uint64_t* sliceOff,
                               const uint64_t* sliceLen, int align4k, void** acc)
{
    uint64_t longest = 0;
    for (uint32_t k = 0; k < n; ++k) longest = sliceLen[k] > longest ? sliceLen[k] : longest;
    void* tmp = malloc((longest ? longest : 1) * r->asz);
    uint64_t* seg = (uint64_t*)malloc(sizeof(uint64_t) * n * n);
    uint64_t* off = (uint64_t*)malloc(sizeof(uint64_t) * n * n);
    if (!tmp || !seg || !off) {
        free(tmp);
        free(seg);
        free(off);
        return ORC_E_INTERNAL;
    }
    for (uint32_t k = 0; k < n; ++k) {
        red_widen(r, cbytes(in[k]) + sliceOff[k] * r->esz, acc[k], sliceLen[k]);
        orc_mesh_chunk_segments(sliceLen[k], n, (uint32_t)r->esz, align4k, seg + (size_t)k * n);
        uint64_t o = 0;
        for (uint32_t i = 0; i + 1 < n; ++i) {
            off[(size_t)k * n + i] = o;
            o += seg[(size_t)k * n + i];
        }
    }
    for (uint32_t step = 0; step + 1 < n; ++step) {
        for (uint32_t i = 0; i + 1 < n; ++i) {
            uint32_t num = step + i + 1;
            if (num >= n) {
                num += 1;
            }
            for (uint32_t sender = 0; sender < n; ++sender) {
                uint32_t next = (sender + num) % n;
                uint32_t owner = (2 * sender + n - next) % n;
                uint64_t cnt = seg[(size_t)owner * n + i];
                uint64_t at = off[(size_t)owner * n + i];
                if (cnt != 0) {
                    red_pair_from_storage(r, bytes(acc[owner]) + at * r->asz,
                                          cbytes(in[sender]) + (sliceOff[owner] + at) * r->esz, cnt, tmp);
                }
            }
        }
    }
    free(tmp);
    free(seg);
    free(off);
    return ORC_OK;
}

static int mesh_chunk_run(const red_t* r, uint32_t n, const void* const* in, const uint64_t* sliceOff,
                          const uint64_t* sliceLen, int align4k, void** acc)
{
    for (uint32_t k = 0; k < n; ++k) {
        acc[k] = malloc((sliceLen[k] ? sliceLen[k] : 1) * r->asz);
        if (!acc[k]) {
            for (uint32_t j = 0; j < k; ++j) free(acc[j]);
            return ORC_E_INTERNAL;
        }
    }
    int rc = mesh_chunk_exchange(r, n, in, sliceOff, sliceLen, align4k, acc);
    if (rc != ORC_OK) {
        for (uint32_t k = 0; k < n; ++k) free(acc[k]);
    }
    return rc;
}

int orc_reduce_scatter_mesh_chunk(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                                  int op, int accMode, uint64_t maxCountPerLoop)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK || recvCount == 0) {
        return rc;
    }
    if (n == 0 || n > ORC_MAX_RANKS) {
        return ORC_E_PARA;
    }
    if (n == 1) {
        memmove(out[0], in[0], recvCount * r.esz);
        return ORC_OK;
    }
    if (maxCountPerLoop == 0) {
        maxCountPerLoop = recvCount;
    }
    uint64_t sliceOff[ORC_MAX_RANKS], sliceLen[ORC_MAX_RANKS];
    void* acc[ORC_MAX_RANKS];
    /* reduce_scatter_sole_executor.cc:250-277: full loops, the last one takes what is left */
    for (uint64_t done = 0; done < recvCount && rc == ORC_OK;) {
        uint64_t cur = recvCount - done < maxCountPerLoop ? recvCount - done : maxCountPerLoop;
        for (uint32_t k = 0; k < n; ++k) {
            sliceOff[k] = (uint64_t)k * recvCount + done;
            sliceLen[k] = cur;
        }
        rc = mesh_chunk_run(&r, n, in, sliceOff, sliceLen, 1, acc);
        if (rc == ORC_OK) {
            for (uint32_t k = 0; k < n; ++k) {
                red_narrow(&r, acc[k], bytes(out[k]) + done * r.esz, cur);
                free(acc[k]);
            }
        }
        done += cur;
    }
    return rc;
}

int orc_reduce_scatter_v_mesh_chunk(uint32_t n, const void* const* in, void* const* out, const uint64_t* counts,
                                    const uint64_t* displs, int dtype, int op, int accMode)
{
    if (dtype == ORC_UINT64 || dtype == ORC_FP64) {
        return ORC_E_NOT_SUPPORT;   /* reduce_scatter_v.cc:231-236 */
    }
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (n == 0 || n > ORC_MAX_RANKS) {
        return ORC_E_PARA;
    }
    if (n == 1) {
        memmove(out[0], in[0], counts[0] * r.esz);     /* op_common.cc:4490-4491: from the start of sendBuf */
        return ORC_OK;
    }
    void* acc[ORC_MAX_RANKS];
    rc = mesh_chunk_run(&r, n, in, displs, counts, 1, acc);     /* always one loop (v_sole_executor.cc:158-171) */
    if (rc == ORC_OK) {
        for (uint32_t k = 0; k < n; ++k) {
            red_narrow(&r, acc[k], out[k], counts[k]);
            free(acc[k]);
        }
    }
    return rc;
}

int orc_all_reduce_mesh_chunk(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                              int accMode, uint64_t maxCountPerLoop)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK || count == 0) {
        return rc;
    }
    if (n == 0 || n > ORC_MAX_RANKS) {
        return ORC_E_PARA;
    }
    if (n == 1) {
        memmove(out[0], in[0], count * r.esz);
        return ORC_OK;
    }
    if (maxCountPerLoop == 0) {
        maxCountPerLoop = count;
    }
    uint64_t sliceOff[ORC_MAX_RANKS], sliceLen[ORC_MAX_RANKS];
    void* acc[ORC_MAX_RANKS];
    for (uint64_t done = 0; done < count && rc == ORC_OK;) {
        uint64_t cur = count - done < maxCountPerLoop ? count - done : maxCountPerLoop;
        uint64_t chunk = orc_round_up(cur, n);          /* two_shot_mesh_chunk.cc:86-112 */
        for (uint32_t k = 0; k < n; ++k) {
            uint64_t at = (uint64_t)k * chunk;
            sliceOff[k] = done + (at < cur ? at : cur);
            sliceLen[k] = at >= cur ? 0 : (cur - at > chunk ? chunk : cur - at);
        }
        rc = mesh_chunk_run(&r, n, in, sliceOff, sliceLen, 0, acc);
        if (rc == ORC_OK) {
            for (uint32_t k = 0; k < n; ++k) {
                for (uint32_t m = 0; m < n; ++m) {
                    red_narrow(&r, acc[k], bytes(out[m]) + sliceOff[k] * r.esz, sliceLen[k]);
                }
                free(acc[k]);
            }
        }
        done += cur;
    }
    return rc;
}

/* ---------------------------------------------------------------------------------------------
 * a13 / a14 / a15: copies
 * ------------------------------------------------------------------------------------------- */
static int copy_dtype_ok(int dtype)
{
    /* Non-reduce ops reject only int128 and invalid values (op_common.cc:4349-4364). */
    return orc_dtype_size(dtype) != 0 && dtype != 12 && dtype != 13;
}

int orc_all_gather(uint32_t n, const void* const* in, void* const* out, uint64_t sendCount, int dtype)
{
    if (!copy_dtype_ok(dtype)) {
        return ORC_E_NOT_SUPPORT;
    }
    size_t esz = orc_dtype_size(dtype);
    /* Gather into a temporary first so that an output aliasing an input stays well defined. */
    uint8_t* all = (uint8_t*)malloc((uint64_t)n * sendCount * esz + 1);
    if (!all) {
        return ORC_E_INTERNAL;
    }
    for (uint32_t r = 0; r < n; ++r) memcpy(all + (uint64_t)r * sendCount * esz, in[r], sendCount * esz);
    for (uint32_t r = 0; r < n; ++r) memcpy(out[r], all, (uint64_t)n * sendCount * esz);
    free(all);
    return ORC_OK;
}

int orc_all_gather_v(uint32_t n, const void* const* in, void* const* out, const uint64_t* counts,
                     const uint64_t* displs, int dtype)
{
    if (!copy_dtype_ok(dtype)) {
        return ORC_E_NOT_SUPPORT;
    }
    size_t esz = orc_dtype_size(dtype);
    /* Non-empty intervals must not overlap (all_gather_v.cc:200-240). */
    for (uint32_t a = 0; a < n; ++a) {
        if (counts[a] == 0) continue;
        if (displs[a] + counts[a] < displs[a]) return ORC_E_PARA;
        for (uint32_t b = a + 1; b < n; ++b) {
            if (counts[b] == 0) continue;
            if (displs[a] < displs[b] + counts[b] && displs[b] < displs[a] + counts[a]) return ORC_E_PARA;
        }
    }
    for (uint32_t dst = 0; dst < n; ++dst) {
        for (uint32_t src = 0; src < n; ++src) {
            memcpy(bytes(out[dst]) + displs[src] * esz, in[src], counts[src] * esz);
        }
    }
    return ORC_OK;
}

int orc_all_to_all_v(uint32_t n, const void* const* in, void* const* out, const uint64_t* sendCounts,
                     const uint64_t* sdispls, const uint64_t* recvCounts, const uint64_t* rdispls, int dtype)
{
    if (!copy_dtype_ok(dtype)) {
        return ORC_E_NOT_SUPPORT;
    }
    size_t esz = orc_dtype_size(dtype);
    for (uint32_t i = 0; i < n; ++i) {
        for (uint32_t j = 0; j < n; ++j) {
            if (recvCounts[(uint64_t)i * n + j] != sendCounts[(uint64_t)j * n + i]) {
                return ORC_E_PARA;
            }
        }
    }
    for (uint32_t i = 0; i < n; ++i) {
        for (uint32_t j = 0; j < n; ++j) {
            uint64_t cnt = sendCounts[(uint64_t)j * n + i];
            memcpy(bytes(out[i]) + rdispls[(uint64_t)i * n + j] * esz, cbytes(in[j]) + sdispls[(uint64_t)j * n + i] * esz,
                   cnt * esz);
        }
    }
    return ORC_OK;
}

int orc_all_to_all(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype)
{
    uint64_t nn = (uint64_t)n * n;
    uint64_t* t = (uint64_t*)malloc(sizeof(uint64_t) * nn * 2 + 1);
    if (!t) {
        return ORC_E_INTERNAL;
    }
    uint64_t* cnt = t;
    uint64_t* dis = t + nn;
    for (uint32_t r = 0; r < n; ++r) {
        uint64_t off = 0;   /* ConvertAlltoAllParam, all_to_all_v.cc:411-421 */
        for (uint32_t i = 0; i < n; ++i) {
            cnt[(uint64_t)r * n + i] = count;
            dis[(uint64_t)r * n + i] = off;
            off += count;
        }
    }
    int rc = orc_all_to_all_v(n, in, out, cnt, dis, cnt, dis, dtype);
    free(t);
    return rc;
}

void orc_all_to_all_vc_params(uint32_t n, uint32_t rank, const uint64_t* matrix, uint64_t* sendCounts,
                              uint64_t* recvCounts, uint64_t* sdispls, uint64_t* rdispls)
{
    uint64_t off = 0;
    for (uint32_t i = 0; i < n; ++i) {   /* all_to_all_v.cc:444-448 */
        sendCounts[i] = matrix[(uint64_t)rank * n + i];
        sdispls[i] = off;
        off += sendCounts[i];
    }
    off = 0;
    for (uint32_t i = 0; i < n; ++i) {   /* :450-455 */
        recvCounts[i] = matrix[(uint64_t)i * n + rank];
        rdispls[i] = off;
        off += recvCounts[i];
    }
}

int orc_all_to_all_vc(uint32_t n, const void* const* in, void* const* out, const uint64_t* matrix, int dtype)
{
    uint64_t nn = (uint64_t)n * n;
    uint64_t* t = (uint64_t*)malloc(sizeof(uint64_t) * nn * 4 + 1);
    if (!t) {
        return ORC_E_INTERNAL;
    }
    for (uint32_t r = 0; r < n; ++r) {
        orc_all_to_all_vc_params(n, r, matrix, t + (uint64_t)r * n, t + nn + (uint64_t)r * n,
                                 t + 2 * nn + (uint64_t)r * n, t + 3 * nn + (uint64_t)r * n);
    }
    int rc = orc_all_to_all_v(n, in, out, t, t + 2 * nn, t + nn, t + 3 * nn, dtype);
    free(t);
    return rc;
}

int orc_reduce_scatter_v_mesh(uint32_t n, const void* const* in, void* const* out, const uint64_t* counts,
                              const uint64_t* displs, int dtype, int op, int accMode)
{
    if (dtype == ORC_UINT64 || dtype == ORC_FP64) {
        return ORC_E_NOT_SUPPORT;   /* reduce_scatter_v.cc:231-236 */
    }
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    for (uint32_t k = 0; k < n; ++k) {
        uint64_t count = counts[k];
        if (count == 0) {
            continue;
        }
        void* acc = malloc(count * r.asz);
        void* tmp = r.accF32 ? malloc(count * r.asz) : NULL;
        if (!acc || (r.accF32 && !tmp)) {
            free(acc);
            free(tmp);
            return ORC_E_INTERNAL;
        }
        uint64_t base = displs[k] * r.esz;
        red_widen(&r, cbytes(in[k]) + base, acc, count);          /* own input first (:127-135) */
        for (uint32_t t = 0; t < n; ++t) {
            if (t != k) {
                red_pair_from_storage(&r, acc, cbytes(in[t]) + base, count, tmp);   /* :145-159 */
            }
        }
        red_narrow(&r, acc, out[k], count);
        free(acc);
        free(tmp);
    }
    return ORC_OK;
}

int orc_reduce_mesh(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                    int accMode, uint32_t root)
{
    if (root >= n) {
        return ORC_E_PARA;
    }
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (count == 0) {
        return ORC_OK;
    }
    void* acc = malloc(count * r.asz);
    void* tmp = r.accF32 ? malloc(count * r.asz) : NULL;
    if (!acc || (r.accF32 && !tmp)) {
        free(acc);
        free(tmp);
        return ORC_E_INTERNAL;
    }
    red_widen(&r, in[0], acc, count);                              /* base slot 0 (:268-281) */
    for (uint32_t idx = 1; idx < n; ++idx) {
        red_pair_from_storage(&r, acc, in[idx], count, tmp);       /* :295-298 */
    }
    red_narrow(&r, acc, out[root], count);
    free(acc);
    free(tmp);
    return ORC_OK;
}

int orc_reduce_two_shot(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                        int accMode, uint32_t root, uint64_t maxCountPerLoop)
{
    if (root >= n) {
        return ORC_E_PARA;
    }
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK || count == 0) {
        return rc;
    }
    if (maxCountPerLoop == 0) {
        maxCountPerLoop = count;
    }
    void* acc = malloc(count * r.asz);
    void* tmp = malloc(count * r.asz);
    if (!acc || !tmp) {
        free(acc);
        free(tmp);
        return ORC_E_INTERNAL;
    }
    /* reduce_sole_executor.cc:203-232: full loops, the last one takes what is left */
    for (uint64_t done = 0; done < count;) {
        uint64_t cur = count - done < maxCountPerLoop ? count - done : maxCountPerLoop;
        uint64_t base = cur / n, rem = cur % n;                       /* CalcSlice :138-162 */
        uint64_t off = done;
        for (uint32_t k = 0; k < n; ++k) {
            uint64_t len = base + (k < rem ? 1 : 0);
            if (len != 0) {
                /* slot k holds rank k's own slice (:191-198); the others fold into it ascending (:254-263) */
                red_widen(&r, cbytes(in[k]) + off * r.esz, acc, len);
                for (uint32_t t = 0; t < n; ++t) {
                    if (t != k) {
                        red_pair_from_storage(&r, acc, cbytes(in[t]) + off * r.esz, len, tmp);
                    }
                }
                red_narrow(&r, acc, bytes(out[root]) + off * r.esz, len);    /* gathered by the root */
            }
            off += len;
        }
        done += cur;
    }
    free(acc);
    free(tmp);
    return ORC_OK;
}

int orc_broadcast(uint32_t n, void* const* buf, uint64_t count, int dtype, uint32_t root)
{
    if (!copy_dtype_ok(dtype)) {
        return ORC_E_NOT_SUPPORT;
    }
    if (root >= n) {
        return ORC_E_PARA;
    }
    size_t esz = orc_dtype_size(dtype);
    for (uint32_t r = 0; r < n; ++r) {
        if (r != root) {
            memcpy(buf[r], buf[root], count * esz);
        }
    }
    return ORC_OK;
}

int orc_scatter(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype, uint32_t root)
{
    if (!copy_dtype_ok(dtype)) {
        return ORC_E_NOT_SUPPORT;
    }
    if (root >= n) {
        return ORC_E_PARA;
    }
    size_t esz = orc_dtype_size(dtype);
    for (uint32_t r = 0; r < n; ++r) {
        memcpy(out[r], cbytes(in[root]) + (uint64_t)r * recvCount * esz, recvCount * esz);
    }
    return ORC_OK;
}

/* a5: LocalCopySlices (wrapper.cc:930-997).  Zero-size slices are skipped; a slice whose source and
 * destination both continue the pending run is merged into it; the pending run is issued when the
 * next slice does not continue it or at the last slice. */
uint32_t orc_local_copy_slices(uint32_t nSlices, const uint64_t* srcOff, const uint64_t* dstOff,
                               const uint64_t* sizes, uint64_t* copies)
{
    if (nSlices == 0) {
        return 0;
    }
    uint32_t issued = 0;
    uint64_t curSrc = srcOff[0], curDst = dstOff[0], curSize = sizes[0];
    for (uint32_t i = 0; i < nSlices; ++i) {
        if (sizes[i] == 0) {
            continue;
        }
        if (i == nSlices - 1) {
            copies[issued * 3 + 0] = curSrc;
            copies[issued * 3 + 1] = curDst;
            copies[issued * 3 + 2] = curSize;
            issued++;
        } else if (srcOff[i + 1] == curSrc + curSize && dstOff[i + 1] == curDst + curSize) {
            curSize += sizes[i + 1];
        } else {
            copies[issued * 3 + 0] = curSrc;
            copies[issued * 3 + 1] = curDst;
            copies[issued * 3 + 2] = curSize;
            issued++;
            curSrc = srcOff[i + 1];
            curDst = dstOff[i + 1];
            curSize = sizes[i + 1];
        }
    }
    return issued;
}

/* ---------------------------------------------------------------------------------------------
 * "All cores" CPU baseline: static split of the element range over threads.
 * ------------------------------------------------------------------------------------------- */
typedef struct {
    int isRs;
    uint32_t n;
    const void* const* in;
    void* const* out;
    uint64_t recvCount, first, count;
    const red_t* r;
    int rc;
} mt_job_t;

static void* mt_worker(void* arg)
{
    mt_job_t* j = (mt_job_t*)arg;
    if (j->isRs) {
        j->rc = reduce_scatter_mesh_range(j->n, j->in, j->out, j->recvCount, j->first, j->count, j->r);
    } else {
        j->rc = all_reduce_mesh_range(j->n, j->in, j->out, j->first, j->count, j->r);
    }
    return NULL;
}

static int run_mt(int isRs, uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                  int accMode, uint32_t nThreads)
{
    red_t r;
    int rc = red_init(&r, dtype, op, accMode);
    if (rc != ORC_OK) {
        return rc;
    }
    if (nThreads == 0) {
        nThreads = 1;
    }
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * nThreads);
    mt_job_t* jobs = (mt_job_t*)malloc(sizeof(mt_job_t) * nThreads);
    uint64_t per = (count + nThreads - 1) / nThreads;
    uint32_t started = 0;
    for (uint32_t t = 0; t < nThreads; ++t) {
        uint64_t first = (uint64_t)t * per;
        if (first >= count) {
            break;
        }
        mt_job_t j = {isRs, n, in, out, count, first, (count - first < per) ? count - first : per, &r, ORC_OK};
        jobs[t] = j;
        pthread_create(&th[t], NULL, mt_worker, &jobs[t]);
        started++;
    }
    for (uint32_t t = 0; t < started; ++t) {
        pthread_join(th[t], NULL);
        if (jobs[t].rc != ORC_OK) {
            rc = jobs[t].rc;
        }
    }
    free(th);
    free(jobs);
    return rc;
}

int orc_reduce_scatter_mesh_mt(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                               int op, int accMode, uint32_t nThreads)
{
    return run_mt(1, n, in, out, recvCount, dtype, op, accMode, nThreads);
}

int orc_all_reduce_mesh_mt(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                           int accMode, uint32_t nThreads)
{
    return run_mt(0, n, in, out, count, dtype, op, accMode, nThreads);
}

/* ---------------------------------------------------------------------------------------------
 * Point to point: BatchSendRecv (batch_send_recv_executor.cc:96-200, 202-275)
 * ------------------------------------------------------------------------------------------- */
typedef struct {
    const orc_send_recv_item_t* item;
    uint32_t flag;     /* peer order of the pair-wise schedule */
    uint32_t index;    /* position in the caller's array: keeps the sort stable */
} bsr_entry_t;

static int bsr_cmp_send(const void* pa, const void* pb)
{
    const bsr_entry_t* a = (const bsr_entry_t*)pa;
    const bsr_entry_t* b = (const bsr_entry_t*)pb;
    if (a->flag != b->flag) return a->flag > b->flag ? -1 : 1;                        /* :109-110 descending */
    if (a->item->count != b->item->count) return a->item->count > b->item->count ? -1 : 1;
    if (a->item->dataType != b->item->dataType) return a->item->dataType > b->item->dataType ? -1 : 1;
    return a->index < b->index ? -1 : 1;
}

static int bsr_cmp_recv(const void* pa, const void* pb)
{
    const bsr_entry_t* a = (const bsr_entry_t*)pa;
    const bsr_entry_t* b = (const bsr_entry_t*)pb;
    if (a->flag != b->flag) return a->flag < b->flag ? -1 : 1;                        /* :121-122 ascending */
    if (a->item->count != b->item->count) return a->item->count > b->item->count ? -1 : 1;
    if (a->item->dataType != b->item->dataType) return a->item->dataType > b->item->dataType ? -1 : 1;
    return a->index < b->index ? -1 : 1;
}

/* Sorted send (isSend) or receive list of one rank; items without elements are dropped (:150). */
static uint32_t bsr_sorted(uint32_t n, uint32_t me, const orc_send_recv_item_t* items, uint32_t itemNum, int isSend,
                           bsr_entry_t* out)
{
    uint32_t k = 0;
    for (uint32_t i = 0; i < itemNum; ++i) {
        if (items[i].count == 0 || (items[i].sendRecvType == 0) != (isSend != 0)) {
            continue;
        }
        uint32_t peer = items[i].remoteRank;
        out[k].item = &items[i];
        out[k].index = i;
        out[k].flag = isSend ? (peer <= me ? peer + n : peer) : (peer < me ? peer + n : peer);   /* :107-108, :119-120 */
        ++k;
    }
    qsort(out, k, sizeof(bsr_entry_t), isSend ? bsr_cmp_send : bsr_cmp_recv);
    return k;
}

int orc_batch_send_recv(uint32_t n, const orc_send_recv_item_t* const* items, const uint32_t* itemNum)
{
    uint32_t most = 0;
    for (uint32_t r = 0; r < n; ++r) {
        most = itemNum[r] > most ? itemNum[r] : most;
        for (uint32_t i = 0; i < itemNum[r]; ++i) {
            const orc_send_recv_item_t* it = &items[r][i];
            if (!copy_dtype_ok(it->dataType)) return ORC_E_NOT_SUPPORT;
            if (it->remoteRank >= n) return ORC_E_PARA;
            if (it->count != 0 && it->buf == NULL) return ORC_E_PTR;
            if (it->count != 0 && it->sendRecvType != 0 && it->sendRecvType != 1) return ORC_E_PARA;
        }
    }
    bsr_entry_t* tx = (bsr_entry_t*)malloc(sizeof(bsr_entry_t) * (most ? most : 1));
    bsr_entry_t* rx = (bsr_entry_t*)malloc(sizeof(bsr_entry_t) * (most ? most : 1));
    if (!tx || !rx) {
        free(tx);
        free(rx);
        return ORC_E_INTERNAL;
    }
    int rc = ORC_OK;
    /* The k-th send of a to b in a's sorted list meets the k-th receive from a in b's sorted list. */
    for (uint32_t a = 0; a < n && rc == ORC_OK; ++a) {
        uint32_t nTx = bsr_sorted(n, a, items[a], itemNum[a], 1, tx);
        for (uint32_t b = 0; b < n && rc == ORC_OK; ++b) {
            uint32_t nRx = bsr_sorted(n, b, items[b], itemNum[b], 0, rx);
            uint32_t i = 0, j = 0;
            for (;;) {
                while (i < nTx && tx[i].item->remoteRank != b) ++i;
                while (j < nRx && rx[j].item->remoteRank != a) ++j;
                if (i >= nTx || j >= nRx) {
                    if (i < nTx || j < nRx) rc = ORC_E_PARA;           /* a transfer without its counterpart */
                    break;
                }
                const orc_send_recv_item_t* s = tx[i].item;
                const orc_send_recv_item_t* d = rx[j].item;
                if (s->count != d->count || s->dataType != d->dataType) {
                    rc = ORC_E_PARA;                                    /* :88-101 for the own rank */
                    break;
                }
                memmove(d->buf, s->buf, s->count * orc_dtype_size(s->dataType));
                ++i;
                ++j;
            }
        }
    }
    free(tx);
    free(rx);
    return rc;
}

/* ---------------------------------------------------------------------------------------------
 * a16: the variable-length argument area of AlltoAllV (all_to_all_v.cc:600-643, template_utils.h:110-159)
 * ------------------------------------------------------------------------------------------- */
/* ConstructVarData: [sendCounts | recvCounts | sdispls | rdispls], n values each. */
void orc_a2a_construct_var_data(uint32_t n, const uint64_t* sendCounts, const uint64_t* recvCounts,
                                const uint64_t* sdispls, const uint64_t* rdispls, uint64_t* varData)
{
    for (uint64_t i = 0; i < 4ull * n; ++i) {
        const uint64_t* from = i / n == 0 ? sendCounts : i / n == 1 ? recvCounts : i / n == 2 ? sdispls : rdispls;
        varData[i] = from[i % n];
    }
}

/* ParseAlltoAllVarData: element counts / displacements and their byte lengths / offsets; the area must hold
 * exactly four vectors (up to five for AlltoAllVC) of n values.  out = 8 arrays of n values:
 * sendCounts, sendLength, recvCounts, recvLength, sendDispls, sendOffset, recvDispls, recvOffset. */
int orc_a2a_parse_var_data(const uint64_t* varData, uint64_t varBytes, uint64_t n, uint64_t elemSize, int isVC,
                           uint64_t* out)
{
    uint64_t minBytes = 4 * n * sizeof(uint64_t);
    uint64_t maxBytes = isVC ? 5 * n * sizeof(uint64_t) : minBytes;
    if (n == 0 || varData == NULL || varBytes < minBytes || varBytes > maxBytes ||
        varBytes % (n * sizeof(uint64_t)) != 0) {
        return ORC_E_PARA;
    }
    for (uint64_t index = 0; index < 4 * n; ++index) {
        uint64_t vec = index / n, rank = index % n;
        out[(2 * vec) * n + rank] = varData[index];
        out[(2 * vec + 1) * n + rank] = varData[index] * elemSize;
    }
    return ORC_OK;
}

/* CalcInputOutputSize: the furthest byte either buffer is touched at. */
void orc_a2a_io_size(uint32_t n, const uint64_t* sendCounts, const uint64_t* recvCounts, const uint64_t* sdispls,
                     const uint64_t* rdispls, uint64_t elemSize, uint64_t* inputBytes, uint64_t* outputBytes)
{
    *inputBytes = 0;
    *outputBytes = 0;
    for (uint32_t i = 0; i < n; ++i) {
        uint64_t in = (sdispls[i] + sendCounts[i]) * elemSize;
        uint64_t out = (rdispls[i] + recvCounts[i]) * elemSize;
        *inputBytes = in > *inputBytes ? in : *inputBytes;
        *outputBytes = out > *outputBytes ? out : *outputBytes;
    }
}

/* a4: LocalReduce (wrapper.cc:901-928) reduces on the host (AicpuReduce) when the type is 64 bits wide or the
 * operation is PROD, otherwise on the device (HcommLocalReduceOnThread). */
int orc_local_reduce_runs_on_host(int dtype, int op)
{
    return dtype == ORC_INT64 || dtype == ORC_UINT64 || dtype == ORC_FP64 || op == 1 /* PROD */;
}
