/*
 * mme_oracle.c -- CPU restatement of the Gaudi3 MME reference arithmetic (plain C, OpenMP over output rows).
 *
 * TEST INFRASTRUCTURE ONLY: the checker for tests/, the smoke entry and the CPU-baseline leg of the benchmark.
 * The product library never links or calls it.
 *
 * How each function is pinned (none is "parity unpinned"):
 *   orc_fp32_to_fp8 / orc_fp8_to_fp32 / orc_fp32_to_bf16 / orc_fp32_to_fp32 / orc_add_fp32 / orc_lfsr32 / orc_tree9 /
 *   orc_fma_vec_* / orc_batch_gemm / orc_convolution / orc_activation
 *     - bit-for-bit against the reference's own sources compiled into oracle/_ref (tests/test_oracle_vs_ref.py), on
 *       structured sweeps (all 256 codes per format/bias/mode, all 65536 high halves of fp32 crossed with low-half
 *       patterns, ties, denormal and overflow edges, every rounding mode) and on seeded random tensors;
 *     - against the known answers the reference's unit tests hold (tests/golden/kat_vectors.json, taken from
 *       mme/tests/unit_tests/mme_unit_test.cpp:13-29,67-172,394-519);
 *     - against vectors written by the compiled reference and committed under tests/golden/ (so the check also runs
 *       where the reference tree is absent);
 *     - against what the mathematics fixes: decode(encode(x)) identities, monotonicity, sign symmetry, agreement of
 *       fp8_152/bias 15 and bf16 RNE with torch's IEEE conversions, exact fp64 dot products bounding the tree,
 *       a direct 7-loop fp64 convolution, and the adjoint identities of dedx / dedw.
 */
#include "mme_oracle.h"

#include <fenv.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum
{
    RM_NE = 0,
    RM_RZ = 1,
    RM_PINF = 2,
    RM_NINF = 3,
    RM_SR = 4,
    RM_HALF_AZ = 6,
    RM_SR_RNE_DNORM = 7
};

static __thread char g_err[512];
static int           g_threads = 0;

const char* orc_last_error(void) { return g_err; }

static int fail(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return -1;
}

void orc_set_num_threads(int n) { g_threads = n; }
int  orc_get_num_threads(void)
{
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}

static inline uint32_t f2u(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float u2f(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline int is_nan32(uint32_t x) { return ((x >> 23) & 0xFF) == 0xFF && (x & 0x7FFFFF) != 0; }
static inline int is_inf32(uint32_t x) { return ((x >> 23) & 0xFF) == 0xFF && (x & 0x7FFFFF) == 0; }
static inline int is_den32(uint32_t x) { return ((x >> 23) & 0xFF) == 0 && (x & 0x7FFFFF) != 0; }
static inline int is_zero32(uint32_t x) { return (x & 0x7FFFFFFF) == 0; }

/* ------------------------------------------------------------------------------------------------------------- */
/* fp8 -> fp32   (fs_fma.cpp:6066-6139)                                                                            */
/* ------------------------------------------------------------------------------------------------------------- */
uint32_t orc_fp8_to_fp32(uint8_t code, int E, int M, int bias, int mode)
{
    (void) E;
    const uint32_t man_all = (1u << M) - 1u;
    const uint32_t exp_all = (0x7Fu >> M);
    uint32_t       man = code & man_all;
    uint32_t       ex = (code & 0x7Fu) >> M;
    uint32_t       sign = code >> 7;

    if ((code & 0x7F) == 0) return sign << 31;
    /* mode 0: exponent all ones is inf (man 0) or NaN; mode 2: only the top code is NaN; mode 1: all finite */
    if ((mode == 0 && ex == exp_all && man != 0) || (mode == 2 && (code & 0x7F) == 0x7F)) return 0x7FFFFFFFu;
    if (mode == 0 && ex == exp_all && man == 0) return (sign << 31) | 0x7F800000u;

    int32_t out_exp = (int32_t) ex - bias + 127;
    if (ex == 0)
    {
        /* denormal: shift the leading one out (lzcnt over M bits, fs_fma.cpp:1393-1404) */
        int lead = M - 1;
        while (!(man & (1u << lead))) lead--;
        int shift = M - 1 - lead;
        man = (man << (shift + 1)) & man_all;
        out_exp -= shift;
    }
    return (sign << 31) | ((uint32_t) out_exp << 23) | (man << (23 - M));
}

/* ------------------------------------------------------------------------------------------------------------- */
/* rounding increment  (fp_accommodate_rounding, fs_fma.cpp:1503-1545)                                             */
/* ------------------------------------------------------------------------------------------------------------- */
static uint32_t round_inc(uint32_t v, int msb, int lsbs, uint32_t sign, int rm, uint32_t lfsr, uint32_t discarded)
{
    switch (rm)
    {
        case RM_RZ: return v;
        case RM_PINF: return v + ((sign == 0) && (msb || lsbs));
        case RM_NINF: return v + ((sign == 1) && (msb || lsbs));
        case RM_HALF_AZ: return v + (msb != 0);
        case RM_SR: return v + (discarded >= lfsr);
        default: /* nearest even, also for unknown values */
            return v + (((v & 1) && msb) || (!(v & 1) && msb && lsbs));
    }
}

/* ------------------------------------------------------------------------------------------------------------- */
/* fp32 -> fp8   (fs_fma.cpp:6731-7027)                                                                            */
/* ------------------------------------------------------------------------------------------------------------- */
uint8_t orc_fp32_to_fp8(uint32_t u, int E, int M, int bias, int rm, uint32_t lfsr, int ftz, int clip, int clip_inf_in,
                        int sftz, int mode)
{
    const int      min_norm = 1 - bias;
    const int      max_exp = ((1 << E) - 1) - bias - 1 + (mode != 0);
    const int      min_exp = min_norm - M - 1;
    const uint32_t exp_all = (1u << E) - 1u;
    const uint32_t man_all = (1u << M) - 1u;
    const int      rm_dn = (rm == RM_SR_RNE_DNORM) ? RM_NE : rm;
    const int      rm_n = (rm == RM_SR_RNE_DNORM) ? RM_SR : rm;
    const uint32_t in_sign = u >> 31;
    const int      toward_zero = (rm == RM_RZ) || (in_sign && rm == RM_PINF) || (!in_sign && rm == RM_NINF);

    uint32_t o_sign = in_sign, o_exp = 0, o_man = 0;
    int      sftz_decision = 0;

    if (is_nan32(u))
    {
        if (mode != 2) o_sign = 0;
        o_exp = exp_all;
        o_man = man_all;
    }
    else if (is_zero32(u))
    {
        o_exp = 0;
        o_man = 0;
    }
    else if (is_inf32(u))
    {
        o_exp = exp_all;
        o_man = (mode == 0) ? 0 : man_all;
    }
    else
    {
        /* a subnormal fp32 input is treated as exponent -127 with the hidden bit set, like the reference (:6830-6831);
         * it is far below every fp8 range so only the directed modes can see the difference */
        const int      e = (int) ((u >> 23) & 0xFF) - 127;
        const uint32_t m = (u & 0x7FFFFF) | (1u << 23);

        if (e > max_exp)
        {
            if (mode == 0)
            {
                if (toward_zero)
                {
                    o_man = man_all;
                    o_exp = (uint32_t) (max_exp + bias);
                }
                else
                {
                    o_exp = exp_all;
                    o_man = 0;
                }
            }
            else if (mode == 1)
            {
                o_exp = exp_all;
                o_man = man_all;
            }
            else
            {
                o_exp = exp_all;
                o_man = toward_zero ? (man_all & ~1u) : man_all;
            }
        }
        else if (e < min_exp)
        {
            uint32_t discarded = 0;
            if (sftz)
            {
                int rc = (23 - M - 1) + (min_norm - e);
                if (ftz) rc += M;
                int sh = 31 - rc;
                if (sh >= 0) discarded = m << sh;
                else if (sh >= -24)
                    discarded = m >> (-sh);
                else
                    discarded = 0;
                if (ftz) sftz_decision = (discarded >= lfsr) && (rm == RM_NE || rm == RM_SR);
            }
            o_man = round_inc(0, 0, 1, in_sign, (sftz && (rm == RM_NE || rm == RM_SR)) ? RM_SR : rm_dn, lfsr, discarded);
            o_exp = 0;
        }
        else
        {
            int out_e = e;
            int rc = (e < min_norm) ? ((23 - M - 1) + (min_norm - e)) : (23 - M - 1);
            if (e < min_norm && ftz && sftz) rc += M;
            const int      sh = 31 - rc;
            const int      msb = (m >> rc) & 1;
            const int      lsbs = (m & ((1u << rc) - 1u)) != 0;
            const uint32_t discarded = m << sh;
            uint32_t       q = m >> (rc + 1);
            if (e < min_norm && ftz && sftz) sftz_decision = (discarded >= lfsr) && (rm == RM_NE || rm == RM_SR);
            q = round_inc(q, msb, lsbs, in_sign, (e < min_norm) ? rm_dn : rm_n, lfsr, discarded);
            if ((e < min_norm && (q & (1u << M))) || (q & (1u << (M + 1)))) out_e++;
            if (out_e > max_exp)
            {
                o_exp = exp_all;
                o_man = (mode == 0) ? 0 : man_all;
            }
            else
            {
                o_exp = (out_e < min_norm) ? 0 : (uint32_t) (out_e + bias);
                o_man = q & man_all;
            }
            if (mode == 2 && toward_zero)
            {
                uint32_t tmp = (o_man | (o_exp << M) | (o_sign << 7)) & 0xFF;
                if (tmp == 0x7F || tmp == 0xFF) o_man -= 1;
            }
        }
    }

    uint8_t out = (uint8_t) (o_man | (o_exp << M) | (o_sign << 7));

    const int out_is_inf = ((uint32_t) (out & 0x7F) >> M) == (0x7Fu >> M) && (out & man_all) == 0;
    if (clip && mode == 0 && out_is_inf && (clip_inf_in || !is_inf32(u))) out = (uint8_t) (out - 1);
    if (clip && mode == 2 && (out == 0x7F || out == 0xFF) && (clip_inf_in || !is_inf32(u)) && !is_nan32(u))
        out = (uint8_t) (out - 1);

    const int out_is_den = (((out & 0x7F) >> M) == 0) && ((out & man_all) != 0);
    if (ftz && (out_is_den || (sftz && sftz_decision)))
    {
        if (rm == RM_PINF && !(out >> 7)) out = (uint8_t) (1u << M);
        else if (rm == RM_NINF && (out >> 7))
            out = (uint8_t) (0x80u | (1u << M));
        else
            out = (uint8_t) ((((sftz && sftz_decision) ? 1u : 0u) << M) | (o_sign << 7));
    }
    return out;
}

/* ------------------------------------------------------------------------------------------------------------- */
/* fp16 / unsigned fp16  <->  fp32   (cfp16_to_fp32 fs_fma.cpp:7239-7310, fp32_to_cfp16 :7033-7237;                */
/* E = 5 with a sign bit, or E = 6 without one; M = 10; no_inf_nan = InfNanMode != 0, fp16.h:94-103)               */
/* ------------------------------------------------------------------------------------------------------------- */
uint32_t orc_cfp16_to_fp32(uint16_t code, int E, int bias, int no_inf_nan)
{
    const int      M = 10;
    const int      uns = (E + M == 16);
    const uint32_t man = code & 0x3FFu;
    const uint32_t ex = ((uint32_t) code >> M) & ((1u << E) - 1u);
    const uint32_t sign = uns ? 0u : ((uint32_t) code >> 15);
    const uint32_t exp_all = (1u << E) - 1u;

    if (ex == 0 && man == 0) return sign << 31;
    if (!no_inf_nan && ex == exp_all) return man ? 0x7FFFFFFFu : ((sign << 31) | 0x7F800000u);

    int32_t  out_exp = (int32_t) ex - bias + 127;
    uint32_t m = man;
    if (ex == 0)
    {
        int lead = M - 1;
        while (!(m & (1u << lead))) lead--;
        const int shift = M - 1 - lead;
        m = (m << (shift + 1)) & 0x3FFu;
        out_exp -= shift;
    }
    return (sign << 31) | ((uint32_t) out_exp << 23) | (m << (23 - M));
}

uint16_t orc_fp32_to_cfp16(uint32_t u, int E, int bias, int rm, uint32_t lfsr, int ftz, int clip, int clip_inf_in,
                           int no_inf_nan)
{
    const int      M = 10;
    const int      uns = (E + M == 16);
    const int      min_norm = 1 - bias;
    const int      max_exp = ((1 << E) - 1) - bias - 1 + (no_inf_nan != 0);
    const int      min_exp = min_norm - M - 1;
    const uint32_t exp_all = (1u << E) - 1u;
    const uint32_t man_all = (1u << M) - 1u;
    const int      rm_dn = (rm == RM_SR_RNE_DNORM) ? RM_NE : rm;
    const int      rm_n = (rm == RM_SR_RNE_DNORM) ? RM_SR : rm;
    const uint32_t in_sign = u >> 31;

    uint32_t o_sign = in_sign, o_exp = 0, o_man = 0;
    if (is_nan32(u))
    {
        o_sign = 0;
        o_exp = exp_all;
        o_man = man_all;
    }
    else if (is_zero32(u) || (uns && in_sign))
    {
        /* the unsigned format has no negative numbers: every negative input, -inf included, gives zero (:7090-7099) */
    }
    else if (is_inf32(u))
    {
        o_exp = exp_all;
        o_man = no_inf_nan ? man_all : 0;
    }
    else
    {
        const int      e = (int) ((u >> 23) & 0xFF) - 127;
        const uint32_t m = (u & 0x7FFFFF) | (1u << 23);
        if (e > max_exp)
        {
            const int toward_zero = (rm == RM_RZ) || (in_sign && rm == RM_PINF) || (!in_sign && rm == RM_NINF);
            if (!no_inf_nan && toward_zero)
            {
                o_man = man_all;
                o_exp = (uint32_t) (max_exp + bias);
            }
            else
            {
                o_exp = exp_all;
                o_man = no_inf_nan ? man_all : 0;
            }
        }
        else if (e < min_exp)
            o_man = round_inc(0, 0, 1, in_sign, rm_dn, lfsr, 0);
        else
        {
            int            out_e = e;
            const int      rc = (e < min_norm) ? ((23 - M - 1) + (min_norm - e)) : (23 - M - 1);
            const int      msb = (m >> rc) & 1;
            const int      lsbs = (m & ((1u << rc) - 1u)) != 0;
            const uint32_t discarded = m << (31 - rc);
            uint32_t       q = m >> (rc + 1);
            q = round_inc(q, msb, lsbs, in_sign, (e < min_norm) ? rm_dn : rm_n, lfsr, discarded);
            if ((e < min_norm && (q & (1u << M))) || (q & (1u << (M + 1)))) out_e++;
            if (out_e > max_exp)
            {
                o_exp = exp_all;
                o_man = no_inf_nan ? man_all : 0;
            }
            else
            {
                o_exp = (out_e < min_norm) ? 0 : (uint32_t) (out_e + bias);
                o_man = q & man_all;
            }
        }
    }
    /* the sign lands on bit E + M, which an unsigned code does not have */
    uint16_t out = (uint16_t) (o_man | (o_exp << M) | (uns ? 0u : (o_sign << 15)));

    const uint32_t out_exp_bits = ((uint32_t) out >> M) & exp_all;
    if (clip && !no_inf_nan && out_exp_bits == exp_all && (out & man_all) == 0 && (clip_inf_in || !is_inf32(u)))
        out = (uint16_t) (out - 1);
    if (ftz && (((uint32_t) out >> M) & exp_all) == 0 && (out & man_all) != 0)
    {
        const uint32_t s = uns ? 0u : ((uint32_t) out >> 15);
        if (rm == RM_PINF && !s) out = (uint16_t) (1u << M);
        else if (rm == RM_NINF && s)
            out = (uint16_t) (0x8000u | (1u << M));
        else
            out = (uint16_t) (s << 15);
    }
    return out;
}

/* ------------------------------------------------------------------------------------------------------------- */
/* fp32 -> tf32   (fp32_to_tf32 = fp32_to_fp19 << 13, fs_fma.cpp:926-987, 1057-1062), nearest-even as the tree     */
/* calls it (rounding mode 0, no LFSR)                                                                             */
/* ------------------------------------------------------------------------------------------------------------- */
uint32_t orc_fp32_to_tf32(uint32_t u, int clip, int clip_inf_in)
{
    uint32_t res; /* the 19-bit code */
    if (is_nan32(u)) res = 0x3FFFFu;
    else if (is_zero32(u) || is_inf32(u))
        res = u >> 13;
    else
    {
        uint32_t  ex = (u >> 23) & 0xFF;
        uint32_t  man = (u >> 13) & 0x3FF;
        const int g = (u >> 12) & 1, rs = (u & 0xFFF) != 0;
        if (ex) man |= 1u << 10;
        if ((g && rs) || (g && !rs && (man & 1)))
        {
            man++;
            if (ex == 0) ex += (man >> 10) & 1;
            else
                ex += (man >> 11) & 1;
        }
        res = ((u >> 31) << 18) | (ex << 10) | (man & 0x3FF);
    }
    if (clip && is_inf32(res << 13) && (clip_inf_in || !is_inf32(u))) res -= 1;
    return res << 13;
}

/* ------------------------------------------------------------------------------------------------------------- */
/* fp32 -> bf16   (fs_fma.cpp:851-924)                                                                             */
/* ------------------------------------------------------------------------------------------------------------- */
uint16_t orc_fp32_to_bf16(uint32_t u, int rm, uint32_t sr, int clip, int ftz_out, int clip_inf_in)
{
    uint16_t res;
    if (is_nan32(u)) res = 0x7FFF;
    else if (is_zero32(u) || is_inf32(u))
        res = (uint16_t) (u >> 16);
    else
    {
        const uint32_t sign = u >> 31;
        const int      g = (u >> 15) & 1;
        const int      rs = (u & 0x7FFF) != 0;
        const uint32_t grs = (u & 0xFFFF) << 16;
        const uint32_t lsb = (u >> 16) & 1;
        int            up;
        switch (rm)
        {
            case RM_PINF: up = (rs || g) && sign == 0; break;
            case RM_NINF: up = (rs || g) && sign == 1; break;
            case RM_NE: up = (g && rs) || (g && !rs && lsb); break;
            case RM_HALF_AZ: up = g; break;
            case RM_SR: up = grs >= sr; break;
            default: up = 0; break; /* RZ, and mode 7 which this converter does not know (:875-879) */
        }
        /* mantissa carry into the exponent is a plain integer carry on the top 16 bits (:880-892) */
        res = (uint16_t) ((u >> 16) + (uint32_t) up);
    }
    const int res_inf = ((res >> 7) & 0xFF) == 0xFF && (res & 0x7F) == 0;
    if (clip && res_inf && (clip_inf_in || !is_inf32(u))) res = (uint16_t) (res - 1);
    const int res_den = ((res >> 7) & 0xFF) == 0 && (res & 0x7F) != 0;
    if (ftz_out && res_den)
    {
        if (rm == RM_PINF && !(res >> 15)) res = 0x0080;
        else if (rm == RM_NINF && (res >> 15))
            res = 0x8080;
        else
            res &= 0x8000;
    }
    return res;
}

/* fp32 -> fp32   (fs_fma.cpp:1064-1088) */
uint32_t orc_fp32_to_fp32(uint32_t u, int rm, int clip, int ftz_out, int clip_inf_in)
{
    (void) clip_inf_in; /* the reference ignores it here */
    uint32_t res = u;
    if (clip && is_inf32(res)) res -= 1;
    if (ftz_out && is_den32(res))
    {
        if (rm == RM_PINF && !(res >> 31)) res = 0x00800000u;
        else if (rm == RM_NINF && (res >> 31))
            res = 0x80800000u;
        else
            res &= 0x80000000u;
    }
    return res;
}

/* add_fp32   (fs_fma.cpp:1271-1321, set_rounding_mode :1097-1116) */
uint32_t orc_add_fp32(uint32_t a, uint32_t b, int rm)
{
    int want;
    switch (rm)
    {
        case RM_RZ: want = FE_TOWARDZERO; break;
        case RM_PINF: want = FE_UPWARD; break;
        case RM_NINF: want = FE_DOWNWARD; break;
        default: want = FE_TONEAREST; break;
    }
    const int   saved = fegetround();
    if (saved != want) fesetround(want);
    volatile float fa = u2f(a), fb = u2f(b);
    volatile float fr = fa + fb;
    if (saved != want) fesetround(saved);
    uint32_t r = f2u(fr);
    if (is_nan32(r)) r = 0x7FFFFFFFu;
    return r;
}

/* ------------------------------------------------------------------------------------------------------------- */
/* memory-write reductions   (doMemoryWrite mme_reference_impl.cpp:718-768 -> executeOp -> ST_TNSR_RMW,             */
/* fs_fma.cpp:2288-2955; fma_bfp16 :27-413 and fma_fp32 :1182-1258 with b = 1, dnorm_ftz = 1)                        */
/* ------------------------------------------------------------------------------------------------------------- */

/* a + c for operands in fp32 format, correctly rounded (rm: 0 nearest even, 1 toward zero, 2 up, 3 down) to a format with
 * man mantissa bits (7: bf16, whose operands arrive widened; 23: fp32) and the fp32 exponent range.  Denormal operands
 * count as zero; a denormal result is flushed: to the smallest normal when the rounding mode points away from zero for
 * its sign, to zero otherwise.  NaN in or inf - inf gives the default NaN (all ones below the sign). */
static uint32_t rmw_add_range(uint32_t a, uint32_t c, int rm, int man, int emin, int emax);
static uint32_t rmw_add(uint32_t a, uint32_t c, int rm, int man) { return rmw_add_range(a, c, rm, man, 1, 254); }

/* the same for a format whose normal numbers have (fp32-biased) exponents emin .. emax: fp16 is man 10, emin 113,
 * emax 142 (fma_fp16_fp16, fs_fma.cpp:1656-2060).  Operands below the smallest normal must arrive as zeros. */
static uint32_t rmw_add_range(uint32_t a, uint32_t c, int rm, int man, int emin, int emax)
{
    const int      drop = 23 - man; /* low bits of the fp32 pattern that the format does not have */
    const uint32_t nan = 0x7FFFFFFFu & ~((1u << drop) - 1u), inf = 0x7F800000u;
    if (((a >> 23) & 0xFF) == 0) a &= 0x80000000u;
    if (((c >> 23) & 0xFF) == 0) c &= 0x80000000u;
    const uint32_t sa = a >> 31, sc = c >> 31;
    if (is_nan32(a) || is_nan32(c)) return nan;
    if (is_inf32(a) || is_inf32(c))
    {
        if (is_inf32(a) && is_inf32(c) && sa != sc) return nan;
        return is_inf32(a) ? a : c;
    }
    if (is_zero32(a) && is_zero32(c)) return ((sa & sc) | ((sa ^ sc) & (uint32_t) (rm == RM_NINF))) << 31;
    if (is_zero32(a)) return c;
    if (is_zero32(c)) return a;
    /* both normal: b = the operand of larger magnitude */
    uint32_t b = a, s = c;
    if ((c & 0x7FFFFFFFu) > (a & 0x7FFFFFFFu))
    {
        b = c;
        s = a;
    }
    const int      eb = (int) ((b >> 23) & 0xFF), es = (int) ((s >> 23) & 0xFF), d = eb - es;
    const uint64_t mb = (uint64_t) ((b & 0x7FFFFFu) | 0x800000u) << 38; /* leading one at bit 61 */
    const uint64_t ms = d <= 38 ? ((uint64_t) ((s & 0x7FFFFFu) | 0x800000u) << 38) >> d : 0;
    int            sticky = d > 38;
    const uint32_t sign = b >> 31;
    uint64_t       r;
    if ((b ^ s) >> 31)
    {
        r = mb - ms - (uint64_t) sticky; /* the true value lies just above r when sticky is set */
        if (r == 0) return (uint32_t) (rm == RM_NINF) << 31;
    }
    else
        r = mb + ms;
    int p = 63;
    while (!((r >> p) & 1)) p--;
    /* bit position of the result's last mantissa bit: normal, or pinned at the denormal quantum 2^(emin - man) */
    int lsb = p - man;
    const int lsb_den = 61 + emin - man - eb;
    const int den = lsb_den > lsb;
    if (den) lsb = lsb_den;
    uint64_t q;
    int      g = 0;
    if (lsb <= 0) q = r << (-lsb);
    else
    {
        q = r >> lsb;
        g = (int) ((r >> (lsb - 1)) & 1);
        sticky |= (r & ((1ull << (lsb - 1)) - 1)) != 0;
    }
    int up;
    switch (rm)
    {
        case RM_RZ: up = 0; break;
        case RM_PINF: up = !sign && (g || sticky); break;
        case RM_NINF: up = sign && (g || sticky); break;
        default: up = g && (sticky || (q & 1)); break;
    }
    q += (uint64_t) up;
    uint32_t res;
    if (den)
    {
        /* q <= 2^man: reaching 2^man is the smallest normal; anything else non-zero is a denormal result, flushed */
        const uint32_t min_normal = (uint32_t) emin << 23;
        if (q >> man) res = min_normal;
        else if (q == 0)
            res = 0;
        else if ((rm == RM_PINF && !sign) || (rm == RM_NINF && sign))
            res = min_normal;
        else
            res = 0;
        return res | (sign << 31);
    }
    else
    {
        int e = eb + (p - 61);
        if (q >> (man + 1))
        {
            q >>= 1;
            e++;
        }
        if (e > emax)
        {
            const int toward_zero = rm == RM_RZ || (rm == RM_PINF && sign) || (rm == RM_NINF && !sign);
            res = toward_zero ? ((((uint32_t) emax + 1) << 23) - (1u << drop)) : inf;
        }
        else
            res = ((uint32_t) e << 23) | (((uint32_t) q & ((1u << man) - 1u)) << drop);
    }
    return res | (sign << 31);
}

/* fp16 (bias 15, full inf/NaN) element of ST_TNSR_RMW: operands widened to fp32 format, the sum rounded to 10 mantissa
 * bits within fp16's exponent range, the result narrowed again */
static uint32_t fp16_widen(uint16_t h, int flush_denormal)
{
    if (flush_denormal && (h & 0x7C00u) == 0) return (uint32_t) (h >> 15) << 31;
    return orc_cfp16_to_fp32(h, 5, 15, 0);
}
static uint16_t fp16_narrow(uint32_t w)
{
    const uint16_t sign = (uint16_t) ((w >> 31) << 15);
    if (is_nan32(w)) return 0x7FFFu;
    if (is_inf32(w)) return (uint16_t) (sign | 0x7C00u);
    if (is_zero32(w)) return sign;
    return (uint16_t) (sign | ((((w >> 23) & 0xFF) - 112u) << 10) | ((w >> 13) & 0x3FFu));
}
/* mem + in, mem - in or max(mem + in, 0) in fp16, before clipping */
static uint16_t rmw_sum_fp16(uint16_t mem, uint16_t in, int op, int rm)
{
    uint16_t r = fp16_narrow(rmw_add_range(fp16_widen(mem, 1), fp16_widen((uint16_t) (op == MME_HIP_REDUCTION_SUB ? in ^ 0x8000u : in), 1), rm, 10,
                                           113, 142));
    if (op == MME_HIP_REDUCTION_MAX_0)
    {
        if (!(u2f(fp16_widen(r, 0)) >= 0.0f)) r = 0; /* MaxFp16(res, 0): NaN fails the comparison (:2186-2207, 2879-2881) */
        if (r == 0x8000u) r = 0;
    }
    return r;
}

/* fp8_152 (bias 15, full inf/NaN) element: the codes are the top bytes of fp16 numbers; sums are formed in fp16 and
 * converted to fp8 with the reduction's rounding mode and denormal results flushed (a second rounding), min / max pick a
 * code (fs_fma.cpp:2410-2436, 2544-2570, 2666-2676, 2772-2782, 2906-2933) */
static uint8_t rmw_elem_fp8_152(uint8_t mem, uint8_t in, int op, int rm, int clip)
{
    const uint16_t m16 = (uint16_t) (mem << 8), i16 = (uint16_t) (in << 8);
    switch (op)
    {
        case MME_HIP_REDUCTION_ADD:
        case MME_HIP_REDUCTION_SUB:
        case MME_HIP_REDUCTION_MAX_0:
        {
            const uint16_t r16 = rmw_sum_fp16(m16, i16, op, rm);
            uint8_t        r = orc_fp32_to_fp8(fp16_widen(r16, 0), 5, 2, 15, rm, 0, 1, 0, 0, 0, 0);
            const int      inf_in = ((mem & 0x7Fu) == 0x7Cu) || ((in & 0x7Fu) == 0x7Cu);
            if (clip && (r & 0x7Fu) == 0x7Cu && !inf_in) r = (uint8_t) (r - 1);
            return r;
        }
        case MME_HIP_REDUCTION_MIN: return (u2f(fp16_widen(m16, 0)) <= u2f(fp16_widen(i16, 0))) ? mem : in;
        case MME_HIP_REDUCTION_MAX: return (u2f(fp16_widen(m16, 0)) >= u2f(fp16_widen(i16, 0))) ? mem : in;
        default: return in;
    }
}

static uint16_t rmw_elem_fp16(uint16_t mem, uint16_t in, int op, int rm, int clip)
{
    const int inf_in = ((mem & 0x7FFFu) == 0x7C00u) || ((in & 0x7FFFu) == 0x7C00u);
    uint16_t  r;
    switch (op)
    {
        case MME_HIP_REDUCTION_ADD:
        case MME_HIP_REDUCTION_SUB:
        case MME_HIP_REDUCTION_MAX_0:
            r = rmw_sum_fp16(mem, in, op, rm);
            if (clip && (r & 0x7FFFu) == 0x7C00u && !inf_in) r = (uint16_t) (r - 1);
            return r;
        case MME_HIP_REDUCTION_MIN: return (u2f(fp16_widen(mem, 0)) <= u2f(fp16_widen(in, 0))) ? mem : in; /* (:2263-2284) */
        case MME_HIP_REDUCTION_MAX: return (u2f(fp16_widen(mem, 0)) >= u2f(fp16_widen(in, 0))) ? mem : in;
        default: return in;
    }
}

/* one element of ST_TNSR_RMW: mem (op) in, both in fp32 format (bf16 widened), result in the same format */
static uint32_t rmw_elem(uint32_t mem, uint32_t in, int op, int rm, int clip, int man)
{
    const int drop = 23 - man;
    uint32_t  r;
    switch (op)
    {
        case MME_HIP_REDUCTION_ADD:
        case MME_HIP_REDUCTION_SUB:
        case MME_HIP_REDUCTION_MAX_0:
            r = rmw_add(mem, op == MME_HIP_REDUCTION_SUB ? in ^ 0x80000000u : in, rm, man);
            if (op == MME_HIP_REDUCTION_MAX_0)
            {
                /* MaxFp32(res, 0): res when res >= 0 as floats (NaN fails the comparison), then -0 -> +0 (:2862-2864) */
                if (!(u2f(r) >= 0.0f)) r = 0;
                if (r == 0x80000000u) r = 0;
            }
            /* clip_fp_inf_input is false in doMemoryWrite (:749) */
            if (clip && is_inf32(r) && !is_inf32(mem) && !is_inf32(in)) r -= 1u << drop;
            return r;
        case MME_HIP_REDUCTION_MIN: return (u2f(mem) <= u2f(in)) ? mem : in; /* (:2221-2258; a NaN operand selects in) */
        case MME_HIP_REDUCTION_MAX: return (u2f(mem) >= u2f(in)) ? mem : in;
        default: return in;
    }
}

uint32_t orc_lfsr32(uint32_t prev, uint32_t polynomial)
{
    uint32_t l = prev >> 1;
    if (prev & 1u) l ^= polynomial;
    return l;
}

/* ------------------------------------------------------------------------------------------------------------- */
/* the 9-input multiply-add tree   (fs_fma_gaudi3.h:392-520, 617-758, 760-1166 with N=9 K=4 c_in_tree=1 no ftz)    */
/* ------------------------------------------------------------------------------------------------------------- */
uint32_t orc_tree9(const uint32_t a[9], const uint32_t b[9], int emul_kind)
{
    const int fp32_emul = emul_kind == 1, half_emul = emul_kind == 2;
    enum { N = 9, K = 4 };
    int     az[N], bz[N], ad[N], bd[N];
    int32_t pexp[N];
    int64_t psig[N];
    int     p_inf[N], p_nan[N], p_neg[N];

    for (int i = 0; i < N; i++)
    {
        az[i] = is_zero32(a[i]);
        bz[i] = is_zero32(b[i]);
        ad[i] = is_den32(a[i]);
        bd[i] = is_den32(b[i]);
    }
    if (fp32_emul)
    {
        /* the eight partial products of one fp32 pair share their zero / denormal indications (:868-903) */
        int allza = 1, allzb = 1, anyda = 0, anydb = 0;
        for (int i = 0; i < 8; i++)
        {
            allza &= az[i];
            allzb &= bz[i];
            anyda |= ad[i];
            anydb |= bd[i];
        }
        for (int i = 0; i < 8; i++)
        {
            az[i] = allza;
            bz[i] = allzb;
            ad[i] = anyda;
            bd[i] = anydb;
        }
    }

    if (half_emul)
    {
        /* fp16 / tf32: the four partial products of one pair share their indications (:819-845) */
        for (int q = 0; q < 8; q += 4)
        {
            int allza = 1, allzb = 1, anyda = 0, anydb = 0;
            for (int i = q; i < q + 4; i++)
            {
                allza &= az[i];
                allzb &= bz[i];
                anyda |= ad[i];
                anydb |= bd[i];
            }
            for (int i = q; i < q + 4; i++)
            {
                az[i] = allza;
                bz[i] = allzb;
                ad[i] = anyda;
                bd[i] = anydb;
            }
        }
    }

    int32_t max_exp = INT32_MIN;
    for (int i = 0; i < N; i++)
    {
        const uint32_t x = a[i], y = b[i];
        const int      emul = (fp32_emul || half_emul) && i != N - 1;
        p_nan[i] = p_inf[i] = p_neg[i] = 0;
        if (is_nan32(x) || is_nan32(y) || (is_inf32(x) && bz[i]) || (is_inf32(y) && az[i]))
        {
            p_nan[i] = 1;
            pexp[i] = 0xFF;
            psig[i] = -1;
        }
        else if (is_inf32(x) || is_inf32(y))
        {
            p_inf[i] = 1;
            p_neg[i] = (x >> 31) ^ (y >> 31);
            pexp[i] = 0xFF;
            psig[i] = 0;
        }
        else if (az[i] || bz[i])
        {
            p_neg[i] = (x >> 31) ^ (y >> 31);
            pexp[i] = -127;
            psig[i] = 0;
        }
        else
        {
            p_neg[i] = (x >> 31) ^ (y >> 31);
            uint32_t ea = (x >> 23) & 0xFF, eb = (y >> 23) & 0xFF;
            uint64_t la, lb;
            if (emul)
            {
                /* which byte-slices carry the hidden one (is_gaudi3 && !fp16_emul branch, :462-468) */
                if (half_emul)
                {
                    /* two slices per operand: the high one carries the hidden one (:469-472) */
                    const int part = i % 4;
                    la = (part == 2 || part == 3);
                    lb = (part == 1 || part == 3);
                }
                else
                {
                    const int part = i % 8;
                    la = (part == 5 || part == 6 || part == 7);
                    lb = (part == 1 || part == 4 || part == 7);
                }
                if (ea == 0) la = 0;
                if (eb == 0) lb = 0;
            }
            else
            {
                la = ea != 0;
                lb = eb != 0;
            }
            if (ea == 0 && ad[i]) ea = 1;
            if (eb == 0 && bd[i]) eb = 1;
            pexp[i] = (int32_t) (ea + eb) - 127;
            const int64_t sa = (int64_t) ((x & 0x7FFFFF) | (la << 23));
            const int64_t sb = (int64_t) ((y & 0x7FFFFF) | (lb << 23));
            psig[i] = sa * sb;
        }
        if (pexp[i] > max_exp) max_exp = pexp[i];
    }
    if (max_exp < -5) max_exp = -5;

    int64_t sum = 0;
    int     all_neg = 1, any_inf = 0, any_nan = 0, inf_neg = 0, pinf = 0, ninf = 0;
    for (int i = 0; i < N; i++)
    {
        int d = max_exp - pexp[i];
        if (d > K + 22) d = K + 22;
        int64_t s = (psig[i] >> (26 - K)) >> d; /* truncation toward zero of the magnitude */
        if (p_neg[i]) s = -s;
        all_neg &= p_neg[i];
        sum += s;
        any_inf |= p_inf[i];
        any_nan |= p_nan[i];
        inf_neg = any_nan ? 0 : (p_inf[i] ? p_neg[i] : inf_neg);
        pinf |= p_inf[i] && !p_neg[i];
        ninf |= p_inf[i] && p_neg[i];
    }
    any_nan |= (pinf && ninf);
    any_inf = any_inf && !any_nan;
    const int is_zero = (sum == 0) && !any_inf && !any_nan;
    const int is_neg = (!any_nan && !any_inf) ? ((is_zero && all_neg) || sum < 0) : inf_neg;

    /* fp_convert with RND_TO_0 and sticky 0 */
    uint32_t result;
    uint64_t mag = (uint64_t) (sum < 0 ? -sum : sum);
    if (any_nan) result = 0x7FFFFFFFu;
    else if (any_inf)
        result = is_neg ? 0xFF800000u : 0x7F800000u;
    else if (is_zero || mag == 0)
        result = is_neg ? 0x80000000u : 0;
    else
    {
        const int lead = 63 - __builtin_clzll(mag);
        int32_t   e = max_exp + 1 + (lead - (21 + K));
        uint32_t  man = (lead >= 23) ? (uint32_t) ((mag >> (lead - 23)) & 0xFFFFFF) : (uint32_t) (mag << (23 - lead));
        if (e > 254) result = is_neg ? 0xFF800000u : 0x7F800000u;
        else if (e < 1)
        {
            int sh = 1 - e;
            if (sh > 31) sh = 31;
            man >>= sh;
            result = ((uint32_t) is_neg << 31) | (man & 0x7FFFFF);
        }
        else
            result = ((uint32_t) is_neg << 31) | ((uint32_t) e << 23) | (man & 0x7FFFFF);
    }
    if (result == 0x80000000u) result = 0; /* "+0/-0 logic disabled" when c is in the tree (:996-1000) */
    return result;
}

uint32_t orc_fma_vec_bf16(const uint16_t* a, ptrdiff_t sa, const uint16_t* b, ptrdiff_t sb, size_t cd)
{
    uint32_t c = 0, ta[9], tb[9];
    tb[8] = 0x3F800000u;
    for (size_t k = 0; k < cd; k += 8)
    {
        for (size_t i = 0; i < 8; i++)
        {
            const int in = (k + i) < cd;
            ta[i] = in ? ((uint32_t) a[(ptrdiff_t) (k + i) * sa] << 16) : 0;
            tb[i] = in ? ((uint32_t) b[(ptrdiff_t) (k + i) * sb] << 16) : 0;
        }
        ta[8] = c;
        c = orc_tree9(ta, tb, 0);
    }
    return c;
}

uint32_t orc_fma_vec_fp8(const uint8_t* a, ptrdiff_t sa, const uint32_t lut_a[256], const uint8_t* b, ptrdiff_t sb,
                         const uint32_t lut_b[256], size_t cd)
{
    uint32_t c = 0, ta[9], tb[9];
    tb[8] = 0x3F800000u;
    for (size_t k = 0; k < cd; k += 8)
    {
        for (size_t i = 0; i < 8; i++)
        {
            const int in = (k + i) < cd;
            /* the tail is padded with the code 0, which decodes to +0 for every format (gaudi3_fma.cpp:104-113) */
            ta[i] = lut_a[in ? a[(ptrdiff_t) (k + i) * sa] : 0];
            tb[i] = lut_b[in ? b[(ptrdiff_t) (k + i) * sb] : 0];
        }
        ta[8] = c;
        c = orc_tree9(ta, tb, 0);
    }
    return c;
}

uint32_t orc_fma_vec_fp32(const uint32_t* a, ptrdiff_t sa, const uint32_t* b, ptrdiff_t sb, size_t cd)
{
    /* byte-slice masks of fs_fma_gaudi3.h:1819-1843: sign+exponent kept, one mantissa slice each */
    static const uint32_t MA[8] = {0xff8000ffu, 0xff8000ffu, 0xff80ff00u, 0xff80ff00u,
                                   0xff80ff00u, 0xffff0000u, 0xffff0000u, 0xffff0000u};
    static const uint32_t MB[8] = {0xff80ff00u, 0xffff0000u, 0xff8000ffu, 0xff80ff00u,
                                   0xffff0000u, 0xff8000ffu, 0xff80ff00u, 0xffff0000u};
    uint32_t c = 0, ta[9], tb[9];
    tb[8] = 0x3F800000u;
    for (size_t k = 0; k < cd; k++)
    {
        const uint32_t x = a[(ptrdiff_t) k * sa], y = b[(ptrdiff_t) k * sb];
        for (int i = 0; i < 8; i++)
        {
            ta[i] = x & MA[i];
            tb[i] = y & MB[i];
        }
        ta[8] = c;
        c = orc_tree9(ta, tb, 1);
    }
    return c;
}

/* the 2-wide fp16 / tf32 step: each element is split in a low (mantissa bits 20..13) and a high (bits 22..21) slice,
 * the four cross products of a pair enter the tree (fs_fma.cpp:3546-3581, 4395-4428) */
static uint32_t half_pair_tree(uint32_t a0, uint32_t b0, uint32_t a1, uint32_t b1, uint32_t c)
{
    const uint32_t LO = 0xff9fe000u, HI = 0xffe00000u;
    const uint32_t ta[9] = {a0 & LO, a0 & LO, a0 & HI, a0 & HI, a1 & LO, a1 & LO, a1 & HI, a1 & HI, c};
    const uint32_t tb[9] = {b0 & LO, b0 & HI, b0 & LO, b0 & HI, b1 & LO, b1 & HI, b1 & LO, b1 & HI, 0x3F800000u};
    return orc_tree9(ta, tb, 2);
}

uint32_t orc_fma_vec_fp16(const uint16_t* a, ptrdiff_t sa, int Ea, int bias_a, int nin_a, const uint16_t* b,
                          ptrdiff_t sb, int Eb, int bias_b, int nin_b, size_t cd)
{
    uint32_t c = 0;
    for (size_t k = 0; k < cd; k += 2)
    {
        const int      in1 = (k + 1) < cd; /* an odd tail is padded with the code 0 (gaudi3_fma.cpp:158-171) */
        const uint32_t a0 = orc_cfp16_to_fp32(a[(ptrdiff_t) k * sa], Ea, bias_a, nin_a);
        const uint32_t b0 = orc_cfp16_to_fp32(b[(ptrdiff_t) k * sb], Eb, bias_b, nin_b);
        const uint32_t a1 = orc_cfp16_to_fp32(in1 ? a[(ptrdiff_t) (k + 1) * sa] : 0, Ea, bias_a, nin_a);
        const uint32_t b1 = orc_cfp16_to_fp32(in1 ? b[(ptrdiff_t) (k + 1) * sb] : 0, Eb, bias_b, nin_b);
        c = half_pair_tree(a0, b0, a1, b1, c);
    }
    return c;
}

uint32_t orc_fma_vec_tf32(const uint32_t* a, ptrdiff_t sa, const uint32_t* b, ptrdiff_t sb, size_t cd, int clip,
                          int clip_inf_in)
{
    uint32_t c = 0;
    for (size_t k = 0; k < cd; k += 2)
    {
        const int      in1 = (k + 1) < cd;
        const uint32_t a0 = orc_fp32_to_tf32(a[(ptrdiff_t) k * sa], clip, clip_inf_in);
        const uint32_t b0 = orc_fp32_to_tf32(b[(ptrdiff_t) k * sb], clip, clip_inf_in);
        const uint32_t a1 = orc_fp32_to_tf32(in1 ? a[(ptrdiff_t) (k + 1) * sa] : 0, clip, clip_inf_in);
        const uint32_t b1 = orc_fp32_to_tf32(in1 ? b[(ptrdiff_t) (k + 1) * sb] : 0, clip, clip_inf_in);
        c = half_pair_tree(a0, b0, a1, b1, c);
    }
    return c;
}

/* ------------------------------------------------------------------------------------------------------------- */
/* descriptors                                                                                                     */
/* ------------------------------------------------------------------------------------------------------------- */
static int dtype_size(int dt)
{
    switch (dt)
    {
        case MME_HIP_FP8_143:
        case MME_HIP_FP8_152: return 1;
        case MME_HIP_BF16:
        case MME_HIP_FP16:
        case MME_HIP_UFP16: return 2;
        case MME_HIP_FP32:
        case MME_HIP_FP32_IEEE:
        case MME_HIP_TF32: return 4;
        default: return 0;
    }
}
static int is_fp8(int dt) { return dt == MME_HIP_FP8_143 || dt == MME_HIP_FP8_152; }
static int is_fp16(int dt) { return dt == MME_HIP_FP16 || dt == MME_HIP_UFP16; }

static void fp8_lut(uint32_t lut[256], const mme_hip_tensor* t)
{
    const int E = t->dtype == MME_HIP_FP8_143 ? 4 : 5;
    for (int c = 0; c < 256; c++) lut[c] = orc_fp8_to_fp32((uint8_t) c, E, 7 - E, (int) t->fp_bias, t->inf_nan_mode);
}

/* one dot product A'(i,:) . B'(:,j) through the chip's fma_vec, dispatching on the element type */
typedef struct
{
    int             dtype;
    const uint32_t *lut_a, *lut_b;
    int             Ea, bias_a, nin_a, Eb, bias_b, nin_b; /* fp16 / ufp16 operands */
    int             clip, clip_inf_in;                    /* tf32 operands */
} dot_ctx;

static void dot_ctx_init(dot_ctx* c, const mme_hip_tensor* a, const mme_hip_tensor* b, uint32_t* lut_a, uint32_t* lut_b,
                         int clip, int clip_inf_in)
{
    memset(c, 0, sizeof *c);
    c->dtype = a->dtype;
    c->lut_a = lut_a;
    c->lut_b = lut_b;
    if (is_fp8(a->dtype))
    {
        fp8_lut(lut_a, a);
        fp8_lut(lut_b, b);
    }
    c->Ea = a->dtype == MME_HIP_UFP16 ? 6 : 5;
    c->Eb = b->dtype == MME_HIP_UFP16 ? 6 : 5;
    c->bias_a = (int) a->fp_bias;
    c->bias_b = (int) b->fp_bias;
    c->nin_a = a->inf_nan_mode != 0;
    c->nin_b = b->inf_nan_mode != 0;
    c->clip = clip;
    c->clip_inf_in = clip_inf_in;
}

static inline uint32_t dot(const dot_ctx* c, const char* a, ptrdiff_t sa, const char* b, ptrdiff_t sb, size_t cd)
{
    switch (c->dtype)
    {
        case MME_HIP_BF16: return orc_fma_vec_bf16((const uint16_t*) a, sa, (const uint16_t*) b, sb, cd);
        case MME_HIP_FP32: return orc_fma_vec_fp32((const uint32_t*) a, sa, (const uint32_t*) b, sb, cd);
        case MME_HIP_FP16:
        case MME_HIP_UFP16:
            return orc_fma_vec_fp16((const uint16_t*) a, sa, c->Ea, c->bias_a, c->nin_a, (const uint16_t*) b, sb, c->Eb,
                                    c->bias_b, c->nin_b, cd);
        case MME_HIP_TF32:
            return orc_fma_vec_tf32((const uint32_t*) a, sa, (const uint32_t*) b, sb, cd, c->clip, c->clip_inf_in);
        default: return orc_fma_vec_fp8((const uint8_t*) a, sa, c->lut_a, (const uint8_t*) b, sb, c->lut_b, cd);
    }
}

static int check_types(const mme_hip_tensor* out, const mme_hip_tensor* a, const mme_hip_tensor* b)
{
    /* Gaudi3 function map: {fp32, tf32, bf16, fp16, ufp16, fp8_143, fp8_152} x fp32 out
     * (mme_reference_impl.cpp:188-196, :591); mixed types only among fp8 and among fp16 / ufp16
     * (gaudi3_fma.cpp:62-66) */
    if (out->dtype != MME_HIP_FP32) return fail("type is not registered in function map !");
    if (!(a->dtype == MME_HIP_BF16 || a->dtype == MME_HIP_FP32 || a->dtype == MME_HIP_TF32 || is_fp8(a->dtype) ||
          is_fp16(a->dtype)))
        return fail("type is not registered in function map !");
    if (!(is_fp8(a->dtype) && is_fp8(b->dtype)) && !(is_fp16(a->dtype) && is_fp16(b->dtype)) && a->dtype != b->dtype)
        return fail("Gaudi3 doesnt support mixed input type flavors");
    return 0;
}

static uint64_t n_elements(const mme_hip_tensor* t)
{
    uint64_t n = 1;
    for (int d = 0; d < 5; d++) n *= t->sizes[d];
    return n;
}

/* bytes spanned by a tensor: stride of the last dimension times its size (setStridesAndGetTensorSize) */
static uint64_t span_elements(const mme_hip_tensor* t)
{
    uint64_t m = 0;
    for (int d = 0; d < 5; d++)
    {
        uint64_t e = (uint64_t) t->strides[d] * t->sizes[d];
        if (e > m) m = e;
    }
    return m;
}

/* ------------------------------------------------------------------------------------------------------------- */
/* doBatchGemm   (mme_reference_impl.cpp:445-539)                                                                  */
/* ------------------------------------------------------------------------------------------------------------- */
int orc_batch_gemm(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, int op)
{
    return orc_batch_gemm_clip(out, x, w, op, 0, 0);
}

int orc_batch_gemm_clip(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, int op, int clip,
                        int clip_inf_in)
{
    if (op < MME_HIP_OP_AB || op > MME_HIP_OP_ATBT) return fail("invalid bgemm op %d", op);
    if (check_types(out, x, w)) return -1;
    for (int d = 2; d < 5; d++)
        if (!((x->sizes[d] == out->sizes[d] || x->sizes[d] == 1) && (w->sizes[d] == out->sizes[d] || w->sizes[d] == 1)))
            return fail("batch dims doesnt match !");
    if (n_elements(x) == 0 || n_elements(w) == 0)
    {
        if (n_elements(x) != n_elements(w)) return fail("One of the input tensors is zero-size, while the other is not");
        memset(out->data, 0, span_elements(out) * 4);
        return 0;
    }
    const int ta = (op == MME_HIP_OP_ATB || op == MME_HIP_OP_ATBT);
    const int tb = (op == MME_HIP_OP_ABT || op == MME_HIP_OP_ATBT);
    const size_t M = ta ? x->sizes[0] : x->sizes[1];
    const size_t Kc = ta ? x->sizes[1] : x->sizes[0];
    const size_t Kb = tb ? w->sizes[0] : w->sizes[1];
    const size_t N = tb ? w->sizes[1] : w->sizes[0];
    if (Kc != Kb) return fail("Common dim doesnt match between input A\\B");
    if (out->sizes[0] != N) return fail("output width doesnt match to inputB width");
    if (out->sizes[1] != M) return fail("output height doesnt match to inputA height");

    uint32_t lut_a[256], lut_b[256];
    dot_ctx  ctx;
    dot_ctx_init(&ctx, x, w, lut_a, lut_b, clip, clip_inf_in);
    const int es = dtype_size(x->dtype);
    /* element strides of A'(i,k) and B'(k,j) */
    const ptrdiff_t a_i = ta ? 1 : x->strides[1], a_k = ta ? x->strides[1] : 1;
    const ptrdiff_t b_k = tb ? 1 : w->strides[1], b_j = tb ? w->strides[1] : 1;

    for (uint32_t b2 = 0; b2 < out->sizes[4]; b2++)
        for (uint32_t b1 = 0; b1 < out->sizes[3]; b1++)
            for (uint32_t b0 = 0; b0 < out->sizes[2]; b0++)
            {
                const uint64_t xo = (uint64_t) (x->sizes[4] == 1 ? 0 : b2) * x->strides[4] +
                                    (uint64_t) (x->sizes[3] == 1 ? 0 : b1) * x->strides[3] +
                                    (uint64_t) (x->sizes[2] == 1 ? 0 : b0) * x->strides[2];
                const uint64_t wo = (uint64_t) (w->sizes[4] == 1 ? 0 : b2) * w->strides[4] +
                                    (uint64_t) (w->sizes[3] == 1 ? 0 : b1) * w->strides[3] +
                                    (uint64_t) (w->sizes[2] == 1 ? 0 : b0) * w->strides[2];
                const uint64_t oo = (uint64_t) b2 * out->strides[4] + (uint64_t) b1 * out->strides[3] +
                                    (uint64_t) b0 * out->strides[2];
                const char* A = (const char*) x->data + xo * es;
                const char* B = (const char*) w->data + wo * es;
                uint32_t*   C = (uint32_t*) out->data + oo;
#pragma omp parallel for schedule(static) num_threads(orc_get_num_threads())
                for (size_t i = 0; i < M; i++)
                    for (size_t j = 0; j < N; j++)
                        C[i * out->strides[1] + j] = dot(&ctx, A + (ptrdiff_t) i * a_i * es, a_k, B + (ptrdiff_t) j * b_j * es, b_k, Kc);
            }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------- */
/* convolution   (mme_reference_impl.cpp:598-659, 770-869, 1055-1120; im2col.cpp:55-172)                           */
/* ------------------------------------------------------------------------------------------------------------- */
typedef struct
{
    const mme_hip_conv_params* p;
    uint32_t                   out_shape[5]; /* the tensor whose dims 1..4 enumerate matrix rows */
    uint32_t                   in_shape[5];  /* the tensor addressed through stride/dilation/padding */
    uint32_t                   kS, kR, kQ;
} im2col_geo;

/* position of matrix row `row` under kernel offset `kidx` in the addressed tensor; returns 0 when it falls into the
 * padding (getCurrentKernelPosition / getCurrentTensorPosition, im2col.cpp:134-172) */
static int im2col_pos(const im2col_geo* g, uint64_t row, uint32_t kidx, int32_t pos[5])
{
    int32_t kc[4];
    kc[0] = (int32_t) (kidx % g->kS);
    kc[1] = (int32_t) ((kidx / g->kS) % g->kR);
    kc[2] = (int32_t) ((kidx / g->kS / g->kR) % g->kQ);
    kc[3] = 0;
    pos[0] = 0;
    uint64_t r = row;
    for (int d = 1; d < 5; d++)
    {
        const uint32_t o = (uint32_t) (r % g->out_shape[d]);
        r /= g->out_shape[d];
        pos[d] = (int32_t) o * g->p->conv_stride[d - 1] + kc[d - 1] * g->p->dilation[d - 1] - g->p->padding[d - 1];
        if (pos[d] < 0 || pos[d] >= (int32_t) g->in_shape[d]) return 0;
    }
    return 1;
}

static uint64_t offset_of(const mme_hip_tensor* t, const int32_t pos[5])
{
    uint64_t o = 0;
    for (int d = 0; d < 5; d++) o += (uint64_t) pos[d] * t->strides[d];
    return o;
}

/* dense copy of a tensor in size order (createBufferWithoutStrides, mme_reference_impl.cpp:245-282) */
static char* densify(const mme_hip_tensor* t)
{
    const int      es = dtype_size(t->dtype);
    const uint64_t n = n_elements(t);
    char*          buf = (char*) malloc((size_t) (n ? n : 1) * es);
    uint64_t       o = 0;
    for (uint32_t i4 = 0; i4 < t->sizes[4]; i4++)
        for (uint32_t i3 = 0; i3 < t->sizes[3]; i3++)
            for (uint32_t i2 = 0; i2 < t->sizes[2]; i2++)
                for (uint32_t i1 = 0; i1 < t->sizes[1]; i1++)
                {
                    const uint64_t src = (uint64_t) i4 * t->strides[4] + (uint64_t) i3 * t->strides[3] +
                                         (uint64_t) i2 * t->strides[2] + (uint64_t) i1 * t->strides[1];
                    memcpy(buf + o * es, (const char*) t->data + src * es, (size_t) t->sizes[0] * es);
                    o += t->sizes[0];
                }
    return buf;
}

int orc_convolution(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w,
                    const mme_hip_tensor* y, const mme_hip_conv_params* p, int op, int rm)
{
    return orc_convolution_clip(out, x, w, y, p, op, rm, 0, 0);
}

int orc_convolution_clip(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w,
                         const mme_hip_tensor* y, const mme_hip_conv_params* p, int op, int rm, int clip,
                         int clip_inf_in)
{
    if (op == MME_HIP_OP_TRANSPOSED_DEDX)
    {
        /* mme_reference_impl.cpp:625-647: the weights arrive with their first two dimensions exchanged (transposeTensor,
         * :366-393) and are read with the S axis reversed (reverseWeightsDimS, :324-364); then a plain dedx */
        if (!w || !w->data) return fail("got null pointer");
        const int       wes = dtype_size(w->dtype);
        const uint64_t  n0 = w->sizes[0], n1 = w->sizes[1], S = w->sizes[2], R = w->sizes[3], Q = w->sizes[4];
        const uint64_t  total = n0 * n1 * S * R * Q;
        char*           buf = (char*) malloc((size_t) (total ? total : 1) * wes);
        mme_hip_tensor  wr = *w;
        uint64_t        acc = 1;
        wr.sizes[0] = (uint32_t) n1;
        wr.sizes[1] = (uint32_t) n0;
        for (int d = 0; d < 5; d++)
        {
            wr.strides[d] = (uint32_t) acc;
            acc *= wr.sizes[d];
        }
        wr.data = buf;
        for (uint64_t q = 0; q < Q; q++)
            for (uint64_t r = 0; r < R; r++)
                for (uint64_t sx = 0; sx < S; sx++)
                    for (uint64_t i1 = 0; i1 < n0; i1++)
                        for (uint64_t i0 = 0; i0 < n1; i0++)
                        {
                            const uint64_t src = i1 * w->strides[0] + i0 * w->strides[1] + (S - 1 - sx) * w->strides[2] + r * w->strides[3] +
                                                 q * w->strides[4];
                            const uint64_t dst = i0 + n1 * (i1 + n0 * (sx + S * (r + R * q)));
                            memcpy(buf + dst * wes, (const char*) w->data + src * wes, (size_t) wes);
                        }
        const int rc = orc_convolution_clip(out, x, &wr, y, p, MME_HIP_OP_DEDX, rm, clip, clip_inf_in);
        free(buf);
        return rc;
    }
    const mme_hip_tensor *A, *B;
    switch (op)
    {
        case MME_HIP_OP_FWD: A = x; B = w; break;
        case MME_HIP_OP_DEDX: A = y; B = w; break;
        case MME_HIP_OP_DEDW: A = x; B = y; break;
        default: return fail("invalid operation");
    }
    if (check_types(out, A, B)) return -1;
    const int es = dtype_size(A->dtype);

    uint32_t lut_a[256], lut_b[256];
    dot_ctx  ctx;
    dot_ctx_init(&ctx, A, B, lut_a, lut_b, clip, clip_inf_in);

    /* the weight-shaped tensor: w for fwd/dedx, out for dedw; the y-shaped tensor: out / y(A) / y(B) */
    const mme_hip_tensor* wt = (op == MME_HIP_OP_DEDW) ? out : w;
    const mme_hip_tensor* yt = (op == MME_HIP_OP_FWD) ? out : y;
    const mme_hip_tensor* xt = (op == MME_HIP_OP_DEDX) ? out : x;
    const uint64_t K = wt->sizes[0], C = wt->sizes[1];
    const uint64_t nk = (uint64_t) wt->sizes[2] * wt->sizes[3] * wt->sizes[4];
    const uint64_t RSC = nk * C;
    const uint64_t BHW = (uint64_t) yt->sizes[1] * yt->sizes[2] * yt->sizes[3] * yt->sizes[4];
    if (xt->sizes[0] != C) return fail("channel dims of x and w differ");
    if (yt->sizes[0] != K) return fail("channel dims of y and w differ");

    im2col_geo g;
    g.p = p;
    memcpy(g.out_shape, yt->sizes, sizeof g.out_shape);
    memcpy(g.in_shape, xt->sizes, sizeof g.in_shape);
    g.kS = wt->sizes[2];
    g.kR = wt->sizes[3];
    g.kQ = wt->sizes[4];

    if (op == MME_HIP_OP_FWD)
    {
        /* Y[row][k] = sum_col im2col(X)[row][col] * W[col][k];   W dense is [RSC][K] */
        char* Wd = densify(w);
        char* zero = (char*) calloc((size_t) C, es);
#pragma omp parallel num_threads(orc_get_num_threads())
        {
            char* arow = (char*) malloc((size_t) RSC * es);
#pragma omp for schedule(static)
            for (uint64_t row = 0; row < BHW; row++)
            {
                int32_t pos[5];
                for (uint32_t kidx = 0; kidx < nk; kidx++)
                {
                    const int in = im2col_pos(&g, row, kidx, pos);
                    memcpy(arow + kidx * C * es, in ? (const char*) x->data + offset_of(x, pos) * es : zero, (size_t) C * es);
                }
                /* output position of this row in the (possibly strided) y tensor */
                int32_t  opos[5] = {0, 0, 0, 0, 0};
                uint64_t r = row;
                for (int d = 1; d < 5; d++)
                {
                    opos[d] = (int32_t) (r % out->sizes[d]);
                    r /= out->sizes[d];
                }
                uint32_t* yrow = (uint32_t*) out->data + offset_of(out, opos);
                for (uint64_t k = 0; k < K; k++) yrow[k] = dot(&ctx, arow, 1, Wd + k * es, (ptrdiff_t) K, RSC);
            }
            free(arow);
        }
        free(zero);
        free(Wd);
    }
    else if (op == MME_HIP_OP_DEDX)
    {
        /* M[row][kidx*C + c] = sum_k dY[row][k] * W[(kidx*C + c)][k];   dX = col2im(M) with fp32 adds */
        char*     Wd = densify(w);
        char*     Yd = densify(y);
        uint32_t* Mx = (uint32_t*) malloc((size_t) BHW * RSC * 4);
#pragma omp parallel for schedule(static) num_threads(orc_get_num_threads())
        for (uint64_t row = 0; row < BHW; row++)
            for (uint64_t col = 0; col < RSC; col++)
                Mx[row * RSC + col] = dot(&ctx, Yd + row * K * es, 1, Wd + col * K * es, 1, K);
        memset(out->data, 0, (size_t) span_elements(out) * 4);
        for (uint32_t kidx = 0; kidx < nk; kidx++)
            for (uint64_t row = 0; row < BHW; row++)
            {
                int32_t pos[5];
                if (!im2col_pos(&g, row, kidx, pos)) continue; /* adds into the discarded padding vector */
                uint32_t* dst = (uint32_t*) out->data + offset_of(out, pos);
                for (uint64_t c = 0; c < C; c++) dst[c] = orc_add_fp32(dst[c], Mx[row * RSC + kidx * C + c], rm);
            }
        free(Mx);
        free(Yd);
        free(Wd);
    }
    else
    {
        /* dW[col][k] = sum_row im2col(X)[row][col] * dY[row][k] */
        char* Yd = densify(y);
        char* At = (char*) malloc((size_t) RSC * BHW * es); /* im2col(X) transposed: [RSC][BHW] */
        for (uint64_t row = 0; row < BHW; row++)
        {
            int32_t pos[5];
            for (uint32_t kidx = 0; kidx < nk; kidx++)
            {
                const int   in = im2col_pos(&g, row, kidx, pos);
                const char* src = in ? (const char*) x->data + offset_of(x, pos) * es : NULL;
                for (uint64_t c = 0; c < C; c++)
                {
                    char* d = At + ((kidx * C + c) * BHW + row) * es;
                    if (src) memcpy(d, src + c * es, (size_t) es);
                    else
                        memset(d, 0, (size_t) es);
                }
            }
        }
#pragma omp parallel for schedule(static) num_threads(orc_get_num_threads())
        for (uint64_t col = 0; col < RSC; col++)
        {
            int32_t  opos[5];
            uint64_t r = col;
            opos[0] = 0;
            for (int d = 1; d < 5; d++)
            {
                opos[d] = (int32_t) (r % out->sizes[d]);
                r /= out->sizes[d];
            }
            uint32_t* dst = (uint32_t*) out->data + offset_of(out, opos);
            for (uint64_t k = 0; k < K; k++) dst[k] = dot(&ctx, At + col * BHW * es, 1, Yd + k * es, (ptrdiff_t) K, BHW);
        }
        free(At);
        free(Yd);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------- */
/* activation / casts   (mme_reference_impl.cpp:661-689, 1132-1141, 1143-1245)                                     */
/* ------------------------------------------------------------------------------------------------------------- */
static int cast_one(void* out, size_t i, int dt, unsigned bias, int mode, uint32_t u, int rm, uint32_t lfsr, int clip,
                    int clip_inf_in, int ftz, int sftz)
{
    switch (dt)
    {
        case MME_HIP_BF16: ((uint16_t*) out)[i] = orc_fp32_to_bf16(u, rm, lfsr, clip, ftz, clip_inf_in); return 0;
        case MME_HIP_FP32: ((uint32_t*) out)[i] = orc_fp32_to_fp32(u, rm, clip, ftz, clip_inf_in); return 0;
        case MME_HIP_FP8_143:
            ((uint8_t*) out)[i] = orc_fp32_to_fp8(u, 4, 3, (int) bias, rm, lfsr, ftz, clip, clip_inf_in, sftz, mode);
            return 0;
        case MME_HIP_FP8_152:
            ((uint8_t*) out)[i] = orc_fp32_to_fp8(u, 5, 2, (int) bias, rm, lfsr, ftz, clip, clip_inf_in, sftz, mode);
            return 0;
        case MME_HIP_FP16:
            ((uint16_t*) out)[i] = orc_fp32_to_cfp16(u, 5, (int) bias, rm, lfsr, ftz, clip, clip_inf_in, mode != 0);
            return 0;
        case MME_HIP_UFP16:
            ((uint16_t*) out)[i] = orc_fp32_to_cfp16(u, 6, (int) bias, rm, lfsr, ftz, clip, clip_inf_in, mode != 0);
            return 0;
        default: return -1;
    }
}

int orc_activation(const mme_hip_tensor* out, const mme_hip_tensor* acc, int relu, int rm, int clip, int clip_inf_in,
                   int ftz, int sftz, uint32_t* lfsr, uint32_t polynomial)
{
    if (acc->dtype != MME_HIP_FP32) return fail("acc element type should be fp32");
    if (acc->dim != out->dim) return fail("dims number of outputTensor doesnt match acc output");
    for (int d = 0; d < 5; d++)
        if (acc->sizes[d] != out->sizes[d]) return fail("sizes of output Tensot doesnt match acc output");
    /* getSizeInElements() is the span in memory, gaps between strided rows included (sim_tensor_base.cpp:177-194) */
    const uint64_t n = span_elements(acc);
    float*         in = (float*) acc->data;
    if (relu) /* std::max((T) 0, x) returns x only when 0 < x: NaN and -0 become +0 (:1132-1141) */
    {
        int contiguous = acc->strides[0] == 1;
        for (int d = 1; d < acc->dim && d < 5; d++) contiguous = contiguous && acc->strides[d] == acc->strides[d - 1] * acc->sizes[d - 1];
        if (!contiguous) return fail("input and output should be flattened"); /* (:1135) */
        for (uint64_t i = 0; i < n; i++) in[i] = (0.0f < in[i]) ? in[i] : 0.0f;
    }
    polynomial &= 0xFFFFu; /* m_polynomial is a uint16_t (mme_reference_impl.h:253) */
    const int reseed = (rm == RM_SR_RNE_DNORM || rm == RM_SR || sftz);
    const int mod = (out->dtype == MME_HIP_BF16 || is_fp16(out->dtype)) ? 64 : 128;
    if (reseed && !lfsr) return fail("stochastic modes need the LFSR state");
    for (uint64_t i = 0; i < n; i++)
    {
        const int      li = (int) (i % mod);
        const uint32_t l = lfsr ? lfsr[li] : 0;
        if (cast_one(out->data, i, out->dtype, out->fp_bias, out->inf_nan_mode, f2u(in[i]), rm, l, clip, clip_inf_in,
                     ftz, sftz))
            return fail("Unsupported type");
        if (reseed && out->dtype != MME_HIP_FP32) lfsr[li] = orc_lfsr32(lfsr[li], polynomial);
    }
    return 0;
}

static inline float pow2f(int e)
{
    /* exact power of two as fp32, e in [-126, 127] */
    return u2f((uint32_t) (e + 127) << 23);
}

int orc_cast_from_fp32(void* out, int dt, unsigned bias, int mode, const float* in, size_t n, int scale_exp,
                       const int32_t* col, size_t n_cols, int relu, int rm, int clip, int clip_inf_in, int ftz)
{
    if (scale_exp < -126 || scale_exp > 126) return fail("scale exponent out of range");
    const float s = pow2f(scale_exp);
    int         bad = 0;
#pragma omp parallel for schedule(static) num_threads(orc_get_num_threads()) reduction(| : bad)
    for (size_t i = 0; i < n; i++)
    {
        volatile float v = in[i];
        if (scale_exp) v = v * s;
        if (col) v = v * pow2f(col[i % n_cols]);
        if (relu) v = (v > 0.0f) ? v : 0.0f; /* std::max(0, x): NaN and -0 become +0 (:1132-1141) */
        bad |= cast_one(out, i, dt, bias, mode, f2u(v), rm, 0, clip, clip_inf_in, ftz, 0) != 0;
    }
    return bad ? fail("Unsupported type") : 0;
}

int orc_cast_to_fp32(float* out, const void* in, int dt, unsigned bias, int mode, size_t n, int scale_exp,
                     const int32_t* col, size_t n_cols)
{
    if (scale_exp < -126 || scale_exp > 126) return fail("scale exponent out of range");
    const float s = pow2f(scale_exp);
    uint32_t    lut[256];
    if (dt == MME_HIP_FP8_143 || dt == MME_HIP_FP8_152)
    {
        const int E = dt == MME_HIP_FP8_143 ? 4 : 5;
        for (int c = 0; c < 256; c++) lut[c] = orc_fp8_to_fp32((uint8_t) c, E, 7 - E, (int) bias, mode);
    }
    else if (dt != MME_HIP_BF16 && !is_fp16(dt))
        return fail("Unsupported type");
#pragma omp parallel for schedule(static) num_threads(orc_get_num_threads())
    for (size_t i = 0; i < n; i++)
    {
        volatile float v = (dt == MME_HIP_BF16) ? u2f((uint32_t) ((const uint16_t*) in)[i] << 16)
                           : is_fp16(dt)        ? u2f(orc_cfp16_to_fp32(((const uint16_t*) in)[i], dt == MME_HIP_UFP16 ? 6 : 5, (int) bias, mode != 0))
                                                : u2f(lut[((const uint8_t*) in)[i]]);
        if (scale_exp) v = v * s;
        if (col) v = v * pow2f(col[i % n_cols]);
        out[i] = v;
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------------------- */
/* bulk forms of the scalar functions, so that sweeps over millions of inputs run at C speed                       */
/* ------------------------------------------------------------------------------------------------------------- */
void orc_fp32_to_fp8_n(uint8_t* out, const uint32_t* in, size_t n, int E, int M, int bias, int rm, const uint32_t* lfsr,
                       int ftz, int clip, int clip_inf_in, int sftz, int mode)
{
    for (size_t i = 0; i < n; i++)
        out[i] = orc_fp32_to_fp8(in[i], E, M, bias, rm, lfsr ? lfsr[i] : 0, ftz, clip, clip_inf_in, sftz, mode);
}
void orc_fp8_to_fp32_n(uint32_t* out, const uint8_t* in, size_t n, int E, int M, int bias, int mode)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_fp8_to_fp32(in[i], E, M, bias, mode);
}
void orc_fp32_to_bf16_n(uint16_t* out, const uint32_t* in, size_t n, int rm, const uint32_t* lfsr, int clip, int ftz,
                        int clip_inf_in)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_fp32_to_bf16(in[i], rm, lfsr ? lfsr[i] : 0, clip, ftz, clip_inf_in);
}
void orc_fp32_to_fp32_n(uint32_t* out, const uint32_t* in, size_t n, int rm, int clip, int ftz, int clip_inf_in)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_fp32_to_fp32(in[i], rm, clip, ftz, clip_inf_in);
}
void orc_add_fp32_n(uint32_t* out, const uint32_t* a, const uint32_t* b, size_t n, int rm)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_add_fp32(a[i], b[i], rm);
}
void orc_tree9_n(uint32_t* out, const uint32_t* a, const uint32_t* b, size_t n, int emul_kind)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_tree9(a + 9 * i, b + 9 * i, emul_kind);
}
void orc_fp32_to_cfp16_n(uint16_t* out, const uint32_t* in, size_t n, int E, int bias, int rm, const uint32_t* lfsr,
                         int ftz, int clip, int clip_inf_in, int no_inf_nan)
{
    for (size_t i = 0; i < n; i++)
        out[i] = orc_fp32_to_cfp16(in[i], E, bias, rm, lfsr ? lfsr[i] : 0, ftz, clip, clip_inf_in, no_inf_nan);
}
void orc_cfp16_to_fp32_n(uint32_t* out, const uint16_t* in, size_t n, int E, int bias, int no_inf_nan)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_cfp16_to_fp32(in[i], E, bias, no_inf_nan);
}
void orc_fp32_to_tf32_n(uint32_t* out, const uint32_t* in, size_t n, int clip, int clip_inf_in)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_fp32_to_tf32(in[i], clip, clip_inf_in);
}

int orc_memory_write(const mme_hip_tensor* memory, const mme_hip_tensor* mme_out, int op, int rm, int clip_fp)
{
    if (!memory || !mme_out || !memory->data || !mme_out->data) return fail("got null pointer");
    const size_t n = (size_t) span_elements(memory);
    if (op == MME_HIP_REDUCTION_NONE)
    {
        memmove(memory->data, mme_out->data, n * (size_t) dtype_size(memory->dtype));
        return 0;
    }
    if (op < 0 || op > MME_HIP_REDUCTION_NONE) return fail("invalid reduction operation");
    if (memory->dtype == MME_HIP_FP32)
    {
        uint32_t*       m = (uint32_t*) memory->data;
        const uint32_t* o = (const uint32_t*) mme_out->data;
        for (size_t i = 0; i < n; i++) m[i] = rmw_elem(m[i], o[i], op, rm, clip_fp, 23);
    }
    else if (memory->dtype == MME_HIP_BF16)
    {
        uint16_t*       m = (uint16_t*) memory->data;
        const uint16_t* o = (const uint16_t*) mme_out->data;
        for (size_t i = 0; i < n; i++) m[i] = (uint16_t) (rmw_elem((uint32_t) m[i] << 16, (uint32_t) o[i] << 16, op, rm, clip_fp, 7) >> 16);
    }
    else if (memory->dtype == MME_HIP_FP16)
    {
        /* the RMW unit knows one fp16: exponent bias 15 with inf and NaN (ST_TNSR_RMW_FP16), whatever the tensor says */
        uint16_t*       m = (uint16_t*) memory->data;
        const uint16_t* o = (const uint16_t*) mme_out->data;
        for (size_t i = 0; i < n; i++) m[i] = rmw_elem_fp16(m[i], o[i], op, rm, clip_fp);
    }
    else if (memory->dtype == MME_HIP_FP8_152)
    {
        uint8_t*       m = (uint8_t*) memory->data;
        const uint8_t* o = (const uint8_t*) mme_out->data;
        for (size_t i = 0; i < n; i++) m[i] = rmw_elem_fp8_152(m[i], o[i], op, rm, clip_fp);
    }
    else
        return fail("reductions exist for fp32, bf16, fp16 and fp8_152 only");
    return 0;
}
