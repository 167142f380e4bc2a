// gemm_fp8_fast.hip -- the fp8 contraction for large aligned problems (the headline path: fp8_143 / fp8_152 operands,
// M and N multiples of 256, K a multiple of 128 and >= 384, 16-byte aligned rows).
//
// Same arithmetic as the general kernel (gemm_impl.hpp): OCP fp8 MFMA with fp32 accumulation, Gaudi's exponent bias
// folded into the epilogue multiplier.  What differs is the data movement, which is what bounds the general kernel:
//
//   tile        256 x 256 outputs per 256-lane workgroup; 4 wavefronts as 2 x 2, 128 x 128 each = 4 x 4 MFMA
//               v_mfma_f32_32x32x64_f8f6f4 tiles -> 256 accumulator registers per lane (AGPRs), one wavefront per SIMD
//   HBM/L2->LDS global_load_lds_dwordx4: 16 bytes per lane straight into LDS, no staging registers.  Ring of 4 stages of
//               64 k-bytes (A 256 x 64 B + B 64 x 256 B = 32 KiB each, 128 KiB of LDS); stage t+3 is requested while
//               stage t feeds the matrix cores, tracked with vmcnt (8 requests per lane and stage)
//   LDS layout  16-byte chunks, placed so that every fragment read is bank-conflict free:
//                 A (k contiguous): chunk (row r, c) at r*4 + (c ^ ((r>>2)&3))       -> ds_read_b128
//                 B (n contiguous): chunk (k, cb)    at k*16 + ((cb + 2*(k&7)) & 15) -> ds_read_b64_tr_b8, the LDS
//                   transpose read of gfx950: a 16-lane group reads 8 k-rows x 16 n-columns and every lane receives
//                   the 8 k-values of its own column, which is the operand layout of the MFMA (k packed per lane)
//               the permutation is applied on the global-address side (each lane fetches the chunk that belongs at its
//               LDS position), the DMA itself writes lanes in order
//   schedule    one barrier per stage, placed right after an MFMA issue so that the 64 cycles of that MFMA cover it;
//               fragment reads of stage t+1 and the 8 DMA requests of stage t+3 are interleaved one per MFMA
//   mapping     workgroup ids are dealt round-robin to the 8 XCDs; ids are remapped so that each XCD owns a compact
//               8 x 4 block of tiles (12 operand panels through its L2 instead of 18)
//
// Replaces, for these shapes, doGemmWorkerFloat + Gaudi3Fp8Fma::fma_vec of the reference
// (mme/mme_reference/mme_reference_impl.cpp:1022-1053, chip_fma/gaudi3_fma.cpp:70-144).
#include <type_traits>

#include "gemm_impl.hpp"

namespace mme
{
namespace
{
typedef int v2i __attribute__((ext_vector_type(2)));
#define LDS3 __attribute__((address_space(3)))

constexpr int FBM = 256, FBN = 256, FBK = 64, FNST = 4;
constexpr int FSTAGE = FBM * FBK + FBK * FBN; // 32 KiB

__device__ __forceinline__ int fa_pos(int r, int c) { return r * 4 + (c ^ ((r >> 2) & 3)); }
__device__ __forceinline__ int fb_pos(int k, int cb) { return k * 16 + ((cb + 2 * (k & 7)) & 15); }

// 16 bytes per lane from global memory to LDS at lds_off + lane * 16 (lds_off is wave-uniform).  Inline assembly keeps
// the request out of the compiler's memory model: it would otherwise order every later LDS read behind it.
__device__ __forceinline__ void dma16(const void* g, uint32_t lds_off)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_off) : "memory");
}

struct Frags
{
    v8i a[4], b[4];
};

__device__ __forceinline__ void read_a(Frags& f, int i, const char* st, int wm, int lane)
{
    const int r = wm * 128 + i * 32 + (lane & 31), c0 = 2 * (lane >> 5);
    const v4i lo = *(const v4i*) (st + fa_pos(r, c0) * 16), hi = *(const v4i*) (st + fa_pos(r, c0 + 1) * 16);
    f.a[i] = v8i {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

// B stored n-contiguous: transposed LDS reads
__device__ __forceinline__ void read_b_tr(Frags& f, int j, const char* st, int wn, int lane)
{
    const int q = lane >> 4, cb = wn * 8 + j * 2 + (q & 1), g = q >> 1, rr = (lane & 15) >> 1, h = lane & 1;
    v2i       t[4];
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
    {
        const int k = g * 32 + 8 * tt + rr;
        t[tt] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LDS3 v2i*) (st + FBM * FBK + fb_pos(k, cb) * 16 + h * 8));
    }
    f.b[j] = v8i {t[0].x, t[0].y, t[1].x, t[1].y, t[2].x, t[2].y, t[3].x, t[3].y};
}

// B stored k-contiguous (the "abt" form): same layout and reads as A
__device__ __forceinline__ void read_b_kc(Frags& f, int j, const char* st, int wn, int lane)
{
    const int r = wn * 128 + j * 32 + (lane & 31), c0 = 2 * (lane >> 5);
    const v4i lo = *(const v4i*) (st + FBM * FBK + fa_pos(r, c0) * 16), hi = *(const v4i*) (st + FBM * FBK + fa_pos(r, c0 + 1) * 16);
    f.b[j] = v8i {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

#define FENCE __builtin_amdgcn_sched_barrier(0)

template<int FMT, bool B_KC>
__global__ __launch_bounds__(256) void gemm_fp8_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    KARG GemmProblem& g = *(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr();
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    if (g.skip_flag && ((*g.skip_flag != 0u) == (g.skip_if != 0))) return;

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), wm = wave >> 1, wn = wave & 1;
    const int tiles_n = g.N / FBN, tiles_m = g.M / FBM;
    int       tm, tn;
    {
        const int b = blockIdx.x, T = tiles_m * tiles_n;
        if ((tiles_m % 8 == 0) && (tiles_n % 4 == 0))
        {
            const int L = (b & 7) * (T >> 3) + (b >> 3), Bx = L >> 5, w = L & 31, nbn = tiles_n >> 2;
            tm = (Bx / nbn) * 8 + (w >> 2);
            tn = (Bx % nbn) * 4 + (w & 3);
        }
        else
        {
            tm = b / tiles_n;
            tn = b % tiles_n;
        }
    }
    int       bz = blockIdx.y;
    const int b0 = bz % g.batch[0];
    bz /= g.batch[0];
    const int       b1 = bz % g.batch[1], b2 = bz / g.batch[1];
    const long long a_off = b0 * g.A.batch_stride[0] + b1 * g.A.batch_stride[1] + b2 * g.A.batch_stride[2];
    const long long b_off = b0 * g.B.batch_stride[0] + b1 * g.B.batch_stride[1] + b2 * g.B.batch_stride[2];
    const int       m0 = tm * FBM, n0 = tn * FBN;
    const long long lda = g.A.stride_f;
    const long long ldb = B_KC ? g.B.stride_f : g.B.stride_k;
    const uint8_t*  A = (const uint8_t*) g.A.base + a_off;
    const uint8_t*  B = (const uint8_t*) g.B.base + b_off;
    const uint32_t  lds_base = (uint32_t) (uintptr_t) lds;

    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    const int nk = g.K / FBK;
    // per-lane global pointers of this wavefront's 4 + 4 request slots (they advance by one stage per step)
    const uint8_t* ga[4];
    const uint8_t* gb[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
    {
        const int t = wave * 4 + u;
        {
            const int r = t * 16 + (lane >> 2), p = lane & 3, c = p ^ ((r >> 2) & 3);
            ga[u] = A + (size_t) (m0 + r) * lda + c * 16;
        }
        if (B_KC)
        {
            const int r = t * 16 + (lane >> 2), p = lane & 3, c = p ^ ((r >> 2) & 3);
            gb[u] = B + (size_t) (n0 + r) * ldb + c * 16;
        }
        else
        {
            const int k = t * 4 + (lane >> 4), p = lane & 15, cb = (p - 2 * (k & 7)) & 15;
            gb[u] = B + (size_t) k * ldb + n0 + cb * 16;
        }
    }
    auto issue_a = [&](int u, int stage, int slot) __attribute__((always_inline))
    {
        dma16(ga[u] + (size_t) stage * FBK, lds_base + slot * FSTAGE + (wave * 4 + u) * 1024);
    };
    auto issue_b = [&](int u, int stage, int slot) __attribute__((always_inline))
    {
        dma16(gb[u] + (B_KC ? (size_t) stage * FBK : (size_t) stage * FBK * ldb), lds_base + slot * FSTAGE + FBM * FBK + (wave * 4 + u) * 1024);
    };
    auto read_b = [&](Frags & f, int j, const char* st) __attribute__((always_inline))
    {
        if (B_KC) read_b_kc(f, j, st, wn, lane);
        else
            read_b_tr(f, j, st, wn, lane);
    };

    for (int t = 0; t < FNST - 1; t++)
    {
#pragma unroll
        for (int u = 0; u < 4; u++)
        {
            issue_a(u, t, t);
            issue_b(u, t, t);
        }
    }
    // s_waitcnt immediate (gfx9): vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14
    __builtin_amdgcn_s_waitcnt(0x4F70); // vmcnt(16): stage 0 has landed
    __syncthreads();
    Frags f0, f1;
#pragma unroll
    for (int i = 0; i < 4; i++)
    {
        read_a(f0, i, lds, wm, lane);
        read_b(f0, i, lds);
    }

#define MMA(i, j) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(cur.a[i], cur.b[j], acc[i][j], FMT & 1, (FMT >> 1) & 1, 0, 0, 0, 0)
#define RA(i) \
    if (RN) read_a(nxt, i, st, wm, lane);
#define RB(j) \
    if (RN) read_b(nxt, j, st);
#define LA(u) \
    if (LOADS) issue_a(u, t + FNST - 1, slot);
#define LB(u) \
    if (LOADS) issue_b(u, t + FNST - 1, slot);
    // One stage: 16 MFMAs on `cur`; after the first one wait until stage t+1 has landed in every wavefront's view
    // (WAITC leaves the younger stages in flight) and fetch its fragments into `nxt`; request stage t+3.
    auto step = [&](int t, Frags& cur, Frags& nxt, auto waitc, auto loads, auto readnext) __attribute__((always_inline))
    {
        constexpr int  WAITC = decltype(waitc)::value;
        constexpr bool LOADS = decltype(loads)::value;
        constexpr bool RN = decltype(readnext)::value;
        const char*    st = lds + ((t + 1) % FNST) * FSTAGE;
        const int      slot = (t + FNST - 1) % FNST;
        MMA(0, 0);
        FENCE;
        if (RN)
        {
            __builtin_amdgcn_s_waitcnt(WAITC);
            __builtin_amdgcn_s_barrier();
        }
        FENCE;
        MMA(0, 1); RA(0) LA(0) FENCE;
        MMA(0, 2); RA(1) FENCE;
        MMA(0, 3); RA(2) LA(1) FENCE;
        MMA(1, 0); RA(3) FENCE;
        MMA(1, 1); RB(0) LA(2) FENCE;
        MMA(1, 2); FENCE;
        MMA(1, 3); RB(1) LA(3) FENCE;
        MMA(2, 0); FENCE;
        MMA(2, 1); RB(2) LB(0) FENCE;
        MMA(2, 2); FENCE;
        MMA(2, 3); RB(3) LB(1) FENCE;
        MMA(3, 0); FENCE;
        MMA(3, 1); LB(2) FENCE;
        MMA(3, 2); FENCE;
        MMA(3, 3); LB(3) FENCE;
        if (RN) __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): `nxt` is complete, this wavefront is done with the stage
    };
    using W8 = std::integral_constant<int, 0x0F78>; // vmcnt(8)
    using W0 = std::integral_constant<int, 0x0F70>; // vmcnt(0)
    using T = std::true_type;
    using F = std::false_type;
    int t = 0;
    for (; t + 5 <= nk; t += 2)
    {
        step(t, f0, f1, W8 {}, T {}, T {});
        step(t + 1, f1, f0, W8 {}, T {}, T {});
    }
    // t == nk - 4 (nk is even and >= 6)
    step(t, f0, f1, W8 {}, T {}, T {});     // requests the last stage
    step(t + 1, f1, f0, W8 {}, F {}, T {}); // stage nk-2 needed, stage nk-1 may be in flight
    step(t + 2, f0, f1, W0 {}, F {}, T {});
    step(t + 3, f1, f0, W0 {}, F {}, F {});
#undef MMA
#undef RA
#undef RB
#undef LA
#undef LB

    // ---- epilogue: alpha, per-column power of two, relu, cast, store (same conversion functions as the general kernel).
    // The output-type dispatch sits outside the fully unrolled accumulator walk so that the accumulators stay in
    // registers.  Addresses are a uniform 64-bit tile base plus 32-bit lane offsets (one add per element).
    const long long c_off = b0 * g.epi.batch_stride[0] + b1 * g.epi.batch_stride[1] + b2 * g.epi.batch_stride[2];
    const long long ldc = g.epi.ld;
    const bool      has_alpha = g.epi.has_alpha != 0;
    const float     alpha = g.epi.alpha;
    const int32_t*  col_exp = g.epi.col_exp;
    const bool      relu = g.epi.fused && g.epi.cast.relu;
    const int       dt = g.epi.fused ? g.epi.out_dtype : DT_FP32;
    const int       esz = (dt == DT_FP32) ? 4 : (dt == DT_BF16 ? 2 : 1);
    char*           tile_base = (char*) g.epi.out + (c_off + (long long) m0 * ldc + n0) * esz; // uniform
    const uint32_t  ldcb = (uint32_t) ldc * esz;                                              // bytes per output row
    const CastParams cp = {g.epi.cast.dtype,       g.epi.cast.exp_bias, g.epi.cast.inf_nan_mode, g.epi.cast.rm,    g.epi.cast.clip_fp,
                           g.epi.cast.clip_inf_in, g.epi.cast.ftz,      g.epi.cast.relu,         g.epi.cast.scale, g.epi.cast.has_scale};
    // value of accumulator (i, j, v) after the power-of-two factors and relu
    auto value = [&](int i, int j, int v, float cs) __attribute__((always_inline))
    {
        float x = acc[i][j][v];
        if (has_alpha) x *= alpha;
        if (col_exp) x *= cs;
        if (relu) x = relu_ref(x);
        return x;
    };
    // generic walk: one store per element
    auto walk = [&](auto store) __attribute__((always_inline))
    {
        const uint32_t lane_off = (uint32_t) (wm * 128 + 4 * (lane >> 5)) * ldcb + (uint32_t) (wn * 128 + (lane & 31)) * esz;
#pragma unroll
        for (int j = 0; j < 4; j++)
        {
            float cs = 1.0f;
            if (col_exp) cs = pow2_of(col_exp[n0 + wn * 128 + j * 32 + (lane & 31)]);
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                    store(tile_base + (lane_off + (uint32_t) (i * 32 + 8 * (v >> 2) + (v & 3)) * ldcb + (uint32_t) (j * 32 * esz)), value(i, j, v, cs));
        }
    };
    if (dt == DT_FP32 && !(g.epi.fused && (g.epi.cast.clip_fp || g.epi.cast.ftz)))
        walk([&](char* p, float x) __attribute__((always_inline)) { *(float*) p = x; });
    else if (dt == DT_BF16 && g.epi.fast_cast)
    {
        // bf16, round to nearest even.  Lanes l and l^1 hold neighbouring columns: they swap one packed pair of rows
        // through DPP so that every lane stores whole dwords (two columns of one row).  NaN, inf and values that round
        // to inf are rare: a per-tile maximum of |x| detects them and that tile takes the element-wise conversion.
        const uint32_t odd = lane & 1;
        const uint32_t sel = odd ? 0x03020706u : 0x05040100u;
        const uint32_t lane_off = (uint32_t) (wm * 128 + 4 * (lane >> 5) + odd) * ldcb + (uint32_t) (wn * 128 + (lane & 30)) * 2;
        const uint32_t lane_off1 = (uint32_t) (wm * 128 + 4 * (lane >> 5)) * ldcb + (uint32_t) (wn * 128 + (lane & 31)) * 2;
#pragma unroll
        for (int j = 0; j < 4; j++)
        {
            float cs = 1.0f;
            if (col_exp) cs = pow2_of(col_exp[n0 + wn * 128 + j * 32 + (lane & 31)]);
#pragma unroll
            for (int i = 0; i < 4; i++)
            {
                uint32_t sum[16], mx = 0;
#pragma unroll
                for (int v = 0; v < 16; v++)
                {
                    const uint32_t u = f2u(value(i, j, v, cs));
                    mx = max(mx, u & 0x7FFFFFFFu);
                    sum[v] = u + 0x7FFFu + ((u >> 16) & 1u); // bf16 code in the high half
                }
                if (__builtin_amdgcn_ballot_w64(mx >= 0x7F7F8000u) == 0)
                {
#pragma unroll
                    for (int v = 0; v < 16; v += 2)
                    {
                        const uint32_t mine = __builtin_amdgcn_perm(sum[v + 1], sum[v], 0x07060302u); // rows v, v+1 of my column
                        const uint32_t theirs = (uint32_t) __builtin_amdgcn_update_dpp(0, (int) mine, 0xB1, 0xF, 0xF, false); // lane ^ 1
                        // even lane: row v = (my col, next col); odd lane: row v+1 = (previous col, my col)
                        const uint32_t word = __builtin_amdgcn_perm(theirs, mine, sel);
                        *(uint32_t*) (tile_base + (lane_off + (uint32_t) (i * 32 + 8 * (v >> 2) + (v & 3)) * ldcb + (uint32_t) (j * 64))) = word;
                    }
                }
                else
                {
#pragma unroll
                    for (int v = 0; v < 16; v++)
                        *(uint16_t*) (tile_base + (lane_off1 + (uint32_t) (i * 32 + 8 * (v >> 2) + (v & 3)) * ldcb + (uint32_t) (j * 64))) =
                            (uint16_t) fp32_to_bf16_rne(f2u(value(i, j, v, cs)), cp.clip_fp, cp.clip_inf_in);
                }
            }
        }
    }
    else if (dt == DT_FP8_143 && g.epi.fast_cast)
        walk([&](char* p, float x) __attribute__((always_inline)) { *(uint8_t*) p = (uint8_t) fp32_to_fp8_rne_mode0<3>(f2u(x), cp.exp_bias, cp.clip_fp, cp.clip_inf_in); });
    else if (dt == DT_FP8_152 && g.epi.fast_cast)
        walk([&](char* p, float x) __attribute__((always_inline)) { *(uint8_t*) p = (uint8_t) fp32_to_fp8_rne_mode0<2>(f2u(x), cp.exp_bias, cp.clip_fp, cp.clip_inf_in); });
    else
    {
        // rare cast settings: element-wise through the out-of-line generic converter (relu is applied there)
        const uint32_t lane_row = wm * 128 + 4 * (lane >> 5), lane_col = wn * 128 + (lane & 31);
#pragma unroll
        for (int j = 0; j < 4; j++)
        {
            float cs = 1.0f;
            if (col_exp) cs = pow2_of(col_exp[n0 + lane_col + j * 32]);
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                {
                    float x = acc[i][j][v];
                    if (has_alpha) x *= alpha;
                    if (col_exp) x *= cs;
                    store_out_slow(g.epi, c_off + (long long) (m0 + lane_row + i * 32 + 8 * (v >> 2) + (v & 3)) * ldc + n0 + lane_col + j * 32, x);
                }
        }
    }
}

template<int FMT>
hipError_t launch_fmt(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[2] = {false, false};
    const bool  bkc = p.B.k_contig != 0;
    const void* fn = bkc ? (const void*) gemm_fp8_fast_kernel<FMT, true> : (const void*) gemm_fp8_fast_kernel<FMT, false>;
    if (!attr_done[bkc])
    {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, FNST * FSTAGE);
        if (e != hipSuccess) return e;
        attr_done[bkc] = true;
    }
    if (bkc) hipLaunchKernelGGL((gemm_fp8_fast_kernel<FMT, true>), grid, dim3(256), FNST * FSTAGE, s, p);
    else
        hipLaunchKernelGGL((gemm_fp8_fast_kernel<FMT, false>), grid, dim3(256), FNST * FSTAGE, s, p);
    return hipGetLastError();
}
} // namespace

bool gemm_fp8_fast_applicable(const GemmProblem& p)
{
    if (!(p.dtype == DT_FP8_143 || p.dtype == DT_FP8_152)) return false;
    if (p.A.kind != VIEW_PLAIN || p.B.kind != VIEW_PLAIN) return false;
    if (!p.A.k_contig || !p.A.vec_ok || !p.B.vec_ok) return false;
    if (p.split_k > 1) return false;
    if (p.M % FBM || p.N % FBN || p.K % (2 * FBK) || p.K < 6 * FBK) return false;
    // epilogue: 32-bit byte offsets inside a tile, dword stores of bf16 pairs
    if (p.epi.ld <= 0 || p.epi.ld * 4 * FBM >= (1ll << 31)) return false;
    if (p.epi.fused && p.epi.out_dtype == DT_BF16)
    {
        if ((p.epi.ld & 1) || ((uintptr_t) p.epi.out & 3)) return false;
        for (int d = 0; d < 3; d++)
            if (p.epi.batch_stride[d] & 1) return false;
    }
    return true;
}

hipError_t launch_gemm_fp8_fast(const GemmProblem& p, hipStream_t s)
{
    const long long nb = (long long) p.batch[0] * p.batch[1] * p.batch[2];
    dim3            grid((p.M / FBM) * (p.N / FBN), (unsigned) nb, 1);
    switch ((p.fmt_a & 1) | ((p.fmt_b & 1) << 1))
    {
        case 0: return launch_fmt<0>(p, grid, s);
        case 1: return launch_fmt<1>(p, grid, s);
        case 2: return launch_fmt<2>(p, grid, s);
        default: return launch_fmt<3>(p, grid, s);
    }
}

} // namespace mme
