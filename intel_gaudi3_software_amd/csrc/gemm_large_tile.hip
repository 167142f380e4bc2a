// gemm_large_tile.hip -- the contraction for large aligned problems (the headline path: fp8_143 / fp8_152 operands, and
// bf16 through the same code; M and N multiples of 256, K a multiple of 128 bytes and >= 384 bytes, 16-byte aligned rows).
//
// Same arithmetic as the general kernel (gemm_impl.hpp): OCP fp8 (or bf16) MFMA with fp32 accumulation, Gaudi's exponent
// bias folded into the epilogue multiplier.  bf16 differs only in the matrix-core instruction (two v_mfma_f32_32x32x16_bf16
// per 64-byte stage and tile pair) and in the transposing read of an n-contiguous B (ds_read_b64_tr_b16).  What differs is the data movement, which is what bounds the general kernel:
//
//   tile        256 x 256 outputs per 512-lane workgroup; 8 wavefronts as 2 x 4, 128 x 64 each = 4 x 2 MFMA
//               v_mfma_f32_32x32x64_f8f6f4 tiles -> 128 accumulator registers per lane, two wavefronts per SIMD: a
//               wavefront cannot issue anything while its own MFMA occupies it, so its neighbour's MFMAs are what
//               cover its LDS reads, DMA requests and waits
//   HBM/L2->LDS global_load_lds_dwordx4: 16 bytes per lane straight into LDS, no staging registers.  Ring of 4 stages of
//               64 k-bytes (A 256 x 64 B + B 64 x 256 B = 32 KiB each, 128 KiB of LDS); stage t+4 is requested while
//               stage t feeds the matrix cores, tracked with vmcnt (4 requests per lane and stage)
//   LDS layout  16-byte chunks, placed so that every fragment read is bank-conflict free:
//                 A (k contiguous): chunk (row r, c) at r*4 + (c ^ ((r>>2)&3))       -> ds_read_b128
//                 B (n contiguous): chunk (k, cb)    at k*16 + ((cb + 2*(k&7)) & 15) -> ds_read_b64_tr_b8, the LDS
//                   transpose read of gfx950: a 16-lane group reads 8 k-rows x 16 n-columns and every lane receives
//                   the 8 k-values of its own column, which is the operand layout of the MFMA (k packed per lane)
//               the permutation is applied on the global-address side (each lane fetches the chunk that belongs at its
//               LDS position), the DMA itself writes lanes in order
//   schedule    one barrier per stage, placed right after an MFMA issue; every fragment register is refilled from
//               stage t+1 right after its last use in stage t, the 4 DMA requests of stage t+4 ride along
//   epilogue    the MFMA takes the B fragment as its first operand, so a lane's accumulator registers run along the
//               output row: one v_permlane32_swap per register pair gives every lane 16 consecutive columns, written
//               with 16-byte stores (bf16 through v_cvt_pk_bf16_f32 with an exact fall-back for NaN / inf / overflow)
//   mapping     workgroup ids are dealt round-robin to the 8 XCDs; ids are remapped so that each XCD owns a compact
//               8 x 4 block of tiles (12 operand panels through its L2 instead of 18)
//
// Replaces, for these shapes, doGemmWorkerFloat + Gaudi3Fp8Fma::fma_vec of the reference
// (mme/mme_reference/mme_reference_impl.cpp:1022-1053, chip_fma/gaudi3_fma.cpp:70-144).
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
template<int FMT, bool B_KC>
__global__ __launch_bounds__(512) void gemm_fp8_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<1, FMT, B_KC>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<bool B_KC, bool A_KC>
__global__ __launch_bounds__(512) void gemm_bf16_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, 0, B_KC, A_KC ? 0 : 2>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

// dedw: pixels along k for both operands, dY plain and n-contiguous
__global__ __launch_bounds__(512) void conv_dedw_bf16_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, 0, false, 3>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<bool B_KC>
__global__ __launch_bounds__(512) void conv_bf16_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, 0, B_KC, 1>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

hipError_t launch_conv_bf16(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[2] = {false, false};
    const bool  bkc = p.B.k_contig != 0;
    const void* fn = bkc ? (const void*) conv_bf16_fast_kernel<true> : (const void*) conv_bf16_fast_kernel<false>;
    if (!attr_done[bkc])
    {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, FNST * FSTAGE);
        if (e != hipSuccess) return e;
        attr_done[bkc] = true;
    }
    if (bkc) hipLaunchKernelGGL((conv_bf16_fast_kernel<true>), grid, dim3(512), FNST * FSTAGE, s, p);
    else
        hipLaunchKernelGGL((conv_bf16_fast_kernel<false>), grid, dim3(512), FNST * FSTAGE, s, p);
    return hipGetLastError();
}

hipError_t launch_bf16(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[5] = {false, false, false, false, false};
    const bool  bkc = p.B.k_contig != 0, akc = p.A.k_contig != 0;
    if (p.A.kind == VIEW_CONV && !p.A.pix_is_f) return launch_fast(conv_dedw_bf16_fast_kernel, attr_done[4], p, grid, s);
    if (akc) return bkc ? launch_fast(gemm_bf16_fast_kernel<true, true>, attr_done[0], p, grid, s)
                        : launch_fast(gemm_bf16_fast_kernel<false, true>, attr_done[1], p, grid, s);
    return bkc ? launch_fast(gemm_bf16_fast_kernel<true, false>, attr_done[2], p, grid, s)
               : launch_fast(gemm_bf16_fast_kernel<false, false>, attr_done[3], p, grid, s);
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
    if (bkc) hipLaunchKernelGGL((gemm_fp8_fast_kernel<FMT, true>), grid, dim3(512), FNST * FSTAGE, s, p);
    else
        hipLaunchKernelGGL((gemm_fp8_fast_kernel<FMT, false>), grid, dim3(512), FNST * FSTAGE, s, p);
    return hipGetLastError();
}
} // namespace

hipError_t launch_gemm_large_tile_f16(const GemmProblem& p, dim3 grid, hipStream_t s); // gemm_large_tile_f16.hip
hipError_t launch_gemm_large_tile_128(const GemmProblem& p, dim3 grid, hipStream_t s); // gemm_large_tile_128.hip
hipError_t launch_gemm_large_tile_conv_fp8(const GemmProblem& p, dim3 grid, hipStream_t s); // gemm_large_tile_conv_fp8.hip
hipError_t launch_gemm_large_tile_fp8_at(const GemmProblem& p, dim3 grid, hipStream_t s); // gemm_large_tile_fp8_at.hip
hipError_t launch_gemm_large_tile_ragged(const GemmProblem& p, dim3 grid, hipStream_t s); // gemm_large_tile_ragged.hip
hipError_t launch_gemm_large_tile_ragged_conv(const GemmProblem& p, dim3 grid, hipStream_t s); // gemm_large_tile_ragged_conv.hip
hipError_t launch_gemm_large_tile_chk(const GemmProblem& p, dim3 grid, hipStream_t s);            // gemm_large_tile_chk.hip
hipError_t launch_gemm_large_tile_w4(const GemmProblem& p, dim3 grid, hipStream_t s);             // gemm_large_tile_w4.hip
hipError_t launch_gemm_large_tile_persistent_chk(const GemmProblem& p, hipStream_t s);            // gemm_large_tile_persistent_chk.hip
bool       gemm_large_tile_persistent_applicable(const GemmProblem& p);                      // gemm_large_tile_persistent.hip
hipError_t launch_gemm_large_tile_persistent(const GemmProblem& p, hipStream_t s);

// the shape is not made of whole tiles (the pixel rows of a convolution view do not count: every kernel handles those)
static bool large_tile_ragged(const GemmProblem& p)
{
    const int tm = p.tile_m == 128 ? 128 : FBM;
    return (p.A.kind != VIEW_CONV && p.M % tm != 0) || p.N % FBN != 0;
}

bool gemm_large_tile_applicable(const GemmProblem& p)
{
    if (!(p.dtype == DT_FP8_143 || p.dtype == DT_FP8_152 || p.dtype == DT_BF16 || p.dtype == DT_FP16)) return false;
    const bool two_byte = p.dtype == DT_BF16 || p.dtype == DT_FP16;
    const int  es = two_byte ? 2 : 1;
    const bool gather = p.A.kind == VIEW_CONV;
    const int  tm = p.tile_m == 128 ? 128 : FBM;
    // the 128-row tile: A plain rows or the fwd / dedx gather; 2-byte operands also with dedw's pixels-along-k view
    if (tm == 128 && !two_byte && !p.A.k_contig) return false;
    if (tm == 128 && !p.A.k_contig && !(gather && !p.A.pix_is_f)) return false;
    if (gather)
    {
        // at most 32 taps, one problem per launch
        if (p.A.ktap[0] * p.A.ktap[1] * p.A.ktap[2] > 32) return false;
        if (p.batch[0] * p.batch[1] * p.batch[2] != 1) return false;
        if (p.A.pix_is_f)
        {
            // fwd / dedx: whole 64-byte stages inside one tap; the gather form of col2im only with unit strides; weights
            // plain or tapped (k-contiguous, same channel count)
            if (p.A.nch % (FBK / es) || p.A.nch * es > GF_ZERO_PAGE_BYTES) return false;
            for (int d = 0; d < 4; d++)
                if (p.A.gather_y && p.A.cstride[d] != 1) return false;
            if (p.B.kind == VIEW_TAPPED && (!p.B.k_contig || p.B.nch != p.A.nch || p.B.stride_k != 1)) return false;
            if (p.B.kind != VIEW_TAPPED && p.B.kind != VIEW_PLAIN) return false;
        }
        else
        {
            // dedw: 16-byte chunks of channels inside one tap, dY plain with its channels contiguous
            if (p.A.gather_y || p.A.nch % (16 / es) || p.B.kind != VIEW_PLAIN || p.B.k_contig) return false;
            // (the kernel keeps the source tensor's strides in bytes in 32-bit registers)
            for (int d = 0; d < 4; d++)
                if (p.A.src_stride[d] < 0 || p.A.src_stride[d] * es >= (1ll << 32)) return false;
        }
    }
    else if (p.A.kind != VIEW_PLAIN || p.B.kind != VIEW_PLAIN)
        return false;
    if (!p.A.vec_ok || !p.B.vec_ok) return false;
    if (gather && p.A.pix_is_f && !p.A.k_contig) return false;
    // whole tiles, except: the convolution views take any pixel count, and the convolutions and the GEMM forms with A
    // k-contiguous have kernels for partial tiles (any M from 64, N a multiple of 16 from 128: a lane's 16 output columns
    // are then all in or all out)
    if (large_tile_ragged(p))
    {
        if ((!gather && !p.A.k_contig) || (gather && !two_byte) || p.M < 64 || p.N % 16 || p.N < FBN / 2) return false;
    }
    if ((p.K * es) % (2 * FBK) || p.K * es < 6 * FBK) return false;
    if (p.split_k > 1)
    {
        // every slice an even number of stages, at least 6
        const int nk = p.K * es / FBK;
        if (nk % (2 * p.split_k) || nk / p.split_k < 6) return false;
    }
    // epilogue: 16-byte stores of 16 consecutive output columns (4 for fp32)
    if (p.epi.ld <= 0) return false;
    {
        const int out_dt = p.epi.fused ? p.epi.out_dtype : DT_FP32;
        if (out_dt == DT_FP16 || out_dt == DT_UFP16) return false; // these outputs take the general kernel's epilogue
        const int per16 = out_dt == DT_FP32 ? 4 : (out_dt == DT_BF16 ? 8 : 16); // elements per 16 bytes
        if ((p.epi.ld % per16) || ((uintptr_t) p.epi.out & 15)) return false;
        for (int d = 0; d < 3; d++)
            if (p.epi.batch_stride[d] % per16) return false;
    }
    return true;
}

// fp8 problems that end up in gemm_fp8_fast_kernel or gemm_fp8_persistent_kernel (see launch_gemm_large_tile): plain views,
// A k-contiguous, whole 256-row tiles
bool gemm_large_tile_checks_operands(const GemmProblem& p)
{
    if (!(p.dtype == DT_FP8_143 || p.dtype == DT_FP8_152) || !gemm_large_tile_applicable(p)) return false;
    return !large_tile_ragged(p) && p.tile_m != 128 && p.A.kind == VIEW_PLAIN && p.B.kind == VIEW_PLAIN && p.A.k_contig;
}

bool gemm_large_tile_takes_mfma_scale(const GemmProblem& p)
{
    return gemm_large_tile_checks_operands(p) && !p.chk && !(p.A.k_contig && gemm_large_tile_persistent_applicable(p));
}

int gemm_fast_pick_tile_m(const GemmProblem& p, int num_cus)
{
    GemmProblem q = p;
    q.split_k = 1;
    q.tile_m = 128;
    if (!gemm_large_tile_applicable(q)) return 0;
    q.tile_m = 0;
    if (!gemm_large_tile_applicable(q)) return 128; // (A contiguous along its rows, M a multiple of 128 only)
    // with at most half of the compute units busy, halving the tile doubles the workgroups without a second round
    const long long tiles = (long long) ((p.M + FBM - 1) / FBM) * ((p.N + FBN - 1) / FBN) * p.batch[0] * p.batch[1] * p.batch[2];
    return 2 * tiles <= num_cus ? 128 : 0;
}

// The fp8 GEMM of whole 256-row tiles has a second form with four wavefronts of 128 x 128 outputs (gemm_large_tile_w4.hip).  Its
// loop takes the same number of cycles per stage and runs at a 2-3 % higher clock on real data (a third less LDS traffic); its
// prologue and its epilogue, with one wavefront per SIMD, take about 4000 cycles more, and fewer wavefronts shorten the launch
// by a microsecond.  Measured on 4096 x 4096 outputs: 1.0-1.4 us faster at K = 4096, 0.8 us slower at K = 1024, equal when the
// tiles need several rounds (8192 x 8192 x 4096).  So: one round of tiles and at least 48 stages per workgroup.
int gemm_fast_pick_waves(const GemmProblem& p, int num_cus)
{
    // (one round: with half as many tiles or fewer the 128-row tiles take over, with more than one round's worth nothing is
    // split, so this form never meets split-k)
    return gemm_large_tile_one_round(p, num_cus) && p.K / FBK >= 48 ? 4 : 8;
}

// An fp8 GEMM of whole 256-row tiles, one workgroup per tile (not the persistent walk, no split-k), whose workgroups are all
// resident at once on a device that does nothing else: the checking instances may then settle special codes among themselves
// (GemmProblem::chk == 2).
bool gemm_large_tile_one_round(const GemmProblem& p, int num_cus)
{
    if (!gemm_large_tile_checks_operands(p) || gemm_large_tile_persistent_applicable(p) || p.split_k > 1) return false;
    return (long long) (p.M / FBM) * (p.N / FBN) * p.batch[0] * p.batch[1] * p.batch[2] <= num_cus;
}

int gemm_fast_pick_split_k(const GemmProblem& p, int num_cus)
{
    GemmProblem q = p;
    q.split_k = 1;
    if (!gemm_large_tile_applicable(q)) return 0;
    const int       tm = p.tile_m == 128 ? 128 : FBM;
    const long long tiles = (long long) ((p.M + tm - 1) / tm) * ((p.N + FBN - 1) / FBN) * p.batch[0] * p.batch[1] * p.batch[2];
    const int       nk = p.K * dt_bytes(p.dtype) / FBK;
    int             best = 1;
    // Splitting the reduction pays when the tiles leave most of the chip idle and the reduction is long: a slice costs a
    // pass of the fp32 output through the workspace plus the reduction kernel.  Rough model in microseconds: a stage (128 bytes of
    // k per row) takes 1.0 as measured on full-size fp8 and bf16 problems, the workspace moves at 3 TB/s (the reduction
    // kernel's measured rate is 2.3 .. 3.1), the extra launch costs 6.  Every slice keeps an even number of stages, at least 6.
    // (0.75 per stage of a 128-row tile: half the matrix work, the same latencies)
    const double stage_us = tm == 128 ? 0.75 : 1.0;
    const double out_bytes = 8.0 * p.M * (double) p.N * p.batch[0] * p.batch[1] * p.batch[2];
    const double t1 = (double) ((tiles + num_cus - 1) / num_cus) * nk * stage_us;
    double       best_t = 0.8 * t1; // a split has to promise a clear gain
    for (int s = 2; s <= 64; s++)
    {
        if (nk % (2 * s) || nk / s < 6) continue;
        const double t = (double) ((tiles * s + num_cus - 1) / num_cus) * (nk / s) * stage_us + s * out_bytes / 3e6 + 6.0;
        if (t < best_t)
        {
            best_t = t;
            best = s;
        }
    }
    return best;
}

hipError_t launch_gemm_large_tile(const GemmProblem& p, hipStream_t s)
{
    const long long nb = (long long) p.batch[0] * p.batch[1] * p.batch[2];
    const int       tm = p.tile_m == 128 ? 128 : FBM;
    dim3            grid(((p.M + tm - 1) / tm) * ((p.N + FBN - 1) / FBN), (unsigned) nb, p.split_k > 1 ? p.split_k : 1);
    if (large_tile_ragged(p)) return p.A.kind == VIEW_CONV ? launch_gemm_large_tile_ragged_conv(p, grid, s) : launch_gemm_large_tile_ragged(p, grid, s);
    if (tm == 128 && p.dtype != DT_BF16 && p.dtype != DT_FP16) return launch_gemm_large_tile_conv_fp8(p, grid, s);
    if (tm == 128) return launch_gemm_large_tile_128(p, grid, s);
    if (p.dtype == DT_FP16) return launch_gemm_large_tile_f16(p, grid, s);
    if (p.A.kind == VIEW_CONV && p.A.pix_is_f) return p.dtype == DT_BF16 ? launch_conv_bf16(p, grid, s) : launch_gemm_large_tile_conv_fp8(p, grid, s);
    if (p.A.k_contig && gemm_large_tile_persistent_applicable(p))
        return p.chk && p.dtype != DT_BF16 ? launch_gemm_large_tile_persistent_chk(p, s) : launch_gemm_large_tile_persistent(p, s);
    if (p.dtype == DT_BF16) return launch_bf16(p, grid, s);
    if (!p.A.k_contig) return launch_gemm_large_tile_fp8_at(p, grid, s);
    if (p.waves == 4) return launch_gemm_large_tile_w4(p, grid, s);
    if (p.chk) return launch_gemm_large_tile_chk(p, grid, s);
    switch ((p.fmt_a & 1) | ((p.fmt_b & 1) << 1))
    {
        case 0: return launch_fmt<0>(p, grid, s);
        case 1: return launch_fmt<1>(p, grid, s);
        case 2: return launch_fmt<2>(p, grid, s);
        default: return launch_fmt<3>(p, grid, s);
    }
}

} // namespace mme
