// conv_fwd_fast.hip -- forward convolution, bf16, 3 x 3 filter, 64 -> 64 channels, stride 1, padding 1 (the ResNet
// 3 x 3 layer of the benchmark configuration: N = 64, H = W = 56).
//
// Implicit GEMM like the general kernel (the im2col matrix of the reference, mme/mme_reference/im2col.cpp:55-91, is
// never built), but organised around what bounds this shape on MI355X: 14.8 GFLOP against 51 MB of compulsory
// traffic puts it within a factor of two of both rooflines, so every input pixel is fetched from memory once, every
// output is written once, and the fetches of the next tile run underneath the matrix-core work of the current one.
//
//   grid        persistent: one workgroup per compute unit (256 lanes = 4 wavefronts), each walking a contiguous run
//               of work units; a unit is 4 output rows x W columns of one image, all 64 output channels
//   LDS         the whole filter, transposed once per workgroup to Wt[out channel][tap * 64 + in channel] (16-byte
//               chunks XOR-swizzled by channel), and two input tiles with halo (6 rows x (W + 2) pixels x 64 channels,
//               16-byte chunks XOR-swizzled by column) filled by global->LDS DMA; pixels outside the image are
//               fetched from a 16-byte page of zeros
//   wavefront   pixel tiles of 32 (tile = wavefront, wavefront + 4), both 32-channel halves: per k-step of 16 channels
//               2 filter fragments + 2 pixel fragments feed 4 v_mfma_f32_32x32x16_bf16 (channels on the rows of the
//               accumulator tile, pixels on its columns, so that a lane ends up with runs of consecutive channels)
//   epilogue    v_permlane32_swap gathers 16 consecutive channels of one pixel per lane; power-of-two factor, relu,
//               cast (same converters as everywhere else), 16-byte stores
//
// Everything else (other filters, channel counts, strides, dtypes) runs on the general kernel.
#include "gemm_impl.hpp"

#include <algorithm>
#include <climits>
#include <type_traits>

namespace mme
{
namespace
{
constexpr int CF_C = 64, CF_K = 64, CF_TAPS = 9, CF_TR = 4;
constexpr int CF_WT_ROW = CF_TAPS * CF_C * 2; // bytes per output-channel row of the transposed filter
constexpr int CF_WT_BYTES = CF_K * CF_WT_ROW; // 73728
constexpr int CF_MAX_W = 56;                  // two halo tiles of 6 x (W + 2) x 128 B next to the filter in 160 KiB
constexpr int CF_MAX_DMA = 11;                // DMA requests per wavefront and tile: ceil(6 * 58 * 8 / 64 / 4)

__device__ __attribute__((aligned(16))) uint32_t cf_zero_page[4];

struct ConvFwdFastArgs
{
    const uint16_t* x;   // [B][H][W][64]
    const uint16_t* w;   // [3][3][64 in][64 out]
    int             B, H, W;
    GemmEpilogue    epi; // out = [B][H][W][64], ld = 64
};

// 16 bytes per lane from global memory to LDS at lds_off + lane * 16 (lds_off is wave-uniform).  Inline assembly keeps
// the request out of the compiler's memory model: it would otherwise order every later LDS read behind it.
__device__ __forceinline__ void cf_dma16(const void* g, uint32_t lds_off)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_off) : "memory");
}

typedef float    cf_v4f __attribute__((ext_vector_type(4)));
typedef uint32_t cf_v4u __attribute__((ext_vector_type(4)));

union CfFrag
{
    uint4 u;
    v8bf  v;
};

__global__ __launch_bounds__(256) void conv_fwd_fast_kernel(ConvFwdFastArgs a_by_value)
{
    (void) a_by_value;
    typedef const __attribute__((address_space(4))) ConvFwdFastArgs& ArgRef;
    ArgRef a = *(const __attribute__((address_space(4))) ConvFwdFastArgs*) __builtin_amdgcn_kernarg_segment_ptr();
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int H = a.H, W = a.W, wp = W + 2;
    const int row_tiles = (H + CF_TR - 1) / CF_TR;
    const int units = a.B * row_tiles;
    const int u_begin = (int) ((long long) blockIdx.x * units / gridDim.x), u_end = (int) ((long long) (blockIdx.x + 1) * units / gridDim.x);
    const int halo_chunks = (CF_TR + 2) * wp * 8;       // 16-byte chunks of one halo tile
    const int halo_bytes = halo_chunks * 16;
    const uint32_t lds_base = (uint32_t) (uintptr_t) lds; // LDS byte address of the dynamic segment
    char*          wt = lds;
    const uint32_t halo_base = CF_WT_BYTES;

    // ---- DMA plan of one halo tile: this lane's chunk in each of the wavefront's requests ------------------------------
    // LDS chunk q = (row * wp + col) * 8 + j holds input channels 8 * (j ^ ((col >> 1) & 7)) .. + 7 of halo pixel (row, col)
    int dma_rel[CF_MAX_DMA]; // element offset from the unit's first input pixel (row h0, column 0); INT_MIN: column outside
    int dma_row[CF_MAX_DMA]; // halo row 0 .. 5, -1: no chunk (tail of the last request)
#pragma unroll
    for (int j = 0; j < CF_MAX_DMA; j++)
    {
        const int q = (wave + 4 * j) * 64 + lane;
        const int pix = q >> 3, row = pix / wp, col = pix - row * wp;
        const int chunk = (q & 7) ^ ((col >> 1) & 7);
        dma_row[j] = q < halo_chunks ? row : -1;
        dma_rel[j] = (col >= 1 && col <= W) ? ((row - 1) * W + (col - 1)) * CF_C + chunk * 8 : INT_MIN;
    }
    auto issue_halo = [&](int u, int buf) __attribute__((always_inline))
    {
        const int       img = u / row_tiles, h0 = (u - img * row_tiles) * CF_TR;
        const uint16_t* org = a.x + ((size_t) img * H + h0) * W * CF_C;
#pragma unroll
        for (int j = 0; j < CF_MAX_DMA; j++)
        {
            const int   h = h0 - 1 + dma_row[j];
            const bool  inside = dma_rel[j] != INT_MIN && h >= 0 && h < H;
            const void* src = inside ? (const void*) (org + dma_rel[j]) : (const void*) cf_zero_page;
            if (dma_row[j] >= 0) cf_dma16(src, lds_base + halo_base + buf * halo_bytes + (wave + 4 * j) * 1024);
        }
    };
    if (u_begin < u_end) issue_halo(u_begin, 0);

    // ---- filter: global [tap][c][k] (k contiguous) -> LDS [k][tap * 64 + c]; 8 x 8 blocks transposed in registers ----
#pragma unroll
    for (int it = 0; it < 3; it++)
    {
        const int blk = tid + it * 256;
        if (blk < (CF_TAPS * CF_C / 8) * (CF_K / 8))
        {
            const int kb = blk & 7, cb = blk >> 3; // cb: block of 8 consecutive (tap, c) rows; kb: block of 8 output channels
            uint4     in[8], out[8];
#pragma unroll
            for (int i = 0; i < 8; i++) in[i] = *reinterpret_cast<const uint4*>(a.w + (size_t) (cb * 8 + i) * CF_K + kb * 8);
            transpose_block<2>(in, out);
#pragma unroll
            for (int j = 0; j < 8; j++) *reinterpret_cast<uint4*>(wt + (kb * 8 + j) * CF_WT_ROW + (cb ^ j) * 16) = out[j];
        }
    }

    // ---- per-lane constants of the contraction -------------------------------------------------------------------------
    const int kg = lane >> 5;
    // filter fragment: row = output channel n * 32 + lane % 32, chunk = tap * 8 + ks * 2 + kg, swizzled by channel & 7
    int wt_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) wt_off[ks] = (lane & 31) * CF_WT_ROW + (((ks * 2 + kg) ^ (lane & 7)) << 4);
    // pixel fragment: this lane's pixel in each of the wavefront's two tiles (clamped into the tile's 4 rows)
    int px_off[2][3][4]; // [tile][s][ks]: byte offset of the chunk in halo row r = 0
#pragma unroll
    for (int t = 0; t < 2; t++)
    {
        int p = (wave + 4 * t) * 32 + (lane & 31);
        p = min(p, CF_TR * W - 1);
        const int prow = p / W, pcol = p - prow * W;
#pragma unroll
        for (int s = 0; s < 3; s++)
#pragma unroll
            for (int ks = 0; ks < 4; ks++)
                px_off[t][s][ks] = ((prow * wp + pcol + s) * 8 + ((ks * 2 + kg) ^ (((pcol + s) >> 1) & 7))) * 16;
    }
    const int row_pitch = wp * 128;

    const bool       fused = a.epi.fused != 0;
    const bool       has_alpha = a.epi.has_alpha != 0;
    const float      alpha = a.epi.alpha;
    const int32_t*   col_exp = a.epi.col_exp;
    const int        dt = fused ? a.epi.out_dtype : DT_FP32;
    const bool       bf16_fast = fused && dt == DT_BF16 && a.epi.fast_cast;
    const CastParams cp = {a.epi.cast.dtype,       a.epi.cast.exp_bias, a.epi.cast.inf_nan_mode, a.epi.cast.rm,    a.epi.cast.clip_fp,
                           a.epi.cast.clip_inf_in, a.epi.cast.ftz,      a.epi.cast.relu,         a.epi.cast.scale, a.epi.cast.has_scale};

    for (int u = u_begin; u < u_end; u++)
    {
        const int buf = (u - u_begin) & 1;
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wavefront's share of the tile has landed
        __syncthreads();                    // ... and everybody else's; nobody still reads the other buffer
        if (u + 1 < u_end) issue_halo(u + 1, buf ^ 1);

        const int   img = u / row_tiles, h0 = (u - img * row_tiles) * CF_TR;
        const int   npix = min(CF_TR, H - h0) * W, ntiles = (npix + 31) >> 5;
        const char* halo = lds + halo_base + buf * halo_bytes;
        const bool  two = wave + 4 < ntiles;
        if (wave >= ntiles) continue;

        v16f acc[2][2];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int n = 0; n < 2; n++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[t][n][v] = 0.0f;

        // k-steps 0 .. 35 = (tap, 16 input channels); the fragments of step i + 1 are fetched between the matrix-core
        // instructions of step i (the scheduling barriers pin that order, the compiler derives the LDS waits from it)
        auto contract = [&](auto nt_c) __attribute__((always_inline))
        {
            constexpr int NT = decltype(nt_c)::value;
            CfFrag        fw[2][2], fx[2][2];
            auto ld_w = [&](int slot, int n, int step) __attribute__((always_inline))
            {
                const int tap = step >> 2, ks = step & 3;
                fw[slot][n].u = *reinterpret_cast<const uint4*>(wt + wt_off[ks] + n * 32 * CF_WT_ROW + tap * 128);
            };
            auto ld_x = [&](int slot, int t, int step) __attribute__((always_inline))
            {
                const int tap = step >> 2, ks = step & 3, r = tap / 3, s = tap - r * 3;
                fx[slot][t].u = *reinterpret_cast<const uint4*>(halo + px_off[t][s][ks] + r * row_pitch);
            };
            auto mm = [&](int slot, int t, int n) __attribute__((always_inline))
            {
                acc[t][n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[slot][n].v, fx[slot][t].v, acc[t][n], 0, 0, 0);
            };
            ld_w(0, 0, 0);
            ld_x(0, 0, 0);
            ld_w(0, 1, 0);
            if (NT == 2) ld_x(0, 1, 0);
#pragma unroll
            for (int step = 0; step < CF_TAPS * 4; step++)
            {
                const int  cur = step & 1, nxt = cur ^ 1;
                const bool more = step + 1 < CF_TAPS * 4;
                if constexpr (NT == 2)
                {
                    if (more) ld_w(nxt, 0, step + 1);
                    mm(cur, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if (more) ld_x(nxt, 0, step + 1);
                    mm(cur, 0, 1);
                    __builtin_amdgcn_sched_barrier(0);
                    if (more) ld_w(nxt, 1, step + 1);
                    mm(cur, 1, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if (more) ld_x(nxt, 1, step + 1);
                    mm(cur, 1, 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
                else
                {
                    if (more) ld_w(nxt, 0, step + 1);
                    if (more) ld_x(nxt, 0, step + 1);
                    mm(cur, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if (more) ld_w(nxt, 1, step + 1);
                    mm(cur, 0, 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        if (two) contract(std::integral_constant<int, 2>());
        else
            contract(std::integral_constant<int, 1>());

        // ---- epilogue: accumulator register v of lane l = channel n * 32 + 8 * (v / 4) + 4 * (l / 32) + v % 4 of pixel l % 32 --
        const long long unit_base = ((long long) img * H + h0) * W * CF_K; // element offset of the unit's first output pixel
#pragma unroll
        for (int t = 0; t < 2; t++)
        {
            if (t == 1 && !two) break;
            const int  p = (wave + 4 * t) * 32 + (lane & 31);
            const bool live = p < npix;
#pragma unroll
            for (int n = 0; n < 2; n++)
            {
                // after the exchange the lane holds channels n * 32 + kg * 16 + 0 .. 15 of its pixel, in order
                float val[16];
#pragma unroll
                for (int g = 0; g < 2; g++)
#pragma unroll
                    for (int i = 0; i < 4; i++)
                    {
                        const float lo = acc[t][n][4 * g + i], hi = acc[t][n][8 + 4 * g + i];
                        const auto  sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
                        val[8 * g + i] = __uint_as_float(sw[0]);
                        val[8 * g + 4 + i] = __uint_as_float(sw[1]);
                    }
                const int ch0 = n * 32 + kg * 16;
#pragma unroll
                for (int c = 0; c < 16; c++)
                {
                    if (has_alpha) val[c] *= alpha;
                    if (col_exp) val[c] *= pow2_of(col_exp[ch0 + c]);
                }
                if (!live) continue;
                const long long idx = unit_base + (long long) p * CF_K + ch0;
                if (!fused)
                {
                    cf_v4f* o = (cf_v4f*) ((float*) a.epi.out + idx);
#pragma unroll
                    for (int c = 0; c < 4; c++) o[c] = cf_v4f {val[4 * c], val[4 * c + 1], val[4 * c + 2], val[4 * c + 3]};
                }
                else if (bf16_fast)
                {
                    uint32_t pk[8];
#pragma unroll
                    for (int c = 0; c < 8; c++)
                        pk[c] = (uint32_t) cast_elem<DT_BF16, true>(val[2 * c], cp) | ((uint32_t) cast_elem<DT_BF16, true>(val[2 * c + 1], cp) << 16);
                    cf_v4u* o = (cf_v4u*) ((uint16_t*) a.epi.out + idx);
                    o[0] = cf_v4u {pk[0], pk[1], pk[2], pk[3]};
                    o[1] = cf_v4u {pk[4], pk[5], pk[6], pk[7]};
                }
                else
                {
#pragma unroll 1
                    for (int c = 0; c < 16; c++) store_out_slow(a.epi, idx + c, val[c]);
                }
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
}
} // namespace

bool conv_fwd_fast_applicable(int dtype, int C, int K, int S, int R, int Q, int W, int H, int D, const int stride[4], const int dil[4],
                              const int pad[4], bool dense)
{
    if (dtype != DT_BF16 || !dense) return false;
    if (C != CF_C || K != CF_K || S != 3 || R != 3 || Q != 1 || D != 1) return false;
    for (int d = 0; d < 4; d++)
        if (stride[d] != 1 || dil[d] != 1) return false;
    if (pad[0] != 1 || pad[1] != 1 || pad[2] != 0 || pad[3] != 0) return false;
    if (W < 1 || W > CF_MAX_W || H < 1) return false;
    return true;
}

hipError_t launch_conv_fwd_fast(const void* x, const void* w, int B, int H, int W, const GemmEpilogue& epi, int num_cus, hipStream_t s)
{
    static bool attr_done = false;
    const int   lds_bytes = CF_WT_BYTES + 2 * (CF_TR + 2) * (W + 2) * 128;
    if (!attr_done)
    {
        hipError_t e = hipFuncSetAttribute((const void*) conv_fwd_fast_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_done = true;
    }
    ConvFwdFastArgs a;
    a.x = (const uint16_t*) x;
    a.w = (const uint16_t*) w;
    a.B = B;
    a.H = H;
    a.W = W;
    a.epi = epi;
    const long long units = (long long) B * ((H + CF_TR - 1) / CF_TR);
    if (units > 0x7fffffffLL) return hipErrorInvalidValue;
    const int grid = (int) std::min<long long>(units, num_cus > 0 ? num_cus : 256);
    hipLaunchKernelGGL(conv_fwd_fast_kernel, dim3(grid), dim3(256), lds_bytes, s, a);
    return hipGetLastError();
}

} // namespace mme
