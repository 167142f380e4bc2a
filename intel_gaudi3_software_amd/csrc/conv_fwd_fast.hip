// conv_fwd_fast.hip -- forward convolution, bf16, 3 x 3 filter, 64 -> 64 channels, stride 1, padding 1 (the ResNet
// 3 x 3 layer of the benchmark configuration: N = 64, H = W = 56).
//
// Implicit GEMM like the general kernel (the im2col matrix of the reference, mme/mme_reference/im2col.cpp:55-91, is
// never built), but organised around what bounds this shape on MI355X: 14.8 GFLOP against 51 MB of compulsory
// traffic puts it within a factor of two of both rooflines, so every input pixel is fetched from memory once, every
// output is written once, and the fetches of the next tile run underneath the matrix-core work of the current one.
//
//   grid        persistent: one workgroup of 512 lanes per compute unit, owning a contiguous run of output rows (row
//               index = image * H + row) cut into units of up to 4 rows of one image.  The 8 wavefronts form two teams
//               of four (one wavefront of each team per SIMD) that take the units alternately: a wavefront cannot
//               issue anything else while its own matrix-core instruction occupies it, so the second team's
//               wavefront on the SIMD is what fills the matrix cores during the first team's loads, stores, waits and
//               epilogue arithmetic.  Teams synchronise among themselves through counters in LDS, not s_barrier
//   LDS         the whole filter in its global order (row = tap * 64 + in channel, 64 out channels each), fetched once
//               per workgroup by global->LDS DMA and read with the transposing ds_read_b64_tr_b16; one input tile with
//               halo per team (6 rows x (W + 2) pixels x 64 channels, 16-byte chunks XOR-swizzled by column), also by
//               DMA, requested as soon as the team has finished with its previous tile.  The halo columns are zeroed
//               once; rows outside the image are fetched from a 16-byte page of zeros
//   wavefront   pixel tiles of 32 (tile = wavefront in team, + 4), both 32-channel halves: per k-step of 16 channels
//               2 filter fragments + 2 pixel fragments, fetched one step ahead, feed 4 v_mfma_f32_32x32x16_bf16
//               (channels on the rows of the accumulator tile, pixels on its columns, so that a lane ends up with
//               runs of consecutive channels)
//   epilogue    v_permlane32_swap gathers 16 consecutive channels of one pixel per lane; power-of-two factor, relu,
//               cast (v_cvt_pk_bf16_f32 where it equals the reference's conversion, the shared converters
//               otherwise), 16-byte stores
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
constexpr int CF_MAX_DMA = 11;                // DMA requests per wavefront and tile: ceil(6 * 58 * 8 / 64 / 4)
constexpr int CF_MAX_W = 56;                  // two halo tiles of 6 x (W + 2) x 128 B next to the filter in 160 KiB

__device__ __attribute__((aligned(16))) uint32_t cf_zero_page[4];

struct ConvFwdFastArgs
{
    const uint16_t* x;   // [B][H][W][64]
    const uint16_t* w;   // [3][3][64 in][64 out]
    int             B, H, W;
    int             rows_per_wg, rows_extra; // B * H output rows = gridDim.x * rows_per_wg + rows_extra (the first rows_extra workgroups take one more)
    GemmEpilogue    epi; // out = [B][H][W][64], ld = 64
    // waits on LDS counters are bounded: after wait_limit polls a wavefront writes CF_GAVE_UP to *status (host-visible
    // memory of the calculator) and goes on, so that a slip in the hand-over logic ends in an error report, not in a hang
    uint32_t*       status;
    uint32_t        wait_limit;
};
constexpr uint32_t CF_GAVE_UP = 0x57414954u; // "WAIT"

__device__ __forceinline__ void cf_wait_for(uint32_t* counter, uint32_t target, uint32_t limit, uint32_t* status)
{
    uint32_t polls = 0;
    while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < target)
    {
        if (polls++ >= limit)
        {
            *status = CF_GAVE_UP;
            break;
        }
        __builtin_amdgcn_s_sleep(1);
    }
}

// 16 bytes per lane from global memory to LDS at lds_off + lane * 16 (lds_off is wave-uniform).  Inline assembly keeps
// the request out of the compiler's memory model: it would otherwise order every later LDS read behind it.
__device__ __forceinline__ void cf_dma16(const void* g, uint32_t lds_off)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_off) : "memory");
}

// the same with the global address given as a wave-uniform base plus a 32-bit byte offset per lane
__device__ __forceinline__ void cf_dma16_off(const void* base, uint32_t off, uint32_t lds_off)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds_off) : "memory");
}

// The arguments are read in place from the kernarg segment where the code needs them; one scalar load per 64-byte line up
// front takes the misses of all lines at once instead of one memory latency each at set-up and in the first epilogue.
__device__ __forceinline__ void cf_warm_kernargs(const __attribute__((address_space(4))) ConvFwdFastArgs& a)
{
    static_assert(sizeof(ConvFwdFastArgs) > 128 && sizeof(ConvFwdFastArgs) <= 192, "three 64-byte lines");
    uint32_t t0, t1, t2;
    asm volatile("s_load_dword %0, %3, 0x0\n\t"
                 "s_load_dword %1, %3, 0x40\n\t"
                 "s_load_dword %2, %3, 0x80\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&s"(t0), "=&s"(t1), "=&s"(t2)
                 : "s"(&a)
                 : "memory");
}

typedef float    cf_v4f __attribute__((ext_vector_type(4)));
typedef uint32_t cf_v4u __attribute__((ext_vector_type(4)));
typedef float    cf_v2f __attribute__((ext_vector_type(2)));
typedef __bf16   cf_v2bf __attribute__((ext_vector_type(2)));

typedef short cf_v4s __attribute__((ext_vector_type(4)));
#define CF_LDS __attribute__((address_space(3)))

union CfFrag
{
    uint4  u;
    v8bf   v;
    cf_v4s h[2];
};

// n / d for 0 <= n < 2^20, 0 < d < 2^10 without the integer-division sequence: a float estimate, corrected by one
__device__ __forceinline__ int cf_div(int n, int d)
{
    int q = (int) ((float) n * __builtin_amdgcn_rcpf((float) d));
    const int r = n - q * d;
    q += (r >= d) - (r < 0);
    return q;
}

// Barrier among the four wavefronts of a team: a counter in LDS that only grows.  (s_barrier would stop the other team
// too.)  Every wavefront of the team reaches every barrier, so the wait ends; it is bounded all the same (cf_wait_for).
__device__ __forceinline__ void cf_team_barrier(uint32_t* counter, uint32_t target, int lane, uint32_t limit, uint32_t* status)
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if (lane == 0) __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    cf_wait_for(counter, target, limit, status);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

__global__ __launch_bounds__(512) void conv_fwd_fast_kernel(ConvFwdFastArgs a_by_value)
{
    (void) a_by_value;
    typedef const __attribute__((address_space(4))) ConvFwdFastArgs& ArgRef;
    ArgRef a = *(const __attribute__((address_space(4))) ConvFwdFastArgs*) __builtin_amdgcn_kernarg_segment_ptr();
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int team = wave >> 2, tw = wave & 3; // two teams of four wavefronts, one of each team per SIMD
    const int H = a.H, W = a.W, wp = W + 2;
    // this workgroup's run of output rows (row index = image * H + row); a unit is up to 4 of them inside one image;
    // the teams take the units of the run alternately
    const int       row_begin = blockIdx.x * a.rows_per_wg + min((int) blockIdx.x, a.rows_extra);
    const int       row_end = row_begin + a.rows_per_wg + ((int) blockIdx.x < a.rows_extra ? 1 : 0);
    const int       halo_bytes = (CF_TR + 2) * wp * 128;
    const uint32_t  lds_base = (uint32_t) (uintptr_t) lds; // LDS byte address of the dynamic segment
    const char*     wt = lds;
    const uint32_t  halo_off = CF_WT_BYTES + team * halo_bytes; // this team's input tile
    const char*     halo = lds + halo_off;
    uint32_t*       counter = (uint32_t*) (lds + CF_WT_BYTES + 2 * halo_bytes) + team;
    if (tid < 2) ((uint32_t*) (lds + CF_WT_BYTES + 2 * halo_bytes))[tid] = 0;

    // ---- input tile with halo by DMA: request i moves LDS chunks 64 * i .. 64 * i + 63, one per lane; wavefront tw of the
    // team issues requests tw, tw + 4, ...  LDS chunk q = (row * wp + col) * 8 + j holds input channels
    // 8 * (j ^ ((col >> 1) & 7)) .. + 7 of halo pixel (row, col) ----------------------------------------------------------
    int dma_rel[CF_MAX_DMA]; // byte offset from the input pixel (row h0 - 1, column 0) of the unit; -1: no chunk to fetch
    int dma_row[CF_MAX_DMA]; // halo row 0 .. 5 (beyond: no such chunk)
    {
        // request j covers halo pixels 32 j + 8 tw + lane / 8: row and column advance incrementally
        int row = cf_div(tw * 8 + (lane >> 3), wp), col = tw * 8 + (lane >> 3) - row * wp;
#pragma unroll
        for (int j = 0; j < CF_MAX_DMA; j++)
        {
            const int chunk = (lane & 7) ^ ((col >> 1) & 7);
            dma_row[j] = row;
            dma_rel[j] = (col >= 1 && col <= W && row < CF_TR + 2) ? ((row * W + (col - 1)) * CF_C + chunk * 8) * 2 : -1;
            col += 32;
            if (wp >= 32)
            {
                const int wrap = col >= wp;
                col -= wrap ? wp : 0;
                row += wrap;
            }
            else
            {
                const int k = cf_div(col, wp);
                col -= k * wp;
                row += k;
            }
        }
    }
    // the halo columns are never fetched: they are zeroed here once, in both tiles
    for (int i = tid; i < 2 * (CF_TR + 2) * 2 * 8; i += 512)
    {
        const int chunk = i & 7, side = (i >> 3) & 1, row = (i >> 4) % (CF_TR + 2), b = (i >> 4) / (CF_TR + 2);
        *reinterpret_cast<uint4*>(lds + CF_WT_BYTES + b * halo_bytes + ((row * wp + (side ? W + 1 : 0)) * 8 + chunk) * 16) = make_uint4(0, 0, 0, 0);
    }
    // A unit whose six halo rows all lie inside the image fetches them all (also those a short unit does not need) with
    // one address per request; a unit at the upper or lower border fetches the missing rows from a page of zeros
    auto issue_halo = [&](int img_, int h0_, int nrows_) __attribute__((always_inline))
    {
        const uint16_t* org = a.x + ((long long) img_ * H + h0_ - 1) * W * CF_C; // input pixel (row h0_ - 1, column 0)
        if (h0_ >= 1 && h0_ + CF_TR + 1 <= H)
        {
#pragma unroll
            for (int j = 0; j < CF_MAX_DMA; j++)
                if (dma_rel[j] >= 0) cf_dma16_off(org, (uint32_t) dma_rel[j], lds_base + halo_off + (tw + 4 * j) * 1024);
        }
        else
        {
#pragma unroll
            for (int j = 0; j < CF_MAX_DMA; j++)
            {
                const int   h = h0_ - 1 + dma_row[j];
                const void* src = (h >= 0 && h < H) ? (const void*) ((const char*) org + dma_rel[j]) : (const void*) cf_zero_page;
                if (dma_rel[j] >= 0 && dma_row[j] < nrows_ + 2) cf_dma16(src, lds_base + halo_off + (tw + 4 * j) * 1024);
            }
        }
    };
    // the team's current unit; advance() steps to the next unit of the run (one call per unit skipped or done)
    int  row = row_begin, img = row_begin / H, h0 = row_begin - img * H, nrows = min(CF_TR, min(H - h0, row_end - row_begin));
    auto advance = [&]() __attribute__((always_inline))
    {
        row += nrows;
        h0 += nrows;
        if (h0 >= H)
        {
            h0 = 0;
            img++;
        }
        nrows = min(CF_TR, min(H - h0, row_end - row));
    };
    if (team == 1) advance();
    if (row < row_end) issue_halo(img, h0, nrows);

    // ---- filter by DMA in its global order: row R = tap * 64 + in channel (128 bytes = 64 out channels), the 32-byte
    // blocks of a row XOR-swizzled by R & 3 so that the transposing reads below touch every bank once.  Each wavefront
    // moves 9 KiB; one M0 setting serves four requests through the instruction offset, which advances the global and the
    // LDS address alike ---------------------------------------------------------------------------------------------------
    {
        constexpr int PER_WAVE = CF_WT_BYTES / 1024 / 8;
        const char*   src = (const char*) a.w + (((lane & ~7) | ((lane & 7) ^ (((lane >> 3) & 3) << 1))) << 4) + wave * (PER_WAVE * 1024);
#pragma unroll
        for (int k = 0; k < PER_WAVE; k += 4)
        {
            const char*    g = src + k * 1024;
            const uint32_t l = lds_base + wave * (PER_WAVE * 1024) + k * 1024;
            if (k + 4 <= PER_WAVE)
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off\n\tglobal_load_lds_dwordx4 %0, off offset:1024\n\t"
                             "global_load_lds_dwordx4 %0, off offset:2048\n\tglobal_load_lds_dwordx4 %0, off offset:3072" ::"v"(g), "s"(l)
                             : "memory");
            else
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(l) : "memory");
        }
    }

    // ---- per-lane constants of the contraction -------------------------------------------------------------------------
    const int kg = lane >> 5;
    // filter fragment (matrix-core rows = out channels n * 32 + lane % 32, k = in channels 8 * kg .. + 7 of the k-step):
    // two ds_read_b64_tr_b16, each handing a lane one out channel of 4 consecutive filter rows; within a group of 16
    // lanes, lane j addresses the 8-byte piece j % 4 of row j / 4
    int wl_off[2];
    {
        const int g = lane >> 4, j = lane & 15;
#pragma unroll
        for (int n = 0; n < 2; n++) wl_off[n] = ((g >> 1) * 8 + (j >> 2)) * 128 + (((n * 2 + (g & 1)) ^ (j >> 2)) << 5) + ((j & 3) << 3);
    }
    // pixel fragment: this lane's pixel in each of the wavefront's two tiles (clamped into the tile's 4 rows)
    int px_off[2][3][4]; // [tile][s][ks]: byte offset of the chunk in halo row r = 0
#pragma unroll
    for (int t = 0; t < 2; t++)
    {
        int p = (tw + 4 * t) * 32 + (lane & 31);
        p = min(p, CF_TR * W - 1);
        const int prow = cf_div(p, W), pcol = p - prow * W;
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
    const bool       scaled = has_alpha || col_exp != nullptr;
    const CastParams cp = {a.epi.cast.dtype,       a.epi.cast.exp_bias, a.epi.cast.inf_nan_mode, a.epi.cast.rm,    a.epi.cast.clip_fp,
                           a.epi.cast.clip_inf_in, a.epi.cast.ftz,      a.epi.cast.relu,         a.epi.cast.scale, a.epi.cast.has_scale};

    // the filter and both teams' first tiles have landed for everybody
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

    uint32_t barriers = 0;     // team barriers passed so far
    int      stores_in_flight = 0; // wave-uniform: 16-byte store instructions issued after the latest DMA requests
    bool     first = true;
    while (row < row_end)
    {
        if (!first)
        {
            // this wavefront's DMA requests for the unit were issued before the previous unit's stores, and vector memory
            // operations retire in issue order: that many stores may still be in flight when the requests have landed
            if (stores_in_flight == 16) __builtin_amdgcn_s_waitcnt(0x4F70);
            else if (stores_in_flight == 8)
                __builtin_amdgcn_s_waitcnt(0x0F78);
            else if (stores_in_flight == 4)
                __builtin_amdgcn_s_waitcnt(0x0F74);
            else
                __builtin_amdgcn_s_waitcnt(0x0F70);
            cf_team_barrier(counter, 4 * ++barriers, lane, a.wait_limit, a.status); // ... and the other three wavefronts' requests as well
        }
        first = false;
        stores_in_flight = 0;

        const int       npix = nrows * W, ntiles = (npix + 31) >> 5;
        const bool      two = tw + 4 < ntiles;
        const long long unit_base = ((long long) img * H + h0) * W * CF_K; // element offset of the unit's first output pixel

        v16f acc[2][2];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int n = 0; n < 2; n++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[t][n][v] = 0.0f;

        // k-steps 0 .. 35 = (tap, 16 input channels); the fragments of step i + 1 are fetched between the matrix-core
        // instructions of step i (the scheduling barriers pin that order, the compiler derives the LDS waits from it);
        // the other team's wavefront on this SIMD fills the issue slots this one leaves open
        auto contract = [&](auto nt_c) __attribute__((always_inline))
        {
            constexpr int NT = decltype(nt_c)::value;
            constexpr int NS = CF_TAPS * 4, AHEAD = 1, RING = AHEAD + 1;
            CfFrag        fw[RING][2], fx[RING][2];
            auto ld_w = [&](int slot, int n, int step) __attribute__((always_inline))
            {
                const int   tap = step >> 2, ks = step & 3;
                const char* p = wt + wl_off[n] + tap * 8192 + ks * 2048;
                fw[slot][n].h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((CF_LDS cf_v4s*) p);
                fw[slot][n].h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((CF_LDS cf_v4s*) (p + 512));
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
#pragma unroll
            for (int step = 0; step < AHEAD; step++)
            {
                ld_w(step, 0, step);
                ld_x(step, 0, step);
                ld_w(step, 1, step);
                if (NT == 2) ld_x(step, 1, step);
            }
#pragma unroll
            for (int step = 0; step < NS; step++)
            {
                const int  cur = step % RING, nxt = (step + AHEAD) % RING;
                const bool more = step + AHEAD < NS;
                if constexpr (NT == 2)
                {
                    if (more) ld_w(nxt, 0, step + AHEAD);
                    mm(cur, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if (more) ld_x(nxt, 0, step + AHEAD);
                    mm(cur, 0, 1);
                    __builtin_amdgcn_sched_barrier(0);
                    if (more) ld_w(nxt, 1, step + AHEAD);
                    mm(cur, 1, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if (more) ld_x(nxt, 1, step + AHEAD);
                    mm(cur, 1, 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
                else
                {
                    if (more) ld_w(nxt, 0, step + AHEAD);
                    if (more) ld_x(nxt, 0, step + AHEAD);
                    mm(cur, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if (more) ld_w(nxt, 1, step + AHEAD);
                    mm(cur, 0, 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        if (tw < ntiles)
        {
            if (two) contract(std::integral_constant<int, 2>());
            else
                contract(std::integral_constant<int, 1>());
        }

        // the team is done with its tile: fetch the tile of its next unit (two units further down the run) underneath
        // the epilogue and the other team's contraction
        const int  img_done = img, h0_done = h0;
        (void) img_done;
        (void) h0_done;
        advance();
        if (row < row_end) advance();
        cf_team_barrier(counter, 4 * ++barriers, lane, a.wait_limit, a.status);
        if (row < row_end) issue_halo(img, h0, nrows);
        if (tw >= ntiles) continue;

        // ---- epilogue: accumulator register v of lane l = channel n * 32 + 8 * (v / 4) + 4 * (l / 32) + v % 4 of pixel
        // l % 32; one v_permlane32_swap per register pair leaves the lane with channels n * 32 + kg * 16 + 0 .. 15 in order --
        auto gather = [&](int t, int n, float (&val)[16]) __attribute__((always_inline))
        {
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
            if (has_alpha)
            {
#pragma unroll
                for (int c = 0; c < 16; c++) val[c] *= alpha;
            }
            if (col_exp)
            {
#pragma unroll
                for (int c = 0; c < 16; c++) val[c] *= pow2_of(col_exp[n * 32 + kg * 16 + c]);
            }
        };
#pragma unroll
        for (int t = 0; t < 2; t++)
        {
            if (t == 1 && !two) break;
            const int p = (tw + 4 * t) * 32 + (lane & 31);
#pragma unroll
            for (int n = 0; n < 2; n++)
            {
                float val[16];
                gather(t, n, val);
                const long long idx = unit_base + (long long) p * CF_K + n * 32 + kg * 16;
                if (bf16_fast)
                {
                    // bf16, round to nearest even: v_cvt_pk_bf16_f32 gives the reference's code for every input except NaN
                    // (checked over all 2^32 inputs); NaN, inf and values that round to inf (where clipping matters) are
                    // rare: the sum of |x| over the lane's 16 values detects them and the block is then converted element
                    // by element
                    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int c = 0; c < 16; c++)
                    {
                        if (cp.relu) val[c] = relu_ref(val[c]);
                        sum[c & 3] += __builtin_fabsf(val[c]);
                    }
                    const bool special = !((sum[0] + sum[1]) + (sum[2] + sum[3]) < 0x1.ffp+127f);
                    uint32_t   pk[8];
                    if (__builtin_amdgcn_ballot_w64(special) == 0)
                    {
#pragma unroll
                        for (int c = 0; c < 8; c++)
                        {
                            const cf_v2bf h = __builtin_convertvector(cf_v2f {val[2 * c], val[2 * c + 1]}, cf_v2bf);
                            __builtin_memcpy(&pk[c], &h, 4);
                        }
                    }
                    else
                    {
#pragma unroll
                        for (int c = 0; c < 8; c++)
                            pk[c] = fp32_to_bf16_rne(f2u(val[2 * c]), cp.clip_fp, cp.clip_inf_in) |
                                    (fp32_to_bf16_rne(f2u(val[2 * c + 1]), cp.clip_fp, cp.clip_inf_in) << 16);
                    }
                    if (p < npix)
                    {
                        cf_v4u* o = (cf_v4u*) ((uint16_t*) a.epi.out + idx);
                        o[0] = cf_v4u {pk[0], pk[1], pk[2], pk[3]};
                        o[1] = cf_v4u {pk[4], pk[5], pk[6], pk[7]};
                    }
                }
                else if (p < npix)
                {
                    if (!fused)
                    {
                        cf_v4f* o = (cf_v4f*) ((float*) a.epi.out + idx);
#pragma unroll
                        for (int c = 0; c < 4; c++) o[c] = cf_v4f {val[4 * c], val[4 * c + 1], val[4 * c + 2], val[4 * c + 3]};
                    }
                    else
                    {
#pragma unroll 1
                        for (int c = 0; c < 16; c++) store_out_slow(a.epi, idx + c, val[c]);
                    }
                }
            }
        }
        stores_in_flight = !fused ? (two ? 16 : 8) : bf16_fast ? (two ? 8 : 4) : 0;
        (void) scaled;
    }
}

// ---------------------------------------------------------------------------------------------------------------------
// Resident form, for runs of output rows whose input fits in LDS at once (the benchmark shape: 14 rows of 56 pixels per
// compute unit).  Nothing is fetched twice and nothing waits in the steady state:
//
//   LDS         every input row the workgroup's run needs ("virtual rows": per image segment of the run its rows plus
//               the one above and the one below, rows outside the image as zeros), (W + 2) pixels each with zeroed
//               halo columns, 16-byte chunks XOR-swizzled by column as above.  All of it is requested in the first
//               microseconds, in row order, so the memory system streams the input while the first tiles are computed
//   filter      lives in registers: a wavefront owns output channels nh * 32 .. + 31 (nh = wavefront & 1) and keeps their 36 k-step
//               fragments (144 registers).  The filter passes through the top 72 KiB of LDS once (DMA in global order,
//               transposing reads); input rows that overlap that area are requested after every wavefront has taken
//               its fragments
//   wavefront   takes pairs of pixel tiles (64 pixels of the run's flattened pixel order) from a queue in LDS, one queue
//               per channel half, in row order: two independent accumulator chains, one ds_read_b128 per matrix-core
//               instruction, fetched five instructions ahead; the epilogue of a pair follows its contraction
//               immediately, which spreads the stores over the whole kernel, and the queue lets the wavefront that
//               gets more of its SIMD's matrix-core time take more pairs
//   sync        two workgroup barriers (filter landed, filter taken and first rows landed); the remaining rows are
//               requested by the second wavefront of every SIMD, which waits for them and raises a counter that the
//               others check before the first pair that needs those rows
constexpr int CR_LDS_BYTES = 160 * 1024;
constexpr int CR_CTRL_OFF = CR_LDS_BYTES - 16;           // three counters: the two tile queues, "all rows landed"
constexpr int CR_STAGE_OFF = CR_CTRL_OFF - CF_WT_BYTES;  // filter staging area: the top of LDS below the counters
constexpr int CR_MAX_TILES = 32;

// number of virtual rows of a run of `rows` output rows that starts at row hs0 of an image of H rows
__host__ __device__ inline int cr_virtual_rows(int rows, int hs0, int H)
{
    const int n0 = rows < H - hs0 ? rows : H - hs0;
    const int rest = rows - n0, full = rest / H, last = rest - full * H;
    return n0 + 2 + full * (H + 2) + (last ? last + 2 : 0);
}

// s_waitcnt vmcnt(n) for a wave-uniform n (the instruction takes an immediate); counts above 15 wait for 15
__device__ __forceinline__ void cr_wait_vmcnt(int n)
{
    switch (n)
    {
        case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;
        case 1: __builtin_amdgcn_s_waitcnt(0x0F71); break;
        case 2: __builtin_amdgcn_s_waitcnt(0x0F72); break;
        case 3: __builtin_amdgcn_s_waitcnt(0x0F73); break;
        case 4: __builtin_amdgcn_s_waitcnt(0x0F74); break;
        case 5: __builtin_amdgcn_s_waitcnt(0x0F75); break;
        case 6: __builtin_amdgcn_s_waitcnt(0x0F76); break;
        case 7: __builtin_amdgcn_s_waitcnt(0x0F77); break;
        case 8: __builtin_amdgcn_s_waitcnt(0x0F78); break;
        case 9: __builtin_amdgcn_s_waitcnt(0x0F79); break;
        case 10: __builtin_amdgcn_s_waitcnt(0x0F7A); break;
        case 11: __builtin_amdgcn_s_waitcnt(0x0F7B); break;
        case 12: __builtin_amdgcn_s_waitcnt(0x0F7C); break;
        case 13: __builtin_amdgcn_s_waitcnt(0x0F7D); break;
        case 14: __builtin_amdgcn_s_waitcnt(0x0F7E); break;
        default:
            if (n < 0) __builtin_amdgcn_s_waitcnt(0x0F70);
            else
                __builtin_amdgcn_s_waitcnt(0x0F7F);
            break;
    }
}

template<int WC> // WC: the image width when it is known at compile time (row pitch and pixel divisions become constants), else 0
__global__ __launch_bounds__(512) void conv_fwd_resident_kernel(ConvFwdFastArgs a_by_value)
{
    (void) a_by_value;
    typedef const __attribute__((address_space(4))) ConvFwdFastArgs& ArgRef;
    ArgRef a = *(const __attribute__((address_space(4))) ConvFwdFastArgs*) __builtin_amdgcn_kernarg_segment_ptr();
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    cf_warm_kernargs(a);

    const int      tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int      nh = wave & 1, kg = lane >> 5;
    const uint32_t lds_base = (uint32_t) (uintptr_t) lds;
    uint32_t*      ctrl = (uint32_t*) (lds + CR_CTRL_OFF);
    if (tid < 4) ctrl[tid] = 0;

    // ---- filter to the staging area, first of all: its addresses need no arithmetic --------------------------------------
    {
        // (the workgroups that share an L2 -- every eighth -- start at different eighths of the filter, so that they do not
        // all ask the same L2 channel for the same line at the same moment)
        constexpr int PER_WAVE = CF_WT_BYTES / 1024 / 8;
        const int     seg = (wave + (blockIdx.x >> 3)) & 7;
        const char*   src = (const char*) a.w + (((lane & ~7) | ((lane & 7) ^ (((lane >> 3) & 3) << 1))) << 4) + seg * (PER_WAVE * 1024);
#pragma unroll
        for (int k = 0; k < PER_WAVE; k += 4)
        {
            const char*    g = src + k * 1024;
            const uint32_t l = lds_base + CR_STAGE_OFF + seg * (PER_WAVE * 1024) + k * 1024;
            if (k + 4 <= PER_WAVE)
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off\n\tglobal_load_lds_dwordx4 %0, off offset:1024\n\t"
                             "global_load_lds_dwordx4 %0, off offset:2048\n\tglobal_load_lds_dwordx4 %0, off offset:3072" ::"v"(g), "s"(l)
                             : "memory");
            else
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(l) : "memory");
        }
    }

    // ---- the run and its virtual rows ------------------------------------------------------------------------------------
    const int H = a.H, W = WC ? WC : a.W, wp = W + 2, row_bytes = wp * 128;
    const int row_begin = blockIdx.x * a.rows_per_wg + min((int) blockIdx.x, a.rows_extra);
    const int rows = a.rows_per_wg + ((int) blockIdx.x < a.rows_extra ? 1 : 0);
    const int img0 = row_begin / H, hs0 = row_begin - img0 * H, n0 = min(H - hs0, rows);
    const int V = rows <= n0 ? rows + 2 : cr_virtual_rows(rows, hs0, H);
    const int npx = rows * W, ntiles = (npx + 31) >> 5, npairs = (ntiles + 1) >> 1;
    // virtual row of the input row above output row o of the run
    auto vtop = [&](int o) __attribute__((always_inline))
    {
        const int u = o - n0, k = cf_div(max(u, 0), H);
        return o < n0 ? o : n0 + 2 + k * (H + 2) + (u - k * H);
    };
    // input row of virtual row v, counted from row 0 of image img0; -1: a row of zeros
    auto vsrc = [&](int v) __attribute__((always_inline))
    {
        const int u = v - (n0 + 2), k = cf_div(max(u, 0), H + 2);
        const int img = v < n0 + 2 ? 0 : 1 + k, h = v < n0 + 2 ? hs0 - 1 + v : u - k * (H + 2) - 1;
        return (h >= 0 && h < H) ? img * H + h : -1;
    };
    // the same two for wave-uniform arguments, in scalar arithmetic
    auto vtop_uniform = [&](int o) __attribute__((always_inline))
    {
        if (o < n0) return o;
        const int u = o - n0, k = u / H;
        return n0 + 2 + k * (H + 2) + (u - k * H);
    };
    auto vsrc_uniform = [&](int v) __attribute__((always_inline))
    {
        int img = 0, h = hs0 - 1 + v;
        if (v >= n0 + 2)
        {
            const int u = v - (n0 + 2), k = u / (H + 2);
            img = 1 + k;
            h = u - k * (H + 2) - 1;
        }
        return (h >= 0 && h < H) ? img * H + h : -1;
    };
    const char* xbase = (const char*) (a.x + (long long) img0 * H * W * CF_C);
    // Requests for virtual rows [va, vb): a request moves 8 consecutive pixels of one input row (64 lanes x 16 bytes) to
    // their 8 slots of the LDS row; chunk i of the slot of LDS column c holds input channels 8 * (i ^ ((c >> 1) & 7)) .. + 7.
    // Request k of a row starts at input column 8 k = LDS column 8 k + 1, so the lane's source offset inside the request is
    // one of two constants (k even / odd), and the instruction's offset field steps through the row in the global and the
    // LDS address alike: a row costs a few scalar instructions.  Whole rows are dealt to the wavefronts in turn; rows of zeros are not requested (zero_rows writes them).  Returns this wavefront's number of requests
    const int      kw = (W + 7) >> 3;
    const int      dj = lane >> 3, di = lane & 7;
    const uint32_t src_even = (uint32_t) (dj * 128 + ((di ^ (((1 + dj) >> 1) & 7)) << 4));
    const uint32_t src_odd = (uint32_t) (dj * 128 + ((di ^ ((4 + ((1 + dj) >> 1)) & 7)) << 4));
    auto issue_rows = [&](int va, int vb, int w0, int nw) __attribute__((always_inline)) // rows to wavefronts w0 .. w0 + nw - 1
    {
        int n = 0;
        if (wave < w0) return n;
        for (int v = va + ((wave - w0 - va) & (nw - 1)); v < vb; v += nw)
        {
            const int g = vsrc_uniform(v);
            if (g < 0) continue;
            // (the values are wave-uniform; readfirstlane tells the compiler so where it cannot prove it)
            const uint64_t src = (uint64_t) (xbase + (long long) g * W * (CF_C * 2));
            uint64_t       src_s = (uint64_t) (uint32_t) __builtin_amdgcn_readfirstlane((uint32_t) src) |
                             ((uint64_t) (uint32_t) __builtin_amdgcn_readfirstlane((uint32_t) (src >> 32)) << 32);
            uint32_t dst = __builtin_amdgcn_readfirstlane(lds_base + (uint32_t) ((v * wp + 1) * 128));
            int      k = 0;
            for (; k + 4 <= (W >> 3); k += 4, src_s += 4096, dst += 4096)
                asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %2\n\tglobal_load_lds_dwordx4 %1, %2 offset:1024\n\t"
                             "global_load_lds_dwordx4 %0, %2 offset:2048\n\tglobal_load_lds_dwordx4 %1, %2 offset:3072" ::"v"(src_even),
                             "v"(src_odd), "s"(src_s), "s"(dst)
                             : "memory");
            for (; k < kw; k++, src_s += 1024, dst += 1024)
                if (8 * k + dj < W) cf_dma16_off((const void*) src_s, (k & 1) ? src_odd : src_even, dst);
            n += kw;
        }
        return n;
    };
    auto zero_cols = [&](int va, int vb, int t0, int nthreads) __attribute__((always_inline))
    {
        for (int i = tid - t0; i < (vb - va) * 16; i += nthreads)
        {
            const int row = va + (i >> 4), side = (i >> 3) & 1, chunk = i & 7;
            *reinterpret_cast<uint4*>(lds + ((row * wp + (side ? W + 1 : 0)) * 8 + chunk) * 16) = make_uint4(0, 0, 0, 0);
        }
    };
    auto zero_rows = [&](int va, int vb, int t0, int nthreads) __attribute__((always_inline))
    {
        auto zero_row = [&](int v) __attribute__((always_inline))
        {
            for (int c = tid - t0; c < wp * 8; c += nthreads) *reinterpret_cast<uint4*>(lds + (v * wp * 8 + c) * 16) = make_uint4(0, 0, 0, 0);
        };
        if (rows <= n0)
        {
            // one image segment: only its first and last virtual row can lie outside the image
            if (hs0 == 0 && va <= 0 && 0 < vb) zero_row(0);
            if (hs0 + n0 == H && va <= n0 + 1 && n0 + 1 < vb) zero_row(n0 + 1);
        }
        else
            for (int v = va; v < vb; v++)
                if (vsrc_uniform(v) < 0) zero_row(v);
    };
    // two groups of rows: [0, g0) is what tiles 0 .. 7 read (as far as it lies below the staging area), requested now;
    // the rest follows when the staging area is free
    const int g1 = min(V, CR_STAGE_OFF / row_bytes);
    const int g0 = min(g1, vtop_uniform((min(npx, 256) - 1) / W) + 3);
    const int n_g0 = issue_rows(0, g0, 0, 8);
    zero_cols(0, g1, 0, 512);
    zero_rows(0, g1, 0, 512);

    const bool       fused = a.epi.fused != 0;
    const bool       has_alpha = a.epi.has_alpha != 0;
    const float      alpha = a.epi.alpha;
    const int32_t*   col_exp = a.epi.col_exp;
    const int        dt = fused ? a.epi.out_dtype : DT_FP32;
    const bool       bf16_fast = fused && dt == DT_BF16 && a.epi.fast_cast;
    const CastParams cp = {a.epi.cast.dtype,       a.epi.cast.exp_bias, a.epi.cast.inf_nan_mode, a.epi.cast.rm,    a.epi.cast.clip_fp,
                           a.epi.cast.clip_inf_in, a.epi.cast.ftz,      a.epi.cast.relu,         a.epi.cast.scale, a.epi.cast.has_scale};

    cr_wait_vmcnt(n_g0); // requests retire in issue order: the filter came first
    __syncthreads();     // every wavefront's part of the filter has landed

    // ---- this wavefront's half of the filter into registers: fragment of k-step (tap, 16 in channels) = out channel
    // nh * 32 + lane % 32, in channels 8 * kg .. + 7 of the step; two ds_read_b64_tr_b16 as in the kernel above ---------------
    CfFrag fw[CF_TAPS * 4];
    {
        const int   g = lane >> 4, j = lane & 15;
        const char* p0 = lds + CR_STAGE_OFF + ((g >> 1) * 8 + (j >> 2)) * 128 + (((nh * 2 + (g & 1)) ^ (j >> 2)) << 5) + ((j & 3) << 3);
#pragma unroll
        for (int step = 0; step < CF_TAPS * 4; step++)
        {
            const char* p = p0 + (step >> 2) * 8192 + (step & 3) * 2048;
            fw[step].h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((CF_LDS cf_v4s*) p);
            fw[step].h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((CF_LDS cf_v4s*) (p + 512));
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70); // this wavefront's requests for the first group of rows
    __syncthreads(); // everybody has taken its fragments: the staging area becomes input rows; the first rows have landed
    // The remaining rows, by the second wavefront of each SIMD: the first one has priority on the matrix cores and starts
    // on the pairs that read only the first rows meanwhile.  The four raise the counter when their requests have landed
    if (wave >= 4)
    {
        issue_rows(g0, V, 4, 4);
        zero_cols(g1, V, 256, 256);
        zero_rows(g1, V, 256, 256);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0) __hip_atomic_fetch_add(ctrl + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }

    bool landed = false; // this wavefront has seen the counter at 4
    while (true)
    {
        uint32_t q = 0;
        if (lane == 0) q = __hip_atomic_fetch_add(ctrl + nh, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        q = __builtin_amdgcn_readfirstlane(q);
        if ((int) q >= npairs) break;
        const int tile0 = 2 * (int) q;
        const int nt = tile0 + 1 < ntiles ? 2 : 1;
        if (!landed && vtop_uniform((min(npx, (tile0 + 2) * 32) - 1) / W) + 3 > g0)
        {
            // every wavefront that raises the counter does so without waiting for anybody: the spin ends
            cf_wait_for(ctrl + 2, 4u, a.wait_limit, a.status);
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            landed = true;
        }

        // LDS address of this lane's pixel under tap (r, s), k-step quarter 0; quarter ks is that ^ (ks << 5).  With a
        // compile-time width the row pitch goes into the instruction's offset field and only r = 0 is kept
        constexpr int XR = WC ? 1 : 3;
        uint32_t      xa[2][XR][3];
#pragma unroll
        for (int t = 0; t < 2; t++)
        {
            const int p = min((tile0 + t) * 32 + (lane & 31), npx - 1);
            const int o = cf_div(p, W), col = p - o * W, vt = vtop(o);
#pragma unroll
            for (int r = 0; r < XR; r++)
#pragma unroll
                for (int s = 0; s < 3; s++)
                    xa[t][r][s] = (uint32_t) (((vt + r) * wp + col + s) * 128) | (uint32_t) ((kg ^ (((col + s) >> 1) & 7)) << 4);
        }
        v16f acc[2];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[t][v] = 0.0f;

        // 36 k-steps x NT tiles = one flat sequence of (pixel fragment read, matrix-core instruction) pairs; the read runs
        // DEPTH pairs ahead of its use through a ring of DEPTH + 1 fragments, which is what hides the LDS latency: a
        // wavefront issues nothing while its own matrix-core instruction runs, so every wait it meets is exposed
        auto contract = [&](auto nt_c) __attribute__((always_inline))
        {
            constexpr int NT = decltype(nt_c)::value;
            constexpr int NQ = CF_TAPS * 4 * NT, DEPTH = WC ? 5 : 2, RING = DEPTH + 1;
            CfFrag        fx[RING];
            auto ld_x = [&](int q) __attribute__((always_inline))
            {
                const int step = q / NT, t = q - step * NT, tap = step >> 2, ks = step & 3, r = tap / 3, s = tap - r * 3;
                if constexpr (WC != 0)
                    fx[q % RING].u = *reinterpret_cast<const uint4*>(lds + (xa[t][0][s] ^ (uint32_t) (ks << 5)) + r * ((WC + 2) * 128));
                else
                    fx[q % RING].u = *reinterpret_cast<const uint4*>(lds + (xa[t][r][s] ^ (uint32_t) (ks << 5)));
            };
#pragma unroll
            for (int q = 0; q < DEPTH; q++) ld_x(q);
#pragma unroll
            for (int q = 0; q < NQ; q++)
            {
                const int step = q / NT, t = q - step * NT;
                if (q + DEPTH < NQ) ld_x(q + DEPTH);
                __builtin_amdgcn_sched_barrier(0);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[step].v, fx[q % RING].v, acc[t], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        if (nt == 2) contract(std::integral_constant<int, 2>());
        else
            contract(std::integral_constant<int, 1>());

        // ---- epilogue of the pair: accumulator register v of lane l = channel nh * 32 + 8 * (v / 4) + 4 * (l / 32) + v % 4
        // of pixel l % 32; v_permlane32_swap leaves the lane with channels nh * 32 + kg * 16 + 0 .. 15 in order -------------
#pragma unroll
        for (int t = 0; t < 2; t++)
        {
            if (t == 1 && nt < 2) break;
            const int p = (tile0 + t) * 32 + (lane & 31);
            float val[16];
#pragma unroll
            for (int g = 0; g < 2; g++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                {
                    const float lo = acc[t][4 * g + i], hi = acc[t][8 + 4 * g + i];
                    const auto  sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
                    val[8 * g + i] = __uint_as_float(sw[0]);
                    val[8 * g + 4 + i] = __uint_as_float(sw[1]);
                }
            if (has_alpha)
            {
#pragma unroll
                for (int c = 0; c < 16; c++) val[c] *= alpha;
            }
            if (col_exp)
            {
#pragma unroll
                for (int c = 0; c < 16; c++) val[c] *= pow2_of(col_exp[nh * 32 + kg * 16 + c]);
            }
            const long long idx = ((long long) row_begin * W + p) * CF_K + nh * 32 + kg * 16;
            if (bf16_fast)
            {
                // v_cvt_pk_bf16_f32 where it gives the reference's code (everything but NaN, and inf / overflow where
                // clipping matters); the sum of |x| over the lane's 16 values detects the rest
                uint32_t pk[8];
                auto     convert = [&](auto relu_c) __attribute__((always_inline))
                {
                    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int c = 0; c < 16; c++)
                    {
                        if (decltype(relu_c)::value) val[c] = relu_ref(val[c]);
                        sum[c & 3] += __builtin_fabsf(val[c]);
                    }
                    const bool special = !((sum[0] + sum[1]) + (sum[2] + sum[3]) < 0x1.ffp+127f);
                    if (__builtin_amdgcn_ballot_w64(special) == 0)
                    {
#pragma unroll
                        for (int c = 0; c < 8; c++)
                        {
                            const cf_v2bf h = __builtin_convertvector(cf_v2f {val[2 * c], val[2 * c + 1]}, cf_v2bf);
                            __builtin_memcpy(&pk[c], &h, 4);
                        }
                    }
                    else
                    {
#pragma unroll
                        for (int c = 0; c < 8; c++)
                            pk[c] = fp32_to_bf16_rne(f2u(val[2 * c]), cp.clip_fp, cp.clip_inf_in) |
                                    (fp32_to_bf16_rne(f2u(val[2 * c + 1]), cp.clip_fp, cp.clip_inf_in) << 16);
                    }
                };
                if (cp.relu) convert(std::true_type());
                else
                    convert(std::false_type());
                if (p < npx)
                {
                    cf_v4u* o = (cf_v4u*) ((uint16_t*) a.epi.out + idx);
                    o[0] = cf_v4u {pk[0], pk[1], pk[2], pk[3]};
                    o[1] = cf_v4u {pk[4], pk[5], pk[6], pk[7]};
                }
            }
            else if (p < npx)
            {
                if (!fused)
                {
                    cf_v4f* o = (cf_v4f*) ((float*) a.epi.out + idx);
#pragma unroll
                    for (int c = 0; c < 4; c++) o[c] = cf_v4f {val[4 * c], val[4 * c + 1], val[4 * c + 2], val[4 * c + 3]};
                }
                else
                {
#pragma unroll 1
                    for (int c = 0; c < 16; c++) store_out_slow(a.epi, idx + c, val[c]);
                }
            }
        }
    }
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

hipError_t launch_conv_fwd_fast(const void* x, const void* w, int B, int H, int W, const GemmEpilogue& epi, int num_cus, uint32_t* status,
                                uint32_t wait_limit, hipStream_t s)
{
    static bool attr_done = false;
    const int   lds_bytes = CF_WT_BYTES + 2 * (CF_TR + 2) * (W + 2) * 128 + 16; // filter, one input tile per team, barrier counters
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
    a.status = status;
    a.wait_limit = wait_limit;
    const long long rows = (long long) B * H;
    if (rows > 0x7fffffffLL) return hipErrorInvalidValue;
    const int grid = (int) std::min<long long>((rows + CF_TR - 1) / CF_TR, num_cus > 0 ? num_cus : 256);
    a.rows_per_wg = (int) (rows / grid);
    a.rows_extra = (int) (rows % grid);
    // the resident form needs every workgroup's input rows in LDS at once and at most four rounds of tiles
    bool resident = (long long) (a.rows_per_wg + 1) * W <= CR_MAX_TILES * 32;
    for (int wg = 0; wg < grid && resident; wg++)
    {
        const long long row_begin = (long long) wg * a.rows_per_wg + std::min(wg, a.rows_extra);
        const int       n = a.rows_per_wg + (wg < a.rows_extra ? 1 : 0);
        if (n * W > CR_MAX_TILES * 32 || cr_virtual_rows(n, (int) (row_begin % H), H) * (W + 2) * 128 > CR_CTRL_OFF) resident = false;
    }
    if (resident)
    {
        static bool attr2_done = false;
        if (!attr2_done)
        {
            for (const void* f : {(const void*) conv_fwd_resident_kernel<0>, (const void*) conv_fwd_resident_kernel<56>,
                                  (const void*) conv_fwd_resident_kernel<28>, (const void*) conv_fwd_resident_kernel<14>})
            {
                hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, CR_LDS_BYTES);
                if (e != hipSuccess) return e;
            }
            attr2_done = true;
        }
        if (W == 56) hipLaunchKernelGGL(conv_fwd_resident_kernel<56>, dim3(grid), dim3(512), CR_LDS_BYTES, s, a);
        else if (W == 28)
            hipLaunchKernelGGL(conv_fwd_resident_kernel<28>, dim3(grid), dim3(512), CR_LDS_BYTES, s, a);
        else if (W == 14)
            hipLaunchKernelGGL(conv_fwd_resident_kernel<14>, dim3(grid), dim3(512), CR_LDS_BYTES, s, a);
        else
            hipLaunchKernelGGL(conv_fwd_resident_kernel<0>, dim3(grid), dim3(512), CR_LDS_BYTES, s, a);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(conv_fwd_fast_kernel, dim3(grid), dim3(512), lds_bytes, s, a);
    return hipGetLastError();
}

} // namespace mme
