// conv_fwd_fast.hip -- forward convolution, bf16, 3 x 3 filter, 64 -> 64 channels, stride 1, padding 1 (the ResNet
// 3 x 3 layer of the benchmark configuration: N = 64, H = W = 56).
//
// Implicit GEMM like the general kernel (the im2col matrix of the reference, mme/mme_reference/im2col.cpp:55-91, is
// never built), but organised around what bounds this shape on MI355X: it is close to the HBM roofline (51 MB of
// compulsory traffic for 14.8 GFLOP), so every input pixel is fetched from memory once and every output written once.
//
//   workgroup   8 output rows x W columns of one image, all 64 output channels; 256 lanes = 4 wavefronts
//   LDS         the input halo tile (10 rows x (W + 2) pixels x 64 channels, zero filled outside the image, 16-byte
//               chunks XOR-swizzled by column) and the whole filter, transposed to k-contiguous rows
//               Wt[out channel][tap * 64 + in channel] (pitch 1168 B: conflict-free 16-byte reads)
//   wavefront   pixel tiles of 32 (tile index = wavefront, +4, +8, ...), both 32-channel halves: per k-step of 16
//               channels 2 filter fragments + up to 4 pixel fragments feed up to 8 v_mfma_f32_32x32x16_bf16
//   epilogue    power-of-two factor, relu, cast (same converters as everywhere else), 2-byte / 4-byte stores
//
// Everything else (other filters, channel counts, strides, dtypes) runs on the general kernel.
#include "gemm_impl.hpp"

namespace mme
{
namespace
{
constexpr int CF_C = 64, CF_K = 64, CF_TAPS = 9, CF_TR = 8;
constexpr int CF_WT_PITCH = CF_TAPS * CF_C * 2 + 16; // bytes per output-channel row of the transposed filter
constexpr int CF_WT_BYTES = CF_K * CF_WT_PITCH;
constexpr int CF_MAX_TILES = 4;                       // pixel tiles per wavefront

struct ConvFwdFastArgs
{
    const uint16_t* x;   // [B][H][W][64]
    const uint16_t* w;   // [3][3][64 in][64 out]
    int             B, H, W;
    GemmEpilogue    epi; // out = [B][H][W][64], ld = 64
};

__device__ __forceinline__ int halo_off(int row, int col, int chunk, int wp)
{
    return ((row * wp + col) * 8 + (chunk ^ ((col >> 1) & 7))) * 16;
}

__global__ __launch_bounds__(256) void conv_fwd_fast_kernel(ConvFwdFastArgs a_by_value)
{
    (void) a_by_value;
    typedef const __attribute__((address_space(4))) ConvFwdFastArgs& ArgRef;
    ArgRef a = *(const __attribute__((address_space(4))) ConvFwdFastArgs*) __builtin_amdgcn_kernarg_segment_ptr();
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    char* wt = lds;                // transposed filter
    char* halo = lds + CF_WT_BYTES; // input tile with halo

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int H = a.H, W = a.W, wp = W + 2;
    const int row_tiles = (H + CF_TR - 1) / CF_TR;
    const int img = blockIdx.x / row_tiles, h0 = (blockIdx.x % row_tiles) * CF_TR;

    // ---- filter: global [tap][c][k] (k contiguous) -> LDS [k][tap * 64 + c]; 8 x 8 blocks transposed in registers ----
    for (int blk = tid; blk < (CF_TAPS * CF_C / 8) * (CF_K / 8); blk += 256)
    {
        const int kb = blk & 7, cb = blk >> 3; // cb: block of 8 consecutive (tap, c) rows; kb: block of 8 output channels
        uint4     in[8], out[8];
#pragma unroll
        for (int i = 0; i < 8; i++) in[i] = *reinterpret_cast<const uint4*>(a.w + (size_t) (cb * 8 + i) * CF_K + kb * 8);
        transpose_block<2>(in, out);
#pragma unroll
        for (int j = 0; j < 8; j++) *reinterpret_cast<uint4*>(wt + (kb * 8 + j) * CF_WT_PITCH + cb * 16) = out[j];
    }
    // ---- input tile with halo: rows h0-1 .. h0+TR, columns -1 .. W; zeros outside the image --------------------------
    const uint16_t* ximg = a.x + (size_t) img * H * W * CF_C;
    for (int c = tid; c < (CF_TR + 2) * wp * 8; c += 256)
    {
        const int chunk = c & 7, pix = c >> 3, row = pix / wp, col = pix - row * wp;
        const int h = h0 - 1 + row, w_ = col - 1;
        uint4     v = make_uint4(0, 0, 0, 0);
        if (h >= 0 && h < H && w_ >= 0 && w_ < W) v = *reinterpret_cast<const uint4*>(ximg + ((size_t) h * W + w_) * CF_C + chunk * 8);
        *reinterpret_cast<uint4*>(halo + halo_off(row, col, chunk, wp)) = v;
    }
    __syncthreads();

    // ---- contraction ----------------------------------------------------------------------------------------------
    const int rows_here = min(CF_TR, H - h0);
    const int npix = rows_here * W, ntiles = (npix + 31) / 32;
    // this lane's pixel in each of the wavefront's tiles (clamped: surplus slots recompute the last pixel, never stored)
    int prow[CF_MAX_TILES], pcol[CF_MAX_TILES];
#pragma unroll
    for (int t = 0; t < CF_MAX_TILES; t++)
    {
        int p = (wave + 4 * t) * 32 + (lane & 31);
        p = min(p, npix - 1);
        prow[t] = p / W;
        pcol[t] = p - prow[t] * W;
    }
    const int kg = lane >> 5;
    v16f      acc[CF_MAX_TILES][2];
#pragma unroll
    for (int t = 0; t < CF_MAX_TILES; t++)
#pragma unroll
        for (int n = 0; n < 2; n++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[t][n][v] = 0.0f;
    const int my_tiles = (ntiles - wave + 3) / 4; // tiles wave, wave+4, ...

    union Frag
    {
        uint4 u;
        v8bf  v;
    };
#pragma unroll 1
    for (int tap = 0; tap < CF_TAPS; tap++)
    {
        const int r = tap / 3, s = tap - r * 3;
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
        {
            Frag fb[2], fa[CF_MAX_TILES];
#pragma unroll
            for (int n = 0; n < 2; n++)
                fb[n].u = *reinterpret_cast<const uint4*>(wt + (n * 32 + (lane & 31)) * CF_WT_PITCH + (tap * CF_C + ks * 16 + kg * 8) * 2);
#pragma unroll
            for (int t = 0; t < CF_MAX_TILES; t++)
                if (t < my_tiles) fa[t].u = *reinterpret_cast<const uint4*>(halo + halo_off(prow[t] + r, pcol[t] + s, ks * 2 + kg, wp));
#pragma unroll
            for (int t = 0; t < CF_MAX_TILES; t++)
                if (t < my_tiles)
                {
#pragma unroll
                    for (int n = 0; n < 2; n++) acc[t][n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[t].v, fb[n].v, acc[t][n], 0, 0, 0);
                }
        }
    }

    // ---- epilogue ---------------------------------------------------------------------------------------------------
    const bool       fused = a.epi.fused != 0;
    const bool       has_alpha = a.epi.has_alpha != 0;
    const float      alpha = a.epi.alpha;
    const int32_t*   col_exp = a.epi.col_exp;
    const int        dt = fused ? a.epi.out_dtype : DT_FP32;
    const CastParams cp = {a.epi.cast.dtype,       a.epi.cast.exp_bias, a.epi.cast.inf_nan_mode, a.epi.cast.rm,    a.epi.cast.clip_fp,
                           a.epi.cast.clip_inf_in, a.epi.cast.ftz,      a.epi.cast.relu,         a.epi.cast.scale, a.epi.cast.has_scale};
    const long long  img_base = ((long long) img * H + h0) * W * CF_K; // element offset of this tile's first output pixel
#pragma unroll
    for (int t = 0; t < CF_MAX_TILES; t++)
    {
        if (t >= my_tiles) continue;
#pragma unroll
        for (int n = 0; n < 2; n++)
        {
            const int ch = n * 32 + (lane & 31);
            float     cs = 1.0f;
            if (col_exp) cs = pow2_of(col_exp[ch]);
#pragma unroll
            for (int v = 0; v < 16; v++)
            {
                const int p = (wave + 4 * t) * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (p >= npix) continue;
                float x = acc[t][n][v];
                if (has_alpha) x *= alpha;
                if (col_exp) x *= cs;
                const long long idx = img_base + (long long) p * CF_K + ch;
                if (!fused) ((float*) a.epi.out)[idx] = x;
                else if (dt == DT_BF16 && a.epi.fast_cast)
                    ((uint16_t*) a.epi.out)[idx] = (uint16_t) cast_elem<DT_BF16, true>(x, cp);
                else
                    store_out_slow(a.epi, idx, x);
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
    if (W < 1 || W > 62 || H < 1) return false;
    if (CF_TR * W > 32 * 4 * CF_MAX_TILES) return false;
    return true;
}

hipError_t launch_conv_fwd_fast(const void* x, const void* w, int B, int H, int W, const GemmEpilogue& epi, hipStream_t s)
{
    static bool     attr_done = false;
    const int       lds_bytes = CF_WT_BYTES + (CF_TR + 2) * (W + 2) * 128;
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
    const int row_tiles = (H + CF_TR - 1) / CF_TR;
    hipLaunchKernelGGL(conv_fwd_fast_kernel, dim3(B * row_tiles), dim3(256), lds_bytes, s, a);
    return hipGetLastError();
}

} // namespace mme
