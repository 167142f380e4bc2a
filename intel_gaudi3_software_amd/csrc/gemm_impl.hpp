// gemm_kernels.hip -- general MFMA contraction kernel for gfx950 (CDNA4).
//
// Replaces the scalar worker loop of the reference calculator (doGemmWorkerFloat,
// mme/mme_reference/mme_reference_impl.cpp:1022-1053, and ChipFma::fma_vec below it) for every contraction on the
// path: batched GEMM in the four transpose forms (:445-539), and convolution fwd / dedx / dedw (:598-659, 770-869)
// as implicit GEMM: the im2col matrix of the reference (im2col.cpp:55-91) is never materialised, its addressing
// (im2col.cpp:134-172) is evaluated while tiles are loaded.  dedx is computed in gather form, so the col2im
// scatter-add (im2col.cpp:93-132) disappears too.
//
// Tiling: 128 x 128 outputs per 256-lane workgroup (4 wavefronts as 2 x 2, 64 x 64 each = 2 x 2 MFMA 32x32 tiles),
// 64 bytes of the reduction dimension per LDS stage, two stages (loads of stage i+1 are in flight while stage i feeds
// the matrix cores).  Every lane reads a 32-byte k-slab per row and stage:
//     fp8  : one v_mfma_f32_32x32x64_f8f6f4 (e4m3 / e5m2 selectable per operand)
//     bf16 : two v_mfma_f32_32x32x16_bf16 (fp16: the same with v_mfma_f32_32x32x16_f16)
//     fp32 : eight v_mfma_f32_32x32x2_f32
// LDS rows are k-contiguous for both operands (row pitch 80 B: conflict-free 16-byte reads); operands whose memory
// layout is contiguous along the free index (B of the "ab" form, x of dedw, ...) are transposed in registers with
// v_perm_b32 on their way into LDS.
//
// Accumulation is fp32 in the MFMA accumulators; the reference accumulates in an 8-wide truncating tree
// (coral-sim/header/gaudi3/fs_core/fs_fma_gaudi3.h:760-1166), so results agree to a tolerance, not bit for bit.
#pragma once
#include "mme_kernels.hpp"

namespace mme
{
namespace
{
typedef int   v8i __attribute__((ext_vector_type(8)));
typedef int   v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// Kernel arguments are read in place from the kernarg segment (constant address space): views are passed on by
// reference to out-of-line helpers without a private copy of the whole problem, and uniform fields stay scalar loads.
#define KARG const __attribute__((address_space(4)))
typedef KARG OperandView& ViewRef;
typedef KARG GemmEpilogue& EpilogueRef;

constexpr int TILE = 128;     // outputs per workgroup along each free index
constexpr int STAGE_BYTES = 64; // bytes of k per row and stage
constexpr int LDS_PITCH = 80; // bytes between rows in LDS
constexpr int THREADS = 256;

// ------------------------------------------------------------------------------------------------------------
// element address of a view
// ------------------------------------------------------------------------------------------------------------
struct PixelPos
{
    int c[4];
};

__device__ __forceinline__ PixelPos decode_pixel(ViewRef v, int pix)
{
    PixelPos p;
    p.c[0] = pix % v.grid[0];
    pix /= v.grid[0];
    p.c[1] = pix % v.grid[1];
    pix /= v.grid[1];
    p.c[2] = pix % v.grid[2];
    p.c[3] = pix / v.grid[2];
    return p;
}

// element offset of (pixel, tap) in the gathered tensor, or -1 when it falls into the padding / between strides
__device__ inline long long conv_offset(ViewRef v, const PixelPos& p, int tap)
{
    int t[4];
    t[0] = tap % v.ktap[0];
    tap /= v.ktap[0];
    t[1] = tap % v.ktap[1];
    t[2] = tap / v.ktap[1];
    t[3] = 0;
    long long off = 0;
#pragma unroll
    for (int d = 0; d < 4; d++)
    {
        int pos;
        if (!v.gather_y) pos = p.c[d] * v.cstride[d] + t[d] * v.dil[d] - v.pad[d];
        else
        {
            const int num = p.c[d] + v.pad[d] - t[d] * v.dil[d];
            if (num < 0) return -1;
            pos = num / v.cstride[d];
            if (pos * v.cstride[d] != num) return -1;
        }
        if (pos < 0 || pos >= v.src[d]) return -1;
        off += (long long) pos * v.src_stride[d];
    }
    return off;
}

// element offset of (f, k) for the gather views; kept out of line: it is long and sits on the slow paths only
__device__ __attribute__((noinline)) long long elem_offset_gather(ViewRef v, int f, int k)
{
    if (v.kind == VIEW_TAPPED)
    {
        const int tap = k / v.nch;
        return (long long) f * v.stride_f + (long long) (k - tap * v.nch) * v.stride_k + (long long) tap * v.tap_stride;
    }
    const int pix = v.pix_is_f ? f : k;
    const int tc = v.pix_is_f ? k : f;
    const int tap = tc / v.nch;
    const int ch = tc - tap * v.nch;
    const long long o = conv_offset(v, decode_pixel(v, pix), tap);
    return o < 0 ? -1 : o + ch;
}

// element offset of (f, k) or -1.  F and Kd are the extents of f and k.
__device__ __forceinline__ long long elem_offset(ViewRef v, int f, int k, int F, int Kd, long long batch_off)
{
    if (f >= F || k >= Kd) return -1;
    if (v.kind == VIEW_PLAIN) return batch_off + (long long) f * v.stride_f + (long long) k * v.stride_k;
    return elem_offset_gather(v, f, k);
}

template<int ES>
__device__ __forceinline__ uint32_t load_elem(const char* base, long long off)
{
    if (off < 0) return 0u;
    if constexpr (ES == 1) return *(const uint8_t*) (base + off);
    else if constexpr (ES == 2)
        return *(const uint16_t*) (base + off * 2);
    else
        return *(const uint32_t*) (base + off * 4);
}

// KV = 16 / ES consecutive elements along the contiguous index, starting at (f, k); along_k says which index runs
template<int ES>
__device__ __forceinline__ uint4 load_vec(ViewRef v, int f, int k, bool along_k, int F, int Kd, long long batch_off)
{
    constexpr int KV = 16 / ES;
    if (v.vec_ok)
    {
        const long long off = elem_offset(v, f, k, F, Kd, batch_off);
        if (off < 0) return make_uint4(0, 0, 0, 0);
        return *reinterpret_cast<const uint4*>(v.base + off * ES);
    }
    // element-wise path (any shape, stride or alignment): not unrolled on purpose, it is the slow path
    unsigned long long lo = 0, hi = 0;
#pragma unroll 1
    for (int i = 0; i < KV; i++)
    {
        const long long off = along_k ? elem_offset(v, f, k + i, F, Kd, batch_off) : elem_offset(v, f + i, k, F, Kd, batch_off);
        const unsigned long long e = load_elem<ES>(v.base, off);
        const int                bit = i * ES * 8;
        if (bit < 64) lo |= e << bit;
        else
            hi |= e << (bit - 64);
    }
    return make_uint4((uint32_t) lo, (uint32_t) (lo >> 32), (uint32_t) hi, (uint32_t) (hi >> 32));
}

// ------------------------------------------------------------------------------------------------------------
// register transposes: in[i] holds KV elements along f for k = i; out[j] holds KV elements along k for f = j
// ------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t w_of(const uint4& v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
__device__ __forceinline__ void     set_w(uint4& v, int i, uint32_t x)
{
    if (i == 0) v.x = x;
    else if (i == 1)
        v.y = x;
    else if (i == 2)
        v.z = x;
    else
        v.w = x;
}

template<int ES>
__device__ __forceinline__ void transpose_block(const uint4 (&in)[16 / ES], uint4 (&out)[16 / ES])
{
    if constexpr (ES == 4)
    {
#pragma unroll
        for (int j = 0; j < 4; j++) out[j] = make_uint4(w_of(in[0], j), w_of(in[1], j), w_of(in[2], j), w_of(in[3], j));
    }
    else if constexpr (ES == 2)
    {
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int kk = 0; kk < 4; kk++)
            {
                const uint32_t lo = w_of(in[2 * kk], j >> 1), hi = w_of(in[2 * kk + 1], j >> 1);
                // v_perm_b32: selector bytes 0-3 pick from the second source, 4-7 from the first
                set_w(out[j], kk, __builtin_amdgcn_perm(hi, lo, (j & 1) ? 0x07060302u : 0x05040100u));
            }
    }
    else
    {
#pragma unroll
        for (int d = 0; d < 4; d++)
#pragma unroll
            for (int kk = 0; kk < 4; kk++)
            {
                const uint32_t r0 = w_of(in[4 * kk], d), r1 = w_of(in[4 * kk + 1], d), r2 = w_of(in[4 * kk + 2], d),
                               r3 = w_of(in[4 * kk + 3], d);
                const uint32_t x01l = __builtin_amdgcn_perm(r1, r0, 0x05010400u); // r0.b0 r1.b0 r0.b1 r1.b1
                const uint32_t x01h = __builtin_amdgcn_perm(r1, r0, 0x07030602u); // r0.b2 r1.b2 r0.b3 r1.b3
                const uint32_t x23l = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
                const uint32_t x23h = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
                set_w(out[4 * d + 0], kk, __builtin_amdgcn_perm(x23l, x01l, 0x05040100u));
                set_w(out[4 * d + 1], kk, __builtin_amdgcn_perm(x23l, x01l, 0x07060302u));
                set_w(out[4 * d + 2], kk, __builtin_amdgcn_perm(x23h, x01h, 0x05040100u));
                set_w(out[4 * d + 3], kk, __builtin_amdgcn_perm(x23h, x01h, 0x07060302u));
            }
    }
}

// ------------------------------------------------------------------------------------------------------------
// staging of one operand tile: global -> registers -> LDS
// ------------------------------------------------------------------------------------------------------------
template<int ES, bool KC>
struct Stager
{
    static constexpr int KV = 16 / ES;
    static constexpr int BK = STAGE_BYTES / ES;
    // k-contiguous: 128 rows x 4 chunks of 16 B = 512 chunks, two per lane.
    // f-contiguous: (BK / KV = 4) x (128 / KV) blocks of KV x KV elements, at most one per lane.
    static constexpr int NBLK = 4 * (TILE / KV);
    static constexpr int NREG = KC ? 2 : KV;
    uint4 r[NREG];

    __device__ __forceinline__ void load(ViewRef v, int f_base, int k0, int F, int Kd, long long boff)
    {
        const int tid = threadIdx.x;
        if constexpr (KC)
        {
#pragma unroll
            for (int j = 0; j < 2; j++)
            {
                const int c = tid + THREADS * j;
                r[j] = load_vec<ES>(v, f_base + (c >> 2), k0 + (c & 3) * KV, true, F, Kd, boff);
            }
        }
        else
        {
            if (tid < NBLK)
            {
                const int kb = tid & 3, fb = tid >> 2;
#pragma unroll
                for (int i = 0; i < KV; i++) r[i] = load_vec<ES>(v, f_base + fb * KV, k0 + kb * KV + i, false, F, Kd, boff);
            }
        }
    }

    __device__ __forceinline__ void store(char* lds)
    {
        const int tid = threadIdx.x;
        if constexpr (KC)
        {
#pragma unroll
            for (int j = 0; j < 2; j++)
            {
                const int c = tid + THREADS * j;
                *reinterpret_cast<uint4*>(lds + (c >> 2) * LDS_PITCH + (c & 3) * 16) = r[j];
            }
        }
        else
        {
            if (tid < NBLK)
            {
                const int kb = tid & 3, fb = tid >> 2;
                uint4     t[KV];
                transpose_block<ES>(r, t);
#pragma unroll
                for (int j = 0; j < KV; j++) *reinterpret_cast<uint4*>(lds + (fb * KV + j) * LDS_PITCH + kb * 16) = t[j];
            }
        }
    }
};

// ------------------------------------------------------------------------------------------------------------
// matrix-core step on one LDS stage
// ------------------------------------------------------------------------------------------------------------
struct Slab
{
    uint4 lo, hi; // 32 bytes of k for one row
};

__device__ __forceinline__ Slab read_slab(const char* lds, int row, int lane)
{
    const char* p = lds + row * LDS_PITCH + (lane >> 5) * 32;
    Slab        s;
    s.lo = *reinterpret_cast<const uint4*>(p);
    s.hi = *reinterpret_cast<const uint4*>(p + 16);
    return s;
}

template<int ES, int FMT>
__device__ __forceinline__ void mma_slab(v16f& acc, const Slab& a, const Slab& b)
{
    if constexpr (ES == 1)
    {
        const v8i va = {(int) a.lo.x, (int) a.lo.y, (int) a.lo.z, (int) a.lo.w, (int) a.hi.x, (int) a.hi.y, (int) a.hi.z, (int) a.hi.w};
        const v8i vb = {(int) b.lo.x, (int) b.lo.y, (int) b.lo.z, (int) b.lo.w, (int) b.hi.x, (int) b.hi.y, (int) b.hi.z, (int) b.hi.w};
        // cbsz / blgp: format of A / B, 0 = fp8 (e4m3), 1 = bf8 (e5m2); scales 0 select the unscaled instruction
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, vb, acc, FMT & 1, (FMT >> 1) & 1, 0, 0, 0, 0);
    }
    else if constexpr (ES == 2)
    {
        union
        {
            uint4 u;
            v8bf  v;
            v8h   h;
        } a0, a1, b0, b1;
        a0.u = a.lo;
        a1.u = a.hi;
        b0.u = b.lo;
        b1.u = b.hi;
        if constexpr (FMT == 1)
        {
            // IEEE half operands
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0.h, b0.h, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1.h, b1.h, acc, 0, 0, 0);
        }
        else
        {
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0.v, b0.v, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1.v, b1.v, acc, 0, 0, 0);
        }
    }
    else
    {
        const uint32_t aw[8] = {a.lo.x, a.lo.y, a.lo.z, a.lo.w, a.hi.x, a.hi.y, a.hi.z, a.hi.w};
        const uint32_t bw[8] = {b.lo.x, b.lo.y, b.lo.z, b.lo.w, b.hi.x, b.hi.y, b.hi.z, b.hi.w};
#pragma unroll
        for (int s = 0; s < 8; s++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u2f(aw[s]), u2f(bw[s]), acc, 0, 0, 0);
    }
}

// ------------------------------------------------------------------------------------------------------------
// epilogue: alpha, per-column power of two, relu, cast, store
// ------------------------------------------------------------------------------------------------------------
// fp16 / ufp16 outputs: one out-of-line copy of the converter, so that the unrolled epilogues of the other output types
// keep their size
__device__ __attribute__((noinline)) uint32_t cast_half_out_of_line(float v, const CastParams& cp, int fast)
{
    if (cp.dtype == DT_UFP16) return cast_elem<DT_UFP16, false>(v, cp);
    return fast ? cast_elem<DT_FP16, true>(v, cp) : cast_elem<DT_FP16, false>(v, cp);
}

__device__ __forceinline__ void store_out(EpilogueRef e, long long idx, float v)
{
    if (!e.fused)
    {
        ((float*) e.out)[idx] = v;
        return;
    }
    const CastParams cp = {e.cast.dtype, e.cast.exp_bias, e.cast.inf_nan_mode, e.cast.rm,    e.cast.clip_fp,
                           e.cast.clip_inf_in, e.cast.ftz, e.cast.relu,    e.cast.scale, e.cast.has_scale};
    switch (e.out_dtype)
    {
        case DT_FP8_143:
            ((uint8_t*) e.out)[idx] = (uint8_t) (e.fast_cast ? cast_elem<DT_FP8_143, true>(v, cp) : cast_elem<DT_FP8_143, false>(v, cp));
            break;
        case DT_FP8_152:
            ((uint8_t*) e.out)[idx] = (uint8_t) (e.fast_cast ? cast_elem<DT_FP8_152, true>(v, cp) : cast_elem<DT_FP8_152, false>(v, cp));
            break;
        case DT_BF16:
            ((uint16_t*) e.out)[idx] = (uint16_t) (e.fast_cast ? cast_elem<DT_BF16, true>(v, cp) : cast_elem<DT_BF16, false>(v, cp));
            break;
        case DT_FP16:
        case DT_UFP16: ((uint16_t*) e.out)[idx] = (uint16_t) cast_half_out_of_line(v, cp, e.fast_cast); break;
        default: ((uint32_t*) e.out)[idx] = cast_elem<DT_FP32, false>(v, cp); break;
    }
}

// out-of-line form for kernels whose epilogue is fully unrolled over many accumulators
__device__ __attribute__((noinline)) void store_out_slow(EpilogueRef e, long long idx, float v) { store_out(e, idx, v); }

__device__ __forceinline__ float pow2_of(int e) { return u2f((uint32_t) (e + 127) << 23); }

// A (f_a, k) x B (f_b, k) -> C[f_a][f_b]
template<int ES, bool A_KC, bool B_KC, int FMT>
__global__ __launch_bounds__(THREADS) void gemm_kernel(GemmProblem g_by_value)
{
    (void) g_by_value; // the only explicit argument: it sits at offset 0 of the kernarg segment
    KARG GemmProblem& g = *(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr();
    constexpr int BK = STAGE_BYTES / ES;
    __shared__ __attribute__((aligned(16))) char lds[2][2][TILE * LDS_PITCH];
    if (g.skip_flag && ((*g.skip_flag == g.skip_epoch) == (g.skip_if != 0))) return;

    const int tiles_n = (g.N + TILE - 1) / TILE;
    const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    // blockIdx.y: batch (dims 2, 3, 4 of the output, dim 2 fastest); blockIdx.z: split-k slice
    int       bz = blockIdx.y;
    const int b0 = bz % g.batch[0];
    bz /= g.batch[0];
    const int       b1 = bz % g.batch[1], b2 = bz / g.batch[1];
    const long long a_off = b0 * g.A.batch_stride[0] + b1 * g.A.batch_stride[1] + b2 * g.A.batch_stride[2];
    const long long b_off = b0 * g.B.batch_stride[0] + b1 * g.B.batch_stride[1] + b2 * g.B.batch_stride[2];

    const int nk_total = (g.K + BK - 1) / BK;
    int       kt_begin = 0, kt_end = nk_total;
    if (g.split_k > 1)
    {
        const int per = (nk_total + g.split_k - 1) / g.split_k;
        kt_begin = blockIdx.z * per;
        kt_end = min(nk_total, kt_begin + per);
    }

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    Stager<ES, A_KC> sa;
    Stager<ES, B_KC> sb;

    if (kt_begin < kt_end)
    {
        sa.load(g.A, tm * TILE, kt_begin * BK, g.M, g.K, a_off);
        sb.load(g.B, tn * TILE, kt_begin * BK, g.N, g.K, b_off);
        sa.store(lds[0][0]);
        sb.store(lds[0][1]);
    }
    __syncthreads();

    for (int kt = kt_begin; kt < kt_end; kt++)
    {
        const int  st = (kt - kt_begin) & 1;
        const bool more = kt + 1 < kt_end;
        if (more)
        {
            sa.load(g.A, tm * TILE, (kt + 1) * BK, g.M, g.K, a_off);
            sb.load(g.B, tn * TILE, (kt + 1) * BK, g.N, g.K, b_off);
        }
        Slab fa[2], fb[2];
#pragma unroll
        for (int i = 0; i < 2; i++) fa[i] = read_slab(lds[st][0], wm * 64 + i * 32 + (lane & 31), lane);
#pragma unroll
        for (int j = 0; j < 2; j++) fb[j] = read_slab(lds[st][1], wn * 64 + j * 32 + (lane & 31), lane);
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) mma_slab<ES, FMT>(acc[i][j], fa[i], fb[j]);
        if (more)
        {
            sa.store(lds[st ^ 1][0]);
            sb.store(lds[st ^ 1][1]);
        }
        __syncthreads();
    }

    // ---- epilogue --------------------------------------------------------------------------------------------
    // MFMA 32x32 accumulator layout: lane l, register v -> row 8 * (v / 4) + 4 * (l / 32) + v % 4, column l % 32
    const bool to_ws = g.split_k > 1;
    const long long c_off = b0 * g.epi.batch_stride[0] + b1 * g.epi.batch_stride[1] + b2 * g.epi.batch_stride[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
    {
        const int n = tn * TILE + wn * 64 + j * 32 + (lane & 31);
        if (n >= g.N) continue;
        float cs = 1.0f;
        if (!to_ws && g.epi.col_exp) cs = pow2_of(g.epi.col_exp[n]);
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++)
            {
                const int m = tm * TILE + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (m >= g.M) continue;
                float x = acc[i][j][v];
                if (to_ws)
                {
                    const long long slab = ((long long) blockIdx.z * gridDim.y + blockIdx.y) * g.M * (long long) g.N;
                    g.workspace[slab + (long long) m * g.N + n] = x;
                }
                else
                {
                    if (g.epi.has_alpha) x *= g.epi.alpha;
                    if (g.epi.col_exp) x *= cs;
                    store_out(g.epi, c_off + (long long) m * g.epi.ld + n, x);
                }
            }
    }
}

template<int ES, int FMT>
void launch_layout(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    const bool akc = p.A.k_contig != 0, bkc = p.B.k_contig != 0;
    if (akc && bkc) hipLaunchKernelGGL((gemm_kernel<ES, true, true, FMT>), grid, dim3(THREADS), 0, s, p);
    else if (akc && !bkc)
        hipLaunchKernelGGL((gemm_kernel<ES, true, false, FMT>), grid, dim3(THREADS), 0, s, p);
    else if (!akc && bkc)
        hipLaunchKernelGGL((gemm_kernel<ES, false, true, FMT>), grid, dim3(THREADS), 0, s, p);
    else
        hipLaunchKernelGGL((gemm_kernel<ES, false, false, FMT>), grid, dim3(THREADS), 0, s, p);
}

} // namespace
} // namespace mme
