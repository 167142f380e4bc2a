// gemm_kernels.hip -- dispatch of the contraction kernels (instantiated per operand type in gemm_inst_*.hip), the
// split-k reduction and the fp8 helper kernels.
#include "gemm_impl.hpp"

namespace mme
{
// one translation unit per operand type / fp8 flavour pair keeps the build parallel
void launch_gemm_bf16(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp16(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp32(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp8_00(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp8_10(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp8_01(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp8_11(const GemmProblem& p, dim3 grid, hipStream_t s);

namespace
{
// sums the split-k partials in slice order (deterministic) and applies the epilogue.  Four consecutive columns per lane
// (16-byte loads, one per slice, up to sixteen slices in flight) when N is a multiple of 4; the sum of an element is formed
// in the same order either way.
__global__ __launch_bounds__(THREADS) void splitk_reduce_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    KARG GemmProblem& g = *(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr();
    if (g.skip_flag && ((*g.skip_flag == g.skip_epoch) == (g.skip_if != 0))) return;
    typedef float r_v4f __attribute__((ext_vector_type(4)));
    const long long mn = (long long) g.M * g.N;
    const long long nb = (long long) g.batch[0] * g.batch[1] * g.batch[2];
    const long long total = mn * nb;
    const int       S = g.split_k;
    auto finish = [&](long long b, long long r, int count, const float* x) __attribute__((always_inline))
    {
        const int m = (int) (r / g.N), n = (int) (r - (long long) m * g.N);
        int       bz = (int) b;
        const int b0 = bz % g.batch[0];
        bz /= g.batch[0];
        const int       b1 = bz % g.batch[1], b2 = bz / g.batch[1];
        const long long c_off = b0 * g.epi.batch_stride[0] + b1 * g.epi.batch_stride[1] + b2 * g.epi.batch_stride[2];
        const long long idx = c_off + (long long) m * g.epi.ld + n;
        float           v[4];
        for (int c = 0; c < count; c++)
        {
            v[c] = x[c];
            if (g.epi.has_alpha) v[c] *= g.epi.alpha;
            if (g.epi.col_exp) v[c] *= pow2_of(g.epi.col_exp[n + c]);
        }
        if (count == 4 && !g.epi.fused && (idx & 3) == 0 && ((uintptr_t) g.epi.out & 15u) == 0)
            *(r_v4f*) ((float*) g.epi.out + idx) = r_v4f {v[0], v[1], v[2], v[3]};
        else
            for (int c = 0; c < count; c++) store_out(g.epi, idx + c, v[c]);
    };
    if ((g.N & 3) == 0 && ((uintptr_t) g.workspace & 15u) == 0)
    {
        const long long groups = total >> 2; // a group of four columns never crosses a row
        for (long long q = (long long) blockIdx.x * THREADS + threadIdx.x; q < groups; q += (long long) gridDim.x * THREADS)
        {
            const long long i = q << 2, b = i / mn, r = i - b * mn;
            const r_v4f*    w = (const r_v4f*) (g.workspace + b * mn + r);
            const long long step = nb * mn / 4; // r_v4f elements between slices
            r_v4f           x = {0.0f, 0.0f, 0.0f, 0.0f};
            // up to sixteen slices in flight per lane, added in slice order
            for (int z0 = 0; z0 < S; z0 += 16)
            {
                r_v4f part[16];
#pragma unroll
                for (int j = 0; j < 16; j++)
                    if (z0 + j < S) part[j] = __builtin_nontemporal_load(w + (z0 + j) * step);
#pragma unroll
                for (int j = 0; j < 16; j++)
                    if (z0 + j < S) x += part[j];
            }
            const float xs[4] = {x.x, x.y, x.z, x.w};
            finish(b, r, 4, xs);
        }
        return;
    }
    for (long long i = (long long) blockIdx.x * THREADS + threadIdx.x; i < total; i += (long long) gridDim.x * THREADS)
    {
        const long long b = i / mn, r = i - b * mn;
        float           x = 0.0f;
        for (int z = 0; z < S; z++) x += g.workspace[(z * nb + b) * mn + r];
        finish(b, r, 1, &x);
    }
}

// ---- fp8 helpers --------------------------------------------------------------------------------------------------
// exponent-all-ones (only_top: 0x7F / 0xFF) codes in one operand; blocks [first, first + count) of the grid take part
__device__ __forceinline__ bool fp8_scan_operand(const uint8_t* data, size_t n, uint32_t exp_mask, int only_top, unsigned first, unsigned count)
{
    const size_t stride = (size_t) count * THREADS;
    uint32_t     hit = 0;
    const size_t n16 = (((uintptr_t) data & 15u) == 0) ? (n >> 4) : 0;
    const uint4* d16 = reinterpret_cast<const uint4*>(data);
    const uint32_t em4 = exp_mask * 0x01010101u;
    auto           test = [&](uint32_t w) {
        if (only_top)
        {
            // a byte equals 0x7F after clearing the sign bit
            const uint32_t x = (w & 0x7F7F7F7Fu) ^ 0x7F7F7F7Fu; // zero byte <=> top code
            hit |= (x - 0x01010101u) & ~x & 0x80808080u;
        }
        else
        {
            const uint32_t x = (w & em4) ^ em4; // zero byte <=> all exponent bits set
            hit |= (x - 0x01010101u) & ~x & 0x80808080u;
        }
    };
    for (size_t i = (size_t) (blockIdx.x - first) * THREADS + threadIdx.x; i < n16; i += stride)
    {
        const uint4 v = d16[i];
        test(v.x);
        test(v.y);
        test(v.z);
        test(v.w);
    }
    for (size_t i = (n16 << 4) + (size_t) (blockIdx.x - first) * THREADS + threadIdx.x; i < n; i += stride)
    {
        const uint32_t c = data[i];
        if (only_top ? ((c & 0x7Fu) == 0x7Fu) : ((c & exp_mask) == exp_mask)) hit |= 1u;
    }
    return hit != 0u;
}

// Both operands in one launch: the first blocks_a blocks scan a, the others b.  A hit stores the call's epoch number;
// the flag is never reset (epochs only grow), so no separate clearing launch is needed.
__global__ __launch_bounds__(THREADS) void fp8_special_scan_kernel(uint32_t* flag, uint32_t epoch, const uint8_t* a, size_t na, uint32_t mask_a,
                                                                   int top_a, unsigned blocks_a, const uint8_t* b, size_t nb, uint32_t mask_b,
                                                                   int top_b)
{
    const bool hit = blockIdx.x < blocks_a ? fp8_scan_operand(a, na, mask_a, top_a, 0, blocks_a)
                                           : fp8_scan_operand(b, nb, mask_b, top_b, blocks_a, gridDim.x - blocks_a);
    if (__any(hit) && (threadIdx.x & 63) == 0) *(volatile uint32_t*) flag = epoch;
}

__device__ __forceinline__ void fp8_decode_operand(uint16_t* out, const uint8_t* in, size_t n, int man_bits, int bias, int mode, unsigned first,
                                                   unsigned count)
{
    const size_t stride = (size_t) count * THREADS;
    for (size_t i = (size_t) (blockIdx.x - first) * THREADS + threadIdx.x; i < n; i += stride)
    {
        // every Gaudi fp8 value (any bias 1..30) is exactly representable in bf16
        const uint32_t f = man_bits == 3 ? fp8_to_fp32<3>(in[i], bias, mode) : fp8_to_fp32<2>(in[i], bias, mode);
        out[i] = (uint16_t) (f >> 16);
    }
}

__global__ __launch_bounds__(THREADS) void fp8_to_bf16_kernel(uint16_t* out_a, const uint8_t* in_a, size_t na, int man_a, int bias_a, int mode_a,
                                                              unsigned blocks_a, uint16_t* out_b, const uint8_t* in_b, size_t nb, int man_b,
                                                              int bias_b, int mode_b, const uint32_t* run_flag, uint32_t epoch)
{
    if (run_flag && *run_flag != epoch) return; // only needed when the scan found codes the hardware formats lack
    if (blockIdx.x < blocks_a) fp8_decode_operand(out_a, in_a, na, man_a, bias_a, mode_a, 0, blocks_a);
    else
        fp8_decode_operand(out_b, in_b, nb, man_b, bias_b, mode_b, blocks_a, gridDim.x - blocks_a);
}
} // namespace

size_t gemm_workspace_bytes(const GemmProblem& p)
{
    if (p.split_k <= 1) return 0;
    return (size_t) p.split_k * p.batch[0] * p.batch[1] * p.batch[2] * (size_t) p.M * p.N * sizeof(float);
}

int gemm_pick_split_k(const GemmProblem& p, int num_cus)
{
    if (const int fast = gemm_fast_pick_split_k(p, num_cus)) return fast; // the large-tile kernel takes this problem
    // split the reduction only when the output tiles cannot fill the chip and the reduction is long
    const long long tiles = (long long) ((p.M + TILE - 1) / TILE) * ((p.N + TILE - 1) / TILE) * p.batch[0] * p.batch[1] * p.batch[2];
    const int       es = dt_bytes(p.dtype);
    const int       nk = (p.K + STAGE_BYTES / es - 1) / (STAGE_BYTES / es);
    if (tiles >= num_cus || nk < 16) return 1;
    long long s = (2LL * num_cus + tiles - 1) / tiles;
    if (s > nk / 8) s = nk / 8;
    if (s > 64) s = 64;
    return s < 2 ? 1 : (int) s;
}

hipError_t launch_gemm(const GemmProblem& p, hipStream_t s)
{
    const long long nb = (long long) p.batch[0] * p.batch[1] * p.batch[2];
    if (p.M <= 0 || p.N <= 0 || nb <= 0) return hipSuccess;
    hipError_t e;
    if (nb > 65535)
    {
        // the batch index is the grid's y dimension (at most 65535): slice the slowest batch dimension that has an extent,
        // one launch per slice with the operands' and the output's base pointers moved on
        const int       d = p.batch[2] > 1 ? 2 : (p.batch[1] > 1 ? 1 : 0);
        const long long inner = nb / p.batch[d];
        const int       step = inner >= 65535 ? 1 : (int) (65535 / inner);
        const int       es = dt_bytes(p.dtype), out_es = p.epi.fused ? dt_bytes(p.epi.out_dtype) : 4;
        for (int b = 0; b < p.batch[d]; b += step)
        {
            GemmProblem q = p;
            q.batch[d] = p.batch[d] - b < step ? p.batch[d] - b : step;
            q.A.base = p.A.base + (long long) b * p.A.batch_stride[d] * es;
            q.B.base = p.B.base + (long long) b * p.B.batch_stride[d] * es;
            q.epi.out = (char*) p.epi.out + (long long) b * p.epi.batch_stride[d] * out_es;
            e = launch_gemm(q, s);
            if (e != hipSuccess) return e;
        }
        return hipSuccess;
    }
    if (gemm_large_tile_applicable(p)) e = launch_gemm_large_tile(p, s);
    else
    {
        const int tiles = ((p.M + TILE - 1) / TILE) * ((p.N + TILE - 1) / TILE);
        dim3      grid(tiles, (unsigned) nb, p.split_k > 1 ? p.split_k : 1);
        switch (p.dtype)
        {
            case DT_BF16: launch_gemm_bf16(p, grid, s); break;
            case DT_FP16: launch_gemm_fp16(p, grid, s); break;
            case DT_FP32: launch_gemm_fp32(p, grid, s); break;
            case DT_FP8_143:
            case DT_FP8_152:
                switch ((p.fmt_a & 1) | ((p.fmt_b & 1) << 1))
                {
                    case 0: launch_gemm_fp8_00(p, grid, s); break;
                    case 1: launch_gemm_fp8_10(p, grid, s); break;
                    case 2: launch_gemm_fp8_01(p, grid, s); break;
                    default: launch_gemm_fp8_11(p, grid, s); break;
                }
                break;
            default: return hipErrorInvalidValue;
        }
        e = hipGetLastError();
    }
    if (e != hipSuccess) return e;
    if (p.split_k > 1)
    {
        const long long total = nb * p.M * (long long) p.N;
        const long long items = (p.N & 3) == 0 && ((uintptr_t) p.workspace & 15u) == 0 ? total >> 2 : total; // four columns per lane
        long long       blocks = (items + THREADS - 1) / THREADS;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned) blocks), dim3(THREADS), 0, s, p);
        e = hipGetLastError();
    }
    return e;
}

namespace
{
__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, size_t n)
{
    const size_t stride = (size_t) gridDim.x * blockDim.x;
    for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = v;
}
} // namespace

hipError_t launch_fill_u32(uint32_t* p, uint32_t v, size_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    size_t blocks = (n + THREADS - 1) / THREADS;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned) blocks), dim3(THREADS), 0, s, p, v, n);
    return hipGetLastError();
}

hipError_t launch_fp8_special_scan2(uint32_t* flag, uint32_t epoch, const void* a, size_t na, int man_bits_a, int mask_kind_a, const void* b,
                                    size_t nb, int man_bits_b, int mask_kind_b, hipStream_t s)
{
    if (mask_kind_a < 0) na = 0;
    if (mask_kind_b < 0) nb = 0;
    if (na + nb == 0) return hipSuccess;
    auto blocks_for = [](size_t n) -> unsigned {
        if (n == 0) return 0;
        size_t blocks = ((n >> 4) + THREADS - 1) / THREADS + 1;
        return (unsigned) (blocks > 1024 ? 1024 : blocks);
    };
    const unsigned ba = blocks_for(na), bb = blocks_for(nb);
    hipLaunchKernelGGL(fp8_special_scan_kernel, dim3(ba + bb), dim3(THREADS), 0, s, flag, epoch, (const uint8_t*) a, na,
                       man_bits_a == 3 ? 0x78u : 0x7Cu, mask_kind_a > 0 ? 1 : 0, ba, (const uint8_t*) b, nb, man_bits_b == 3 ? 0x78u : 0x7Cu,
                       mask_kind_b > 0 ? 1 : 0);
    return hipGetLastError();
}

hipError_t launch_fp8_to_bf16_2(uint16_t* out_a, const uint8_t* in_a, size_t na, int man_bits_a, int bias_a, int mode_a, uint16_t* out_b,
                                const uint8_t* in_b, size_t nb, int man_bits_b, int bias_b, int mode_b, const uint32_t* run_flag, uint32_t epoch,
                                hipStream_t s)
{
    if (na + nb == 0) return hipSuccess;
    auto blocks_for = [](size_t n) -> unsigned {
        if (n == 0) return 0;
        size_t blocks = (n + 8 * THREADS - 1) / (8 * THREADS);
        return (unsigned) (blocks > 1024 ? 1024 : blocks);
    };
    const unsigned ba = blocks_for(na), bb = blocks_for(nb);
    hipLaunchKernelGGL(fp8_to_bf16_kernel, dim3(ba + bb), dim3(THREADS), 0, s, out_a, in_a, na, man_bits_a, bias_a, mode_a, ba, out_b, in_b, nb,
                       man_bits_b, bias_b, mode_b, run_flag, epoch);
    return hipGetLastError();
}

} // namespace mme
