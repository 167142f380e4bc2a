// gemm_kernels.hip -- dispatch of the contraction kernels (instantiated per operand type in gemm_inst_*.hip), the
// split-k reduction and the fp8 helper kernels.
#include "gemm_impl.hpp"

namespace mme
{
// one translation unit per operand type / fp8 flavour pair keeps the build parallel
void launch_gemm_bf16(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp32(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp8_00(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp8_10(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp8_01(const GemmProblem& p, dim3 grid, hipStream_t s);
void launch_gemm_fp8_11(const GemmProblem& p, dim3 grid, hipStream_t s);

namespace
{
// sums the split-k partials in slice order (deterministic) and applies the epilogue
__global__ __launch_bounds__(THREADS) void splitk_reduce_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    KARG GemmProblem& g = *(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr();
    if (g.skip_flag && ((*g.skip_flag != 0u) == (g.skip_if != 0))) return;
    const long long mn = (long long) g.M * g.N;
    const long long nb = (long long) g.batch[0] * g.batch[1] * g.batch[2];
    const long long total = mn * nb;
    for (long long i = (long long) blockIdx.x * THREADS + threadIdx.x; i < total; i += (long long) gridDim.x * THREADS)
    {
        const long long b = i / mn, r = i - b * mn;
        float           x = 0.0f;
        for (int z = 0; z < g.split_k; z++) x += g.workspace[(z * nb + b) * mn + r];
        const int m = (int) (r / g.N), n = (int) (r - (long long) m * g.N);
        int       bz = (int) b;
        const int b0 = bz % g.batch[0];
        bz /= g.batch[0];
        const int       b1 = bz % g.batch[1], b2 = bz / g.batch[1];
        const long long c_off = b0 * g.epi.batch_stride[0] + b1 * g.epi.batch_stride[1] + b2 * g.epi.batch_stride[2];
        if (g.epi.has_alpha) x *= g.epi.alpha;
        if (g.epi.col_exp) x *= pow2_of(g.epi.col_exp[n]);
        store_out(g.epi, c_off + (long long) m * g.epi.ld + n, x);
    }
}

// ---- fp8 helpers --------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(THREADS) void fp8_special_scan_kernel(uint32_t* flag, const uint8_t* data, size_t n, uint32_t exp_mask,
                                                                   int only_top)
{
    const size_t stride = (size_t) gridDim.x * THREADS;
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
    for (size_t i = (size_t) blockIdx.x * THREADS + threadIdx.x; i < n16; i += stride)
    {
        const uint4 v = d16[i];
        test(v.x);
        test(v.y);
        test(v.z);
        test(v.w);
    }
    for (size_t i = (n16 << 4) + (size_t) blockIdx.x * THREADS + threadIdx.x; i < n; i += stride)
    {
        const uint32_t c = data[i];
        if (only_top ? ((c & 0x7Fu) == 0x7Fu) : ((c & exp_mask) == exp_mask)) hit |= 1u;
    }
    if (__any(hit != 0u) && (threadIdx.x & 63) == 0) atomicOr(flag, 1u);
}

__global__ __launch_bounds__(THREADS) void fp8_to_bf16_kernel(uint16_t* out, const uint8_t* in, size_t n, int man_bits, int bias, int mode,
                                                              const uint32_t* run_flag)
{
    if (run_flag && *run_flag == 0u) return; // only needed when the scan found codes the hardware formats lack
    const size_t stride = (size_t) gridDim.x * THREADS;
    for (size_t i = (size_t) blockIdx.x * THREADS + threadIdx.x; i < n; i += stride)
    {
        // every Gaudi fp8 value (any bias 1..30) is exactly representable in bf16
        const uint32_t f = man_bits == 3 ? fp8_to_fp32<3>(in[i], bias, mode) : fp8_to_fp32<2>(in[i], bias, mode);
        out[i] = (uint16_t) (f >> 16);
    }
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
    const int       es = (p.dtype == DT_BF16) ? 2 : (p.dtype == DT_FP32 ? 4 : 1);
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
    if (gemm_fp8_fast_applicable(p)) e = launch_gemm_fp8_fast(p, s);
    else
    {
        const int tiles = ((p.M + TILE - 1) / TILE) * ((p.N + TILE - 1) / TILE);
        dim3      grid(tiles, (unsigned) nb, p.split_k > 1 ? p.split_k : 1);
        switch (p.dtype)
        {
            case DT_BF16: launch_gemm_bf16(p, grid, s); break;
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
        long long       blocks = (total + THREADS - 1) / THREADS;
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

hipError_t launch_fp8_special_scan(uint32_t* flag, const void* data, size_t n, int man_bits, int mask_kind, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    const uint32_t exp_mask = man_bits == 3 ? 0x78u : 0x7Cu;
    size_t         blocks = ((n >> 4) + THREADS - 1) / THREADS + 1;
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL(fp8_special_scan_kernel, dim3((unsigned) blocks), dim3(THREADS), 0, s, flag, (const uint8_t*) data, n, exp_mask,
                       mask_kind);
    return hipGetLastError();
}

hipError_t launch_fp8_to_bf16(uint16_t* out, const uint8_t* in, size_t n, int man_bits, int bias, int mode, const uint32_t* run_flag,
                              hipStream_t s)
{
    if (n == 0) return hipSuccess;
    size_t blocks = (n + THREADS - 1) / THREADS;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(fp8_to_bf16_kernel, dim3((unsigned) blocks), dim3(THREADS), 0, s, out, in, n, man_bits, bias, mode, run_flag);
    return hipGetLastError();
}

} // namespace mme
