// cast_kernels.hip -- bandwidth-bound elementwise kernels: fp32 -> {fp8_143, fp8_152, bf16, fp32} (cast / quantize),
// {fp8, bf16} -> fp32 (dequantize), in-place relu, absmax.
//
// Each follows convertToOutputDataType (mme/mme_reference/mme_reference_impl.cpp:1143-1245) element by element; the
// arithmetic lives in mme_numeric.hpp.  Layout: flat arrays.  A wavefront reads 64 x 16 B = 1 KiB per load
// instruction (fully coalesced) and keeps four such loads in flight per lane; algorithmic traffic is 4 + sizeof(out)
// bytes per element (5 B for fp8, 6 B for bf16), the kernels are HBM-bound.
#include "mme_kernels.hpp"

namespace mme
{
namespace
{
typedef float    v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

constexpr int CAST_THREADS = 256;
constexpr int CAST_UNROLL = 4; // float4 loads in flight per lane
constexpr int DEQUANT_UNROLL = 8; // loads of four codes in flight per lane in cast_to_fp32_kernel

template<int DT>
struct OutVec; // four converted elements
template<>
struct OutVec<DT_FP8_143>
{
    using type = uint32_t;
};
template<>
struct OutVec<DT_FP8_152>
{
    using type = uint32_t;
};
template<>
struct OutVec<DT_BF16>
{
    using type = v2u;
};
template<>
struct OutVec<DT_FP16>
{
    using type = v2u;
};
template<>
struct OutVec<DT_UFP16>
{
    using type = v2u;
};
template<>
struct OutVec<DT_FP32>
{
    using type = v4u;
};

// the per-tensor power of two; skipped (not multiplied by 1) when absent so that NaN payloads reach an fp32 output intact
__device__ __forceinline__ float descale(float v, const CastParams& p) { return p.has_scale ? v * p.scale : v; }

template<int DT, bool FAST>
__device__ __forceinline__ typename OutVec<DT>::type cast4(const v4f& v, const CastParams& p, const v4f& cs)
{
    const uint32_t a = cast_elem<DT, FAST>(descale(v.x, p) * cs.x, p), b = cast_elem<DT, FAST>(descale(v.y, p) * cs.y, p),
                   c = cast_elem<DT, FAST>(descale(v.z, p) * cs.z, p), d = cast_elem<DT, FAST>(descale(v.w, p) * cs.w, p);
    if constexpr (dt_bytes(DT) == 1) return a | (b << 8) | (c << 16) | (d << 24);
    else if constexpr (dt_bytes(DT) == 2)
        return v2u {a | (b << 16), c | (d << 16)};
    else
        return v4u {a, b, c, d};
}
template<int DT, bool FAST>
__device__ __forceinline__ typename OutVec<DT>::type cast4(const v4f& v, const CastParams& p)
{
    const uint32_t a = cast_elem<DT, FAST>(descale(v.x, p), p), b = cast_elem<DT, FAST>(descale(v.y, p), p),
                   c = cast_elem<DT, FAST>(descale(v.z, p), p), d = cast_elem<DT, FAST>(descale(v.w, p), p);
    if constexpr (dt_bytes(DT) == 1) return a | (b << 8) | (c << 16) | (d << 24);
    else if constexpr (dt_bytes(DT) == 2)
        return v2u {a | (b << 16), c | (d << 16)};
    else
        return v4u {a, b, c, d};
}

template<int DT>
__device__ __forceinline__ void store1(void* out, size_t i, uint32_t v)
{
    if constexpr (dt_bytes(DT) == 1) ((uint8_t*) out)[i] = (uint8_t) v;
    else if constexpr (dt_bytes(DT) == 2)
        ((uint16_t*) out)[i] = (uint16_t) v;
    else
        ((uint32_t*) out)[i] = v;
}

__device__ __forceinline__ float pow2_of(int e) { return u2f((uint32_t) (e + 127) << 23); }

// n4 = number of whole float4 groups; the tail (n % 4 elements) is handled by the last lanes of block 0.
// COL: multiply element i by 2^col_exp[i % n_cols] as well (n_cols % 4 == 0 is required by the launcher for COL).
template<int DT, bool FAST, bool COL>
__global__ __launch_bounds__(CAST_THREADS) void cast_from_fp32_kernel(void* __restrict__ out,
                                                                      const float* __restrict__ in,
                                                                      size_t n,
                                                                      CastParams p,
                                                                      const int32_t* __restrict__ col_exp,
                                                                      uint32_t n_cols)
{
    using OV = typename OutVec<DT>::type;
    const size_t  n4 = n >> 2;
    const v4f*    in4 = reinterpret_cast<const v4f*>(in);
    OV*           out4 = reinterpret_cast<OV*>(out);
    // A workgroup owns contiguous chunks of CAST_UNROLL x 256 float4 (16 KiB of input): four fully coalesced 1 KiB
    // loads per wavefront are issued back to back, then converted and stored.  Streaming (non-temporal) accesses and
    // one chunk per workgroup measured fastest on MI355X (6.2 TB/s against 4.5 TB/s for a grid-stride loop).
    constexpr size_t CHUNK = (size_t) CAST_UNROLL * CAST_THREADS;
    const size_t     n_chunks = (n4 + CHUNK - 1) / CHUNK;
    for (size_t c = blockIdx.x; c < n_chunks; c += gridDim.x)
    {
        const size_t i = c * CHUNK + threadIdx.x;
        if (c * CHUNK + CHUNK <= n4)
        {
            v4f v[CAST_UNROLL];
#pragma unroll
            for (int j = 0; j < CAST_UNROLL; j++) v[j] = __builtin_nontemporal_load(in4 + i + j * CAST_THREADS);
#pragma unroll
            for (int j = 0; j < CAST_UNROLL; j++)
            {
                OV o;
                if constexpr (COL)
                {
                    const uint32_t c0 = (uint32_t) (((i + j * CAST_THREADS) << 2) % n_cols);
                    const int4     ce = *reinterpret_cast<const int4*>(col_exp + c0);
                    o = cast4<DT, FAST>(v[j], p, v4f {pow2_of(ce.x), pow2_of(ce.y), pow2_of(ce.z), pow2_of(ce.w)});
                }
                else
                    o = cast4<DT, FAST>(v[j], p);
                __builtin_nontemporal_store(o, out4 + i + j * CAST_THREADS);
            }
        }
        else
        {
            for (size_t k = i; k < n4; k += CAST_THREADS)
            {
                const v4f v = in4[k];
                OV        o;
                if constexpr (COL)
                {
                    const uint32_t c0 = (uint32_t) ((k << 2) % n_cols);
                    const int4     ce = *reinterpret_cast<const int4*>(col_exp + c0);
                    o = cast4<DT, FAST>(v, p, v4f {pow2_of(ce.x), pow2_of(ce.y), pow2_of(ce.z), pow2_of(ce.w)});
                }
                else
                    o = cast4<DT, FAST>(v, p);
                out4[k] = o;
            }
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3))
    {
        const size_t k = (n4 << 2) + threadIdx.x;
        float        v = in[k];
        if (p.has_scale) v *= p.scale;
        if constexpr (COL) v *= pow2_of(col_exp[k % n_cols]);
        store1<DT>(out, k, cast_elem<DT, FAST>(v, p));
    }
}

// scalar form for per-column scales whose period is not a multiple of 4, or unaligned buffers
template<int DT, bool FAST>
__global__ __launch_bounds__(CAST_THREADS) void cast_from_fp32_scalar_kernel(void* __restrict__ out,
                                                                             const float* __restrict__ in,
                                                                             size_t n,
                                                                             CastParams p,
                                                                             const int32_t* __restrict__ col_exp,
                                                                             uint32_t n_cols)
{
    const size_t stride = (size_t) gridDim.x * CAST_THREADS;
    for (size_t i = (size_t) blockIdx.x * CAST_THREADS + threadIdx.x; i < n; i += stride)
    {
        float v = in[i];
        if (p.has_scale) v *= p.scale;
        if (col_exp) v *= pow2_of(col_exp[i % n_cols]);
        store1<DT>(out, i, cast_elem<DT, FAST>(v, p));
    }
}

// ---- dequantize -----------------------------------------------------------------------------------------------
// fp8 -> fp32 in a handful of vector instructions (the bulk dequantiser spends more time on the step-by-step decoder than on
// memory: 25 instructions per element).  The magnitude bits, shifted so that the exponent fields line up, are an fp32 number
// with the wrong exponent bias: 2^(e - 127) x 1.m, or the fp32 denormal m x 2^(-149 + 23 - M) for e = 0.  Multiplied by
// 2^(127 - bias) that is the code's value either way (the product of an fp32 denormal and a power of two is exact, and
// fp32 denormals are not flushed in these kernels); the codes that are inf / NaN in the tensor's mode are patched in after.
// Equal to fp8_to_fp32 for all 256 codes, every bias and mode (tested exhaustively through the kernel).
template<int M>
__device__ __forceinline__ float fp8_to_fp32_by_scaling(uint32_t code, float two_pow_127_minus_bias, int mode)
{
    constexpr uint32_t exp_all = (0x7Fu >> M) << M;
    const uint32_t     sign = (code & 0x80u) << 24, mag = code & 0x7Fu;
    uint32_t           r = f2u(u2f(mag << (23 - M)) * two_pow_127_minus_bias) | sign;
    if (mode == 0 && (mag & exp_all) == exp_all) r = (mag & ~exp_all) ? 0x7FFFFFFFu : (sign | 0x7F800000u);
    if (mode == 2 && mag == 0x7Fu) r = 0x7FFFFFFFu;
    return u2f(r);
}

template<int DT>
__device__ __forceinline__ float decode1(uint32_t code, int bias, int mode)
{
    if constexpr (DT == DT_FP8_143) return fp8_to_fp32_by_scaling<3>(code, u2f((uint32_t) (254 - bias) << 23), mode);
    else if constexpr (DT == DT_FP8_152)
        return fp8_to_fp32_by_scaling<2>(code, u2f((uint32_t) (254 - bias) << 23), mode);
    else if constexpr (DT == DT_FP16)
        return u2f(cfp16_to_fp32<5>(code, bias, mode != 0));
    else if constexpr (DT == DT_UFP16)
        return u2f(cfp16_to_fp32<6>(code, bias, mode != 0));
    else
        return u2f(code << 16);
}

template<int DT>
__global__ __launch_bounds__(CAST_THREADS) void cast_to_fp32_kernel(float* __restrict__ out,
                                                                    const void* __restrict__ in,
                                                                    size_t n,
                                                                    int bias,
                                                                    int mode,
                                                                    float scale,
                                                                    int has_scale,
                                                                    const int32_t* __restrict__ col_exp,
                                                                    uint32_t n_cols,
                                                                    int vec_ok,
                                                                    const uint32_t* __restrict__ run_flag,
                                                                    uint32_t run_epoch)
{
    if (run_flag && *run_flag != run_epoch) return; // predicated launch: runs only when the flag holds this call's epoch
    const size_t stride = (size_t) gridDim.x * CAST_THREADS;
    const size_t t = (size_t) blockIdx.x * CAST_THREADS + threadIdx.x;
    size_t       done = 0;
    if (vec_ok)
    {
        // four elements per lane and step: one 4 B (fp8) / 8 B (bf16) load, one 16 B streaming store; a workgroup owns
        // contiguous chunks of 8 x 256 such groups (32 KiB of output; measured on 2^28 fp8 codes: 238 us with 4 x 256, 222 us
        // with 8, 265 us with 16; fewer, looping workgroups are slower still)
        constexpr int    CAST_UNROLL = DEQUANT_UNROLL;
        const size_t     n4 = n >> 2;
        v4f*             out4 = reinterpret_cast<v4f*>(out);
        constexpr size_t CHUNK = (size_t) CAST_UNROLL * CAST_THREADS;
        const size_t     n_chunks = (n4 + CHUNK - 1) / CHUNK;
        for (size_t ch = blockIdx.x; ch < n_chunks; ch += gridDim.x)
        {
            uint32_t raw[CAST_UNROLL][2];
#pragma unroll
            for (int u = 0; u < CAST_UNROLL; u++)
            {
                const size_t i = ch * CHUNK + threadIdx.x + (size_t) u * CAST_THREADS;
                raw[u][0] = raw[u][1] = 0;
                if (i < n4)
                {
                    if constexpr (dt_bytes(DT) == 2)
                    {
                        const v2u r = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(in) + i);
                        raw[u][0] = r.x;
                        raw[u][1] = r.y;
                    }
                    else
                        raw[u][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(in) + i);
                }
            }
#pragma unroll
            for (int u = 0; u < CAST_UNROLL; u++)
            {
                const size_t i = ch * CHUNK + threadIdx.x + (size_t) u * CAST_THREADS;
                if (i >= n4) continue;
                uint32_t c[4];
                if constexpr (dt_bytes(DT) == 2)
                {
                    c[0] = raw[u][0] & 0xFFFFu;
                    c[1] = raw[u][0] >> 16;
                    c[2] = raw[u][1] & 0xFFFFu;
                    c[3] = raw[u][1] >> 16;
                }
                else
                {
                    c[0] = raw[u][0] & 0xFFu;
                    c[1] = (raw[u][0] >> 8) & 0xFFu;
                    c[2] = (raw[u][0] >> 16) & 0xFFu;
                    c[3] = raw[u][0] >> 24;
                }
                float f[4];
#pragma unroll
                for (int j = 0; j < 4; j++)
                {
                    f[j] = decode1<DT>(c[j], bias, mode);
                    if (has_scale) f[j] *= scale;
                    if (col_exp) f[j] *= pow2_of(col_exp[((i << 2) + j) % n_cols]);
                }
                __builtin_nontemporal_store(v4f {f[0], f[1], f[2], f[3]}, out4 + i);
            }
        }
        done = n4 << 2;
    }
    for (size_t i = done + t; i < n; i += stride)
    {
        uint32_t c;
        if constexpr (dt_bytes(DT) == 2) c = reinterpret_cast<const uint16_t*>(in)[i];
        else
            c = reinterpret_cast<const uint8_t*>(in)[i];
        float f = decode1<DT>(c, bias, mode);
        if (has_scale) f *= scale;
        if (col_exp) f *= pow2_of(col_exp[i % n_cols]);
        out[i] = f;
    }
}

// ---- stochastic conversions ---------------------------------------------------------------------------------------
// The reference keeps LFSR registers and hands element i the value of register i % L (L = 128 for fp8, 64 for bf16),
// stepping that register once after every use (convertToOutputDataType, mme/mme_reference/mme_reference_impl.cpp:
// 1143-1245).  Element i therefore sees register i % L after i / L steps.  The step is linear over GF(2), so a thread
// reaches step t directly: jump[k * 32 + b] is the image of bit b under 2^k steps, built on the host for the
// calculator's polynomial.  Thread g owns register g % L for STOCH_STEPS consecutive steps; at every step the L threads
// of a group touch L consecutive elements.
constexpr int STOCH_STEPS = 32;

__device__ __forceinline__ uint32_t lfsr_jump(uint32_t s, unsigned long long t, const uint32_t* __restrict__ jump)
{
    for (int k = 0; t != 0; k++, t >>= 1)
        if (t & 1ull)
        {
            uint32_t y = 0;
#pragma unroll
            for (int b = 0; b < 32; b++) y ^= ((s >> b) & 1u) ? jump[k * 32 + b] : 0u;
            s = y;
        }
    return s;
}

template<int DT>
__global__ __launch_bounds__(CAST_THREADS) void cast_stochastic_kernel(void* __restrict__ out,
                                                                       const float* __restrict__ in,
                                                                       size_t n,
                                                                       CastParams p,
                                                                       int sftz,
                                                                       int reseed,
                                                                       uint32_t polynomial,
                                                                       LfsrRegisters regs,
                                                                       const uint32_t* __restrict__ jump)
{
    constexpr int    L = (dt_bytes(DT) == 2) ? 64 : 128;
    const size_t     g = (size_t) blockIdx.x * CAST_THREADS + threadIdx.x;
    const int        r = (int) (g & (L - 1));
    const size_t     t0 = (g / L) * STOCH_STEPS;
    uint32_t         state = regs.v[r];
    if (t0 * L + r >= n) return;
    if (reseed) state = lfsr_jump(state, t0, jump);
    for (int j = 0; j < STOCH_STEPS; j++)
    {
        const size_t i = (t0 + j) * L + r;
        if (i >= n) break;
        const uint32_t u = f2u(in[i]);
        if constexpr (DT == DT_BF16) ((uint16_t*) out)[i] = (uint16_t) fp32_to_bf16_stochastic(u, p.rm, state, p.clip_fp, p.ftz, p.clip_inf_in);
        else if constexpr (DT == DT_FP16 || DT == DT_UFP16)
            ((uint16_t*) out)[i] = (uint16_t) fp32_to_cfp16<(DT == DT_UFP16) ? 6 : 5>(u, p.exp_bias, p.rm, state, p.ftz, p.clip_fp, p.clip_inf_in,
                                                                                     p.inf_nan_mode != 0);
        else
            ((uint8_t*) out)[i] = (uint8_t) fp32_to_fp8_stochastic<(DT == DT_FP8_143) ? 3 : 2>(u, p.exp_bias, p.rm, state, p.ftz, p.clip_fp,
                                                                                               p.clip_inf_in, sftz, p.inf_nan_mode);
        if (reseed) state = lfsr32_step(state, polynomial);
    }
}

__global__ __launch_bounds__(CAST_THREADS) void relu_inplace_kernel(float* __restrict__ x, size_t n)
{
    const size_t stride = (size_t) gridDim.x * CAST_THREADS;
    for (size_t i = (size_t) blockIdx.x * CAST_THREADS + threadIdx.x; i < n; i += stride) x[i] = relu_ref(x[i]);
}

// ---- absmax: wavefront reduction with DPP-free shuffles, one atomicMax on the bit pattern per block -------------
__global__ __launch_bounds__(CAST_THREADS) void absmax_kernel(uint32_t* __restrict__ out_bits,
                                                              const float* __restrict__ in,
                                                              size_t n,
                                                              int vec_ok)
{
    const size_t stride = (size_t) gridDim.x * CAST_THREADS;
    const size_t t = (size_t) blockIdx.x * CAST_THREADS + threadIdx.x;
    uint32_t     m = 0; // |x| of non-NaN fp32 values orders like the unsigned bit pattern
    auto         acc = [&](float f) {
        const uint32_t a = f2u(f) & 0x7FFFFFFFu;
        if (a <= 0x7F800000u) m = max(m, a);
    };
    size_t done = 0;
    if (vec_ok)
    {
        const size_t  n4 = n >> 2;
        const v4f*    in4 = reinterpret_cast<const v4f*>(in);
        for (size_t i = t; i < n4; i += stride)
        {
            const v4f v = __builtin_nontemporal_load(in4 + i);
            acc(v.x);
            acc(v.y);
            acc(v.z);
            acc(v.w);
        }
        done = n4 << 2;
    }
    for (size_t i = done + t; i < n; i += stride) acc(in[i]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = max(m, (uint32_t) __shfl_xor((int) m, off, 64));
    __shared__ uint32_t wave_max[CAST_THREADS / 64];
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        uint32_t b = wave_max[0];
        for (int w = 1; w < CAST_THREADS / 64; w++) b = max(b, wave_max[w]);
        atomicMax(out_bits, b);
    }
}

__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, size_t n)
{
    const size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

int grid_for(size_t work_items, int max_blocks)
{
    size_t b = (work_items + CAST_THREADS - 1) / CAST_THREADS;
    if (b < 1) b = 1;
    if (b > (size_t) max_blocks) b = (size_t) max_blocks;
    return (int) b;
}

template<int DT, bool FAST>
void launch_cast_dt(void* out, const float* in, size_t n, const CastParams& p, const int32_t* col, size_t n_cols,
                    hipStream_t s)
{
    const bool aligned = (((uintptr_t) out | (uintptr_t) in) & 15u) == 0;
    if (aligned && (!col || ((n_cols & 3u) == 0 && ((uintptr_t) col & 15u) == 0)))
    {
        // one 16 KiB chunk per workgroup, up to 2^20 workgroups (a 16 GiB input) before workgroups loop
        const int grid = grid_for(((n >> 2) / CAST_UNROLL + 1) , 1 << 20);
        if (col)
            hipLaunchKernelGGL((cast_from_fp32_kernel<DT, FAST, true>), dim3(grid), dim3(CAST_THREADS), 0, s, out, in, n, p,
                               col, (uint32_t) n_cols);
        else
            hipLaunchKernelGGL((cast_from_fp32_kernel<DT, FAST, false>), dim3(grid), dim3(CAST_THREADS), 0, s, out, in, n,
                               p, col, (uint32_t) n_cols);
    }
    else
    {
        const int grid = grid_for(n, 8192);
        hipLaunchKernelGGL((cast_from_fp32_scalar_kernel<DT, FAST>), dim3(grid), dim3(CAST_THREADS), 0, s, out, in, n, p,
                           col, (uint32_t) (n_cols ? n_cols : 1));
    }
}
} // namespace

hipError_t launch_cast_from_fp32(void* out, const float* in, size_t n, const CastParams& p, const int32_t* col,
                                 size_t n_cols, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    const bool fast = cast_params_fast(p);
    switch (p.dtype)
    {
        case DT_FP8_143:
            fast ? launch_cast_dt<DT_FP8_143, true>(out, in, n, p, col, n_cols, s)
                 : launch_cast_dt<DT_FP8_143, false>(out, in, n, p, col, n_cols, s);
            break;
        case DT_FP8_152:
            fast ? launch_cast_dt<DT_FP8_152, true>(out, in, n, p, col, n_cols, s)
                 : launch_cast_dt<DT_FP8_152, false>(out, in, n, p, col, n_cols, s);
            break;
        case DT_BF16:
            fast ? launch_cast_dt<DT_BF16, true>(out, in, n, p, col, n_cols, s)
                 : launch_cast_dt<DT_BF16, false>(out, in, n, p, col, n_cols, s);
            break;
        case DT_FP16:
            fast ? launch_cast_dt<DT_FP16, true>(out, in, n, p, col, n_cols, s) : launch_cast_dt<DT_FP16, false>(out, in, n, p, col, n_cols, s);
            break;
        case DT_UFP16:
            fast ? launch_cast_dt<DT_UFP16, true>(out, in, n, p, col, n_cols, s) : launch_cast_dt<DT_UFP16, false>(out, in, n, p, col, n_cols, s);
            break;
        case DT_FP32: launch_cast_dt<DT_FP32, false>(out, in, n, p, col, n_cols, s); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_cast_to_fp32(float* out, const void* in, int dtype, int bias, int mode, size_t n, float scale,
                               int has_scale, const int32_t* col, size_t n_cols, hipStream_t s, const uint32_t* run_flag, uint32_t run_epoch)
{
    if (n == 0) return hipSuccess;
    const int vec_ok = (((uintptr_t) out & 15u) == 0) && (((uintptr_t) in & 7u) == 0);
    const int grid = vec_ok ? grid_for((n >> 2) / DEQUANT_UNROLL + 1, 1 << 20) : grid_for(n, 8192);
    const uint32_t nc = (uint32_t) (n_cols ? n_cols : 1);
    switch (dtype)
    {
        case DT_FP8_143:
            hipLaunchKernelGGL((cast_to_fp32_kernel<DT_FP8_143>), dim3(grid), dim3(CAST_THREADS), 0, s, out, in, n, bias,
                               mode, scale, has_scale, col, nc, vec_ok, run_flag, run_epoch);
            break;
        case DT_FP8_152:
            hipLaunchKernelGGL((cast_to_fp32_kernel<DT_FP8_152>), dim3(grid), dim3(CAST_THREADS), 0, s, out, in, n, bias,
                               mode, scale, has_scale, col, nc, vec_ok, run_flag, run_epoch);
            break;
        case DT_BF16:
            hipLaunchKernelGGL((cast_to_fp32_kernel<DT_BF16>), dim3(grid), dim3(CAST_THREADS), 0, s, out, in, n, bias, mode,
                               scale, has_scale, col, nc, vec_ok, run_flag, run_epoch);
            break;
        case DT_FP16:
            hipLaunchKernelGGL((cast_to_fp32_kernel<DT_FP16>), dim3(grid), dim3(CAST_THREADS), 0, s, out, in, n, bias, mode, scale, has_scale, col, nc,
                               vec_ok, run_flag, run_epoch);
            break;
        case DT_UFP16:
            hipLaunchKernelGGL((cast_to_fp32_kernel<DT_UFP16>), dim3(grid), dim3(CAST_THREADS), 0, s, out, in, n, bias, mode, scale, has_scale, col, nc,
                               vec_ok, run_flag, run_epoch);
            break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_cast_stochastic(void* out, const float* in, size_t n, const CastParams& p, int sftz, int reseed, uint32_t polynomial,
                                  const LfsrRegisters& regs, const uint32_t* jump, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    const size_t L = dt_bytes(p.dtype) == 2 ? 64 : 128;
    const size_t groups = ((n + L - 1) / L + STOCH_STEPS - 1) / STOCH_STEPS;
    const size_t blocks = (groups * L + CAST_THREADS - 1) / CAST_THREADS;
    if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
    switch (p.dtype)
    {
        case DT_FP8_143:
            hipLaunchKernelGGL((cast_stochastic_kernel<DT_FP8_143>), dim3((unsigned) blocks), dim3(CAST_THREADS), 0, s, out, in, n, p, sftz, reseed,
                               polynomial, regs, jump);
            break;
        case DT_FP8_152:
            hipLaunchKernelGGL((cast_stochastic_kernel<DT_FP8_152>), dim3((unsigned) blocks), dim3(CAST_THREADS), 0, s, out, in, n, p, sftz, reseed,
                               polynomial, regs, jump);
            break;
        case DT_BF16:
            hipLaunchKernelGGL((cast_stochastic_kernel<DT_BF16>), dim3((unsigned) blocks), dim3(CAST_THREADS), 0, s, out, in, n, p, sftz, reseed,
                               polynomial, regs, jump);
            break;
        case DT_FP16:
            hipLaunchKernelGGL((cast_stochastic_kernel<DT_FP16>), dim3((unsigned) blocks), dim3(CAST_THREADS), 0, s, out, in, n, p, sftz, reseed,
                               polynomial, regs, jump);
            break;
        case DT_UFP16:
            hipLaunchKernelGGL((cast_stochastic_kernel<DT_UFP16>), dim3((unsigned) blocks), dim3(CAST_THREADS), 0, s, out, in, n, p, sftz, reseed,
                               polynomial, regs, jump);
            break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// ---- weights of transposed_dedx: out[i0][i1][s][r][q] = in[i1][i0][S - 1 - s][r][q] (first index contiguous on both
// sides), i.e. transposeTensor + reverseWeightsDimS of the reference (mme_reference_impl.cpp:324-393, 625-647) -----------
template<typename T>
__global__ __launch_bounds__(CAST_THREADS) void repack_transposed_weights_kernel(T* __restrict__ out, const T* __restrict__ in, uint32_t n0, uint32_t n1,
                                                                                 uint32_t S, size_t total)
{
    const size_t stride = (size_t) gridDim.x * CAST_THREADS;
    for (size_t i = (size_t) blockIdx.x * CAST_THREADS + threadIdx.x; i < total; i += stride)
    {
        // i = i0 + n1 * (i1 + n0 * (s + S * rq))
        const size_t   a = i / n1, b = a / n0, rq = b / S;
        const uint32_t i0 = (uint32_t) (i - a * n1), i1 = (uint32_t) (a - b * n0), s = (uint32_t) (b - rq * S);
        out[i] = in[i1 + (size_t) n0 * (i0 + (size_t) n1 * ((S - 1 - s) + (size_t) S * rq))];
    }
}

hipError_t launch_repack_transposed_weights(void* out, const void* in, int elem_size, uint32_t n0, uint32_t n1, uint32_t S, size_t total, hipStream_t s)
{
    if (total == 0) return hipSuccess;
    const dim3 grid(grid_for(total, 4096)), block(CAST_THREADS);
    switch (elem_size)
    {
        case 1: hipLaunchKernelGGL(repack_transposed_weights_kernel<uint8_t>, grid, block, 0, s, (uint8_t*) out, (const uint8_t*) in, n0, n1, S, total); break;
        case 2: hipLaunchKernelGGL(repack_transposed_weights_kernel<uint16_t>, grid, block, 0, s, (uint16_t*) out, (const uint16_t*) in, n0, n1, S, total); break;
        case 4: hipLaunchKernelGGL(repack_transposed_weights_kernel<uint32_t>, grid, block, 0, s, (uint32_t*) out, (const uint32_t*) in, n0, n1, S, total); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// ---- memory-write reductions: memory = memory (op) mme_out, element by element (doMemoryWrite, mme_reference_impl.cpp:
// 718-768).  16 bytes per lane where both buffers are 16-byte aligned; 12 B/elt (fp32) or 6 B/elt (bf16) of traffic ------
template<int DT>
__global__ __launch_bounds__(CAST_THREADS) void memory_write_reduce_kernel(void* __restrict__ memory, const void* __restrict__ mme_out, size_t n,
                                                                           int op, int rm, int clip, int vec_ok)
{
    const size_t stride = (size_t) gridDim.x * CAST_THREADS;
    const size_t t = (size_t) blockIdx.x * CAST_THREADS + threadIdx.x;
    constexpr int PER = 16 / dt_bytes(DT); // elements per 16 bytes
    size_t        done = 0;
    if (vec_ok)
    {
        const size_t nv = n / PER;
        v4u*         m4 = reinterpret_cast<v4u*>(memory);
        const v4u*   o4 = reinterpret_cast<const v4u*>(mme_out);
        for (size_t i = t; i < nv; i += stride)
        {
            const v4u a = m4[i], b = o4[i];
            v4u       r;
#pragma unroll
            for (int w = 0; w < 4; w++)
            {
                if constexpr (DT == DT_FP32) r[w] = rmw_elem<23>(a[w], b[w], op, rm, clip);
                else if constexpr (DT == DT_FP16)
                    r[w] = rmw_elem_fp16(a[w] & 0xFFFFu, b[w] & 0xFFFFu, op, rm, clip) | (rmw_elem_fp16(a[w] >> 16, b[w] >> 16, op, rm, clip) << 16);
                else if constexpr (DT == DT_FP8_152)
                {
                    r[w] = 0u;
#pragma unroll
                    for (int k = 0; k < 4; k++) r[w] |= rmw_elem_fp8_152((a[w] >> (8 * k)) & 0xFFu, (b[w] >> (8 * k)) & 0xFFu, op, rm, clip) << (8 * k);
                }
                else
                    r[w] = (rmw_elem<7>(a[w] << 16, b[w] << 16, op, rm, clip) >> 16) |
                           (rmw_elem<7>(a[w] & 0xFFFF0000u, b[w] & 0xFFFF0000u, op, rm, clip) & 0xFFFF0000u);
            }
            m4[i] = r;
        }
        done = nv * PER;
    }
    for (size_t i = done + t; i < n; i += stride)
    {
        if constexpr (DT == DT_FP32) ((uint32_t*) memory)[i] = rmw_elem<23>(((uint32_t*) memory)[i], ((const uint32_t*) mme_out)[i], op, rm, clip);
        else if constexpr (DT == DT_FP16)
            ((uint16_t*) memory)[i] = (uint16_t) rmw_elem_fp16(((uint16_t*) memory)[i], ((const uint16_t*) mme_out)[i], op, rm, clip);
        else if constexpr (DT == DT_FP8_152)
            ((uint8_t*) memory)[i] = (uint8_t) rmw_elem_fp8_152(((uint8_t*) memory)[i], ((const uint8_t*) mme_out)[i], op, rm, clip);
        else
            ((uint16_t*) memory)[i] =
                (uint16_t) (rmw_elem<7>((uint32_t) ((uint16_t*) memory)[i] << 16, (uint32_t) ((const uint16_t*) mme_out)[i] << 16, op, rm, clip) >> 16);
    }
}

hipError_t launch_memory_write_reduce(void* memory, const void* mme_out, int dtype, size_t n, int op, int rm, int clip, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    const int  vec_ok = (((uintptr_t) memory | (uintptr_t) mme_out) & 15u) == 0;
    const dim3 grid(grid_for(n / 4 + 1, 2048)), block(CAST_THREADS);
    if (dtype == DT_FP32) hipLaunchKernelGGL(memory_write_reduce_kernel<DT_FP32>, grid, block, 0, s, memory, mme_out, n, op, rm, clip, vec_ok);
    else if (dtype == DT_BF16)
        hipLaunchKernelGGL(memory_write_reduce_kernel<DT_BF16>, grid, block, 0, s, memory, mme_out, n, op, rm, clip, vec_ok);
    else if (dtype == DT_FP16)
        hipLaunchKernelGGL(memory_write_reduce_kernel<DT_FP16>, grid, block, 0, s, memory, mme_out, n, op, rm, clip, vec_ok);
    else if (dtype == DT_FP8_152)
        hipLaunchKernelGGL(memory_write_reduce_kernel<DT_FP8_152>, grid, block, 0, s, memory, mme_out, n, op, rm, clip, vec_ok);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

// ---- operands of the tf32 flavour: fp32 words rounded to tf32 on entry (Gaudi3Tf32Fma::fma_vec, chip_fma/gaudi3_fma.cpp:237-272)
__global__ __launch_bounds__(CAST_THREADS) void round_to_tf32_kernel(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, size_t n, int clip,
                                                                     int clip_inf_in, const uint32_t* __restrict__ run_flag, uint32_t run_epoch)
{
    if (run_flag && *run_flag != run_epoch) return;
    const size_t stride = (size_t) gridDim.x * CAST_THREADS;
    for (size_t i = (size_t) blockIdx.x * CAST_THREADS + threadIdx.x; i < n; i += stride) out[i] = fp32_to_tf32(in[i], clip, clip_inf_in);
}

hipError_t launch_round_to_tf32(void* out, const void* in, size_t n, int clip, int clip_inf_in, hipStream_t s, const uint32_t* run_flag,
                                uint32_t run_epoch)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(round_to_tf32_kernel, dim3(grid_for(n, 8192)), dim3(CAST_THREADS), 0, s, (uint32_t*) out, (const uint32_t*) in, n, clip,
                       clip_inf_in, run_flag, run_epoch);
    return hipGetLastError();
}

// ---- fp16 / ufp16 / tf32 operands as two bf16 parts -------------------------------------------------------------------
// These types carry 11 significant bits; bf16 carries 8.  value = hi + lo with hi = the value truncated to bf16 and lo = the
// exact remainder (at most 3 significant bits), so a * b = hi_a hi_b + hi_a lo_b + lo_a hi_b + lo_a lo_b with every product
// exact in fp32: the contraction becomes one bf16 contraction over 4 K, operand A laid out as [hi | hi | lo | lo] along k and
// operand B as [hi | lo | hi | lo].  The copies are dense: (batch, f, 4 K) when the source is k-contiguous, (batch, 4 K, f)
// otherwise; batch dimensions the source broadcasts (stride 0) have extent 1 in the copy.  A value that is not finite
// cannot be split (inf * 0 appears among the partial products), nor can a value so small that its low part would fall
// under bf16's normal range (below 2^-100 for fp32, 2^-112 for the 11-bit types): either stores `epoch` into *flag and the
// caller's predicated launches take the fp32 path instead.  V elements per lane along the contiguous index (8 with 16-byte accesses, or 1).
// fp32 operands (24 significant bits) take three parts, value = hi + mid + lo of 8 bits each, and six K-blocks: A as
// [hi | hi | mid | hi | lo | mid], B as [hi | mid | hi | lo | hi | mid]; the three products left out (mid lo, lo mid, lo lo)
// are below 2^-23 of hi hi, the rounding step of the fp32 accumulation itself.
template<int DT, int V>
__global__ __launch_bounds__(CAST_THREADS) void split_bf16_kernel(uint16_t* __restrict__ out, const void* __restrict__ in, SplitBf16Args a)
{
    const long long C = a.k_contig ? a.K : a.F, O = a.k_contig ? a.F : a.K, groups = C / V;
    const long long total = groups * O * a.e[0] * a.e[1] * a.e[2];
    const long long part = a.k_contig ? (long long) a.K : (long long) a.K * a.F; // elements between the K-blocks
    const int       hi_part1 = a.is_b ? 2 : 1, lo_part0 = a.is_b ? 1 : 2;          // hi -> parts 0 and hi_part1, lo -> lo_part0 and 3
    constexpr int   NB = DT == DT_FP32 ? 6 : 4;                                    // K-blocks
    // three parts: which part (0 hi, 1 mid, 2 lo) each of the six K-blocks holds
    const int       p3[6] = {0, a.is_b ? 1 : 0, a.is_b ? 0 : 1, a.is_b ? 2 : 0, a.is_b ? 0 : 2, 1};
    bool            special = false;
    for (long long t = (long long) blockIdx.x * CAST_THREADS + threadIdx.x; t < total; t += (long long) gridDim.x * CAST_THREADS)
    {
        const long long cg = t % groups, r = t / groups, o = r % O;
        long long       b = r / O;
        const long long f = a.k_contig ? o : cg * V, k = a.k_contig ? cg * V : o;
        const long long dst = a.k_contig ? (b * a.F + f) * NB * a.K + k : (b * NB * a.K + k) * a.F + f;
        const int       b0 = (int) (b % a.e[0]);
        b /= a.e[0];
        const int       b1 = (int) (b % a.e[1]), b2 = (int) (b / a.e[1]);
        const long long src = b0 * a.bs[0] + b1 * a.bs[1] + b2 * a.bs[2] + f * a.sf + k * a.sk;
        uint32_t        raw[V];
        if constexpr (V == 8 && (DT == DT_TF32 || DT == DT_FP32))
        {
            const v4u x = *(const v4u*) ((const uint32_t*) in + src), y = *(const v4u*) ((const uint32_t*) in + src + 4);
            raw[0] = x.x, raw[1] = x.y, raw[2] = x.z, raw[3] = x.w, raw[4] = y.x, raw[5] = y.y, raw[6] = y.z, raw[7] = y.w;
        }
        else if constexpr (V == 8)
        {
            const v4u x = *(const v4u*) ((const uint16_t*) in + src);
            raw[0] = x.x & 0xFFFFu, raw[1] = x.x >> 16, raw[2] = x.y & 0xFFFFu, raw[3] = x.y >> 16;
            raw[4] = x.z & 0xFFFFu, raw[5] = x.z >> 16, raw[6] = x.w & 0xFFFFu, raw[7] = x.w >> 16;
        }
        else if constexpr (DT == DT_TF32 || DT == DT_FP32)
            raw[0] = ((const uint32_t*) in)[src];
        else
            raw[0] = ((const uint16_t*) in)[src];
        uint32_t hi[V], lo[V], mid[V];
#pragma unroll
        for (int j = 0; j < V; j++)
        {
            uint32_t u;
            if constexpr (DT == DT_TF32) u = fp32_to_tf32(raw[j], a.clip, a.clip_inf_in);
            else if constexpr (DT == DT_FP32)
                u = raw[j];
            else
                u = f2u(decode1<DT>(raw[j], a.bias, a.mode));
            special = special || ((u & 0x7F800000u) == 0x7F800000u);
            // the lowest part ends at the value's last significant bit, 2^-23 (fp32) or 2^-10 (the 11-bit types) below its
            // exponent, and has to be a normal bf16 number itself (smallest 2^-126) so that no matrix instruction may flush
            // it: a non-zero value below 2^-100 (fp32) / 2^-112 cannot be split either
            constexpr uint32_t MIN_EXP_FIELD = DT == DT_FP32 ? 127 - 100 : 127 - 112;
            special = special || ((u & 0x7FFFFFFFu) != 0 && ((u >> 23) & 0xFFu) < MIN_EXP_FIELD);
            const uint32_t h = u & 0xFFFF0000u;
            hi[j] = h >> 16;
            const float rest = u2f(u) - u2f(h);
            if constexpr (DT == DT_FP32)
            {
                const uint32_t m = f2u(rest) & 0xFFFF0000u;
                mid[j] = m >> 16;
                lo[j] = f2u(rest - u2f(m)) >> 16;
            }
            else
            {
                mid[j] = 0;
                lo[j] = f2u(rest) >> 16;
            }
        }
        if constexpr (DT == DT_FP32)
        {
            // six K-blocks
#pragma unroll
            for (int blk = 0; blk < 6; blk++)
            {
                const int which = p3[blk];
                if constexpr (V == 8)
                {
                    uint32_t w[8];
#pragma unroll
                    for (int j = 0; j < 8; j++) w[j] = which == 0 ? hi[j] : (which == 1 ? mid[j] : lo[j]);
                    *(v4u*) (out + dst + blk * part) = v4u {w[0] | (w[1] << 16), w[2] | (w[3] << 16), w[4] | (w[5] << 16), w[6] | (w[7] << 16)};
                }
                else
                    out[dst + blk * part] = (uint16_t) (which == 0 ? hi[0] : (which == 1 ? mid[0] : lo[0]));
            }
        }
        else if constexpr (V == 8)
        {
            const v4u h4 = {hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16), hi[4] | (hi[5] << 16), hi[6] | (hi[7] << 16)};
            const v4u l4 = {lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16), lo[4] | (lo[5] << 16), lo[6] | (lo[7] << 16)};
            *(v4u*) (out + dst) = h4;
            *(v4u*) (out + dst + hi_part1 * part) = h4;
            *(v4u*) (out + dst + lo_part0 * part) = l4;
            *(v4u*) (out + dst + 3 * part) = l4;
        }
        else
        {
            out[dst] = (uint16_t) hi[0];
            out[dst + hi_part1 * part] = (uint16_t) hi[0];
            out[dst + lo_part0 * part] = (uint16_t) lo[0];
            out[dst + 3 * part] = (uint16_t) lo[0];
        }
    }
    if (special) *a.flag = a.epoch;
}

template<int DT>
static hipError_t launch_split_dt(uint16_t* out, const void* in, const SplitBf16Args& a, hipStream_t s)
{
    const long long contig_stride = a.k_contig ? a.sk : a.sf, other = a.k_contig ? a.sf : a.sk, C = a.k_contig ? a.K : a.F;
    const int       es = DT == DT_TF32 ? 4 : 2;
    bool            vec = contig_stride == 1 && C % 8 == 0 && other % 8 == 0 && ((uintptr_t) in % 16 == 0) && ((uintptr_t) out % 16 == 0);
    for (int i = 0; i < 3; i++) vec = vec && a.bs[i] % 8 == 0;
    (void) es;
    const long long total = (long long) a.F * a.K * a.e[0] * a.e[1] * a.e[2] / (vec ? 8 : 1);
    if (total == 0) return hipSuccess;
    const int grid = grid_for((size_t) total, 1 << 20);
    if (vec) hipLaunchKernelGGL((split_bf16_kernel<DT, 8>), dim3(grid), dim3(CAST_THREADS), 0, s, out, in, a);
    else
        hipLaunchKernelGGL((split_bf16_kernel<DT, 1>), dim3(grid), dim3(CAST_THREADS), 0, s, out, in, a);
    return hipGetLastError();
}

hipError_t launch_split_bf16(uint16_t* out, const void* in, int dtype, const SplitBf16Args& a, hipStream_t s)
{
    switch (dtype)
    {
        case DT_FP16: return launch_split_dt<DT_FP16>(out, in, a, s);
        case DT_UFP16: return launch_split_dt<DT_UFP16>(out, in, a, s);
        case DT_TF32: return launch_split_dt<DT_TF32>(out, in, a, s);
        case DT_FP32: return launch_split_dt<DT_FP32>(out, in, a, s);
        default: return hipErrorInvalidValue;
    }
}

template<class T>
__global__ __launch_bounds__(CAST_THREADS) void strided_copy_kernel(T* __restrict__ dst, const T* __restrict__ src, StridedCopyArgs a, size_t total)
{
    for (size_t i = (size_t) blockIdx.x * CAST_THREADS + threadIdx.x; i < total; i += (size_t) gridDim.x * CAST_THREADS)
    {
        size_t r = i, so = 0, d_o = 0;
#pragma unroll
        for (int d = 0; d < 5; d++)
        {
            const size_t c = r % a.sizes[d];
            r /= a.sizes[d];
            so += c * a.src_strides[d];
            d_o += c * a.dst_strides[d];
        }
        dst[d_o] = src[so];
    }
}

hipError_t launch_strided_copy(void* dst, const void* src, int elem_size, const StridedCopyArgs& a, hipStream_t s)
{
    size_t total = 1;
    for (int d = 0; d < 5; d++) total *= a.sizes[d];
    if (total == 0) return hipSuccess;
    const int grid = grid_for(total, 1 << 16);
    switch (elem_size)
    {
        case 1: hipLaunchKernelGGL((strided_copy_kernel<uint8_t>), dim3(grid), dim3(CAST_THREADS), 0, s, (uint8_t*) dst, (const uint8_t*) src, a, total); break;
        case 2: hipLaunchKernelGGL((strided_copy_kernel<uint16_t>), dim3(grid), dim3(CAST_THREADS), 0, s, (uint16_t*) dst, (const uint16_t*) src, a, total); break;
        case 4: hipLaunchKernelGGL((strided_copy_kernel<uint32_t>), dim3(grid), dim3(CAST_THREADS), 0, s, (uint32_t*) dst, (const uint32_t*) src, a, total); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_relu_inplace(float* x, size_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(relu_inplace_kernel, dim3(grid_for(n, 8192)), dim3(CAST_THREADS), 0, s, x, n);
    return hipGetLastError();
}

hipError_t launch_absmax(float* out, const float* in, size_t n, hipStream_t s)
{
    // the result cell is cleared by a one-lane fill kernel (not a memset node) so the sequence can be graph-captured
    hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(1), 0, s, (uint32_t*) out, 0u, (size_t) 1);
    if (n == 0) return hipGetLastError();
    const int vec_ok = ((uintptr_t) in & 15u) == 0;
    hipLaunchKernelGGL(absmax_kernel, dim3(grid_for(vec_ok ? (n >> 2) + 1 : n, 2048)), dim3(CAST_THREADS), 0, s,
                       (uint32_t*) out, in, n, vec_ok);
    return hipGetLastError();
}

} // namespace mme
