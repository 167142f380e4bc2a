// mme_kernels.hpp -- internal (C++) interface between the C ABI layer and the HIP kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include "mme_numeric.hpp"

namespace mme
{
// ---- elementwise (cast_kernels.hip) ---------------------------------------------------------------------------
hipError_t launch_cast_from_fp32(void* out, const float* in, size_t n, const CastParams& p, const int32_t* col_exp,
                                 size_t n_cols, hipStream_t s);
// run_flag (device, may be NULL): the kernel does nothing unless *run_flag == run_epoch
hipError_t launch_cast_to_fp32(float* out, const void* in, int dtype, int bias, int mode, size_t n, float scale,
                               int has_scale, const int32_t* col_exp, size_t n_cols, hipStream_t s, const uint32_t* run_flag = nullptr,
                               uint32_t run_epoch = 0);
// stochastic rounding / stochastic flush: regs = the calculator's LFSR registers 0 .. 127 before the call, jump = device table of
// LFSR_JUMP_LEVELS x 32 words (image of every state bit under 2^k steps); reseed: step a register after every use
constexpr int LFSR_JUMP_LEVELS = 40;
struct LfsrRegisters
{
    uint32_t v[128];
};
hipError_t launch_cast_stochastic(void* out, const float* in, size_t n, const CastParams& p, int sftz, int reseed, uint32_t polynomial,
                                  const LfsrRegisters& regs, const uint32_t* jump, hipStream_t s);
// weights of transposed_dedx (dense, n0 x n1 x S x R x Q, n0 contiguous) -> n1 x n0 x S x R x Q with the S axis reversed
hipError_t launch_repack_transposed_weights(void* out, const void* in, int elem_size, uint32_t n0, uint32_t n1, uint32_t S, size_t total,
                                            hipStream_t s);
// memory[i] = memory[i] (op) mme_out[i] for fp32 / bf16 (op: 0 add, 1 sub, 2 min, 3 max, 4 max(sum, 0); rm: 0 nearest even, 1 toward
// zero, 2 up, 3 down)
hipError_t launch_memory_write_reduce(void* memory, const void* mme_out, int dtype, size_t n, int op, int rm, int clip, hipStream_t s);
hipError_t launch_relu_inplace(float* x, size_t n, hipStream_t s);
// copies the logical elements of a 5-d tensor between two layouts: element (i0 .. i4) from src + sum i_d * src_strides[d] to
// dst + sum i_d * dst_strides[d] (strides in elements of elem_size bytes); used to make a dense copy of a tensor whose
// strides the contraction kernels cannot follow, and to write a dense result back into such a tensor
struct StridedCopyArgs
{
    uint32_t sizes[5];
    uint32_t src_strides[5], dst_strides[5];
};
hipError_t launch_strided_copy(void* dst, const void* src, int elem_size, const StridedCopyArgs& a, hipStream_t s);
// fp32 words -> the same words rounded to tf32 (nearest even, 10 mantissa bits), out of place
hipError_t launch_round_to_tf32(void* out, const void* in, size_t n, int clip, int clip_inf_in, hipStream_t s, const uint32_t* run_flag = nullptr,
                                uint32_t run_epoch = 0);
// fp16 / ufp16 / tf32 operand (a plain view: F x K per batch entry, strides in elements) -> dense bf16 copy holding the value
// as hi + lo parts, four K-blocks along k: [hi | hi | lo | lo] (is_b = 0) or [hi | lo | hi | lo] (is_b = 1); (batch, f, 4 K)
// when k_contig, else (batch, 4 K, f).  e[]: batch extents of the copy (1 where the source broadcasts).  A value that is not
// finite stores epoch into *flag.
struct SplitBf16Args
{
    int       F, K, e[3];
    long long sf, sk, bs[3];
    int       k_contig, is_b;
    int       bias, mode, clip, clip_inf_in; // decode parameters (bias / mode: fp16 flavours; clip*: tf32 rounding)
    uint32_t* flag;
    uint32_t  epoch;
};
hipError_t launch_split_bf16(uint16_t* out, const void* in, int dtype, const SplitBf16Args& a, hipStream_t s);
hipError_t launch_absmax(float* out, const float* in, size_t n, hipStream_t s);

// ---- contraction (gemm_kernels.hip) ---------------------------------------------------------------------------
//
// Every contraction of the path is C[f_a][f_b] = sum_k A(f_a, k) * B(f_b, k) over one "view" per operand.
// A view maps (free index f, reduction index k) to an element address, either as a plain strided matrix or through
// the im2col / col2im addressing of the reference (mme/mme_reference/im2col.cpp:134-172).

enum : int
{
    VIEW_PLAIN = 0,  // base + f * stride_f + k * stride_k (+ batch offset)
    VIEW_CONV = 1,   // (pixel, tap, channel) gather, see below
    VIEW_TAPPED = 2  // k = tap * nch + ch:  base + f * stride_f + ch * stride_k + tap * tap_stride  (weights of dedx)
};

struct OperandView
{
    const char* base;
    int         kind;
    int         k_contig; // 1: consecutive k are adjacent in memory, 0: consecutive f are
    int         vec_ok;   // 16-byte vector loads along the contiguous index are legal and never straddle a boundary
    // VIEW_PLAIN
    long long stride_f, stride_k; // elements
    long long batch_stride[3];    // elements, 0 where the operand is broadcast
    long long tap_stride;         // VIEW_TAPPED only
    // VIEW_CONV: element = src[pos(pixel, tap)][channel]
    int       pix_is_f;   // 1: f = pixel, k = tap * nch + channel;  0: k = pixel, f = tap * nch + channel
    int       gather_y;   // 0: pos = pixel * stride + tap * dilation - padding (read x at an output pixel)
                          // 1: pos = (pixel + padding - tap * dilation) / stride, exact division only (read dy at an
                          //    input pixel: the gather form of col2im)
    int       nch;        // channels per tap
    int       grid[4];    // extents of the pixel index space (dims 1..4 of the tensor that enumerates pixels)
    int       src[4];     // extents of dims 1..4 of the tensor being read
    long long src_stride[4];
    int       ktap[3];    // S, R, Q
    int       cstride[4], dil[4], pad[4];
};

struct GemmEpilogue
{
    void*          out;
    long long      ld;              // elements between consecutive f_a rows of the output
    long long      batch_stride[3];
    int            out_dtype;       // DT_*
    CastParams     cast;            // used when fused != 0
    int            fused;           // 0: raw fp32 accumulators (times alpha)
    float          alpha;           // exact power of two folded into the accumulators (fp8 bias fold, descale)
    int            has_alpha;
    const int32_t* col_exp;         // per f_b power-of-two exponents or NULL
    int            fast_cast;
    // the host can rule out NaN, infinite and overflowing values before the cast (operands without such codes, a bounded
    // reduction, one known power-of-two factor): the fast converters then need not look for them
    int            finite;
    // fp8 large-tile kernels: power-of-two exponent handed to the matrix instruction's block-scale operand instead of a
    // multiplication per output (the host folds alpha into it when no product or sum can leave the fp32 range either way;
    // has_alpha is then 0)
    int            mfma_scale_exp;
};

struct GemmProblem
{
    int          dtype;      // operand element type (DT_*); fp8 operands may differ in flavour
    int          fmt_a, fmt_b; // fp8 only: 0 = 4-bit exponent (e4m3), 1 = 5-bit exponent (e5m2)
    int          M, N, K;    // extents of f_a, f_b, k
    int          batch[3];
    OperandView  A, B;
    GemmEpilogue epi;
    int          tile_m;     // large-tile kernel: rows of the output tile, 128 or 0 / 256 (chosen by gemm_fast_pick_tile_m)
    int          waves;      // large-tile kernel: wavefronts per workgroup, 4 or 0 / 8 (chosen by gemm_fast_pick_waves)
    int          split_k;    // >1: partial sums go to workspace and are reduced in a fixed order
    float*       workspace;  // split_k * batch * M * N floats
    // device-side predicate: when skip_flag != NULL the whole launch returns at once if (*skip_flag == skip_epoch) == skip_if
    // (the scan of the call with that epoch number found something; the flag is never reset, epochs only grow).
    // Lets the fp8 path enqueue "native fp8" and "decoded bf16" variants back to back without a host round trip.
    const uint32_t* skip_flag;
    int             skip_if;
    uint32_t        skip_epoch;
    // chk != 0 (fp8 operands, large-tile kernels that have the variant, see gemm_large_tile_checks_operands): the launch never
    // skips; instead the kernel looks at the operand bytes it multiplies and stores skip_epoch into *skip_flag when a byte b
    // of operand A (B) has (b & chk_mask_a) + chk_add_a >= 0x80, i.e. a code the hardware's fp8 formats read differently
    // (mask 0: that operand needs no check).  The caller then enqueues the exact fall-back behind it, predicated on the flag.
    int             chk;
    uint32_t        chk_mask_a, chk_add_a, chk_mask_b, chk_add_b; // the byte constants replicated over a 32-bit word
    // The four-wavefront form (chk == 2; one round of tiles, every workgroup resident) settles the matter inside the launch: the
    // looks are shared out the same way, but what they find is noted per operand panel in chk_state (zero before the launch,
    // row panels + column panels words per batch element: finished lookers in the low half, finds in the high half), and a workgroup
    // whose panels hold such a code computes its tile once more, exactly, from operands decoded with Gaudi's meaning of the
    // codes (inf / NaN modes below; the hardware formats' exponent bias, so that the epilogue's factor stays the same).
    int             chk_inf_nan_a, chk_inf_nan_b;
    uint32_t*       chk_state;
    // diagnostics (NULL: off): CLOCK_PROBE_WORKGROUPS x 4 cells in which the large-tile kernels note, per workgroup, the shader
    // clock counter and the 100 MHz counter at its start and at its end
    uint64_t*       clock_probe;
};
constexpr int CLOCK_PROBE_WORKGROUPS = 4096;
// the page of zeros that the convolution gathers of the large-tile kernels read where a filter tap falls into the padding: as long
// as the channels of one tap may be (a padding lane adds the stage's channel offset like every other lane)
constexpr int GF_ZERO_PAGE_BYTES = 4096;

// diagnostics: `iters` x 8 dependent-free 32x32 matrix instructions per wavefront on 256 workgroups of 8 wavefronts, operands in
// registers (zero, or four sets of random codes used in turn); kind 0: fp8 (32x32x64), 1: bf16 (32x32x16).  stamps: 256 x 2
// cells, shader clocks and 100 MHz ticks each workgroup's loop took.
hipError_t launch_matrix_core_rate(int kind, int random_operands, int iters, uint64_t* stamps, hipStream_t s);

size_t     gemm_workspace_bytes(const GemmProblem& p);
int        gemm_pick_split_k(const GemmProblem& p, int num_cus);
// 128 when the large-tile kernel should run this problem with 128-row tiles (few tiles, 2-byte operands, A k-contiguous), else 0
int        gemm_fast_pick_tile_m(const GemmProblem& p, int num_cus);
hipError_t launch_gemm(const GemmProblem& p, hipStream_t s);
// large aligned fp8 problems (gemm_large_tile.hip); launch_gemm routes to it when applicable
bool       gemm_large_tile_applicable(const GemmProblem& p);
int        gemm_fast_pick_split_k(const GemmProblem& p, int num_cus); // 0: the large-tile kernel does not take this problem
int        gemm_fast_pick_waves(const GemmProblem& p, int num_cus);   // (after tile_m and split_k have been chosen)
bool       gemm_large_tile_one_round(const GemmProblem& p, int num_cus); // (likewise)
hipError_t launch_gemm_large_tile(const GemmProblem& p, hipStream_t s);
// the kernel this problem takes can check its fp8 operands for special codes itself (GemmProblem::chk)
bool       gemm_large_tile_checks_operands(const GemmProblem& p);
// the kernel this problem takes applies GemmEpilogue::mfma_scale_exp (the plain fp8 kernel with one workgroup per 256 x 256 tile)
bool       gemm_large_tile_takes_mfma_scale(const GemmProblem& p);

// forward convolution fast path (conv_fwd_fast.hip): bf16, 3x3, 64 -> 64 channels, stride 1, padding 1, dense NHWC
bool       conv_fwd_fast_applicable(int dtype, int C, int K, int S, int R, int Q, int W, int H, int D, const int stride[4], const int dil[4],
                                    const int pad[4], bool dense);
// status: host-visible word that a kernel sets when it gives up a bounded wait (after wait_limit polls)
hipError_t launch_conv_fwd_fast(const void* x, const void* w, int B, int H, int W, const GemmEpilogue& epi, int num_cus, uint32_t* status,
                                uint32_t wait_limit, hipStream_t s);

// flags every exponent-all-ones code of an fp8 buffer (inf / NaN in Gaudi's full mode, finite for the hardware's
// e4m3): *flag |= 1.  mask_kind 0: any code with all exponent bits set; 1: only 0x7F / 0xFF.
// one launch for both operands: mask_kind < 0 leaves an operand out; a hit stores `epoch` into *flag
hipError_t launch_fp8_special_scan2(uint32_t* flag, uint32_t epoch, const void* a, size_t na, int man_bits_a, int mask_kind_a, const void* b,
                                    size_t nb, int man_bits_b, int mask_kind_b, hipStream_t s);

// dense or strided 5-d fp8 -> bf16 exact decode (used when the hardware's fp8 formats cannot represent the operand)
// run_flag (device, may be NULL): the kernel does nothing when *run_flag == 0
// both operands in one launch; runs only when *run_flag == epoch (run_flag may be NULL: always)
hipError_t launch_fp8_to_bf16_2(uint16_t* out_a, const uint8_t* in_a, size_t na, int man_bits_a, int bias_a, int mode_a, uint16_t* out_b,
                                const uint8_t* in_b, size_t nb, int man_bits_b, int bias_b, int mode_b, const uint32_t* run_flag, uint32_t epoch,
                                hipStream_t s);
// one-lane fill of n 32-bit cells (kernels instead of memset nodes keep call sequences graph-capturable)
hipError_t launch_fill_u32(uint32_t* p, uint32_t v, size_t n, hipStream_t s);

} // namespace mme
