// mme_api.hip -- the C ABI declared in include/mme_hip.h: handle, validation (the reference's MME_ASSERT conditions),
// mapping of tensor descriptors to kernel problems, host-pointer staging.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "../../include/mme_hip.h"
#include "mme_kernels.hpp"

using namespace mme;

// Scratch memory of the entry point that allocates nothing (mme_hip_batch_gemm_dev_noalloc): one array per device, held from
// the moment the library's code is loaded on that device until the process ends.  Bytes 0 .. 255 hold the flag cell of the
// fp8 / split-operand fall-backs, the rest is handed out per call (split-k partial sums, decoded operand copies).  In host
// code the array's name is only a stand-in: its device address is asked for once per device (mme_hip_create, with that
// device current) and kept in g_scratch_ptr.
static __device__ __align__(256) unsigned char scratch[MME_HIP_NOALLOC_SCRATCH_BYTES];

namespace
{
constexpr int         MAX_DEVICES = 64;
void*                 g_scratch_ptr[MAX_DEVICES];      // device address of `scratch` on each device, null until asked for
std::atomic<uint32_t> g_scratch_epoch[MAX_DEVICES];    // epoch numbers of the flag cell in `scratch`: shared by every handle of a device
std::mutex            g_scratch_mutex;

thread_local std::string g_create_error = "";

// A grow-only block of device memory.  Launches enqueued earlier may still read or write the old block when a larger one is
// asked for, and launches recorded into a HIP graph refer to it for as long as the graph lives: the new block is allocated
// before the old one is given up (a failed allocation leaves the buffer as it was), and with keep_old the old block is not
// freed but retired until the buffer is destroyed.
struct DeviceBuffer
{
    void*              p = nullptr;
    size_t             bytes = 0;
    std::vector<void*> retired;
    ~DeviceBuffer()
    {
        if (p) (void) hipFree(p);
        for (void* q : retired) (void) hipFree(q);
    }
    hipError_t reserve(size_t n, bool keep_old = false)
    {
        if (n <= bytes) return hipSuccess;
        void*      q = nullptr;
        hipError_t e = hipMalloc(&q, n);
        if (e != hipSuccess) return e;
        if (p)
        {
            if (keep_old) retired.push_back(p);
            else
                (void) hipFree(p);
        }
        p = q;
        bytes = n;
        return hipSuccess;
    }
};
} // namespace

struct mme_hip_calc
{
    int                   chip = MME_HIP_CHIP_GAUDI3;
    int                   device = 0;
    int                   num_cus = 256;
    hipStream_t           own_stream = nullptr;
    hipStream_t           stream = nullptr;
    unsigned              num_threads = 1;
    std::vector<uint32_t> lfsr;            // the reference's m_lfsr: advanced by every stochastic conversion
    uint32_t              polynomial = 0;
    int                   operand_clip_fp = 0, operand_clip_inf_in = 0; // clipFp / clipFpInfIn of the tf32 operand conversion
    std::vector<uint32_t> lfsr_jump;       // LFSR_JUMP_LEVELS x 32 words, built when the calculator is created
    DeviceBuffer          lfsr_jump_dev;
    DeviceBuffer          weights_ws;      // repacked weights of transposed_dedx
    std::string           error;
    DeviceBuffer          split_ws;  // split-k partial sums
    DeviceBuffer          decode_ws; // bf16 copies of fp8 operands the hardware formats cannot express
    // host-pointer entry points: device copies of the call's tensors (grow-only, kept between calls) and two pinned bounce
    // buffers with the events that say when the device has consumed / filled them
    // one word of pinned host memory that kernels with bounded waits write when they give one up (read after a
    // synchronisation), its device-side address, and the number of polls such a wait may take
    uint32_t*             status_host = nullptr;
    uint32_t*             status_dev = nullptr;
    uint32_t              wait_limit = 1u << 22;
    DeviceBuffer          stage_dev[3];
    void*                 bounce[2] = {nullptr, nullptr};
    hipEvent_t            bounce_ev[2] = {nullptr, nullptr};
    DeviceBuffer          pack_ws[3]; // dense copies of convolution tensors whose strides the kernels cannot follow (weights, dy, output)
    DeviceBuffer          stoch_ws;  // fp32 results of a contraction whose fused epilogue rounds stochastically
    DeviceBuffer          flag;      // one 32-bit cell: epoch number of the latest call whose operands held codes the hardware formats lack
    uint32_t              specials_epoch = 0; // epoch number of the latest call that scanned
    int                   fp8_specials_policy = 0;
    int                   last_form[4] = {0, 256, 1, 8}; // mme_hip_last_contraction_form
    // panel words of the fp8 GEMMs that settle special codes inside their launch (GemmProblem::chk_state): a ring of regions, one per launch, all cleared by
    // one fill launch every CHK_STATE_RING launches
    DeviceBuffer          chk_state;
    unsigned              chk_state_launches = 0;
    // set for the duration of a call through the entry point that allocates nothing: every workspace comes out of the
    // device's static scratch array (noalloc_used: bytes handed out so far in this call)
    bool                  noalloc = false;
    size_t                noalloc_used = 0;
    // recording: the stream of the current call is being captured into a HIP graph.  graph_seen: some call of this handle
    // has been; from then on the work spaces never free a block they outgrow (a graph may replay launches that point into it)
    bool                  recording = false;
    bool                  graph_seen = false;
    // a handle without a device that only answers "which kernel form would this call launch" (mme_hip_plan_*): it goes
    // through the same checks and the same planning as a real call, allocates nothing and skips every launch
    bool                  dry_run = false;
    // diagnostics: per-workgroup clock stamps of the large-tile kernels (mme_hip_clock_probe), NULL while switched off
    DeviceBuffer          clock_probe_buf;
    uint64_t*             clock_probe = nullptr;
};

namespace
{
int fail(mme_hip_handle h, int code, const char* fmt, ...)
{
    char    buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (h) h->error = buf;
    else
        g_create_error = buf;
    return code;
}

int build_lfsr_jump(mme_hip_handle h);

// a kernel launch of a contraction or conversion path: skipped by a planning handle (mme_hip_calc::dry_run)
#define LAUNCH_TRY(h, expr)                  \
    do                                       \
    {                                        \
        if (!(h)->dry_run) HIP_TRY(h, expr); \
    } while (0)

int hip_fail(mme_hip_handle h, hipError_t e, const char* what)
{
    return fail(h, e == hipErrorOutOfMemory ? MME_HIP_ENOMEM : MME_HIP_EHIP, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(h, expr)                                          \
    do                                                            \
    {                                                             \
        hipError_t e_ = (expr);                                   \
        if (e_ != hipSuccess) return hip_fail((h), e_, #expr);    \
    } while (0)

// First thing in every device-pointer entry point: is the call being recorded into a graph?  (A stream whose state cannot be
// read counts as recording: the careful side.)
void note_recording(mme_hip_handle h)
{
    if (h->dry_run) return;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(h->stream, &st) != hipSuccess)
    {
        (void) hipGetLastError();
        st = hipStreamCaptureStatusActive;
    }
    h->recording = st != hipStreamCaptureStatusNone;
    if (h->recording) h->graph_seen = true;
}

// grows one of the handle's buffers (see DeviceBuffer)
hipError_t grow(mme_hip_handle h, DeviceBuffer& buf, size_t bytes) { return h->dry_run ? hipSuccess : buf.reserve(bytes, h->graph_seen); }

// Work space of `bytes` for the current call: the handle's grow-only buffer `buf`, or, in a call that may not allocate, the
// next piece of the device's static scratch array.
// panel words of the fp8 GEMMs that settle special codes inside their launch: words per launch (row panels + column panels per
// batch element, at most 256 tiles in all) and launches per clearing
constexpr size_t   CHK_STATE_REGION_WORDS = 2048;
constexpr unsigned CHK_STATE_RING = 64;

int take_ws(mme_hip_handle h, DeviceBuffer& buf, size_t bytes, void** out)
{
    if (h->dry_run)
    {
        *out = (void*) (uintptr_t) 4096; // (a planning handle never touches it; aligned and not null, like a real one)
        return MME_HIP_OK;
    }
    if (!h->noalloc)
    {
        HIP_TRY(h, grow(h, buf, bytes));
        *out = buf.p;
        return MME_HIP_OK;
    }
    const size_t need = (bytes + 255) & ~(size_t) 255;
    if (h->noalloc_used + need > (size_t) MME_HIP_NOALLOC_SCRATCH_BYTES)
        return fail(h, MME_HIP_ENOMEM,
                    "this call needs %zu more bytes of work space, the static scratch of the allocation-free entry point has %zu of %zu left; use "
                    "mme_hip_batch_gemm_dev",
                    need, (size_t) MME_HIP_NOALLOC_SCRATCH_BYTES - h->noalloc_used, (size_t) MME_HIP_NOALLOC_SCRATCH_BYTES);
    *out = (unsigned char*) g_scratch_ptr[h->device] + h->noalloc_used;
    h->noalloc_used += need;
    return MME_HIP_OK;
}

int elem_size(int dt)
{
    switch (dt)
    {
        case MME_HIP_FP8_143:
        case MME_HIP_FP8_152: return 1;
        case MME_HIP_BF16:
        case MME_HIP_FP16:
        case MME_HIP_UFP16: return 2;
        case MME_HIP_FP32:
        case MME_HIP_FP32_IEEE:
        case MME_HIP_TF32: return 4;
        default: return 0;
    }
}
bool is_fp8(int dt) { return dt == MME_HIP_FP8_143 || dt == MME_HIP_FP8_152; }
bool is_fp16(int dt) { return dt == MME_HIP_FP16 || dt == MME_HIP_UFP16; }

uint64_t n_elements(const mme_hip_tensor* t)
{
    uint64_t n = 1;
    for (int d = 0; d < 5; d++) n *= t->sizes[d];
    return n;
}
// elements spanned in memory: the largest stride * size (setStridesAndGetTensorSize, sim_tensor_base.cpp:351-374)
uint64_t span_elements(const mme_hip_tensor* t)
{
    uint64_t m = 0;
    for (int d = 0; d < 5; d++) m = std::max<uint64_t>(m, (uint64_t) t->strides[d] * t->sizes[d]);
    return m;
}
// dims 1..4 enumerate rows of one dense-pitched matrix: stride[d+1] == stride[d] * size[d]
bool rows_collapsible(const mme_hip_tensor* t)
{
    for (int d = 1; d < 4; d++)
        if (t->sizes[d + 1] > 1 && (uint64_t) t->strides[d + 1] != (uint64_t) t->strides[d] * t->sizes[d]) return false;
    return true;
}

int check_tensor(mme_hip_handle h, const mme_hip_tensor* t, const char* name)
{
    if (!t) return fail(h, MME_HIP_EINVAL, "%s: got null pointer", name);
    if (elem_size(t->dtype) == 0) return fail(h, MME_HIP_EINVAL, "%s: type not supported", name);
    if (t->strides[0] != 1) return fail(h, MME_HIP_EINVAL, "%s: the first dimension must be contiguous", name);
    if (n_elements(t) >= (1ull << 31)) return fail(h, MME_HIP_EINVAL, "%s: more than 2^31 elements", name);
    if (n_elements(t) && !t->data) return fail(h, MME_HIP_EINVAL, "%s: got null pointer", name);
    return MME_HIP_OK;
}

// the reference's registration table for Gaudi3 (mme_reference_impl.cpp:188-196) and its type pairing rule
// (chip_fma/gaudi3_fma.cpp:62-66)
int check_operand_types(mme_hip_handle h, const mme_hip_tensor* a, const mme_hip_tensor* b)
{
    const int ta = a->dtype, tb = b->dtype;
    if (!(ta == MME_HIP_BF16 || ta == MME_HIP_FP32 || ta == MME_HIP_TF32 || is_fp8(ta) || is_fp16(ta)))
        return fail(h, MME_HIP_EINVAL, "type is not registered in function map !");
    if (!(is_fp8(ta) && is_fp8(tb)) && !(is_fp16(ta) && is_fp16(tb)) && ta != tb)
        return fail(h, MME_HIP_EINVAL, "Gaudi3 doesnt support mixed input type flavors");
    for (const mme_hip_tensor* t : {a, b})
        if (is_fp16(t->dtype) && t->fp_bias > (t->dtype == MME_HIP_FP16 ? 31u : 63u))
            return fail(h, MME_HIP_EINVAL, "fp16 / ufp16 exponent bias exceeds the exponent field");
    for (const mme_hip_tensor* t : {a, b})
        if (is_fp8(t->dtype))
        {
            if (t->dtype == MME_HIP_FP8_143 && !(t->fp_bias == 3 || t->fp_bias == 7 || t->fp_bias == 11 || t->fp_bias == 15))
                return fail(h, MME_HIP_EINVAL, "fp8_143 exponent bias must be 3, 7, 11 or 15");
            if (t->dtype == MME_HIP_FP8_152 && (t->fp_bias < 1 || t->fp_bias > 30))
                return fail(h, MME_HIP_EINVAL, "fp8_152 exponent bias must be in 1..30");
            if (t->inf_nan_mode < 0 || t->inf_nan_mode > 2) return fail(h, MME_HIP_EINVAL, "invalid infNanMode");
        }
    return MME_HIP_OK;
}

int check_out_type(mme_hip_handle h, const mme_hip_tensor* out, const mme_hip_epilogue* epi)
{
    if (!epi)
    {
        if (out->dtype != MME_HIP_FP32) return fail(h, MME_HIP_EINVAL, "type is not registered in function map !");
        return MME_HIP_OK;
    }
    if (!(out->dtype == MME_HIP_FP32 || out->dtype == MME_HIP_BF16 || is_fp8(out->dtype) || is_fp16(out->dtype)))
        return fail(h, MME_HIP_EINVAL, "Unsupported type");
    if (is_fp16(out->dtype) && out->fp_bias > (out->dtype == MME_HIP_FP16 ? 31u : 63u))
        return fail(h, MME_HIP_EINVAL, "fp16 / ufp16 exponent bias exceeds the exponent field");
    {
        const int rm = epi->rounding_mode;
        if (!(rm == 0 || rm == 1 || rm == 2 || rm == 3 || rm == 4 || rm == 6 || rm == 7)) return fail(h, MME_HIP_EINVAL, "invalid rounding mode %d", rm);
    }
    if (epi->scale_exp < -126 || epi->scale_exp > 126) return fail(h, MME_HIP_EINVAL, "scale exponent out of range");
    return MME_HIP_OK;
}

CastParams make_cast(int dtype, unsigned bias, int mode, int rm, int clip, int clip_inf, int ftz, int relu, int scale_exp)
{
    CastParams c;
    c.dtype = dtype == MME_HIP_FP32_IEEE ? DT_FP32 : dtype;
    c.exp_bias = (int) bias;
    c.inf_nan_mode = mode;
    c.rm = rm;
    c.clip_fp = clip;
    c.clip_inf_in = clip_inf;
    c.ftz = ftz;
    c.relu = relu;
    c.has_scale = scale_exp != 0;
    uint32_t bits = (uint32_t) (scale_exp + 127) << 23;
    memcpy(&c.scale, &bits, 4);
    return c;
}

float pow2f(int e)
{
    uint32_t bits = (uint32_t) (e + 127) << 23;
    float    f;
    memcpy(&f, &bits, 4);
    return f;
}

// ---- fp8 operands: fold Gaudi's exponent bias into a power of two, decide whether the hardware formats suffice -------
struct Fp8Plan
{
    int fold_exp = 0;     // accumulators are multiplied by 2^fold_exp
    int scan_kind[2] = {-1, -1}; // -1: every code is exact in the hardware format; 0 / 1: mask kind to scan for
    // mask kind whose absence also rules out inf and NaN among the operand's values (-1: the scan above already does, or the
    // format has none): 0 any exponent-all-ones code, 1 only 0x7F / 0xFF
    int nonfinite_kind[2] = {-1, -1};
};

Fp8Plan plan_fp8(const mme_hip_tensor* a, const mme_hip_tensor* b)
{
    Fp8Plan               p;
    const mme_hip_tensor* t[2] = {a, b};
    for (int i = 0; i < 2; i++)
    {
        if (t[i]->dtype == MME_HIP_FP8_143)
        {
            p.fold_exp += 7 - (int) t[i]->fp_bias; // hardware e4m3 has bias 7
            // full mode: exponent 15 is inf / NaN (finite 256..448 for the hardware); no-inf-nan mode: 0x7F is finite
            // (NaN for the hardware); minimal mode is the hardware's own format
            p.scan_kind[i] = t[i]->inf_nan_mode == 0 ? 0 : (t[i]->inf_nan_mode == 1 ? 1 : -1);
            p.nonfinite_kind[i] = t[i]->inf_nan_mode == 2 ? 1 : -1; // minimal mode: 0x7F / 0xFF are NaN for Gaudi and hardware alike
        }
        else
        {
            p.fold_exp += 15 - (int) t[i]->fp_bias; // hardware e5m2 has bias 15
            // full mode is the hardware's own format; the other modes give finite meaning to exponent-31 codes
            p.scan_kind[i] = t[i]->inf_nan_mode == 0 ? -1 : 0;
            p.nonfinite_kind[i] = t[i]->inf_nan_mode == 0 ? 0 : -1; // full mode: exponent 31 is inf / NaN for Gaudi and hardware alike
        }
    }
    return p;
}

void set_plain_view(OperandView& v, const void* base, long long stride_f, long long stride_k, bool k_contig, int es, int extent_contig,
                    const long long bstride[3])
{
    memset(&v, 0, sizeof v);
    v.base = (const char*) base;
    v.kind = VIEW_PLAIN;
    v.stride_f = stride_f;
    v.stride_k = stride_k;
    v.k_contig = k_contig;
    const int       kv = 16 / es;
    const long long other = k_contig ? stride_f : stride_k;
    bool            ok = ((uintptr_t) base % 16 == 0) && (other % kv == 0) && (extent_contig % kv == 0);
    for (int i = 0; i < 3; i++)
    {
        v.batch_stride[i] = bstride[i];
        ok = ok && (bstride[i] % kv == 0);
    }
    v.vec_ok = ok;
}

// The flag cell of this call and a fresh epoch number for it.  A call that may not allocate uses the cell at the start of the
// device's static scratch array (zero when the code is loaded) with epoch numbers that every handle of the device draws
// from one counter, so that a stale value of another handle's call never equals this call's number.
int next_flag_epoch(mme_hip_handle h, uint32_t** flag, uint32_t* epoch)
{
    if (h->noalloc)
    {
        *flag = (uint32_t*) g_scratch_ptr[h->device];
        *epoch = ++g_scratch_epoch[h->device];
        return MME_HIP_OK;
    }
    if (!h->flag.p)
    {
        HIP_TRY(h, grow(h, h->flag, 256));
        LAUNCH_TRY(h, launch_fill_u32((uint32_t*) h->flag.p, 0u, 64, h->stream)); // epoch numbers start at 1
    }
    *flag = (uint32_t*) h->flag.p;
    *epoch = ++h->specials_epoch;
    return MME_HIP_OK;
}

// Runs one contraction, taking care of fp8 operands: native MFMA formats when every code is exact there, otherwise an
// exact fp8 -> bf16 decode followed by the bf16 kernel.  Both variants are enqueued, a device flag picks one, so the
// call never waits for the device.
// multiplies the epilogue's power-of-two factor by 2^fold
int fold_alpha(mme_hip_handle h, GemmEpilogue& e, int fold)
{
    uint32_t bits;
    memcpy(&bits, &e.alpha, 4);
    int ex = e.has_alpha ? (int) ((bits >> 23) & 0xFF) - 127 : 0;
    ex += fold;
    if (ex < -126 || ex > 126) return fail(h, MME_HIP_EINVAL, "exponent bias and scale exponents exceed the fp32 range");
    e.alpha = pow2f(ex);
    e.has_alpha = ex != 0;
    return MME_HIP_OK;
}

// picks tile height and k-slices of a problem and makes sure the split-k workspace can hold its partial sums
int plan_launch(mme_hip_handle h, GemmProblem& g)
{
    g.tile_m = gemm_fast_pick_tile_m(g, h->num_cus);
    g.split_k = gemm_pick_split_k(g, h->num_cus);
    g.waves = gemm_fast_pick_waves(g, h->num_cus);
    h->last_form[0] = gemm_large_tile_applicable(g) ? 1 : 0;
    h->last_form[1] = g.tile_m == 128 ? 128 : 256;
    h->last_form[2] = g.split_k > 1 ? g.split_k : 1;
    h->last_form[3] = g.waves == 4 ? 4 : 8;
    g.workspace = nullptr;
    g.clock_probe = h->clock_probe;
    if (g.split_k > 1)
    {
        void* ws = nullptr;
        if (int rc = take_ws(h, h->split_ws, gemm_workspace_bytes(g), &ws)) return rc;
        g.workspace = (float*) ws;
    }
    return MME_HIP_OK;
}

// fp16 / ufp16 / tf32 operands.  Two fp16 operands in full inf/NaN mode are IEEE half with the exponent bias as a power of
// two: they go to the fp16 matrix instruction as they are (returns with g.dtype = DT_FP16, nothing launched).  Every other
// combination (unsigned fp16 with its 6-bit exponent, exponent-all-ones codes that are finite, tf32) is contracted here:
//  - plain GEMMs of some size: each operand is written as two bf16 parts that add up to its exact value and the bf16 kernels
//    contract the 4 K long rows (split_bf16_kernel); operands that hold inf or NaN raise a device flag, which skips that
//    contraction and lets the fp32 one below run instead, so the call never waits for the device.  fp32 operands take the
//    same route with three bf16 parts and six of the nine cross products (6 K long rows; the fall-back then reads the
//    operands themselves);
//  - everything else: fp32 words holding the operands' exact values (tf32: the rounded ones), in the operands' own layout,
//    contracted by the fp32 instantiation.
int run_half_contraction(mme_hip_handle h, GemmProblem& g, const mme_hip_tensor* ta, const mme_hip_tensor* tb, const void* a_base, const void* b_base,
                         bool& done)
{
    done = false;
    if (ta->dtype == MME_HIP_FP16 && tb->dtype == MME_HIP_FP16 && ta->inf_nan_mode == 0 && tb->inf_nan_mode == 0)
    {
        g.dtype = DT_FP16;
        return fold_alpha(h, g.epi, (15 - (int) ta->fp_bias) + (15 - (int) tb->fp_bias));
    }
    done = true;
    const bool      fp32_in = ta->dtype == MME_HIP_FP32;
    const int       kblocks = fp32_in ? 6 : 4; // K-blocks of the split copies
    const long long nbatch = (long long) g.batch[0] * g.batch[1] * g.batch[2];
    bool            two_part = g.A.kind == VIEW_PLAIN && g.B.kind == VIEW_PLAIN && (long long) g.M * g.N * g.K * nbatch >= (1ll << 26) &&
                          g.K <= (1 << 27);
    if (fp32_in && !two_part)
    {
        done = false; // plain fp32 contraction: the caller launches it
        return MME_HIP_OK;
    }
    const size_t na = span_elements(ta), nb = span_elements(tb);
    const size_t na_pad = (na + 3) & ~(size_t) 3;
    size_t       part_elems[2] = {0, 0};
    long long    eff[2][3];
    OperandView* view[2] = {&g.A, &g.B};
    const int    free_extent[2] = {g.M, g.N};
    if (two_part)
        for (int i = 0; i < 2; i++)
        {
            part_elems[i] = (size_t) free_extent[i] * g.K * kblocks;
            for (int d = 0; d < 3; d++)
            {
                eff[i][d] = view[i]->batch_stride[d] ? g.batch[d] : 1;
                part_elems[i] *= (size_t) eff[i][d];
            }
            part_elems[i] = (part_elems[i] + 7) & ~(size_t) 7;
        }
    if (two_part && (part_elems[0] + part_elems[1]) * 2 > ((size_t) 16 << 30))
    {
        // the split copies would need more than 16 GiB of work space: contract the operands as they are
        if (fp32_in)
        {
            done = false;
            return MME_HIP_OK;
        }
        two_part = false;
        part_elems[0] = part_elems[1] = 0;
    }
    const size_t fp32_copies = fp32_in ? 0 : na_pad + ((nb + 3) & ~(size_t) 3);
    void* decode_ws = nullptr;
    if (int rc = take_ws(h, h->decode_ws, (fp32_copies + 4) * 4 + (part_elems[0] + part_elems[1]) * 2, &decode_ws)) return rc;
    float*    da = (float*) decode_ws;
    float*    db = da + na_pad;
    uint16_t* parts = (uint16_t*) ((float*) decode_ws + fp32_copies);
    const mme_hip_tensor* t[2] = {ta, tb};
    const void*           src[2] = {a_base, b_base};
    uint32_t*             flag = nullptr;
    uint32_t              epoch = 0;
    GemmProblem           g2 = g;
    if (two_part)
    {
        if (int rc = next_flag_epoch(h, &flag, &epoch)) return rc;
        OperandView* v2[2] = {&g2.A, &g2.B};
        uint16_t*    dst = parts;
        for (int i = 0; i < 2; i++)
        {
            SplitBf16Args a;
            a.F = free_extent[i];
            a.K = g.K;
            a.sf = view[i]->stride_f;
            a.sk = view[i]->stride_k;
            a.k_contig = view[i]->k_contig;
            a.is_b = i;
            a.bias = (int) t[i]->fp_bias;
            a.mode = t[i]->inf_nan_mode;
            a.clip = h->operand_clip_fp;
            a.clip_inf_in = h->operand_clip_inf_in;
            a.flag = flag;
            a.epoch = epoch;
            long long bstride[3], run = (long long) a.F * a.K * kblocks;
            for (int d = 0; d < 3; d++)
            {
                a.e[d] = (int) eff[i][d];
                a.bs[d] = view[i]->batch_stride[d];
                bstride[d] = view[i]->batch_stride[d] ? run : 0;
                run *= eff[i][d];
            }
            LAUNCH_TRY(h, launch_split_bf16(dst, src[i], t[i]->dtype, a, h->stream));
            if (a.k_contig) set_plain_view(*v2[i], dst, (long long) kblocks * a.K, 1, true, 2, kblocks * a.K, bstride);
            else
                set_plain_view(*v2[i], dst, 1, a.F, false, 2, a.F, bstride);
            dst += part_elems[i];
        }
        g2.dtype = DT_BF16;
        g2.K = kblocks * g.K;
    }
    // the fp32 contraction: the only one, or the one that runs when an operand holds inf / NaN
    for (int i = 0; i < 2 && !fp32_in; i++)
    {
        float* d = i ? db : da;
        if (t[i]->dtype == MME_HIP_TF32)
            LAUNCH_TRY(h, launch_round_to_tf32(d, src[i], i ? nb : na, h->operand_clip_fp, h->operand_clip_inf_in, h->stream, flag, epoch));
        else
            LAUNCH_TRY(h, launch_cast_to_fp32(d, src[i], t[i]->dtype, (int) t[i]->fp_bias, t[i]->inf_nan_mode, i ? nb : na, 1.0f, 0, nullptr, 0, h->stream,
                                           flag, epoch));
    }
    g.dtype = DT_FP32;
    if (!fp32_in)
    {
        g.A.base = (const char*) da;
        g.B.base = (const char*) db;
    }
    g.skip_flag = flag;
    g.skip_epoch = epoch;
    g.skip_if = 0; // runs when the flag holds this call's epoch
    if (two_part)
    {
        // both contractions may slice k; size the shared workspace for the larger request before either is launched
        GemmProblem probe = g;
        if (int rc = plan_launch(h, probe)) return rc;
        g2.skip_flag = flag;
        g2.skip_epoch = epoch;
        g2.skip_if = 1;
        if (int rc = plan_launch(h, g2)) return rc; // (the workspace only grows: it now fits either request)
        LAUNCH_TRY(h, launch_gemm(g2, h->stream));
    }
    if (int rc = plan_launch(h, g)) return rc;
    LAUNCH_TRY(h, launch_gemm(g, h->stream));
    return MME_HIP_OK;
}

int run_contraction(mme_hip_handle h, GemmProblem& g, const mme_hip_tensor* ta, const mme_hip_tensor* tb, const void* a_base,
                    const void* b_base)
{
    g.skip_flag = nullptr;
    g.skip_if = 0;
    if (is_fp16(g.dtype) || g.dtype == MME_HIP_TF32 || g.dtype == MME_HIP_FP32)
    {
        bool done = false;
        if (int rc = run_half_contraction(h, g, ta, tb, a_base, b_base, done)) return rc;
        if (done) return MME_HIP_OK;
    }
    if (int rc = plan_launch(h, g)) return rc;
    if (!is_fp8(g.dtype))
    {
        LAUNCH_TRY(h, launch_gemm(g, h->stream));
        return MME_HIP_OK;
    }
    const Fp8Plan plan = plan_fp8(ta, tb);
    g.fmt_a = ta->dtype == MME_HIP_FP8_152;
    g.fmt_b = tb->dtype == MME_HIP_FP8_152;
    const int fold = plan.fold_exp;
    // alpha so far holds the caller's descale (or 1); fold the bias difference into the same multiplication
    if (int rc = fold_alpha(h, g.epi, fold)) return rc;
    const bool need_scan = (plan.scan_kind[0] >= 0 || plan.scan_kind[1] >= 0) && h->fp8_specials_policy == 0;
    // Can a value that is not finite reach the output conversion?  Not when no operand holds an inf or NaN code (the caller's
    // promise, or the checks below), the accumulators stay below 2^(log2 K + 18 / 25 / 32, by operand formats) in the hardware formats' units, and the only
    // factor is the one power of two known here: the fast converters then skip their look-out for such values.
    const bool in_kernel_check = need_scan && gemm_large_tile_checks_operands(g);
    // a launch whose workgroups are all resident at once settles special codes inside the launch (panel words, see
    // GemmProblem::chk_state); it needs those words, which the allocation-free entry point does not have
    const size_t panel_words = (size_t) g.batch[0] * g.batch[1] * g.batch[2] * (size_t) (g.M / 256 + g.N / 256);
    bool         in_launch_check = in_kernel_check && gemm_large_tile_one_round(g, h->num_cus) && !h->noalloc && panel_words <= CHK_STATE_REGION_WORDS;
    if (in_launch_check)
    {
        // A launch recorded into a graph is replayed with the panel words as its last run left them, counts already at their
        // final values: a workgroup would look at a panel before this run's lookers have reported.  Recorded calls take the
        // epoch flag below, which a replay may find set by an earlier run (then the exact kernels run: slower, never wrong).
        in_launch_check = !h->recording;
    }
    {
        bool finite = h->fp8_specials_policy == MME_HIP_FP8_SPECIALS_ASSUME_NONE || in_kernel_check ||
                      (plan.nonfinite_kind[0] < 0 && plan.nonfinite_kind[1] < 0 && need_scan);
        uint32_t bits;
        memcpy(&bits, &g.epi.alpha, 4);
        const int ex = g.epi.has_alpha ? (int) ((bits >> 23) & 0xFF) - 127 : 0;
        int       log2k = 0;
        while ((1ll << log2k) < g.K) log2k++;
        // a product of two codes in the hardware formats' units stays below 2^18 (e4m3 x e4m3: 448^2), 2^25 (mixed: 448 x 57344)
        // or 2^32 (e5m2 x e5m2: 57344^2), a sum of K of them below 2^(log2 K + that)
        const int prod_log2 = g.fmt_a && g.fmt_b ? 32 : (g.fmt_a || g.fmt_b ? 25 : 18);
        const int acc_log2 = log2k + prod_log2;
        g.epi.finite = finite && !g.epi.col_exp && acc_log2 + ex < 127;

        // The plain large-tile fp8 kernel can hand that power of two to the matrix instruction (its block-scale operand) and
        // save a multiplication per output.  Scaling before the fp32 accumulation equals scaling after it as long as nothing
        // leaves the normal fp32 range either way: the smallest product is 2^-32 in the hardware formats' units (two e5m2
        // denormals) and sums stay below 2^acc_log2.
        if (g.epi.has_alpha && !in_kernel_check && ex >= -94 && ex <= 100 && acc_log2 + ex < 127 && gemm_large_tile_takes_mfma_scale(g))
        {
            g.epi.mfma_scale_exp = ex;
            g.epi.alpha = 1.0f;
            g.epi.has_alpha = 0;
        }
    }
    if (!need_scan)
    {
        LAUNCH_TRY(h, launch_gemm(g, h->stream));
        return MME_HIP_OK;
    }
    // the constants of the in-kernel look: a byte b is special when (b & m) == m, m = the exponent field (kind 0) or all of 0x7F
    // (kind 1: only 0x7F / 0xFF).  An operand in its hardware-native mode is looked at as well, for its inf / NaN codes: the
    // exact fall-back converts those values like any other, and the native kernel's epilogue may count on finite accumulators.
    auto set_check_constants = [&]()
    {
        const mme_hip_tensor* t[2] = {ta, tb};
        uint32_t              mask[2], add[2];
        for (int i = 0; i < 2; i++)
        {
            const int      kind = plan.scan_kind[i] >= 0 ? plan.scan_kind[i] : plan.nonfinite_kind[i];
            const uint32_t m = kind < 0 ? 0u : (kind == 1 ? 0x7Fu : (t[i]->dtype == MME_HIP_FP8_143 ? 0x78u : 0x7Cu));
            mask[i] = m * 0x01010101u;
            add[i] = m ? (0x80u - m) * 0x01010101u : 0u;
        }
        g.chk_mask_a = mask[0], g.chk_add_a = add[0], g.chk_mask_b = mask[1], g.chk_add_b = add[1];
        g.chk_inf_nan_a = ta->inf_nan_mode, g.chk_inf_nan_b = tb->inf_nan_mode;
    };
    if (in_launch_check)
    {
        if (!h->chk_state.p) HIP_TRY(h, grow(h, h->chk_state, (size_t) CHK_STATE_RING * CHK_STATE_REGION_WORDS * sizeof(uint32_t)));
        const unsigned slot = h->chk_state_launches++ % CHK_STATE_RING;
        if (slot == 0) LAUNCH_TRY(h, launch_fill_u32((uint32_t*) h->chk_state.p, 0u, (size_t) CHK_STATE_RING * CHK_STATE_REGION_WORDS, h->stream));
        g.chk = 2;
        g.chk_state = (uint32_t*) h->chk_state.p + (size_t) slot * CHK_STATE_REGION_WORDS;
        set_check_constants();
        LAUNCH_TRY(h, launch_gemm(g, h->stream));
        return MME_HIP_OK;
    }
    // the flag holds the epoch of the latest call that met such a code; the native kernel either finds them itself while it
    // multiplies (the large-tile kernels that can) or is skipped when a scan launch in front of it found one; decode + bf16
    // kernel run only when the flag holds this call's epoch, and then write the whole output
    uint32_t* flag = nullptr;
    uint32_t  epoch = 0;
    if (int rc = next_flag_epoch(h, &flag, &epoch)) return rc;
    g.skip_flag = flag;
    g.skip_epoch = epoch;
    g.skip_if = 1; // native variant: skipped when the scan found something
    if (in_kernel_check)
    {
        g.chk = 1;
        set_check_constants();
    }
    else
        LAUNCH_TRY(h, launch_fp8_special_scan2(flag, epoch, a_base, span_elements(ta), ta->dtype == MME_HIP_FP8_143 ? 3 : 2, plan.scan_kind[0], b_base,
                                            span_elements(tb), tb->dtype == MME_HIP_FP8_143 ? 3 : 2, plan.scan_kind[1], h->stream));
    LAUNCH_TRY(h, launch_gemm(g, h->stream));

    const size_t na = span_elements(ta), nb = span_elements(tb);
    const size_t na_pad = (na + 7) & ~(size_t) 7;
    void* decode_ws = nullptr;
    if (int rc = take_ws(h, h->decode_ws, (na_pad + nb + 8) * 2, &decode_ws)) return rc;
    uint16_t* da = (uint16_t*) decode_ws;
    uint16_t* db = da + na_pad;
    LAUNCH_TRY(h, launch_fp8_to_bf16_2(da, (const uint8_t*) a_base, na, ta->dtype == MME_HIP_FP8_143 ? 3 : 2, (int) ta->fp_bias, ta->inf_nan_mode, db,
                                    (const uint8_t*) b_base, nb, tb->dtype == MME_HIP_FP8_143 ? 3 : 2, (int) tb->fp_bias, tb->inf_nan_mode, flag,
                                    epoch, h->stream));
    GemmProblem g2 = g;
    g2.chk = 0;
    g2.dtype = DT_BF16;
    g2.A.base = (const char*) da;
    g2.B.base = (const char*) db;
    // the decoded copies keep the operands' layout; vector legality: 8 bf16 per 16 bytes is a weaker requirement than
    // 16 fp8 per 16 bytes on every stride, and both copies start 16-byte aligned
    {
        uint32_t bits;
        memcpy(&bits, &g.epi.alpha, 4);
        int e = (g.epi.has_alpha ? (int) ((bits >> 23) & 0xFF) - 127 : 0) + g.epi.mfma_scale_exp;
        e -= fold; // decoded operands carry their true values
        g2.epi.alpha = pow2f(e);
        g2.epi.has_alpha = e != 0;
        g2.epi.mfma_scale_exp = 0;
        g2.epi.finite = 0; // (the decoded operands may hold inf and NaN)
    }
    g2.skip_if = 0; // decoded variant: skipped unless the scan found something
    g2.split_k = g.split_k;
    LAUNCH_TRY(h, launch_gemm(g2, h->stream));
    return MME_HIP_OK;
}

int fill_epilogue(mme_hip_handle h, GemmEpilogue& e, const mme_hip_tensor* out, const mme_hip_epilogue* epi)
{
    memset(&e, 0, sizeof e);
    e.out = out->data;
    e.out_dtype = out->dtype == MME_HIP_FP32_IEEE ? DT_FP32 : out->dtype;
    e.alpha = 1.0f;
    if (epi)
    {
        e.fused = 1;
        e.cast = make_cast(out->dtype, out->fp_bias, out->inf_nan_mode, epi->rounding_mode, epi->clip_fp, epi->clip_inf_in,
                           epi->flush_denorms, epi->relu, 0);
        e.fast_cast = cast_params_fast(e.cast);
        e.alpha = pow2f(epi->scale_exp);
        e.has_alpha = epi->scale_exp != 0;
        e.col_exp = epi->col_scale_exp;
    }
    (void) h;
    return MME_HIP_OK;
}
// after the stream has been synchronised: did a kernel give up one of its bounded waits since the last look?
int check_status(mme_hip_handle h)
{
    const uint32_t code = *(volatile uint32_t*) h->status_host;
    if (code == 0) return MME_HIP_OK;
    *(volatile uint32_t*) h->status_host = 0;
    return fail(h, MME_HIP_EHIP, "a kernel gave up a bounded wait on its workgroup's counters (code 0x%08x): the output of the calls since the last synchronisation is not valid", code);
}

bool stochastic_epilogue(const mme_hip_epilogue* epi)
{
    return epi && (epi->rounding_mode == MME_HIP_RM_STOCHASTIC || epi->rounding_mode == MME_HIP_RM_STOCHASTIC_AND_NEAREST);
}
} // namespace

extern "C" int mme_hip_activation_dev(mme_hip_handle h, const mme_hip_tensor* out, const mme_hip_tensor* acc, int relu, int rm, int clip_fp,
                                      int clip_inf_in, int flush_denorms, int stochastic_ftz);

namespace
{
// A fused epilogue with a stochastic rounding mode.  The reference draws element i's random bits from LFSR register i % L
// after i / L steps (convertToOutputDataType, mme_reference_impl.cpp:1153-1240), an order that belongs to the flat output
// buffer, not to a tile walk; so the contraction writes its scaled (and rectified) fp32 results into a work space laid out
// like the output, and the stochastic cast kernel of doActivation converts that, with the calculator's registers and in the
// reference's order.  `contraction(tmp, epilogue)` runs the contraction into the fp32 tensor tmp.
template<class F>
int with_stochastic_epilogue(mme_hip_handle h, const mme_hip_tensor* out, const mme_hip_epilogue* epi, F&& contraction)
{
    mme_hip_tensor tmp = *out;
    tmp.dtype = MME_HIP_FP32;
    tmp.fp_bias = 0;
    tmp.inf_nan_mode = MME_HIP_FULL_INF_NAN;
    const size_t n = (size_t) span_elements(out);
    void*        p = nullptr;
    if (int rc = take_ws(h, h->stoch_ws, (n ? n : 1) * sizeof(float), &p)) return rc;
    tmp.data = p;
    // gaps between strided rows are converted too (the cast runs over the tensor's span): they hold zeros, as a freshly
    // allocated accumulator tensor of the reference would
    if (n != n_elements(out)) LAUNCH_TRY(h, launch_fill_u32((uint32_t*) p, 0u, n, h->stream));
    mme_hip_epilogue plain = *epi;
    plain.rounding_mode = MME_HIP_RM_NEAREST_EVEN;
    plain.clip_fp = plain.clip_inf_in = plain.flush_denorms = 0;
    if (int rc = contraction(&tmp, &plain)) return rc;
    return mme_hip_activation_dev(h, out, &tmp, 0, epi->rounding_mode, epi->clip_fp, epi->clip_inf_in, epi->flush_denorms, 0);
}
} // namespace

// =====================================================================================================================
extern "C" {

const char* mme_hip_version(void) { return "mme-hip 0.1 gfx950"; }

const char* mme_hip_last_error(mme_hip_handle h) { return h ? h->error.c_str() : g_create_error.c_str(); }

int mme_hip_create(mme_hip_handle* out, int chip, int max_tensor_dims, int max_conv_dims, unsigned seed, uint32_t lfsr_num_regs,
                   const uint32_t* lfsr, uint32_t polynomial)
{
    if (!out) return fail(nullptr, MME_HIP_EINVAL, "got null pointer");
    *out = nullptr;
    if (max_tensor_dims != MME_HIP_MAX_TENSOR_DIMS || max_conv_dims != MME_HIP_MAX_CONV_DIMS)
        return fail(nullptr, MME_HIP_EINVAL, "dynamic value different than static value");
    if (chip != MME_HIP_CHIP_GAUDI3)
    {
        if (chip == MME_HIP_CHIP_GAUDI || chip == MME_HIP_CHIP_GAUDI2)
            return fail(nullptr, MME_HIP_EUNSUPPORTED, "only the Gaudi3 numerics are built in this library");
        return fail(nullptr, MME_HIP_EINVAL, "unknown chip type");
    }
    mme_hip_calc* h = new (std::nothrow) mme_hip_calc;
    if (!h) return fail(nullptr, MME_HIP_ENOMEM, "out of host memory");
    hipError_t e = hipGetDevice(&h->device);
    if (e == hipSuccess)
    {
        hipDeviceProp_t prop;
        e = hipGetDeviceProperties(&prop, h->device);
        if (e == hipSuccess)
        {
            h->num_cus = prop.multiProcessorCount;
            if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            {
                std::string arch = prop.gcnArchName;
                delete h;
                return fail(nullptr, MME_HIP_EHIP, "this library holds gfx950 code objects only, device is %s", arch.c_str());
            }
        }
    }
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&h->own_stream, hipStreamNonBlocking);
    if (e != hipSuccess)
    {
        delete h;
        return fail(nullptr, MME_HIP_EHIP, "no usable HIP device: %s", hipGetErrorString(e));
    }
    h->stream = h->own_stream;
    e = hipHostMalloc((void**) &h->status_host, 256, hipHostMallocMapped);
    if (e == hipSuccess)
    {
        memset(h->status_host, 0, 256);
        e = hipHostGetDevicePointer((void**) &h->status_dev, h->status_host, 0);
    }
    if (e != hipSuccess)
    {
        mme_hip_destroy(h);
        return fail(nullptr, MME_HIP_EHIP, "no host-visible status word: %s", hipGetErrorString(e));
    }
    if (h->device < 0 || h->device >= MAX_DEVICES)
    {
        const int dev = h->device;
        mme_hip_destroy(h);
        return fail(nullptr, MME_HIP_EHIP, "device index %d is beyond the %d devices this library keeps scratch addresses for", dev, MAX_DEVICES);
    }
    {
        // the device address of this device's copy of the static scratch array (the current device is the handle's)
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (!g_scratch_ptr[h->device])
        {
            void* p = nullptr;
            e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !p)
            {
                mme_hip_destroy(h);
                return fail(nullptr, MME_HIP_EHIP, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
            }
            g_scratch_ptr[h->device] = p;
        }
    }
    // LFSR registers and polynomial exactly as the reference seeds them (mme_reference_impl.cpp:146-170)
    h->lfsr.resize(lfsr_num_regs);
    for (uint32_t i = 0; i < lfsr_num_regs; i++) h->lfsr[i] = lfsr ? lfsr[i] : i + 2;
    if (polynomial == 0)
    {
        std::mt19937                    gen(seed);
        std::uniform_int_distribution<> distr(25, 63);
        h->polynomial = (uint32_t) distr(gen);
    }
    else
        h->polynomial = polynomial & 0xFFFFu; // the reference keeps it in a uint16_t member (mme_reference_impl.h:253)
    // the LFSR's jump table and its device copy are made here, not on the first stochastic conversion: that call may come
    // through the entry point that allocates nothing, or while its stream records a graph
    if (int rc = build_lfsr_jump(h))
    {
        g_create_error = h->error;
        mme_hip_destroy(h);
        return rc;
    }
    *out = h;
    return MME_HIP_OK;
}

void mme_hip_destroy(mme_hip_handle h)
{
    if (!h) return;
    if (h->own_stream)
    {
        (void) hipStreamSynchronize(h->own_stream);
        (void) hipStreamDestroy(h->own_stream);
    }
    if (h->status_host) (void) hipHostFree(h->status_host);
    for (int i = 0; i < 2; i++)
    {
        if (h->bounce_ev[i]) (void) hipEventDestroy(h->bounce_ev[i]);
        if (h->bounce[i]) (void) hipHostFree(h->bounce[i]);
    }
    delete h;
}

int mme_hip_limit_num_of_threads(mme_hip_handle h, unsigned n)
{
    if (!h) return MME_HIP_EINVAL;
    h->num_threads = n;
    return MME_HIP_OK;
}

void* mme_hip_stream(mme_hip_handle h) { return h ? (void*) h->stream : nullptr; }

int mme_hip_set_stream(mme_hip_handle h, void* s)
{
    if (!h) return MME_HIP_EINVAL;
    h->stream = s ? (hipStream_t) s : h->own_stream;
    h->chk_state_launches = 0; // (the panel words are cleared in stream order: start a fresh ring on the new stream)
    return MME_HIP_OK;
}

int mme_hip_synchronize(mme_hip_handle h)
{
    if (!h) return MME_HIP_EINVAL;
    HIP_TRY(h, hipStreamSynchronize(h->stream));
    return check_status(h);
}

int mme_hip_set_wait_limit(mme_hip_handle h, unsigned polls)
{
    if (!h) return MME_HIP_EINVAL;
    h->wait_limit = polls;
    return MME_HIP_OK;
}

int mme_hip_clock_probe(mme_hip_handle h, int enable)
{
    if (!h) return MME_HIP_EINVAL;
    h->clock_probe = nullptr;
    if (!enable) return MME_HIP_OK;
    const size_t bytes = (size_t) CLOCK_PROBE_WORKGROUPS * 4 * sizeof(uint64_t);
    HIP_TRY(h, hipSetDevice(h->device));
    HIP_TRY(h, grow(h, h->clock_probe_buf, bytes));
    LAUNCH_TRY(h, launch_fill_u32((uint32_t*) h->clock_probe_buf.p, 0, bytes / 4, h->stream));
    h->clock_probe = (uint64_t*) h->clock_probe_buf.p;
    return MME_HIP_OK;
}

int mme_hip_clock_probe_read(mme_hip_handle h, double* shader_mhz, double* mean_us, double* max_us, int* workgroups)
{
    if (!h) return MME_HIP_EINVAL;
    if (!h->clock_probe) return fail(h, MME_HIP_EINVAL, "mme_hip_clock_probe_read: the probe is switched off");
    const size_t          cells = (size_t) CLOCK_PROBE_WORKGROUPS * 4;
    std::vector<uint64_t> host(cells);
    HIP_TRY(h, hipSetDevice(h->device));
    HIP_TRY(h, hipMemcpyAsync(host.data(), h->clock_probe, cells * sizeof(uint64_t), hipMemcpyDeviceToHost, h->stream));
    LAUNCH_TRY(h, launch_fill_u32((uint32_t*) h->clock_probe, 0, cells * 2, h->stream));
    HIP_TRY(h, hipStreamSynchronize(h->stream));
    double clocks = 0, ticks = 0, worst = 0;
    int    n = 0;
    for (int wg = 0; wg < CLOCK_PROBE_WORKGROUPS; wg++)
    {
        const uint64_t* c = &host[4 * (size_t) wg];
        if (!c[1] || c[3] <= c[1]) continue; // this workgroup did not run (or not to its end) since the last read
        clocks += (double) (c[2] - c[0]);
        ticks += (double) (c[3] - c[1]);
        worst = std::max(worst, (double) (c[3] - c[1]));
        n++;
    }
    if (workgroups) *workgroups = n;
    if (shader_mhz) *shader_mhz = n ? clocks / ticks * 100.0 : 0.0;
    if (mean_us) *mean_us = n ? ticks / n / 100.0 : 0.0;
    if (max_us) *max_us = worst / 100.0;
    return MME_HIP_OK;
}

int mme_hip_last_contraction_form(mme_hip_handle h, int* large_tile, int* tile_rows, int* split_k, int* wavefronts)
{
    if (!h) return MME_HIP_EINVAL;
    if (large_tile) *large_tile = h->last_form[0];
    if (tile_rows) *tile_rows = h->last_form[1];
    if (split_k) *split_k = h->last_form[2];
    if (wavefronts) *wavefronts = h->last_form[3];
    return MME_HIP_OK;
}

int mme_hip_matrix_core_rate(mme_hip_handle h, int dtype, int random_operands, int iters, int launches, double* tflops, double* shader_mhz)
{
    if (!h || iters < 1 || launches < 1) return MME_HIP_EINVAL;
    if (dtype != MME_HIP_FP8_143 && dtype != MME_HIP_BF16) return fail(h, MME_HIP_EUNSUPPORTED, "mme_hip_matrix_core_rate: fp8_143 or bf16");
    const int kind = dtype == MME_HIP_FP8_143 ? 0 : 1;
    HIP_TRY(h, hipSetDevice(h->device));
    uint64_t* stamps = nullptr;
    HIP_TRY(h, hipMalloc((void**) &stamps, 513 * sizeof(uint64_t)));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    for (int i = 0; i < 2 && e == hipSuccess; i++) e = launch_matrix_core_rate(kind, random_operands, iters, stamps, h->stream);
    if (e == hipSuccess) e = hipEventRecord(e0, h->stream);
    for (int i = 0; i < launches && e == hipSuccess; i++) e = launch_matrix_core_rate(kind, random_operands, iters, stamps, h->stream);
    if (e == hipSuccess) e = hipEventRecord(e1, h->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(h->stream);
    float                 ms = 0;
    std::vector<uint64_t> host(512);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e == hipSuccess) e = hipMemcpy(host.data(), stamps, 512 * sizeof(uint64_t), hipMemcpyDeviceToHost);
    if (e0) (void) hipEventDestroy(e0);
    if (e1) (void) hipEventDestroy(e1);
    (void) hipFree(stamps);
    if (e != hipSuccess) return hip_fail(h, e, "mme_hip_matrix_core_rate");
    double clocks = 0, ticks = 0;
    for (int wg = 0; wg < 256; wg++)
    {
        clocks += (double) host[2 * wg];
        ticks += (double) host[2 * wg + 1];
    }
    // 256 workgroups x 8 wavefronts x iters x 8 accumulators x one 32x32x64 step (fp8: one instruction, bf16: two of 32x32x16... x2)
    const double flop_per_acc_step = kind == 0 ? 2.0 * 32 * 32 * 64 : 2.0 * 2.0 * 32 * 32 * 16;
    if (tflops) *tflops = 256.0 * 8 * iters * 8 * flop_per_acc_step * launches / (ms * 1e-3) / 1e12;
    if (shader_mhz) *shader_mhz = ticks > 0 ? clocks / ticks * 100.0 : 0.0;
    return MME_HIP_OK;
}

int mme_hip_set_operand_clip(mme_hip_handle h, int clip_fp, int clip_fp_inf_in)
{
    if (!h) return MME_HIP_EINVAL;
    h->operand_clip_fp = clip_fp != 0;
    h->operand_clip_inf_in = clip_fp_inf_in != 0;
    return MME_HIP_OK;
}

int mme_hip_set_fp8_specials_policy(mme_hip_handle h, int policy)
{
    if (!h) return MME_HIP_EINVAL;
    if (policy != MME_HIP_FP8_SPECIALS_CHECK && policy != MME_HIP_FP8_SPECIALS_ASSUME_NONE)
        return fail(h, MME_HIP_EINVAL, "unknown fp8 specials policy %d", policy);
    h->fp8_specials_policy = policy;
    return MME_HIP_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// batched GEMM
// ---------------------------------------------------------------------------------------------------------------------
int mme_hip_batch_gemm_dev(mme_hip_handle h, const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, int op,
                           const mme_hip_epilogue* epi)
{
    if (!h) return MME_HIP_EINVAL;
    note_recording(h);
    if (int rc = check_tensor(h, out, "output")) return rc;
    if (int rc = check_tensor(h, x, "x")) return rc;
    if (int rc = check_tensor(h, w, "w")) return rc;
    if (op < MME_HIP_OP_AB || op > MME_HIP_OP_ATBT) return fail(h, MME_HIP_EINVAL, "invalid bgemm op %d", op);
    if (int rc = check_operand_types(h, x, w)) return rc;
    if (int rc = check_out_type(h, out, epi)) return rc;
    if (stochastic_epilogue(epi) && out->dtype != MME_HIP_FP32)
        return with_stochastic_epilogue(h, out, epi, [&](const mme_hip_tensor* tmp, const mme_hip_epilogue* e) { return mme_hip_batch_gemm_dev(h, tmp, x, w, op, e); });
    for (int d = 2; d < 5; d++)
        if (!((x->sizes[d] == out->sizes[d] || x->sizes[d] == 1) && (w->sizes[d] == out->sizes[d] || w->sizes[d] == 1)))
            return fail(h, MME_HIP_EINVAL, "batch dims doesnt match !");
    const int out_es = elem_size(out->dtype);
    if (n_elements(x) == 0 || n_elements(w) == 0)
    {
        // zero common dimension: the output is all zeros (handleZeroCdCase, mme_reference_impl.cpp:204-216)
        if (n_elements(x) != n_elements(w)) return fail(h, MME_HIP_EINVAL, "One of the input tensors is zero-size, while the other is not");
        const size_t bytes = span_elements(out) * out_es;
        if (bytes % 4) return fail(h, MME_HIP_EUNSUPPORTED, "zero-size contraction into an output whose byte size is not a multiple of 4");
        LAUNCH_TRY(h, launch_fill_u32((uint32_t*) out->data, 0u, bytes / 4, h->stream));
        return MME_HIP_OK;
    }
    const bool ta = (op == MME_HIP_OP_ATB || op == MME_HIP_OP_ATBT);
    const bool tb = (op == MME_HIP_OP_ABT || op == MME_HIP_OP_ATBT);
    const int  M = ta ? x->sizes[0] : x->sizes[1];
    const int  Ka = ta ? x->sizes[1] : x->sizes[0];
    const int  Kb = tb ? w->sizes[0] : w->sizes[1];
    const int  N = tb ? w->sizes[1] : w->sizes[0];
    if (Ka != Kb) return fail(h, MME_HIP_EINVAL, "Common dim doesnt match between input A\\B");
    if ((int) out->sizes[0] != N) return fail(h, MME_HIP_EINVAL, "output width doesnt match to inputB width");
    if ((int) out->sizes[1] != M) return fail(h, MME_HIP_EINVAL, "output height doesnt match to inputA height");

    GemmProblem g;
    memset(&g, 0, sizeof g);
    g.dtype = x->dtype;
    g.M = M;
    g.N = N;
    g.K = Ka;
    const int es = elem_size(x->dtype);
    long long abs_[3], bbs[3];
    for (int d = 0; d < 3; d++)
    {
        g.batch[d] = out->sizes[d + 2];
        abs_[d] = x->sizes[d + 2] == 1 ? 0 : x->strides[d + 2];
        bbs[d] = w->sizes[d + 2] == 1 ? 0 : w->strides[d + 2];
    }
    // A(m, k): x[m * s1 + k] or, transposed, x[k * s1 + m];   B(n, k): w[k * s1 + n] or, transposed, w[n * s1 + k]
    set_plain_view(g.A, x->data, ta ? 1 : x->strides[1], ta ? x->strides[1] : 1, !ta, es, ta ? M : Ka, abs_);
    set_plain_view(g.B, w->data, tb ? w->strides[1] : 1, tb ? 1 : w->strides[1], tb, es, tb ? Kb : N, bbs);
    if (int rc = fill_epilogue(h, g.epi, out, epi)) return rc;
    g.epi.ld = out->strides[1];
    for (int d = 0; d < 3; d++) g.epi.batch_stride[d] = out->strides[d + 2];
    return run_contraction(h, g, x, w, x->data, w->data);
}

int mme_hip_batch_gemm_dev_noalloc(mme_hip_handle h, const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, int op,
                                   const mme_hip_epilogue* epi)
{
    if (!h) return MME_HIP_EINVAL;
    if (!g_scratch_ptr[h->device]) return fail(h, MME_HIP_EHIP, "the static scratch array has no address on device %d", h->device);
    // every work space request of this call is served from the static array; nothing below allocates or frees
    struct Scope
    {
        mme_hip_handle h;
        explicit Scope(mme_hip_handle h_) : h(h_)
        {
            h->noalloc = true;
            h->noalloc_used = 256; // the flag cell
        }
        ~Scope() { h->noalloc = false; }
    } scope(h);
    return mme_hip_batch_gemm_dev(h, out, x, w, op, epi);
}

// ---------------------------------------------------------------------------------------------------------------------
// convolution
// ---------------------------------------------------------------------------------------------------------------------
int mme_hip_convolution_dev(mme_hip_handle h, const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w,
                            const mme_hip_tensor* y, const mme_hip_conv_params* cp, int op, const mme_hip_epilogue* epi)
{
    if (!h) return MME_HIP_EINVAL;
    note_recording(h);
    if (!cp) return fail(h, MME_HIP_EINVAL, "got null pointer");
    // (deterministic_dedw is a descriptor-generation variant: the reference's calculator rejects it too, mme_reference_impl.cpp:656-657)
    if (op == MME_HIP_OP_TRANSPOSED_DEDX)
    {
        // mme_reference_impl.cpp:625-647: exchange the first two weight dimensions, reverse the S axis, then dedx.  The
        // weights are small; they are repacked into a workspace by one launch, as the reference does on the host
        if (int rc = check_tensor(h, w, "inputB")) return rc;
        uint64_t acc = 1;
        bool     dense = true;
        for (int d = 0; d < 5; d++)
        {
            dense = dense && !(w->sizes[d] > 1 && w->strides[d] != acc);
            acc *= w->sizes[d];
        }
        const int   es = elem_size(w->dtype);
        const void* w_dense = w->data;
        void*       ws = nullptr;
        if (!dense)
        {
            // strided weights: a dense copy first
            if (int rc = take_ws(h, h->pack_ws[0], (size_t) acc * es + 16, &ws)) return rc;
            StridedCopyArgs a;
            uint32_t        run = 1;
            for (int i = 0; i < 5; i++)
            {
                a.sizes[i] = w->sizes[i], a.src_strides[i] = w->strides[i], a.dst_strides[i] = run;
                run *= w->sizes[i];
            }
            LAUNCH_TRY(h, launch_strided_copy(ws, w->data, es, a, h->stream));
            w_dense = ws;
        }
        if (int rc = take_ws(h, h->weights_ws, (size_t) acc * es + 16, &ws)) return rc;
        LAUNCH_TRY(h, launch_repack_transposed_weights(ws, w_dense, es, w->sizes[0], w->sizes[1], w->sizes[2], (size_t) acc, h->stream));
        mme_hip_tensor wr = *w;
        wr.data = ws;
        wr.sizes[0] = w->sizes[1];
        wr.sizes[1] = w->sizes[0];
        acc = 1;
        for (int d = 0; d < 5; d++)
        {
            wr.strides[d] = (uint32_t) acc;
            acc *= wr.sizes[d];
        }
        return mme_hip_convolution_dev(h, out, x, &wr, y, cp, MME_HIP_OP_DEDX, epi);
    }
    if (op != MME_HIP_OP_FWD && op != MME_HIP_OP_DEDX && op != MME_HIP_OP_DEDW) return fail(h, MME_HIP_EINVAL, "invalid operation");
    // operand roles (mme_reference_impl.cpp:611-655): fwd A=x B=w; dedx A=y B=w; dedw A=x B=y
    const mme_hip_tensor* A = op == MME_HIP_OP_DEDX ? y : x;
    const mme_hip_tensor* B = op == MME_HIP_OP_DEDW ? y : w;
    if (int rc = check_tensor(h, out, "output")) return rc;
    if (int rc = check_tensor(h, A, "inputA")) return rc;
    if (int rc = check_tensor(h, B, "inputB")) return rc;
    if (int rc = check_operand_types(h, A, B)) return rc;
    if (int rc = check_out_type(h, out, epi)) return rc;
    if (stochastic_epilogue(epi) && out->dtype != MME_HIP_FP32)
        return with_stochastic_epilogue(h, out, epi, [&](const mme_hip_tensor* tmp, const mme_hip_epilogue* e) {
            // the output tensor also stands in the argument list under its role's name
            return mme_hip_convolution_dev(h, tmp, op == MME_HIP_OP_DEDX ? tmp : x, op == MME_HIP_OP_DEDW ? tmp : w, op == MME_HIP_OP_FWD ? tmp : y, cp, op, e);
        });
    for (int i = 0; i < 4; i++)
        if (cp->conv_stride[i] < 1 || cp->dilation[i] < 1) return fail(h, MME_HIP_EINVAL, "convolution stride and dilation must be positive");

    const mme_hip_tensor* wt = op == MME_HIP_OP_DEDW ? out : w; // weight-shaped  [K, C, S, R, Q]
    const mme_hip_tensor* yt = op == MME_HIP_OP_FWD ? out : y;  // output-shaped  [K, W', H', D', B]
    const mme_hip_tensor* xt = op == MME_HIP_OP_DEDX ? out : x; // input-shaped   [C, W, H, D, B]
    const int Kc = wt->sizes[0], C = wt->sizes[1];
    const int taps = wt->sizes[2] * wt->sizes[3] * wt->sizes[4];
    if ((int) xt->sizes[0] != C) return fail(h, MME_HIP_EINVAL, "channel dims of x and w differ");
    if ((int) yt->sizes[0] != Kc) return fail(h, MME_HIP_EINVAL, "channel dims of y and w differ");
    const long long y_pix = (long long) yt->sizes[1] * yt->sizes[2] * yt->sizes[3] * yt->sizes[4];
    const long long x_pix = (long long) xt->sizes[1] * xt->sizes[2] * xt->sizes[3] * xt->sizes[4];
    if (y_pix >= (1ll << 31) || x_pix >= (1ll << 31) || (long long) taps * std::max(C, Kc) >= (1ll << 31))
        return fail(h, MME_HIP_EINVAL, "convolution extents exceed 2^31");
    if (n_elements(out) == 0) return MME_HIP_OK;

    // The kernels address the weights as one matrix with a single row pitch (rows of K output channels, one per (channel,
    // tap)), the output as rows of one pitch, and dedw's dy likewise.  A tensor whose strides do not collapse that way (the
    // reference takes any strides, createBufferWith/WithoutStrides, mme_reference_impl.cpp:245-319) is contracted through a
    // dense copy: inputs are gathered into one first, a result is computed densely and scattered into the caller's layout
    // afterwards (only the tensor's own elements are written, what lies between them is left alone).
    {
        const mme_hip_tensor* w_in = op == MME_HIP_OP_DEDW ? nullptr : w;
        const mme_hip_tensor* y_in = op == MME_HIP_OP_DEDW ? y : nullptr;
        const bool            pack_w = w_in && !rows_collapsible(w_in), pack_y = y_in && !rows_collapsible(y_in), pack_out = !rows_collapsible(out);
        if (pack_w || pack_y || pack_out)
        {
            auto dense_of = [](const mme_hip_tensor* t, void* data) {
                mme_hip_tensor d = *t;
                uint32_t       acc = 1;
                for (int i = 0; i < 5; i++)
                {
                    d.strides[i] = acc;
                    acc *= t->sizes[i];
                }
                d.data = data;
                return d;
            };
            auto copy = [&](const mme_hip_tensor* dst, const mme_hip_tensor* src) {
                StridedCopyArgs a;
                for (int i = 0; i < 5; i++) a.sizes[i] = src->sizes[i], a.src_strides[i] = src->strides[i], a.dst_strides[i] = dst->strides[i];
                return launch_strided_copy(dst->data, src->data, elem_size(src->dtype), a, h->stream);
            };
            mme_hip_tensor wd, yd, od;
            void*          p = nullptr;
            if (pack_w)
            {
                if (int rc = take_ws(h, h->pack_ws[0], (size_t) n_elements(w) * elem_size(w->dtype) + 16, &p)) return rc;
                wd = dense_of(w, p);
                LAUNCH_TRY(h, copy(&wd, w));
            }
            if (pack_y)
            {
                if (int rc = take_ws(h, h->pack_ws[1], (size_t) n_elements(y) * elem_size(y->dtype) + 16, &p)) return rc;
                yd = dense_of(y, p);
                LAUNCH_TRY(h, copy(&yd, y));
            }
            if (pack_out)
            {
                if (int rc = take_ws(h, h->pack_ws[2], (size_t) n_elements(out) * elem_size(out->dtype) + 16, &p)) return rc;
                od = dense_of(out, p);
            }
            const mme_hip_tensor* o2 = pack_out ? &od : out;
            const mme_hip_tensor* x2 = op == MME_HIP_OP_DEDX ? o2 : x;
            const mme_hip_tensor* w2 = op == MME_HIP_OP_DEDW ? o2 : (pack_w ? &wd : w);
            const mme_hip_tensor* y2 = op == MME_HIP_OP_FWD ? o2 : (pack_y ? &yd : y);
            if (int rc = mme_hip_convolution_dev(h, o2, x2, w2, y2, cp, op, epi)) return rc;
            if (pack_out) LAUNCH_TRY(h, copy(out, &od));
            return MME_HIP_OK;
        }
    }
    const long long w_ld = (long long) taps * C > 1 ? (long long) wt->strides[1] : Kc;
    if (w_ld < Kc) return fail(h, MME_HIP_EINVAL, "weight rows overlap");

    const int es = elem_size(A->dtype);
    const int kv = 16 / es;

    if (op == MME_HIP_OP_FWD)
    {
        auto dense = [](const mme_hip_tensor* t) {
            uint64_t acc = 1;
            for (int d = 0; d < 5; d++)
            {
                if (t->sizes[d] > 1 && t->strides[d] != acc) return false;
                acc *= t->sizes[d];
            }
            return ((uintptr_t) t->data % 16) == 0;
        };
        const int st[4] = {cp->conv_stride[0], cp->conv_stride[1], cp->conv_stride[2], cp->conv_stride[3]};
        const int di[4] = {cp->dilation[0], cp->dilation[1], cp->dilation[2], cp->dilation[3]};
        const int pa[4] = {cp->padding[0], cp->padding[1], cp->padding[2], cp->padding[3]};
        const bool same = out->sizes[1] == x->sizes[1] && out->sizes[2] == x->sizes[2] && out->sizes[3] == 1 && out->sizes[4] == x->sizes[4];
        if (same && x->dtype == MME_HIP_BF16 && w->dtype == MME_HIP_BF16 && !is_fp16(out->dtype) &&
            conv_fwd_fast_applicable(x->dtype, C, Kc, w->sizes[2], w->sizes[3], w->sizes[4], x->sizes[1], x->sizes[2], x->sizes[3], st, di, pa,
                                     dense(x) && dense(w) && dense(out)))
        {
            GemmEpilogue e;
            if (int rc = fill_epilogue(h, e, out, epi)) return rc;
            e.ld = Kc;
            h->last_form[0] = 2, h->last_form[1] = 0, h->last_form[2] = 1, h->last_form[3] = 8; // (the 3 x 3, 64 -> 64 channel forward kernel)
            LAUNCH_TRY(h, launch_conv_fwd_fast(x->data, w->data, x->sizes[4], x->sizes[2], x->sizes[1], e, h->num_cus, h->status_dev, h->wait_limit, h->stream));
            return MME_HIP_OK;
        }
    }

    GemmProblem g;
    memset(&g, 0, sizeof g);
    g.dtype = A->dtype;
    g.batch[0] = g.batch[1] = g.batch[2] = 1;
    const long long zero3[3] = {0, 0, 0};

    auto conv_view = [&](OperandView& v, const mme_hip_tensor* src, const mme_hip_tensor* pixels, int nch, int pix_is_f, int gather_y) {
        memset(&v, 0, sizeof v);
        v.base = (const char*) src->data;
        v.kind = VIEW_CONV;
        v.pix_is_f = pix_is_f;
        v.gather_y = gather_y;
        v.nch = nch;
        v.k_contig = pix_is_f; // channels are contiguous; they run along k when pixels run along f
        bool ok = ((uintptr_t) src->data % 16 == 0) && (nch % kv == 0);
        for (int d = 0; d < 4; d++)
        {
            v.grid[d] = pixels->sizes[d + 1];
            v.src[d] = src->sizes[d + 1];
            v.src_stride[d] = src->strides[d + 1];
            v.cstride[d] = cp->conv_stride[d];
            v.dil[d] = cp->dilation[d];
            v.pad[d] = cp->padding[d];
            ok = ok && (src->strides[d + 1] % kv == 0);
        }
        for (int d = 0; d < 3; d++) v.ktap[d] = wt->sizes[d + 2];
        v.vec_ok = ok;
    };

    if (op == MME_HIP_OP_FWD)
    {
        // Y[pix][k] = sum_{tap, c} X[pos(pix, tap)][c] * W[(tap * C + c)][k]
        g.M = (int) y_pix;
        g.N = Kc;
        g.K = taps * C;
        conv_view(g.A, x, out, C, 1, 0);
        set_plain_view(g.B, w->data, 1, w_ld, false, es, Kc, zero3);
    }
    else if (op == MME_HIP_OP_DEDX)
    {
        // dX[pix][c] = sum_{tap, k} dY[src(pix, tap)][k] * W[(tap * C + c)][k]     (gather form of col2im)
        g.M = (int) x_pix;
        g.N = C;
        g.K = taps * Kc;
        conv_view(g.A, y, out, Kc, 1, 1);
        memset(&g.B, 0, sizeof g.B);
        g.B.base = (const char*) w->data;
        g.B.kind = VIEW_TAPPED;
        g.B.k_contig = 1;
        g.B.stride_f = w_ld;
        g.B.stride_k = 1;
        g.B.tap_stride = w_ld * C;
        g.B.nch = Kc;
        g.B.vec_ok = ((uintptr_t) w->data % 16 == 0) && (Kc % kv == 0) && (w_ld % kv == 0);
    }
    else
    {
        // dW[(tap * C + c)][k] = sum_pix X[pos(pix, tap)][c] * dY[pix][k]
        g.M = taps * C;
        g.N = Kc;
        g.K = (int) y_pix;
        conv_view(g.A, x, y, C, 0, 0);
        set_plain_view(g.B, y->data, 1, y->strides[1], false, es, Kc, zero3);
    }
    if (int rc = fill_epilogue(h, g.epi, out, epi)) return rc;
    g.epi.ld = out->strides[1];
    return run_contraction(h, g, A, B, A->data, B->data);
}

namespace
{
// a handle for planning only: no device, no stream, nothing allocated; the registers and the jump table that a stochastic
// epilogue's host bookkeeping reads are there (all zero)
void make_planning_handle(mme_hip_calc& h, int num_cus, int fp8_specials_policy)
{
    h.dry_run = true;
    h.num_cus = num_cus > 0 ? num_cus : 256;
    h.fp8_specials_policy = fp8_specials_policy;
    h.lfsr.assign(256, 0u);
    h.lfsr_jump.assign((size_t) LFSR_JUMP_LEVELS * 32, 0u);
}

int planned_form(mme_hip_calc& h, int rc, int form[4], char* error, size_t error_bytes)
{
    for (int i = 0; i < 4; i++) form[i] = rc == MME_HIP_OK ? h.last_form[i] : 0;
    if (error && error_bytes)
    {
        snprintf(error, error_bytes, "%s", rc == MME_HIP_OK ? "" : h.error.c_str());
    }
    return rc;
}
} // namespace

int mme_hip_plan_batch_gemm(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, int op, const mme_hip_epilogue* epi,
                            int num_cus, int fp8_specials_policy, int form[4], char* error, size_t error_bytes)
{
    if (!form) return MME_HIP_EINVAL;
    mme_hip_calc h;
    make_planning_handle(h, num_cus, fp8_specials_policy);
    h.last_form[0] = -1; // (a zero-size contraction launches no contraction kernel at all)
    return planned_form(h, mme_hip_batch_gemm_dev(&h, out, x, w, op, epi), form, error, error_bytes);
}

int mme_hip_plan_convolution(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, const mme_hip_tensor* y,
                             const mme_hip_conv_params* cp, int op, const mme_hip_epilogue* epi, int num_cus, int fp8_specials_policy, int form[4],
                             char* error, size_t error_bytes)
{
    if (!form) return MME_HIP_EINVAL;
    mme_hip_calc h;
    make_planning_handle(h, num_cus, fp8_specials_policy);
    h.last_form[0] = -1;
    return planned_form(h, mme_hip_convolution_dev(&h, out, x, w, y, cp, op, epi), form, error, error_bytes);
}

namespace
{
// jump table of the handle's LFSR: entry [k][b] = state reached from the one-bit state 1 << b after 2^k steps (built once, when
// the calculator is created)
int build_lfsr_jump(mme_hip_handle h)
{
    std::vector<uint32_t> t((size_t) LFSR_JUMP_LEVELS * 32);
    for (int b = 0; b < 32; b++) t[b] = lfsr32_step(1u << b, h->polynomial);
    for (int k = 1; k < LFSR_JUMP_LEVELS; k++)
        for (int b = 0; b < 32; b++)
        {
            // two times 2^(k-1) steps
            const uint32_t x = t[(size_t) (k - 1) * 32 + b];
            uint32_t       y = 0;
            for (int c = 0; c < 32; c++)
                if ((x >> c) & 1u) y ^= t[(size_t) (k - 1) * 32 + c];
            t[(size_t) k * 32 + b] = y;
        }
    HIP_TRY(h, h->lfsr_jump_dev.reserve(t.size() * 4));
    HIP_TRY(h, hipMemcpy(h->lfsr_jump_dev.p, t.data(), t.size() * 4, hipMemcpyHostToDevice));
    h->lfsr_jump = std::move(t);
    return MME_HIP_OK;
}

uint32_t lfsr_jump_host(mme_hip_handle h, uint32_t s, unsigned long long steps)
{
    for (int k = 0; steps != 0 && k < LFSR_JUMP_LEVELS; k++, steps >>= 1)
        if (steps & 1ull)
        {
            uint32_t y = 0;
            for (int b = 0; b < 32; b++)
                if ((s >> b) & 1u) y ^= h->lfsr_jump[(size_t) k * 32 + b];
            s = y;
        }
    return s;
}
} // namespace

// ---------------------------------------------------------------------------------------------------------------------
// activation / casts
// ---------------------------------------------------------------------------------------------------------------------
int mme_hip_activation_dev(mme_hip_handle h, const mme_hip_tensor* out, const mme_hip_tensor* acc, int relu, int rm, int clip_fp,
                           int clip_inf_in, int flush_denorms, int stochastic_ftz)
{
    if (!h) return MME_HIP_EINVAL;
    note_recording(h);
    if (int rc = check_tensor(h, out, "output")) return rc;
    if (int rc = check_tensor(h, acc, "acc")) return rc;
    if (acc->dtype != MME_HIP_FP32) return fail(h, MME_HIP_EINVAL, "acc element type should be fp32");
    if (acc->dim != out->dim) return fail(h, MME_HIP_EINVAL, "dims number of outputTensor doesnt match acc output");
    for (int d = 0; d < 5; d++)
        if (acc->sizes[d] != out->sizes[d]) return fail(h, MME_HIP_EINVAL, "sizes of output Tensot doesnt match acc output");
    if (!(out->dtype == MME_HIP_FP32 || out->dtype == MME_HIP_BF16 || is_fp8(out->dtype) || is_fp16(out->dtype)))
        return fail(h, MME_HIP_EINVAL, "Unsupported type");
    if (!(rm == 0 || rm == 1 || rm == 2 || rm == 3 || rm == 4 || rm == 6 || rm == 7)) return fail(h, MME_HIP_EINVAL, "invalid rounding mode %d", rm);
    // the reference converts the first getSizeInElements() elements of both flat buffers (:1155), and that count is the
    // tensor's span in memory, gaps between strided rows included (sim_tensor_base.cpp:177-194)
    const size_t n = span_elements(acc);
    if (span_elements(out) < n) return fail(h, MME_HIP_EINVAL, "the output tensor spans fewer elements than acc");
    if (relu)
    {
        // doRelu insists on a tensor without gaps (mme_reference_impl.cpp:1135)
        bool contiguous = acc->strides[0] == 1;
        for (int d = 1; d < acc->dim && d < MME_HIP_MAX_TENSOR_DIMS; d++) contiguous = contiguous && acc->strides[d] == acc->strides[d - 1] * acc->sizes[d - 1];
        if (!contiguous) return fail(h, MME_HIP_EINVAL, "input and output should be flattened");
        LAUNCH_TRY(h, launch_relu_inplace((float*) acc->data, n, h->stream));
    }
    const CastParams c = make_cast(out->dtype, out->fp_bias, out->inf_nan_mode, rm, clip_fp, clip_inf_in, flush_denorms, 0, 0);
    const bool       reseed = rm == MME_HIP_RM_STOCHASTIC || rm == MME_HIP_RM_STOCHASTIC_AND_NEAREST || stochastic_ftz;
    if (reseed && out->dtype != MME_HIP_FP32)
    {
        // element i takes LFSR register i % L and steps it (mme_reference_impl.cpp:1153-1240); the registers live in the
        // handle between calls, like m_lfsr in the reference's calculator
        const size_t L = (out->dtype == MME_HIP_BF16 || is_fp16(out->dtype)) ? 64 : 128;
        if (h->lfsr.size() < L) return fail(h, MME_HIP_EINVAL, "stochastic modes need %zu LFSR registers, the calculator has %zu", L, h->lfsr.size());
        LfsrRegisters regs;
        memset(&regs, 0, sizeof regs);
        for (size_t r = 0; r < L; r++) regs.v[r] = h->lfsr[r];
        LAUNCH_TRY(h, launch_cast_stochastic(out->data, (const float*) acc->data, n, c, stochastic_ftz, 1, h->polynomial, regs,
                                          (const uint32_t*) h->lfsr_jump_dev.p, h->stream));
        for (size_t r = 0; r < L && r < n; r++) h->lfsr[r] = lfsr_jump_host(h, h->lfsr[r], (n - r + L - 1) / L);
        return MME_HIP_OK;
    }
    LAUNCH_TRY(h, launch_cast_from_fp32(out->data, (const float*) acc->data, n, c, nullptr, 0, h->stream));
    return MME_HIP_OK;
}

int mme_hip_cast_from_fp32_dev(mme_hip_handle h, void* out, int out_dtype, unsigned out_fp_bias, int out_inf_nan_mode, const float* in,
                               size_t n, int scale_exp, const int32_t* col_scale_exp, size_t n_cols, int relu, int rm, int clip_fp,
                               int clip_inf_in, int flush_denorms)
{
    if (!h) return MME_HIP_EINVAL;
    if (!(out_dtype == MME_HIP_FP32 || out_dtype == MME_HIP_BF16 || is_fp8(out_dtype) || is_fp16(out_dtype)))
        return fail(h, MME_HIP_EINVAL, "Unsupported type");
    if (!(rm == 0 || rm == 1 || rm == 2 || rm == 3 || rm == 6))
        return fail(h, rm == 4 || rm == 7 ? MME_HIP_EUNSUPPORTED : MME_HIP_EINVAL, "rounding mode %d is not available here", rm);
    if (scale_exp < -126 || scale_exp > 126) return fail(h, MME_HIP_EINVAL, "scale exponent out of range");
    if (col_scale_exp && n_cols == 0) return fail(h, MME_HIP_EINVAL, "n_cols must be positive with per-column scales");
    if (n && (!out || !in)) return fail(h, MME_HIP_EINVAL, "got null pointer");
    const CastParams c = make_cast(out_dtype, out_fp_bias, out_inf_nan_mode, rm, clip_fp, clip_inf_in, flush_denorms, relu, scale_exp);
    LAUNCH_TRY(h, launch_cast_from_fp32(out, in, n, c, col_scale_exp, n_cols, h->stream));
    return MME_HIP_OK;
}

int mme_hip_cast_to_fp32_dev(mme_hip_handle h, float* out, const void* in, int in_dtype, unsigned in_fp_bias, int in_inf_nan_mode, size_t n,
                             int scale_exp, const int32_t* col_scale_exp, size_t n_cols)
{
    if (!h) return MME_HIP_EINVAL;
    if (!(in_dtype == MME_HIP_BF16 || is_fp8(in_dtype) || is_fp16(in_dtype))) return fail(h, MME_HIP_EINVAL, "Unsupported type");
    if (scale_exp < -126 || scale_exp > 126) return fail(h, MME_HIP_EINVAL, "scale exponent out of range");
    if (col_scale_exp && n_cols == 0) return fail(h, MME_HIP_EINVAL, "n_cols must be positive with per-column scales");
    if (n && (!out || !in)) return fail(h, MME_HIP_EINVAL, "got null pointer");
    LAUNCH_TRY(h, launch_cast_to_fp32(out, in, in_dtype, (int) in_fp_bias, in_inf_nan_mode, n, pow2f(scale_exp), scale_exp != 0, col_scale_exp,
                                   n_cols, h->stream));
    return MME_HIP_OK;
}

int mme_hip_absmax_dev(mme_hip_handle h, float* out_absmax, const float* in, size_t n)
{
    if (!h) return MME_HIP_EINVAL;
    if (!out_absmax || (n && !in)) return fail(h, MME_HIP_EINVAL, "got null pointer");
    LAUNCH_TRY(h, launch_absmax(out_absmax, in, n, h->stream));
    return MME_HIP_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// host-pointer entry points: stage through device memory, run the _dev form, copy back, synchronise
// ---------------------------------------------------------------------------------------------------------------------
namespace
{
// Host memory <-> device memory for the reference-compatible entry points.  The caller's buffers are ordinary pageable
// memory: they are moved through two pinned bounce buffers in chunks, the host-side copy of one chunk (a few threads)
// running while the DMA engine moves the other, so that a large tensor travels at close to the link's rate.
constexpr size_t BOUNCE_BYTES = (size_t) 16 << 20;
constexpr size_t BOUNCE_THREAD_BYTES = (size_t) 2 << 20; // one host thread per this many bytes of a chunk, at most four

void host_copy(void* dst, const void* src, size_t n)
{
    const size_t nt = std::min<size_t>(4, n / BOUNCE_THREAD_BYTES);
    if (nt < 2)
    {
        memcpy(dst, src, n);
        return;
    }
    std::vector<std::thread> workers;
    const size_t             per = ((n / nt) + 4095) & ~(size_t) 4095;
    for (size_t i = 1; i < nt; i++)
    {
        const size_t off = i * per, len = off >= n ? 0 : std::min(per, n - off);
        if (len) workers.emplace_back([=] { memcpy((char*) dst + off, (const char*) src + off, len); });
    }
    memcpy(dst, src, std::min(per, n));
    for (auto& w : workers) w.join();
}

int ensure_bounce(mme_hip_handle h)
{
    for (int i = 0; i < 2; i++)
    {
        if (!h->bounce[i]) HIP_TRY(h, hipHostMalloc(&h->bounce[i], BOUNCE_BYTES, hipHostMallocDefault));
        if (!h->bounce_ev[i]) HIP_TRY(h, hipEventCreateWithFlags(&h->bounce_ev[i], hipEventDisableTiming));
    }
    return MME_HIP_OK;
}

int host_to_device(mme_hip_handle h, void* dst, const void* src, size_t bytes)
{
    if (int rc = ensure_bounce(h)) return rc;
    int k = 0;
    for (size_t off = 0; off < bytes; off += BOUNCE_BYTES, k++)
    {
        const int    slot = k & 1;
        const size_t n = std::min(BOUNCE_BYTES, bytes - off);
        if (k >= 2) HIP_TRY(h, hipEventSynchronize(h->bounce_ev[slot])); // the DMA of chunk k - 2 has read this buffer
        host_copy(h->bounce[slot], (const char*) src + off, n);
        HIP_TRY(h, hipMemcpyAsync((char*) dst + off, h->bounce[slot], n, hipMemcpyHostToDevice, h->stream));
        HIP_TRY(h, hipEventRecord(h->bounce_ev[slot], h->stream));
    }
    // the bounce buffers are reused by the next transfer: it waits for these events first
    for (int i = 0; i < 2 && i < k; i++) HIP_TRY(h, hipEventSynchronize(h->bounce_ev[(k - 1 - i) & 1]));
    return MME_HIP_OK;
}

int device_to_host(mme_hip_handle h, void* dst, const void* src, size_t bytes)
{
    if (int rc = ensure_bounce(h)) return rc;
    const size_t chunks = (bytes + BOUNCE_BYTES - 1) / BOUNCE_BYTES;
    for (size_t k = 0; k <= chunks; k++)
    {
        if (k < chunks)
        {
            const size_t off = k * BOUNCE_BYTES, n = std::min(BOUNCE_BYTES, bytes - off);
            HIP_TRY(h, hipMemcpyAsync(h->bounce[k & 1], (const char*) src + off, n, hipMemcpyDeviceToHost, h->stream));
            HIP_TRY(h, hipEventRecord(h->bounce_ev[k & 1], h->stream));
        }
        if (k >= 1)
        {
            // chunk k - 1 has landed in its bounce buffer: hand it to the caller while chunk k is on its way
            const size_t off = (k - 1) * BOUNCE_BYTES, n = std::min(BOUNCE_BYTES, bytes - off);
            HIP_TRY(h, hipEventSynchronize(h->bounce_ev[(k - 1) & 1]));
            host_copy((char*) dst + off, h->bounce[(k - 1) & 1], n);
        }
    }
    return MME_HIP_OK;
}

struct Staged
{
    mme_hip_tensor t;
    void*          host = nullptr;
    size_t         bytes = 0;
};

// slot: which of the handle's three device-side staging buffers holds this tensor during the call
int stage_in(mme_hip_handle h, Staged& s, int slot, const mme_hip_tensor* src, bool copy)
{
    s.t = *src;
    s.host = src->data;
    s.bytes = (size_t) span_elements(src) * elem_size(src->dtype);
    HIP_TRY(h, grow(h, h->stage_dev[slot], s.bytes ? s.bytes : 16));
    s.t.data = h->stage_dev[slot].p;
    if (copy && s.bytes) return host_to_device(h, s.t.data, s.host, s.bytes);
    return MME_HIP_OK;
}
// (returns with the bytes in the caller's buffer: the copy waits for the stream's work before it)
int stage_out(mme_hip_handle h, Staged& s)
{
    if (s.bytes) return device_to_host(h, s.host, s.t.data, s.bytes);
    return MME_HIP_OK;
}
bool has_gaps(const mme_hip_tensor* t) { return span_elements(t) != n_elements(t); }
// the host entry points carry clipFp / clipFpInfIn per call: set them on the handle for the call's duration
struct OperandClipScope
{
    mme_hip_handle h;
    int            old_clip, old_inf;
    OperandClipScope(mme_hip_handle h_, int clip, int inf) : h(h_), old_clip(h_->operand_clip_fp), old_inf(h_->operand_clip_inf_in)
    {
        h->operand_clip_fp = clip != 0;
        h->operand_clip_inf_in = inf != 0;
    }
    ~OperandClipScope()
    {
        h->operand_clip_fp = old_clip;
        h->operand_clip_inf_in = old_inf;
    }
};
} // namespace

int mme_hip_batch_gemm(mme_hip_handle h, const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, int op, int rm, int clip_fp,
                       int clip_fp_inf_in)
{
    (void) rm; // the Gaudi3 tree hard-codes round-to-zero
    if (!h) return MME_HIP_EINVAL;
    // clipFp / clipFpInfIn reach the tf32 operand conversion only; the other FMA classes drop them (gaudi3_fma.h:43,79,96-98)
    const OperandClipScope clip_scope(h, clip_fp, clip_fp_inf_in);
    if (int rc = check_tensor(h, out, "output")) return rc;
    if (int rc = check_tensor(h, x, "x")) return rc;
    if (int rc = check_tensor(h, w, "w")) return rc;
    Staged so, sx, sw;
    // a strided output keeps the bytes between its rows: copy them in first
    if (int rc = stage_in(h, so, 0, out, has_gaps(out))) return rc;
    if (int rc = stage_in(h, sx, 1, x, true)) return rc;
    if (int rc = stage_in(h, sw, 2, w, true)) return rc;
    if (int rc = mme_hip_batch_gemm_dev(h, &so.t, &sx.t, &sw.t, op, nullptr)) return rc;
    if (int rc = stage_out(h, so)) return rc;
    HIP_TRY(h, hipStreamSynchronize(h->stream));
    return MME_HIP_OK;
}

int mme_hip_convolution(mme_hip_handle h, const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, const mme_hip_tensor* y,
                        const mme_hip_conv_params* cp, int op, int rm, int clip_fp, int clip_fp_inf_in)
{
    (void) rm; // reaches only col2im's additions in the reference; all taps share one accumulator here
    if (!h) return MME_HIP_EINVAL;
    const OperandClipScope clip_scope(h, clip_fp, clip_fp_inf_in);
    // (any other operation is an error, and the device-pointer form reports it before it touches a tensor; never hand it a
    // valid operation here: the tensors hold host pointers)
    if (op != MME_HIP_OP_FWD && op != MME_HIP_OP_DEDX && op != MME_HIP_OP_DEDW && op != MME_HIP_OP_TRANSPOSED_DEDX)
        return fail(h, MME_HIP_EINVAL, "invalid operation");
    if (!out || !x || !w || !y) return fail(h, MME_HIP_EINVAL, "got null pointer");
    const bool            dedx = op == MME_HIP_OP_DEDX || op == MME_HIP_OP_TRANSPOSED_DEDX; // the same roles, the weights laid out differently
    const mme_hip_tensor* A = dedx ? y : x;
    const mme_hip_tensor* B = op == MME_HIP_OP_DEDW ? y : w;
    if (int rc = check_tensor(h, out, "output")) return rc;
    if (int rc = check_tensor(h, A, "inputA")) return rc;
    if (int rc = check_tensor(h, B, "inputB")) return rc;
    Staged so, sa, sb;
    if (int rc = stage_in(h, so, 0, out, has_gaps(out))) return rc;
    if (int rc = stage_in(h, sa, 1, A, true)) return rc;
    if (int rc = stage_in(h, sb, 2, B, true)) return rc;
    const mme_hip_tensor* dx = dedx ? &so.t : &sa.t;
    const mme_hip_tensor* dw = op == MME_HIP_OP_DEDW ? &so.t : &sb.t;
    const mme_hip_tensor* dy = op == MME_HIP_OP_FWD ? &so.t : (dedx ? &sa.t : &sb.t);
    if (int rc = mme_hip_convolution_dev(h, &so.t, dx, dw, dy, cp, op, nullptr)) return rc;
    if (int rc = stage_out(h, so)) return rc;
    HIP_TRY(h, hipStreamSynchronize(h->stream));
    return check_status(h);
}

int mme_hip_activation(mme_hip_handle h, const mme_hip_tensor* out, const mme_hip_tensor* acc, int relu, int rm, int clip_fp, int clip_inf_in,
                       int flush_denorms, int stochastic_ftz)
{
    if (!h) return MME_HIP_EINVAL;
    if (int rc = check_tensor(h, out, "output")) return rc;
    if (int rc = check_tensor(h, acc, "acc")) return rc;
    Staged so, sa;
    if (int rc = stage_in(h, so, 0, out, true)) return rc;
    if (int rc = stage_in(h, sa, 1, acc, true)) return rc;
    if (int rc = mme_hip_activation_dev(h, &so.t, &sa.t, relu, rm, clip_fp, clip_inf_in, flush_denorms, stochastic_ftz)) return rc;
    if (int rc = stage_out(h, so)) return rc;
    if (relu)
        if (int rc = stage_out(h, sa)) return rc; // relu rewrites acc in place in the reference (:683-686)
    HIP_TRY(h, hipStreamSynchronize(h->stream));
    return MME_HIP_OK;
}

int mme_hip_memory_write_dev(mme_hip_handle h, const mme_hip_tensor* memory, const mme_hip_tensor* mme_out, int reduction_op, int reduction_rm,
                             int clip_fp)
{
    if (!h) return MME_HIP_EINVAL;
    note_recording(h);
    if (!memory || !mme_out) return fail(h, MME_HIP_EINVAL, "got null pointer");
    if (reduction_op < 0 || reduction_op > MME_HIP_REDUCTION_NONE) return fail(h, MME_HIP_EINVAL, "invalid reduction operation %d", reduction_op);
    const size_t n = (size_t) span_elements(memory);
    if (n && (!memory->data || !mme_out->data)) return fail(h, MME_HIP_EINVAL, "got null pointer");
    if (reduction_op == MME_HIP_REDUCTION_NONE)
    {
        // a byte copy of the destination tensor's size (mme_reference_impl.cpp:725-729)
        const size_t bytes = n * elem_size(memory->dtype);
        if (bytes) HIP_TRY(h, hipMemcpyAsync(memory->data, mme_out->data, bytes, hipMemcpyDeviceToDevice, h->stream));
        return MME_HIP_OK;
    }
    // element types of a reduction: convertDataTypeToDataTypeRMW, mme_reference_impl.cpp:691-716
    switch (memory->dtype)
    {
        case MME_HIP_BF16:
        case MME_HIP_FP16:    // (the unit's fp16 and fp8_152: exponent bias 15 with inf and NaN, whatever the tensor's fields say)
        case MME_HIP_FP8_152:
        case MME_HIP_FP32: break;
        case MME_HIP_FP8_143: return fail(h, MME_HIP_EINVAL, "fp8_143 is not supported in reduction");
        case MME_HIP_UFP16: return fail(h, MME_HIP_EINVAL, "ufp16 is not supported in reduction");
        default: return fail(h, MME_HIP_EINVAL, "Unsupported data type when converting to reduction RMW data type");
    }
    if (mme_out->dtype != memory->dtype) return fail(h, MME_HIP_EINVAL, "element types of memory and mmeOut differ");
    if (reduction_rm < 0 || reduction_rm > 3) return fail(h, MME_HIP_EINVAL, "invalid reduction rounding mode %d", reduction_rm);
    LAUNCH_TRY(h, launch_memory_write_reduce(memory->data, mme_out->data, memory->dtype, n, reduction_op, reduction_rm,
                                          clip_fp, h->stream));
    return MME_HIP_OK;
}

int mme_hip_memory_write(mme_hip_handle h, const mme_hip_tensor* memory, const mme_hip_tensor* mme_out, int reduction_op, int reduction_rm,
                         int clip_fp)
{
    if (!h) return MME_HIP_EINVAL;
    if (!memory || !mme_out) return fail(h, MME_HIP_EINVAL, "got null pointer");
    if (reduction_op == MME_HIP_REDUCTION_NONE)
    {
        // reduction none: a byte copy of the destination tensor's size (mme_reference_impl.cpp:725-729), host to host
        const size_t bytes = (size_t) span_elements(memory) * elem_size(memory->dtype);
        if (bytes) memmove(memory->data, mme_out->data, bytes);
        return MME_HIP_OK;
    }
    // the reduction reads memory's span of elements from both buffers
    mme_hip_tensor o = *mme_out;
    for (int d = 0; d < 5; d++)
    {
        o.sizes[d] = memory->sizes[d];
        o.strides[d] = memory->strides[d];
    }
    Staged sm, so;
    if (int rc = stage_in(h, sm, 0, memory, true)) return rc;
    if (int rc = stage_in(h, so, 1, &o, true)) return rc;
    if (int rc = mme_hip_memory_write_dev(h, &sm.t, &so.t, reduction_op, reduction_rm, clip_fp)) return rc;
    if (int rc = stage_out(h, sm)) return rc;
    HIP_TRY(h, hipStreamSynchronize(h->stream));
    return MME_HIP_OK;
}

} // extern "C"
