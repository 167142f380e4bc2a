// gemm_large_tile_impl.hpp -- body of the large-tile contraction kernels (256 x 256 outputs per workgroup, operands brought
// into LDS by DMA, matrix-core instructions fed from a four-stage ring).  The translation units that include it
// instantiate the kernels: gemm_large_tile.hip (fp8, bf16; its header comment describes the design) and
// gemm_large_tile_f16.hip (IEEE half).
#pragma once
#include <type_traits>

#include "gemm_impl.hpp"

namespace mme
{
namespace
{
typedef int v2i __attribute__((ext_vector_type(2)));
#define LDS3 __attribute__((address_space(3)))

constexpr int FBM = 256, FBN = 256, FBK = 64, FNST = 4;
constexpr int FSTAGE = FBM * FBK + FBK * FBN; // 32 KiB

__device__ __forceinline__ int fa_pos(int r, int c) { return r * 4 + (c ^ ((r >> 2) & 3)); }
__device__ __forceinline__ int fb_pos(int k, int cb) { return k * 16 + ((cb + 2 * (k & 7)) & 15); }

// 16 bytes per lane from global memory to LDS at lds_off + lane * 16 (lds_off is wave-uniform).  Inline assembly keeps
// the request out of the compiler's memory model: it would otherwise order every later LDS read behind it.
__device__ __forceinline__ void dma16(const void* g, uint32_t lds_off)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_off) : "memory");
}

// operand fragments of one stage: four 32-row blocks of A, NJ 32-column blocks of B
template<int NJ>
struct FragsT
{
    v8i a[4], b[NJ];
};

// (row0: first row of this wavefront's block of the staged A tile; the B readers take the address of the stage's B part)
template<class FR>
__device__ __forceinline__ void read_a(FR& f, int i, const char* st, int row0, int lane)
{
    const int r = row0 + i * 32 + (lane & 31), c0 = 2 * (lane >> 5);
    const v4i lo = *(const v4i*) (st + fa_pos(r, c0) * 16), hi = *(const v4i*) (st + fa_pos(r, c0 + 1) * 16);
    f.a[i] = v8i {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

// B stored n-contiguous: transposed LDS reads (cb0: the wavefront's first 16-column chunk of the tile)
template<class FR>
__device__ __forceinline__ void read_b_tr(FR& f, int j, const char* st, int cb0, int lane)
{
    const int q = lane >> 4, cb = cb0 + j * 2 + (q & 1), g = q >> 1, rr = (lane & 15) >> 1, h = lane & 1;
    v2i       t[4];
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
    {
        const int k = g * 32 + 8 * tt + rr;
        t[tt] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LDS3 v2i*) (st + fb_pos(k, cb) * 16 + h * 8));
    }
    f.b[j] = v8i {t[0].x, t[0].y, t[1].x, t[1].y, t[2].x, t[2].y, t[3].x, t[3].y};
}

// bf16, B stored n-contiguous: a stage is 32 k-rows x 256 columns x 2 B = 32 chunks of 16 B per row, the 32-byte blocks of a
// row XOR-swizzled by k & 3.  ds_read_b64_tr_b16: within a group of 16 lanes, lane q addresses the 8-byte piece q % 4 of
// row q / 4 and receives 4 consecutive k of its own column.  The fragment's k order ({0-7, 16-23} then {8-15, 24-31}
// for the two lane halves) is the one the k-contiguous reads of the other operand produce.
template<class FR>
__device__ __forceinline__ void read_b_tr16(FR& f, int j, const char* st, int cb0, int lane)
{
    typedef short v4s __attribute__((ext_vector_type(4)));
    const int g = lane >> 4, q = lane & 15, h = g >> 1, block = cb0 + j * 2 + (g & 1);
    union
    {
        v4s h4[4];
        v8i v;
    } u;
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
    {
        // reads 0, 1 -> k = 16 h + 0 .. 7 (first MFMA), reads 2, 3 -> k = 16 h + 8 .. 15 (second MFMA)
        const int k = 16 * h + 4 * tt + (q >> 2);
        u.h4[tt] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS3 v4s*) (st + k * 512 + ((block ^ (k & 3)) << 5) + ((q & 3) << 3)));
    }
    f.b[j] = u.v;
}

// bf16, A stored f-contiguous: the same stage layout and reads as an n-contiguous B, over the wavefront's TM / 2 rows
// (a k-row of the stage is TM elements = TM / 16 blocks of 32 bytes)
template<int TM, class FR>
__device__ __forceinline__ void read_a_tr16(FR& f, int i, const char* st, int wm, int lane)
{
    typedef short v4s __attribute__((ext_vector_type(4)));
    const int g = lane >> 4, q = lane & 15, h = g >> 1, block = wm * (TM / 32) + i * 2 + (g & 1);
    union
    {
        v4s h4[4];
        v8i v;
    } u;
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
    {
        const int k = 16 * h + 4 * tt + (q >> 2);
        u.h4[tt] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS3 v4s*) (st + k * (TM * 2) + ((block ^ (k & 3)) << 5) + ((q & 3) << 3)));
    }
    f.a[i] = u.v;
}

// fp8, A stored f-contiguous: the stage layout and reads of an n-contiguous fp8 B (64 k-rows x 256 bytes), over the
// wavefront's 128 rows = 8 chunks of 16
template<class FR>
__device__ __forceinline__ void read_a_tr8(FR& f, int i, const char* st, int wm, int lane)
{
    const int q = lane >> 4, cb = wm * 8 + i * 2 + (q & 1), g = q >> 1, rr = (lane & 15) >> 1, h = lane & 1;
    v2i       t[4];
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
    {
        const int k = g * 32 + 8 * tt + rr;
        t[tt] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LDS3 v2i*) (st + fb_pos(k, cb) * 16 + h * 8));
    }
    f.a[i] = v8i {t[0].x, t[0].y, t[1].x, t[1].y, t[2].x, t[2].y, t[3].x, t[3].y};
}

// B stored k-contiguous (the "abt" form): same layout and reads as A
template<class FR>
__device__ __forceinline__ void read_b_kc(FR& f, int j, const char* st, int cb0, int lane)
{
    const int r = cb0 * 16 + j * 32 + (lane & 31), c0 = 2 * (lane >> 5);
    const v4i lo = *(const v4i*) (st + fa_pos(r, c0) * 16), hi = *(const v4i*) (st + fa_pos(r, c0 + 1) * 16);
    f.b[j] = v8i {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

#define FENCE __builtin_amdgcn_sched_barrier(0)

// s_waitcnt immediate that waits until at most n of this wavefront's memory requests are outstanding and leaves the other
// counters alone (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14)
constexpr int vm_wait(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

// The problem description is read in place from the kernarg segment, field by field where the code needs it: every 64-byte
// line touched for the first time (tile set-up, gather set-up, epilogue) would be a miss of its own, one memory latency
// each, in series.  One scalar load per line up front takes all those misses at once.
__device__ __forceinline__ void warm_kernargs(KARG GemmProblem& g)
{
    static_assert(sizeof(GemmProblem) > 640 && sizeof(GemmProblem) <= 704, "one load per 64-byte line of the problem description");
    uint32_t t0, t1, t2, t3, t4, t5, t6, t7, t8, t9, t10;
    asm volatile("s_load_dword %0, %11, 0x0\n\t"
                 "s_load_dword %1, %11, 0x40\n\t"
                 "s_load_dword %2, %11, 0x80\n\t"
                 "s_load_dword %3, %11, 0xc0\n\t"
                 "s_load_dword %4, %11, 0x100\n\t"
                 "s_load_dword %5, %11, 0x140\n\t"
                 "s_load_dword %6, %11, 0x180\n\t"
                 "s_load_dword %7, %11, 0x1c0\n\t"
                 "s_load_dword %8, %11, 0x200\n\t"
                 "s_load_dword %9, %11, 0x240\n\t"
                 "s_load_dword %10, %11, 0x280\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5), "=&s"(t6), "=&s"(t7), "=&s"(t8), "=&s"(t9), "=&s"(t10)
                 : "s"(&g)
                 : "memory");
}

// ES = 1: fp8 (FMT selects e4m3 / e5m2 per operand), ES = 2: bf16 (FMT 0) or IEEE half (FMT 1).  Everything up to the matrix-core instruction is
// byte-based and shared: a stage is 64 bytes of k per row for both.
// GATHER: A is a convolution view with pixels along f (im2col addressing of mme/mme_reference/im2col.cpp:134-172 for the
// forward pass, its gather-form inverse for dedx): row r of the tile is a pixel, a 64-byte stage is a run of channels
// of one filter tap, so a request's address is (pixel's offset for tap 0) + (the tap's uniform offset) + channel, or a
// page of zeros where the tap falls outside the source tensor.  B may then be a tapped weight view (dedx).
__device__ __attribute__((aligned(16))) uint32_t gf_zero_page[GF_ZERO_PAGE_BYTES / 4];

//
// AMODE says how operand A is addressed: 0 plain, k contiguous; 1 convolution view with pixels along f (GATHER above);
// 2 plain, f contiguous (the "atb" forms; bf16 only: the stage then holds 32 k-rows x 256 f like an n-contiguous B and is
// read with ds_read_b64_tr_b16); 3 convolution view with pixels along k (dedw: f = tap * channels + channel is fixed per
// lane, the pixel advances by 32 per stage and is decoded incrementally).
// TM: rows of the output tile, 256 or 128 (128 for problems whose 256-row tiles would leave most of the chip idle; AMODE
// 0, 1 and 3).  A wavefront then owns TM / 2 rows x 64 columns; an f-contiguous A stage is 32 k-rows of TM elements, one
// request of 16 bytes per lane covers 2 (TM 256) or 4 (TM 128) of them.
// RG ("ragged", not for AMODE 2): N is any multiple of 16 and, for AMODE 0, M any count (the convolution views take any pixel
// count as they are): the loads of a partial tile are clamped to the operand's last row / last 16-byte chunk and its stores
// are predicated.  A separate instantiation, so that the kernels for whole tiles stay free of the clamps and predicates.
// PERSIST (AMODE 0, whole 256-row tiles, 1- or 2-byte fused outputs, no split-k; gridDim = (256, 1, 1) and 160 KiB of LDS):
// a workgroup walks over tiles id, id + 256, ... of all batch elements.  Once the last fragments of a tile have left the
// ring, the first four stages of the next tile are requested, and the epilogue of the finished tile (which stages its
// stores in the 32 KiB of LDS behind the ring) runs while they arrive: pipeline fill and epilogue overlap.
// CHK (fp8, AMODE 0, whole 256-row tiles): the kernel inspects the operand bytes on their way to the matrix cores for codes
// that the hardware's fp8 formats read differently from Gaudi's (GemmProblem::chk_*) and raises the problem's flag when it
// meets one.  Every 64-byte stage of an operand row is looked at by exactly one of the workgroups that read it (stage t of
// the A rows by the tile column t mod tiles_n, of the B columns by the tile row t mod tiles_m): when its turn comes, each
// wavefront reads an eighth of that part of the stage once more from LDS and tests the bytes, a few vector instructions in
// the shadow of the matrix instructions, so a clean operand costs no extra pass over memory and no extra launch.  With one
// workgroup per tile and one round of tiles (GemmProblem::chk == 2) the hit is not handed to the host's fall-back but
// settled inside the launch: see SELFCHK in the body.
// NST: stages of the ring (4 to 6, default 4; every instantiation uses the default: six stages of the 128-row tile's 24 KiB
// measured 2-3 % slower than four on the 3 x 3 convolutions of 32 x 28 x 28 x 256, whose steps then divide by six to find a slot).
// The reduction has to be at least NST stages long.
// NW: wavefronts of the workgroup, 8 (2 x 4, each TM / 2 rows x 64 columns, two per SIMD) or 4 (2 x 2, each 128 rows x 128
// columns with its 256 accumulator registers in the upper half of the 512-register file, one per SIMD: a stage then costs
// 64 KiB of LDS reads instead of 96; fp8 and AMODE 0 with whole 256-row tiles only).
template<int ES, int FMT, bool B_KC, int AMODE = 0, int TM = FBM, bool RG = false, bool PERSIST = false, bool CHK = false, int NST = FNST, int NW = 8>
__device__ __forceinline__ void gemm_fast_body_impl(KARG GemmProblem& g)
{
    static_assert(NST >= 4 && NST <= 6 && (!PERSIST || NST == FNST), "ring depth");
    static_assert(NW == 8 || (NW == 4 && AMODE == 0 && TM == FBM && !RG && !PERSIST && NST == FNST), "four wavefronts: plain k-contiguous A, whole 256-row tiles");
    static_assert(!CHK || (ES == 1 && AMODE == 0 && TM == FBM && !RG), "operand checks: fp8, plain k-contiguous A, whole 256-row tiles");
    static_assert(!PERSIST || (AMODE == 0 && TM == FBM && !RG), "the persistent schedule: plain k-contiguous A, whole 256-row tiles");
    static_assert(TM == 256 || (TM == 128 && AMODE != 2), "the 128-row tile is not instantiated for plain f-contiguous A");
    static_assert(TM == 256 || ES == 2 || AMODE < 2, "fp8 operands that are contiguous along the tile's rows: 256-row tiles only");
    constexpr int  WR = TM / 2;                   // rows per wavefront
    constexpr int  NI = WR / 32;                  // A fragments (32-row blocks) per wavefront
    constexpr int  WGN = NW / 2;                  // the wavefronts form a 2 x WGN grid over the tile
    constexpr int  WC = FBN / WGN;                // columns per wavefront
    constexpr int  NJ = WC / 32;                  // B fragments (32-column blocks) per wavefront
    constexpr int  NUA = TM * FBK / 1024 / NW;    // A requests per lane and stage (16 rows x 64 bytes per wavefront and request)
    constexpr int  NUB = FBN * FBK / 1024 / NW;   // B requests per lane and stage
    constexpr int  A_BYTES = TM * FBK;            // A part of a stage; the B part follows
    constexpr int  STAGE = A_BYTES + FBK * FBN;   // 32 KiB or 24 KiB
    constexpr int  NREQ = NUA + NUB;              // requests per lane and stage
    using Frags = FragsT<NJ>;
    constexpr bool GATHER = AMODE == 1;           // tap masks + uniform tap offsets
    static_assert(!RG || AMODE != 2, "partial tiles are not instantiated for plain f-contiguous A");
    constexpr bool RAGGED_M = AMODE == 1 || AMODE == 3 || RG; // the last row tile may be partial
    // (RG: the last column tile may be partial too; N is a multiple of 16, so a lane's 16 columns are all in or all out)
    constexpr bool A_KC = AMODE < 2;
    // CHK, one workgroup per tile: when the host says so (chk == 2: one round of tiles, every workgroup resident) the workgroups
    // note per operand panel what their looks found and how many of a panel's lookers are done; after its epilogue a workgroup
    // waits for the lookers of its own two panels (long done by then) and, if one of them met such a code, computes its tile
    // once more, exactly, inside the same launch (below, after the loop).  No flag for the host then, nothing enqueued behind
    // the kernel.
    constexpr bool SELFCHK = CHK && !PERSIST;
    const bool     in_launch = SELFCHK && g.chk == 2;
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    warm_kernargs(g);
    if (!CHK && g.skip_flag && ((*g.skip_flag == g.skip_epoch) == (g.skip_if != 0))) return;

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), wm = wave / WGN, wn = wave % WGN;
    const int tiles_n = RG ? (g.N + FBN - 1) / FBN : g.N / FBN, tiles_m = (g.M + TM - 1) / TM;
    const int tiles_total = tiles_m * tiles_n;
    int       m0 = 0, n0 = 0, b0 = 0, b1 = 0, b2 = 0, cur_tm = 0, cur_tn = 0;
    uint32_t  chk_bad = 0; // CHK: bit 7 of a byte is set once a special code has been seen
    const long long lda = (A_KC ? g.A.stride_f : g.A.stride_k) * ES; // bytes between rows of the staged A tile
    const long long ldb = (B_KC ? g.B.stride_f : g.B.stride_k) * ES;
    const uint8_t*  A = nullptr;
    const uint8_t*  B = nullptr;
    // tile L of the walk (each XCD owns a compact 8 x 4 block of tiles at a time) and batch element bz -> m0, n0, A, B
    auto locate = [&](int L, int bz) __attribute__((always_inline))
    {
        int tm, tn;
        if ((tiles_m % 8 == 0) && (tiles_n % 4 == 0))
        {
            const int Bx = L >> 5, w = L & 31, nbn = tiles_n >> 2;
            tm = (Bx / nbn) * 8 + (w >> 2);
            tn = (Bx % nbn) * 4 + (w & 3);
        }
        else
        {
            tm = L / tiles_n;
            tn = L % tiles_n;
        }
        b0 = bz % g.batch[0];
        bz /= g.batch[0];
        b1 = bz % g.batch[1];
        b2 = bz / g.batch[1];
        const long long a_off = b0 * g.A.batch_stride[0] + b1 * g.A.batch_stride[1] + b2 * g.A.batch_stride[2];
        const long long b_off = b0 * g.B.batch_stride[0] + b1 * g.B.batch_stride[1] + b2 * g.B.batch_stride[2];
        m0 = tm * TM;
        n0 = tn * FBN;
        cur_tm = tm;
        cur_tn = tn;
        A = (const uint8_t*) g.A.base + a_off * ES;
        B = (const uint8_t*) g.B.base + b_off * ES;
    };
    // workgroup ids are dealt round-robin to the 8 XCDs
    const int walk_first = PERSIST ? (int) ((blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3)) : 0;
    const int walk_total = PERSIST ? tiles_total * g.batch[0] * g.batch[1] * g.batch[2] : 0;
    // split-k launches (grid = tiles x 1 x slices): the workgroups that land on one XCD (every eighth of the linear order) take
    // consecutive (slice, tile) pairs, so the tiles of a k-slice, which all read the same slice of B and overlapping slices of
    // A, find them in one L2 instead of fetching them into all eight
    int kslice = 0, split_tile = (int) blockIdx.x;
    if (!PERSIST && g.split_k > 1)
    {
        kslice = (int) blockIdx.z;
        if (gridDim.y == 1)
        {
            const int total = (int) (gridDim.x * gridDim.z), lin = (int) (blockIdx.x + gridDim.x * blockIdx.z);
            const int x = lin & 7, p = x * (total >> 3) + min(x, total & 7) + (lin >> 3); // a bijection of [0, total)
            kslice = p / (int) gridDim.x;
            split_tile = p - kslice * (int) gridDim.x;
        }
    }
    if constexpr (PERSIST) locate(walk_first % tiles_total, walk_first / tiles_total);
    else if (g.split_k > 1)
        locate(split_tile, blockIdx.y);
    else if ((tiles_m % 8 == 0) && (tiles_n % 4 == 0))
        locate((blockIdx.x & 7) * (tiles_total >> 3) + (blockIdx.x >> 3), blockIdx.y);
    else
        locate(blockIdx.x, blockIdx.y);
    const uint32_t  lds_base = (uint32_t) (uintptr_t) lds;

    v16f acc[NI][NJ];
#pragma unroll
    for (int i = 0; i < NI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // split-k: slice `kslice` takes an equal share of the stages and writes raw partial sums to the workspace
    const int nk = g.K * ES / FBK / (g.split_k > 1 ? g.split_k : 1), kt_begin = kslice * nk;
    // per-lane global pointers of this wavefront's request slots (they advance by one stage per step)
    const uint8_t* ga[NUB];
    const uint8_t* gb[NUB];
    auto setup_ptrs = [&]() __attribute__((always_inline))
    {
#pragma unroll
    for (int u = 0; u < NUB; u++)
    {
        const int t = wave * NUB + u;
        ga[u] = nullptr;
        if constexpr (AMODE == 0)
        {
            if (u < NUA)
            {
                const int r = (wave * NUA + u) * 16 + (lane >> 2), p = lane & 3, c = p ^ ((r >> 2) & 3);
                ga[u] = A + (size_t) (RG ? min(m0 + r, g.M - 1) : m0 + r) * lda + c * 16 + (size_t) kt_begin * FBK;
            }
        }
        if constexpr (AMODE == 2 && ES == 2)
        {
            const int k = t * 2 + (lane >> 5), p = lane & 31, chunk = p ^ ((k & 3) << 1);
            ga[u] = A + (size_t) (k + kt_begin * (FBK / 2)) * lda + m0 * 2 + chunk * 16;
        }
        if constexpr (AMODE == 2 && ES == 1)
        {
            const int k = t * 4 + (lane >> 4), p = lane & 15, cb = (p - 2 * (k & 7)) & 15;
            ga[u] = A + (size_t) (k + kt_begin * FBK) * lda + m0 + cb * 16;
        }
        if (B_KC)
        {
            const int r = t * 16 + (lane >> 2), p = lane & 3, c = p ^ ((r >> 2) & 3);
            gb[u] = B + (size_t) (RG ? min(n0 + r, g.N - 1) : n0 + r) * ldb + c * 16 + (size_t) kt_begin * FBK;
        }
        else if (GATHER && g.B.kind == VIEW_TAPPED)
            gb[u] = nullptr; // (tapped weights are k-contiguous: B_KC)
        else if (ES == 1)
        {
            const int k = t * 4 + (lane >> 4), p = lane & 15, cb = (p - 2 * (k & 7)) & 15;
            gb[u] = B + (size_t) (k + kt_begin * FBK) * ldb + (RG ? min(n0 + cb * 16, g.N - 16) : n0 + cb * 16);
        }
        else
        {
            const int k = t * 2 + (lane >> 5), p = lane & 31, chunk = p ^ ((k & 3) << 1);
            gb[u] = B + (size_t) (k + kt_begin * (FBK / 2)) * ldb + (RG ? min(n0 + chunk * 8, g.N - 8) : n0 + chunk * 8) * 2;
        }
    }
    };
    setup_ptrs();
    // ---- GATHER: per-row tap masks and the running (tap, channel) position of the stage being requested ----------------
    uint32_t  tap_ok[NUB] = {};        // bit t: tap t of this lane's row (request slot u) reads inside the source tensor
    int       g_tap = 0, g_ch = 0;     // uniform: tap and first channel of the next stage to request
    int       g_t[3] = {0, 0, 0};      // g_tap as (s, r, q)
    int       g_chb = 0;               // uniform: g_ch in bytes
    long long g_delta_b = 0;           // uniform byte offset of that stage in the weights (tapped: tap + channel; plain: stage)
    long long g_step_b = 0;            // plain weights: bytes from one stage to the next
    // per lane and request slot: where the current tap's channels of this lane's row start, or the zero page when the tap
    // falls into the padding (the zero page is as long as a row's channels, so every lane adds the same channel offset)
    const uint8_t* a_tap[NUB] = {};
    const int stage_ch = FBK / ES;     // channels per stage
    // (values that are the same in every lane are handed back to scalar registers after the vector arithmetic of a tap change)
    auto uniform32 = [](int x) __attribute__((always_inline)) { return __builtin_amdgcn_readfirstlane(x); };
    auto uniform64 = [](long long x) __attribute__((always_inline))
    {
        const uint32_t lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) x), hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) ((unsigned long long) x >> 32));
        return (long long) (((unsigned long long) hi << 32) | lo);
    };
    // a new tap (once per nch / stage_ch stages): its offset in the gathered tensor and in the tapped weights, and every
    // lane's base address for it
    auto gather_offsets = [&]() __attribute__((always_inline))
    {
        long long d = 0;
#pragma unroll
        for (int q = 0; q < 3; q++) d += (long long) g_t[q] * g.A.dil[q] * g.A.src_stride[q];
        const long long tap_a = uniform64((g.A.gather_y ? -d : d) * ES);
        if (g.B.kind == VIEW_TAPPED) g_delta_b = uniform64(((long long) g_tap * g.B.tap_stride + g_ch) * ES);
        g_chb = uniform32(g_ch * ES);
#pragma unroll
        for (int u = 0; u < NUA; u++)
        {
            const bool ok = (tap_ok[u] >> g_tap) & 1u;
            a_tap[u] = ok ? ga[u] + tap_a : (const uint8_t*) gf_zero_page;
        }
    };
    auto gather_advance = [&]() __attribute__((always_inline))
    {
        g_ch += stage_ch;
        if (g_ch >= g.A.nch)
        {
            g_ch = 0;
            g_tap = uniform32(g_tap + 1);
            if (++g_t[0] == g.A.ktap[0])
            {
                g_t[0] = 0;
                if (++g_t[1] == g.A.ktap[1])
                {
                    g_t[1] = 0;
                    g_t[2]++;
                }
            }
#pragma unroll
            for (int q = 0; q < 3; q++) g_t[q] = uniform32(g_t[q]);
            gather_offsets();
        }
        else
        {
            // same tap, next channels: the common case costs two scalar additions
            g_chb += FBK;
            if (g.B.kind == VIEW_TAPPED) g_delta_b += FBK;
        }
        // (plain weights: the stage's offset does not depend on the tap)
        if (g.B.kind != VIEW_TAPPED) g_delta_b += g_step_b;
    };
    if constexpr (GATHER)
    {
        const int ntaps = g.A.ktap[0] * g.A.ktap[1] * g.A.ktap[2];
#pragma unroll
        for (int u = 0; u < NUA; u++)
        {
            const int r = (wave * NUA + u) * 16 + (lane >> 2), p = lane & 3, c = p ^ ((r >> 2) & 3);
            const int pix = min(m0 + r, g.M - 1);
            const PixelPos pp = decode_pixel(g.A, pix);
            long long      off0 = 0;
#pragma unroll
            for (int d = 0; d < 4; d++)
                off0 += (long long) (g.A.gather_y ? pp.c[d] + g.A.pad[d] : pp.c[d] * g.A.cstride[d] - g.A.pad[d]) * g.A.src_stride[d];
            ga[u] = A + off0 * ES + c * 16;
            if (m0 + r < g.M)
            {
                // which taps land inside the tensor: range checks per dimension, the taps counted up as (s, r, q) digits
                // (no division: the gather form of col2im comes here with unit strides only)
                int ts[3] = {0, 0, 0};
                for (int t = 0; t < ntaps; t++)
                {
                    bool ok = true;
#pragma unroll
                    for (int d = 0; d < 4; d++)
                    {
                        const int td = d < 3 ? ts[d] * g.A.dil[d] : 0;
                        const int pos = g.A.gather_y ? pp.c[d] + g.A.pad[d] - td : pp.c[d] * g.A.cstride[d] + td - g.A.pad[d];
                        ok = ok && pos >= 0 && pos < g.A.src[d];
                    }
                    tap_ok[u] |= (ok ? 1u : 0u) << t;
                    if (++ts[0] == g.A.ktap[0])
                    {
                        ts[0] = 0;
                        if (++ts[1] == g.A.ktap[1])
                        {
                            ts[1] = 0;
                            ts[2]++;
                        }
                    }
                }
            }
        }
        if (g.B.kind == VIEW_TAPPED)
#pragma unroll
            for (int u = 0; u < 2; u++)
            {
                const int r = (wave * 2 + u) * 16 + (lane >> 2), p = lane & 3, c = p ^ ((r >> 2) & 3);
                gb[u] = B + (size_t) (RG ? min(n0 + r, g.N - 1) : n0 + r) * ldb + c * 16;
            }
        // first stage of this workgroup's k range
        const int k0 = kt_begin * stage_ch;
        g_tap = k0 / g.A.nch;
        g_ch = k0 - g_tap * g.A.nch;
        g_step_b = uniform64(B_KC ? (long long) FBK : (long long) (FBK / ES) * ldb);
        g_delta_b = 0; // (plain weights: gb[u] points at this workgroup's first stage)
        g_t[0] = g_tap % g.A.ktap[0];
        g_t[1] = (g_tap / g.A.ktap[0]) % g.A.ktap[1];
        g_t[2] = g_tap / (g.A.ktap[0] * g.A.ktap[1]);
        gather_offsets();
    }
    // ---- AMODE 3: this lane's (tap, channel) per request slot and the pixel of the next stage to request -----------------
    int       w_pc[2][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}}; // pixel coordinates (dims 1..4 of the tensor that enumerates pixels)
    int       w_tc[2][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}}; // this lane's tap in the source tensor's coordinates: tap * dilation - padding
    int       w_chb[2] = {0, 0};                         // channel byte offset, < 0: f beyond M
    int       w_step[4] = {0, 0, 0, 0};                  // the pixels of one stage as digits in the radix of the pixel grid
    // what every request of the loop needs of the problem description, read once and pinned in scalar registers (a read
    // inside a step would wait on the counter that the step's LDS reads share): the convolution strides, the source
    // tensor's extents and its strides in bytes (below 2^32, the host sees to that) and the extents of the pixel grid
    int      w_cs[4] = {0, 0, 0, 0}, w_src[4] = {0, 0, 0, 0}, w_grid[3] = {0, 0, 0};
    uint32_t w_sb[4] = {0, 0, 0, 0};
    if constexpr (AMODE == 3)
    {
#pragma unroll
        for (int d = 0; d < 4; d++)
        {
            w_cs[d] = g.A.cstride[d];
            w_src[d] = g.A.src[d];
            w_sb[d] = (uint32_t) (g.A.src_stride[d] * ES);
            asm volatile("" : "+s"(w_cs[d]), "+s"(w_src[d]), "+s"(w_sb[d]));
        }
#pragma unroll
        for (int d = 0; d < 3; d++)
        {
            w_grid[d] = g.A.grid[d];
            asm volatile("" : "+s"(w_grid[d]));
        }
        {
            int rest = FBK / ES;
#pragma unroll
            for (int d = 0; d < 3; d++)
            {
                w_step[d] = __builtin_amdgcn_readfirstlane(rest % w_grid[d]);
                rest = __builtin_amdgcn_readfirstlane(rest / w_grid[d]);
            }
            w_step[3] = rest;
#pragma unroll
            for (int d = 0; d < 4; d++) asm volatile("" : "+s"(w_step[d]));
        }
#pragma unroll
        for (int u = 0; u < 2; u++)
        {
            if (u >= NUA) break;
            constexpr int RPQ = ES == 1 ? 4 : 512 / TM; // k-rows per request
            const int     kr = (wave * NUA + u) * RPQ + lane / (64 / RPQ);
            // 16-byte chunk of the row that this lane fetches (the swizzles of the two stage layouts)
            const int chunk = ES == 1 ? ((lane & 15) - 2 * (kr & 7)) & 15 : (lane & (64 / RPQ - 1)) ^ ((kr & 3) << 1);
            const int f = m0 + chunk * (16 / ES), tap = f / g.A.nch;
            w_chb[u] = f < g.M ? (f - tap * g.A.nch) * ES : -1;
            w_tc[u][0] = (tap % g.A.ktap[0]) * g.A.dil[0] - g.A.pad[0];
            w_tc[u][1] = ((tap / g.A.ktap[0]) % g.A.ktap[1]) * g.A.dil[1] - g.A.pad[1];
            w_tc[u][2] = (tap / (g.A.ktap[0] * g.A.ktap[1])) * g.A.dil[2] - g.A.pad[2];
            w_tc[u][3] = -g.A.pad[3];
            const PixelPos pp = decode_pixel(g.A, kt_begin * (FBK / ES) + kr);
#pragma unroll
            for (int d = 0; d < 4; d++) w_pc[u][d] = pp.c[d];
        }
    }
    // the address of the zero page, fetched once and pinned in two scalar registers: left to itself the compiler re-reads it
    // from the global offset table in every step, and the wait for that scalar load also waits for the step's LDS reads
    uint32_t zero_lo = 0, zero_hi = 0;
    if constexpr (AMODE == 3 || GATHER)
    {
        const uint64_t z = (uint64_t) (uintptr_t) gf_zero_page;
        zero_lo = (uint32_t) z;
        zero_hi = (uint32_t) (z >> 32);
        asm volatile("" : "+s"(zero_lo), "+s"(zero_hi));
    }
    auto zero_page = [&]() __attribute__((always_inline)) { return (const uint8_t*) (uintptr_t) (((uint64_t) zero_hi << 32) | zero_lo); };
    auto issue_a = [&](int u, int stage, int slot) __attribute__((always_inline))
    {
        if constexpr (AMODE == 3)
        {
            // x[pos(pixel, tap)][channel .. + 7], or zeros where the tap falls into the padding
            // (a position outside the tensor fails the unsigned comparison whether it is negative or too large; its offset is
            // then not used)
            uint64_t off = (uint64_t) (uint32_t) w_chb[u];
            bool     ok = w_chb[u] >= 0;
#pragma unroll
            for (int d = 0; d < 4; d++)
            {
                const int pos = w_pc[u][d] * w_cs[d] + w_tc[u][d];
                ok = ok && (uint32_t) pos < (uint32_t) w_src[d];
                off += (uint64_t) (uint32_t) pos * w_sb[d];
            }
            const uint8_t* src = ok ? A + off : zero_page();
            dma16(src, lds_base + slot * STAGE + (wave * NUA + u) * 1024);
            // next stage: 32 (2-byte elements) or 64 (fp8) pixels further, added digit by digit in the mixed radix of the pixel
            // grid (a digit of the step is smaller than its radix, so one conditional subtraction per digit is enough)
            int carry = 0;
#pragma unroll
            for (int d = 0; d < 3; d++)
            {
                const int v = w_pc[u][d] + w_step[d] + carry;
                carry = v >= w_grid[d] ? 1 : 0;
                w_pc[u][d] = v - (carry ? w_grid[d] : 0);
            }
            w_pc[u][3] += w_step[3] + carry;
        }
        else if constexpr (AMODE == 2)
            dma16(ga[u] + (size_t) stage * (FBK / ES) * lda, lds_base + slot * STAGE + (wave * 2 + u) * 1024);
        else if constexpr (GATHER)
        {
            dma16(a_tap[u] + g_chb, lds_base + slot * STAGE + (wave * NUA + u) * 1024);
        }
        else
            dma16(ga[u] + (size_t) stage * FBK, lds_base + slot * STAGE + (wave * NUA + u) * 1024);
    };
    auto issue_b = [&](int u, int stage, int slot) __attribute__((always_inline))
    {
        if constexpr (GATHER)
        {
            // one running offset for both kinds of weights, so the step has no branch on the kind
            dma16(gb[u] + g_delta_b, lds_base + slot * STAGE + A_BYTES + (wave * NUB + u) * 1024);
            if (u == NUB - 1) gather_advance(); // the stage's last request
            return;
        }
        dma16(gb[u] + (B_KC ? (size_t) stage * FBK : (size_t) stage * (FBK / ES) * ldb), lds_base + slot * STAGE + A_BYTES + (wave * NUB + u) * 1024);
    };
    auto read_b = [&](Frags & f, int j, const char* st) __attribute__((always_inline))
    {
        // (the wavefront's first 16-column chunk of the tile)
        if (B_KC) read_b_kc(f, j, st + A_BYTES, wn * (WC / 16), lane);
        else if (ES == 1)
            read_b_tr(f, j, st + A_BYTES, wn * (WC / 16), lane);
        else
            read_b_tr16(f, j, st + A_BYTES, wn * (WC / 16), lane);
    };

    // all four slots of the ring are requested up front: a slot is free again as soon as its stage has been copied into
    // fragment registers, which happens one step before the stage is multiplied
    auto issue_prologue = [&]() __attribute__((always_inline))
    {
        for (int t = 0; t < NST; t++)
        {
#pragma unroll
            for (int u = 0; u < NUB; u++)
            {
                if (u < NUA) issue_a(u, t, t);
                issue_b(u, t, t);
            }
        }
    };
    issue_prologue();
    for (int walk_it = 0;;) // (one pass unless PERSIST)
    {
    // s_waitcnt immediate (gfx9): vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14
    if (!PERSIST || walk_it == 0) __builtin_amdgcn_s_waitcnt(vm_wait((NST - 1) * NREQ)); // all stages but the first may still be in flight: stage 0 has landed
    else
    {
        // a later tile: its four stages were requested before the previous tile's epilogue, whose stores share the counter
        __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
        for (int i = 0; i < NI; i++)
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
    }
    __syncthreads();
    auto read_a_any = [&](Frags & fr, int i, const char* st) __attribute__((always_inline))
    {
        if constexpr (A_KC) read_a(fr, i, st, wm * WR, lane);
        else if constexpr (ES == 1)
            read_a_tr8(fr, i, st, wm, lane);
        else
            read_a_tr16<TM>(fr, i, st, wm, lane);
    };
    Frags f;
#pragma unroll
    for (int i = 0; i < NI; i++) read_a_any(f, i, lds);
#pragma unroll
    for (int j = 0; j < NJ; j++) read_b(f, j, lds);

    constexpr bool MSCALE = ES == 1 && AMODE == 0 && TM == FBM && !RG && !PERSIST && !CHK;
    const int      mfma_scale_a = 127 + (MSCALE ? g.epi.mfma_scale_exp : 0);
    auto mma = [&](int i, int j) __attribute__((always_inline))
    {
        if constexpr (ES == 1)
        {
            // the block-scale operands are exponents (2^(byte - 127), byte 0 of the register): the first carries the
            // epilogue's power-of-two factor when the host folded it in, the second is 2^0
            // (only in the plain instances, see gemm_large_tile_takes_mfma_scale: with the scale operands the register allocator
            // spills in the instances that walk over tiles or check their operands -- also in the four-wavefront checking
            // instance, 16 registers, which cost it more than the multiplication in the epilogue that the scale operand saves)
            if constexpr (!MSCALE) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.b[j], f.a[i], acc[i][j], (FMT >> 1) & 1, FMT & 1, 0, 0, 0, 0);
            else
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.b[j], f.a[i], acc[i][j], (FMT >> 1) & 1, FMT & 1, 0, mfma_scale_a, 0, 127);
        }
        else
        {
            union
            {
                v8i  v;
                v8bf h[2];
                v8h  f[2];
            } ua, ub;
            ua.v = f.a[i];
            ub.v = f.b[j];
            if constexpr (FMT == 1)
            {
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ub.f[0], ua.f[0], acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ub.f[1], ua.f[1], acc[i][j], 0, 0, 0);
            }
            else
            {
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ub.h[0], ua.h[0], acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ub.h[1], ua.h[1], acc[i][j], 0, 0, 0);
            }
        }
    };
#define MMA(i, j) mma(i, j)
#define RA(i) \
    if (RN) read_a_any(f, i, st);
#define RB(j) \
    if (RN) read_b(f, j, st);
#define LA(u) \
    if (LOADS) issue_a(u, t + NST, slot);
#define LB(u) \
    if (LOADS) issue_b(u, t + NST, slot);
    // the look itself: this wavefront's share (2 KiB of eight wavefronts, 4 KiB of four) of one operand's part of a stage, straight from LDS (the swizzled
    // placement does not matter, every byte of the part is an operand byte)
    uint32_t chk_bad_b = 0; // SELFCHK keeps what it found in B apart from what it found in A (chk_bad)
    auto chk_scan = [&](const char* part, uint32_t mask, uint32_t add, uint32_t& chk_bad) __attribute__((always_inline))
    {
#pragma unroll
        for (int q = 0; q < 8 / NW; q++)
        {
            const char* mine = part + wave * (16384 / NW) + q * 2048 + lane * 16;
            const v4i   x0 = *(const v4i*) mine, x1 = *(const v4i*) (mine + 1024);
            chk_bad |= (((uint32_t) x0.x & mask) + add) | (((uint32_t) x0.y & mask) + add);
            chk_bad |= (((uint32_t) x0.z & mask) + add) | (((uint32_t) x0.w & mask) + add);
            chk_bad |= (((uint32_t) x1.x & mask) + add) | (((uint32_t) x1.y & mask) + add);
            chk_bad |= (((uint32_t) x1.z & mask) + add) | (((uint32_t) x1.w & mask) + add);
        }
    };
    // steps until this workgroup's next turn to look at the A part / B part of a stage: stage s of the A rows falls to the tile
    // column s mod tiles_n, of the B columns to the tile row s mod tiles_m; step t looks at stage t + 1 (stage 0 right here)
    int chk_ca = (cur_tn + tiles_n - 1) % tiles_n, chk_cb = (cur_tm + tiles_m - 1) % tiles_m;
    // the constants of the check, read from the kernel arguments once and pinned in scalar registers: a read inside a step
    // would wait on the counter that the step's LDS reads share
    uint32_t chk_ma = 0, chk_aa = 0, chk_mb = 0, chk_ab = 0;
    bool     chk_a_mine = false, chk_b_mine = false;
    if constexpr (CHK)
    {
        chk_ma = g.chk_mask_a, chk_aa = g.chk_add_a, chk_mb = g.chk_mask_b, chk_ab = g.chk_add_b;
        asm volatile("" : "+s"(chk_ma), "+s"(chk_aa), "+s"(chk_mb), "+s"(chk_ab));
        chk_a_mine = chk_ma != 0;
        chk_b_mine = chk_mb != 0;
        if (cur_tn == 0 && chk_a_mine) chk_scan(lds, chk_ma, chk_aa, chk_bad);
        if (cur_tm == 0 && chk_b_mine) chk_scan(lds + A_BYTES, chk_mb, chk_ab, SELFCHK ? chk_bad_b : chk_bad);
    }
    // One stage: 8 MFMAs; after the first one wait until stage t+1 has landed in every wavefront's view (WAITC leaves the
    // younger stages in flight); each fragment register is refilled from stage t+1 right after its last use in stage t (the
    // other wavefront on the SIMD covers the tail of that latency); request stage t+4 into the slot of stage t, whose
    // fragments every wavefront read during the previous step (the barrier above orders those reads before this request).
    int  slot_of_step = 0; // t mod NST of the next step
    auto step = [&](int t, auto waitc, auto loads, auto readnext) __attribute__((always_inline))
    {
        constexpr int  WAITC = decltype(waitc)::value;
        constexpr bool LOADS = decltype(loads)::value;
        constexpr bool RN = decltype(readnext)::value;
        // slots of stage t (to be refilled) and of stage t+1 (to be read): the steps run in order from t = 0, so a ring whose
        // depth is not a power of two counts its slots up instead of dividing
        int slot, next_slot;
        if constexpr ((NST & (NST - 1)) == 0)
        {
            slot = t % NST;
            next_slot = (t + 1) % NST;
        }
        else
        {
            slot = slot_of_step;
            next_slot = slot_of_step + 1 == NST ? 0 : slot_of_step + 1;
            slot_of_step = next_slot;
        }
        const char* st = lds + next_slot * STAGE;
        MMA(0, 0);
        FENCE;
        if (RN)
        {
            __builtin_amdgcn_s_waitcnt(WAITC);
            __builtin_amdgcn_s_barrier();
            if constexpr (CHK)
            {
                // stage t + 1 has landed: one branch per step, the look is a cold block that touches no fragment register
                const bool do_a = chk_ca == 0 && chk_a_mine, do_b = chk_cb == 0 && chk_b_mine;
                chk_ca = chk_ca == 0 ? tiles_n - 1 : chk_ca - 1;
                chk_cb = chk_cb == 0 ? tiles_m - 1 : chk_cb - 1;
                if (__builtin_expect(do_a || do_b, 0))
                {
                    if (do_a) chk_scan(st, chk_ma, chk_aa, chk_bad);
                    if (do_b) chk_scan(st + A_BYTES, chk_mb, chk_ab, SELFCHK ? chk_bad_b : chk_bad);
                }
            }
        }
        FENCE;
        if constexpr (NJ == 4)
        {
            // one wavefront per SIMD, 16 MFMAs per stage: column by column through rows 0 and 1, then through rows 2 and 3.  A
            // fragment is refilled right after its last use and then has six or more MFMAs (400 cycles) until its next use in
            // the following stage; the eight requests ride along in the first half
            MMA(1, 0); FENCE;
            LA(0) MMA(0, 1); FENCE;
            LA(1) MMA(1, 1); FENCE;
            LA(2) MMA(0, 2); FENCE;
            LA(3) MMA(1, 2); FENCE;
            LB(0) MMA(0, 3); FENCE;
            RA(0) LB(1) MMA(1, 3); FENCE;
            RA(1) LB(2) MMA(2, 0); FENCE;
            LB(3) MMA(3, 0); FENCE;
            RB(0) MMA(2, 1); FENCE;
            MMA(3, 1); FENCE;
            RB(1) MMA(2, 2); FENCE;
            MMA(3, 2); FENCE;
            RB(2) MMA(2, 3); FENCE;
            RA(2) MMA(3, 3); FENCE;
            RB(3) RA(3) FENCE;
            return;
        }
        MMA(0, 1); FENCE;
        if constexpr (NI == 4)
        {
            RA(0) LA(0) MMA(1, 0); FENCE;
            MMA(1, 1); FENCE;
            RA(1) LA(1) MMA(2, 0); FENCE;
            MMA(2, 1); FENCE;
            RA(2) LB(0) MMA(3, 0); FENCE;
            RB(0) LB(1) MMA(3, 1); FENCE;
            RA(3) RB(1) FENCE;
        }
        else
        {
            // 128-row tile: four MFMAs per stage, three requests
            RA(0) LA(0) MMA(1, 0); FENCE;
            RB(0) LB(0) MMA(1, 1); FENCE;
            RA(1) RB(1) LB(1) FENCE;
        }
    };
    // at the wait of step t the stages t+1 .. t+NST-1 have been requested; stage t+1 is needed, so the younger NST-2 stages of
    // this wavefront's requests may stay in flight
    using WM = std::integral_constant<int, vm_wait((NST - 2) * NREQ)>;
    using T = std::true_type;
    using F = std::false_type;
    int t = 0;
    // steps 0 .. nk-NST-1 request stages NST .. nk-1.  The 128-row tile walks the four-stage ring four steps at a time: t is
    // then a multiple of four, the slots of a step are compile-time constants and the LDS addresses of its reads and
    // requests need no arithmetic; what is left of the steps (a pair, the count is even) follows.
    if constexpr ((TM == 128 || NW == 4) && NST == 4 && !PERSIST)
        for (; t + NST + 3 < nk; t += 4)
        {
            step(t, WM {}, T {}, T {});
            step(t + 1, WM {}, T {}, T {});
            step(t + 2, WM {}, T {}, T {});
            step(t + 3, WM {}, T {}, T {});
        }
    for (; t + NST + 1 < nk; t += 2)
    {
        step(t, WM {}, T {}, T {});
        step(t + 1, WM {}, T {}, T {});
    }
    if constexpr (NST % 2 != 0) // (the number of stages is even: an odd ring leaves one more step before the drain)
    {
        step(t, WM {}, T {}, T {});
        t++;
    }
    // t == nk - NST (nk >= NST): everything has been requested; step nk-NST+i needs stage nk-NST+i+1 with NST-2-i younger stages
    // behind it, the last step reads nothing
    auto drain = [&](auto ic) __attribute__((always_inline))
    {
        constexpr int I = decltype(ic)::value;
        if constexpr (I < NST - 1) step(t + I, std::integral_constant<int, vm_wait((NST - 2 - I) * NREQ)> {}, F {}, T {});
    };
    if constexpr (NST == 4)
    {
        step(t, std::integral_constant<int, vm_wait(2 * NREQ)> {}, F {}, T {});
        step(t + 1, std::integral_constant<int, vm_wait(NREQ)> {}, F {}, T {});
        step(t + 2, std::integral_constant<int, vm_wait(0)> {}, F {}, T {});
        step(t + 3, std::integral_constant<int, vm_wait(0)> {}, F {}, F {});
    }
    else
    {
        drain(std::integral_constant<int, 0> {});
        drain(std::integral_constant<int, 1> {});
        drain(std::integral_constant<int, 2> {});
        drain(std::integral_constant<int, 3> {});
        drain(std::integral_constant<int, 4> {});
        step(t + NST - 1, std::integral_constant<int, vm_wait(0)> {}, F {}, F {});
    }
#undef MMA
#undef RA
#undef RB
#undef LA
#undef LB
    if constexpr (CHK)
    {
        if (!in_launch)
        {
            if ((chk_bad | chk_bad_b) & 0x80808080u) *const_cast<uint32_t*>((const uint32_t*) g.skip_flag) = g.skip_epoch;
            chk_bad = 0;
        }
    }
    // In-launch settling: what this workgroup's looks found goes into the launch's panel words (GemmProblem::chk_state, zero
    // before the launch; per batch element one word per row panel of A, then one per column panel of B): one device-scope
    // addition per panel that counts this workgroup as a finished looker in the low half of the word and a find in the high
    // half.  Count and flag travel together, so a reader needs one look per panel and no ordering between words.  (Relaxed
    // accesses: the words are the only data that pass between workgroups, there is nothing for a release to write back or
    // an acquire to invalidate -- with release / acquire every workgroup flushed and invalidated its L2, 2 us per launch.)
    bool      tile_exact = false;
    uint32_t* panel_a = nullptr;
    uint32_t* panel_b = nullptr;
    if (in_launch)
    {
        uint32_t* st = g.chk_state + (size_t) blockIdx.y * (unsigned) (tiles_m + tiles_n);
        panel_a = st + cur_tm;
        panel_b = st + tiles_m + cur_tn;
        const bool bad_a = __syncthreads_or((chk_bad & 0x80808080u) != 0u) != 0, bad_b = __syncthreads_or((chk_bad_b & 0x80808080u) != 0u) != 0;
        chk_bad = 0;
        if (threadIdx.x == 0)
        {
            __hip_atomic_fetch_add(panel_a, 1u + (bad_a ? 0x10000u : 0u), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_fetch_add(panel_b, 1u + (bad_b ? 0x10000u : 0u), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // The tile once more, from operands decoded to bf16 with Gaudi's meaning of the codes (every fp8 value is a bf16 value;
    // decoded with the hardware formats' exponent bias, so the epilogue's factor applies unchanged): fragments straight from
    // global memory, 16 k at a time, v_mfma_f32_32x32x16_bf16 into the same accumulators.  Rare and slow by design (about a
    // millisecond for K = 4096).
    auto recompute_exactly = [&]() __attribute__((always_inline))
    {
        if constexpr (SELFCHK)
        {
            const int mode_a = g.chk_inf_nan_a, mode_b = g.chk_inf_nan_b;
            // eight codes (two registers) -> eight bf16 (four registers)
            auto decode8 = [&](uint32_t lo, uint32_t hi, auto e5m2, int mode) __attribute__((always_inline))
            {
                uint32_t h[8];
#pragma unroll
                for (int q = 0; q < 8; q++)
                {
                    const uint32_t code = ((q < 4 ? lo : hi) >> (8 * (q & 3))) & 0xFFu;
                    h[q] = (decltype(e5m2)::value ? fp8_to_fp32<2>(code, 15, mode) : fp8_to_fp32<3>(code, 7, mode)) >> 16;
                }
                union
                {
                    uint32_t w[4];
                    v8bf     v;
                } u;
#pragma unroll
                for (int q = 0; q < 4; q++) u.w[q] = h[2 * q] | (h[2 * q + 1] << 16);
                return u.v;
            };
#pragma unroll
            for (int i = 0; i < NI; i++)
#pragma unroll
                for (int j = 0; j < NJ; j++)
#pragma unroll
                    for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
            const int kh = 8 * (lane >> 5), r32 = lane & 31;
#pragma unroll 1
            for (int k0 = 0; k0 < g.K; k0 += 16)
            {
                v8bf fa[NI], fb[NJ];
#pragma unroll
                for (int i = 0; i < NI; i++)
                {
                    const uint2 raw = *(const uint2*) (A + (size_t) (m0 + wm * WR + i * 32 + r32) * lda + k0 + kh);
                    fa[i] = decode8(raw.x, raw.y, std::integral_constant<bool, (FMT & 1) != 0>(), mode_a);
                }
#pragma unroll
                for (int j = 0; j < NJ; j++)
                {
                    uint32_t lo = 0, hi = 0;
                    if constexpr (B_KC)
                    {
                        const uint2 raw = *(const uint2*) (B + (size_t) (n0 + wn * WC + j * 32 + r32) * ldb + k0 + kh);
                        lo = raw.x;
                        hi = raw.y;
                    }
                    else
                    {
                        const uint8_t* col = B + (size_t) (k0 + kh) * ldb + n0 + wn * WC + j * 32 + r32;
#pragma unroll
                        for (int q = 0; q < 4; q++)
                        {
                            lo |= (uint32_t) col[(size_t) q * ldb] << (8 * q);
                            hi |= (uint32_t) col[(size_t) (q + 4) * ldb] << (8 * q);
                        }
                    }
                    fb[j] = decode8(lo, hi, std::integral_constant<bool, ((FMT >> 1) & 1) != 0>(), mode_b);
                }
#pragma unroll
                for (int i = 0; i < NI; i++)
#pragma unroll
                    for (int j = 0; j < NJ; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
            }
        }
    };

    // ---- epilogue: alpha, per-column power of two, relu, cast, store (same conversion functions as the general kernel).
    // The matrix-core operands are swapped (B fragment first), so accumulator register v of lane l is output column
    // 8 * (v / 4) + 4 * (l / 32) + v % 4 of row l % 32 of its 32 x 32 block: one v_permlane32_swap per register pair leaves
    // every lane with 16 consecutive columns of one row, stored 16 bytes at a time.  The output-type dispatch sits
    // outside the unrolled block walk so that the accumulators stay in registers.
    const long long c_off = b0 * g.epi.batch_stride[0] + b1 * g.epi.batch_stride[1] + b2 * g.epi.batch_stride[2];
    const int       em0 = m0, en0 = n0; // the finished tile (m0, n0 move on to the next one below)
    bool            has_next = false;
    if constexpr (PERSIST)
    {
        walk_it++;
        const int L = walk_it * (int) gridDim.x + walk_first;
        has_next = L < walk_total;
        if (has_next)
        {
            __syncthreads(); // the slowest wavefront has taken its last fragments out of the ring
            locate(L % tiles_total, L / tiles_total);
            setup_ptrs();
            issue_prologue();
        }
    }
    // (PERSIST: the epilogue's lane- and wavefront-dependent values are derived from laundered copies, so that the
    // compiler does not hoist them out of the walk over tiles and keep them in registers through the main loop)
    int elane = lane, ewave = wave;
    if constexpr (PERSIST)
    {
        asm volatile("" : "+v"(elane));
        asm volatile("" : "+s"(ewave));
    }
    const int ewm = ewave / WGN, ewn = ewave % WGN;
    const long long ldc = g.epi.ld;
    const bool      has_alpha = g.epi.has_alpha != 0;
    const float     alpha = g.epi.alpha;
    const int32_t*  col_exp = g.epi.col_exp;
    const bool      relu = g.epi.fused && g.epi.cast.relu;
    const int       dt = g.epi.fused ? g.epi.out_dtype : DT_FP32;
    const int       esz = (dt == DT_FP32) ? 4 : (dt == DT_BF16 ? 2 : 1);
    const CastParams cp = {g.epi.cast.dtype,       g.epi.cast.exp_bias, g.epi.cast.inf_nan_mode, g.epi.cast.rm,    g.epi.cast.clip_fp,
                           g.epi.cast.clip_inf_in, g.epi.cast.ftz,      g.epi.cast.relu,         g.epi.cast.scale, g.epi.cast.has_scale};
    const int       kg = elane >> 5;
    const bool      finite = g.epi.finite != 0; // (SELFCHK: a tile computed again from the decoded operands, which may hold inf and NaN, goes out through the generic converter)
    // element offset of this elane's first value in block (0, 0): row em0 + ewm * WR + elane % 32, column en0 + ewn * WC + 16 kg
    const long long lane_elem = c_off + (long long) (em0 + ewm * WR + (elane & 31)) * ldc + en0 + ewn * WC + kg * 16;
    // (four wavefronts: the 256 accumulators live in the accumulation registers; reading each one from there where it is used
    // keeps the register allocator from moving them all to vector registers, and from there to scratch memory, at once)
    auto acc_value = [&](float x) __attribute__((always_inline))
    {
        if constexpr (NW == 4)
        {
            float y;
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(y) : "a"(x));
            return y;
        }
        else
            return x;
    };
    // block (i, j) -> the elane's 16 values after the power-of-two factors and relu
    auto gather = [&](int i, int j, float (&val)[16], auto raw_c) __attribute__((always_inline))
    {
#pragma unroll
        for (int q = 0; q < 2; q++)
#pragma unroll
            for (int r = 0; r < 4; r++)
            {
                const float lo = acc_value(acc[i][j][4 * q + r]), hi = acc_value(acc[i][j][8 + 4 * q + r]);
                const auto  sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
                val[8 * q + r] = __uint_as_float(sw[0]);
                val[8 * q + 4 + r] = __uint_as_float(sw[1]);
            }
        if constexpr (decltype(raw_c)::value) return;
        if (has_alpha)
        {
#pragma unroll
            for (int c = 0; c < 16; c++) val[c] *= alpha;
        }
        if (col_exp)
        {
#pragma unroll
            for (int c = 0; c < 16; c++) val[c] *= pow2_of(col_exp[RG ? min(en0 + ewn * WC + j * 32 + kg * 16 + c, g.N - 1) : en0 + ewn * WC + j * 32 + kg * 16 + c]);
        }
        if (relu)
        {
#pragma unroll
            for (int c = 0; c < 16; c++) val[c] = relu_ref(val[c]);
        }
    };
    typedef float    e_v4f __attribute__((ext_vector_type(4)));
    typedef uint32_t e_v4u __attribute__((ext_vector_type(4)));
    typedef float    e_v2f __attribute__((ext_vector_type(2)));
    typedef __bf16   e_v2bf __attribute__((ext_vector_type(2)));
    // Converted values pass through LDS on their way out (the ring is idle by now): a elane holds 16 columns of one row, and
    // stored from there a 128-byte line of the output would arrive as four to eight separate pieces.  Each wavefront stages
    // one 32-row block of 64 of its columns (16-byte chunks XOR-swizzled by row, conflict-free both ways) and stores it back
    // with consecutive lanes on consecutive chunks of a row: whole lines per request.
    auto walk_to = [&](auto esz_c, auto raw_c, uint8_t* outb, long long pitch, auto pack) __attribute__((always_inline))
    {
        constexpr int ESZ = decltype(esz_c)::value; // bytes per output element = 16-byte chunks per elane and block
        constexpr int RB = 64 * ESZ, CPR = RB / 16, NRD = RB / 32;
        // (PERSIST: behind the ring, which already holds the next tile; 1- and 2-byte outputs only, the host sees to that)
        char*         stg = lds + (PERSIST && ESZ <= 2 ? NST * STAGE : 0) + ewave * (32 * RB);
        const int     row = elane & 31, swz = (row * CPR / 16) & (CPR - 1);
        constexpr bool RAW = decltype(raw_c)::value; // partial sums of a k-slice: no factors, no relu
        if constexpr (!PERSIST) __syncthreads(); // the slowest wavefront has taken its last fragments out of the ring
        if constexpr (NW == 4)
        {
            // One wavefront per SIMD: nothing else covers the two LDS round trips of a block, so the blocks are pipelined by
            // hand through two staging buffers: while block n comes back from LDS, block n + 1 is converted; while block n's
            // stores leave, block n + 1 goes into the other buffer.
            constexpr int NB = NI * (NJ / 2), BUF = NW * 32 * RB;
            uint32_t      p0[4 * ESZ], p1[4 * ESZ];
            auto convert = [&](int n) __attribute__((always_inline))
            {
                float val[16];
                gather(n / (NJ / 2), (n % (NJ / 2)) * 2, val, raw_c);
                pack(val, p0);
                gather(n / (NJ / 2), (n % (NJ / 2)) * 2 + 1, val, raw_c);
                pack(val, p1);
            };
            auto lds_put = [&](int buf) __attribute__((always_inline))
            {
#pragma unroll
                for (int h = 0; h < ESZ; h++)
                {
                    *(e_v4u*) (stg + buf * BUF + row * RB + ((((0 * 2 + kg) * ESZ + h) ^ swz) << 4)) = e_v4u {p0[4 * h], p0[4 * h + 1], p0[4 * h + 2], p0[4 * h + 3]};
                    *(e_v4u*) (stg + buf * BUF + row * RB + ((((1 * 2 + kg) * ESZ + h) ^ swz) << 4)) = e_v4u {p1[4 * h], p1[4 * h + 1], p1[4 * h + 2], p1[4 * h + 3]};
                }
            };
            convert(0);
            lds_put(0);
#pragma unroll
            for (int n = 0; n < NB; n++)
            {
                const int i = n / (NJ / 2), jh = n % (NJ / 2);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                e_v4u v[NRD];
#pragma unroll
                for (int r = 0; r < NRD; r++)
                {
                    const int q = r * 64 + elane, rr = q / CPR, lc = q % CPR;
                    v[r] = *(const e_v4u*) (stg + (n & 1) * BUF + rr * RB + ((lc ^ ((rr * CPR / 16) & (CPR - 1))) << 4));
                }
                if (n + 1 < NB) convert(n + 1);
#pragma unroll
                for (int r = 0; r < NRD; r++)
                {
                    const int q = r * 64 + elane, rr = q / CPR, lc = q % CPR;
                    if ((!RAGGED_M || em0 + ewm * WR + i * 32 + rr < g.M) && (!RG || en0 + ewn * WC + jh * 64 + lc * (16 / ESZ) < g.N))
                        __builtin_nontemporal_store(v[r], (e_v4u*) (outb + (long long) (i * 32 + rr) * pitch + jh * RB + lc * 16));
                }
                if (n + 1 < NB) lds_put((n + 1) & 1);
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < NI; i++)
#pragma unroll
        for (int jh = 0; jh < NJ / 2; jh++) // (64 columns at a time)
        {
#pragma unroll
            for (int j = 0; j < 2; j++)
            {
                float    val[16];
                uint32_t pk[4 * ESZ];
                gather(i, jh * 2 + j, val, raw_c);
                pack(val, pk);
#pragma unroll
                for (int h = 0; h < ESZ; h++)
                    *(e_v4u*) (stg + row * RB + ((((j * 2 + kg) * ESZ + h) ^ swz) << 4)) = e_v4u {pk[4 * h], pk[4 * h + 1], pk[4 * h + 2], pk[4 * h + 3]};
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int r = 0; r < NRD; r++)
            {
                const int   q = r * 64 + elane, rr = q / CPR, lc = q % CPR;
                const e_v4u v = *(const e_v4u*) (stg + rr * RB + ((lc ^ ((rr * CPR / 16) & (CPR - 1))) << 4));
                if ((!RAGGED_M || em0 + ewm * WR + i * 32 + rr < g.M) && (!RG || en0 + ewn * WC + jh * 64 + lc * (16 / ESZ) < g.N))
                    __builtin_nontemporal_store(v, (e_v4u*) (outb + (long long) (i * 32 + rr) * pitch + jh * RB + lc * 16));
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        (void) RAW;
    };
    auto walk = [&](auto esz_c, auto pack) __attribute__((always_inline))
    {
        constexpr int ESZ = decltype(esz_c)::value;
        walk_to(esz_c, std::false_type(), (uint8_t*) g.epi.out + (c_off + (long long) (em0 + ewm * WR) * ldc + en0 + ewn * WC) * ESZ, ldc * ESZ, pack);
    };
    // element-wise through the out-of-line generic converter (which applies relu itself): rare cast settings, and the tiles
    // that the four-wavefront checking form computed again
    auto store_generic = [&]() __attribute__((always_inline))
    {
#pragma unroll 1
        for (int i = 0; i < NI; i++)
#pragma unroll 1
            for (int j = 0; j < NJ; j++)
            {
                float val[16];
#pragma unroll
                for (int q = 0; q < 2; q++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                    {
                        // (dynamic block index: read the accumulators through a switch-free copy)
                        float lo = 0.0f, hi = 0.0f;
#pragma unroll
                        for (int ii = 0; ii < NI; ii++)
#pragma unroll
                            for (int jj = 0; jj < NJ; jj++)
                                if (ii == i && jj == j)
                                {
                                    lo = acc_value(acc[ii][jj][4 * q + r]);
                                    hi = acc_value(acc[ii][jj][8 + 4 * q + r]);
                                }
                        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
                        val[8 * q + r] = __uint_as_float(sw[0]);
                        val[8 * q + 4 + r] = __uint_as_float(sw[1]);
                    }
                for (int c = 0; c < 16; c++)
                {
                    float x = val[c];
                    if (has_alpha) x *= alpha;
                    if (col_exp) x *= pow2_of(col_exp[RG ? min(en0 + ewn * WC + j * 32 + kg * 16 + c, g.N - 1) : en0 + ewn * WC + j * 32 + kg * 16 + c]);
                    if ((!RAGGED_M || em0 + ewm * WR + i * 32 + (elane & 31) < g.M) && (!RG || en0 + ewn * WC + j * 32 + kg * 16 < g.N)) store_out_slow(g.epi, lane_elem + (long long) (i * 32) * ldc + j * 32 + c, x);
                }
            }
    };
    if (!PERSIST && g.split_k > 1)
    {
        // raw partial sums; splitk_reduce_kernel adds the slices in order and applies the epilogue
        float* ws = g.workspace + ((long long) kslice * gridDim.y + blockIdx.y) * g.M * (long long) g.N + (long long) (em0 + ewm * WR) * g.N + en0 + ewn * WC;
        walk_to(std::integral_constant<int, 4>(), std::true_type(), (uint8_t*) ws, (long long) g.N * 4, [&](const float (&val)[16], uint32_t (&pk)[16]) __attribute__((always_inline)) {
#pragma unroll
            for (int c = 0; c < 16; c++) pk[c] = __float_as_uint(val[c]);
        });
    }
    else if (!PERSIST && dt == DT_FP32 && !(g.epi.fused && (g.epi.cast.clip_fp || g.epi.cast.ftz)))
        walk(std::integral_constant<int, 4>(), [&](const float (&val)[16], uint32_t (&pk)[16]) __attribute__((always_inline)) {
#pragma unroll
            for (int c = 0; c < 16; c++) pk[c] = __float_as_uint(val[c]);
        });
    else if (dt == DT_BF16 && g.epi.fast_cast)
        // bf16, round to nearest even: v_cvt_pk_bf16_f32 gives the reference's code for every input except NaN (checked over
        // all 2^32 inputs); NaN, inf and values that round to inf (where clipping matters) are rare: the sum of |x| over
        // the elane's 16 values detects them and the block is then converted element by element
        walk(std::integral_constant<int, 2>(), [&](const float (&val)[16], uint32_t (&pk)[8]) __attribute__((always_inline)) {
            bool special = false;
            if (!finite)
            {
                float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int c = 0; c < 16; c++) sum[c & 3] += __builtin_fabsf(val[c]);
                special = !((sum[0] + sum[1]) + (sum[2] + sum[3]) < 0x1.ffp+127f);
            }
            if (finite || __builtin_amdgcn_ballot_w64(special) == 0)
            {
#pragma unroll
                for (int c = 0; c < 8; c++)
                {
                    const e_v2bf h = __builtin_convertvector(e_v2f {val[2 * c], val[2 * c + 1]}, e_v2bf);
                    __builtin_memcpy(&pk[c], &h, 4);
                }
            }
            else
            {
#pragma unroll
                for (int c = 0; c < 8; c++)
                    pk[c] = fp32_to_bf16_rne(f2u(val[2 * c]), cp.clip_fp, cp.clip_inf_in) | (fp32_to_bf16_rne(f2u(val[2 * c + 1]), cp.clip_fp, cp.clip_inf_in) << 16);
            }
        });
    else if ((dt == DT_FP8_143 || dt == DT_FP8_152) && g.epi.fast_cast)
    {
        auto fp8_store = [&](auto m_c) __attribute__((always_inline))
        {
            constexpr int MAN = decltype(m_c)::value;
            walk(std::integral_constant<int, 1>(), [&](const float (&val)[16], uint32_t (&pk)[4]) __attribute__((always_inline)) {
                // the hardware converter equals the reference's conversion on finite inputs; a block that holds inf or
                // NaN (sum of magnitudes not finite) takes the exact converter
                bool special = false;
                if (!finite)
                {
                    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int c = 0; c < 16; c++) sum[c & 3] += __builtin_fabsf(val[c]);
                    special = !((sum[0] + sum[1]) + (sum[2] + sum[3]) <= 0x1.fffffep+127f);
                }
                if (finite || __builtin_amdgcn_ballot_w64(special) == 0)
                {
#pragma unroll
                    for (int c = 0; c < 4; c++) pk[c] = fp8_hw_pack4<MAN>(val[4 * c], val[4 * c + 1], val[4 * c + 2], val[4 * c + 3], cp.exp_bias, cp.clip_fp);
                }
                else
                {
#pragma unroll
                    for (int c = 0; c < 4; c++)
                    {
                        pk[c] = 0;
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            pk[c] |= (fp32_to_fp8_rne_mode0<MAN>(f2u(val[4 * c + e]), cp.exp_bias, cp.clip_fp, cp.clip_inf_in) & 0xFFu) << (8 * e);
                    }
                }
            });
        };
        if (dt == DT_FP8_143) fp8_store(std::integral_constant<int, 3>());
        else
            fp8_store(std::integral_constant<int, 2>());
    }
    else if (!PERSIST)
        store_generic();
    if (in_launch)
    {
        // every looker of this tile's row panel of A (one workgroup per tile column) and of its column panel of B has finished
        // its loop before it started the epilogue that this workgroup has just finished as well, so the wait is a formality
        // unless the device is shared; it is bounded, and a workgroup that cannot tell computes its tile again to be safe
        bool again = false;
        if (threadIdx.x == 0)
        {
            bool     all_in = false;
            uint32_t wa = 0, wb = 0;
            for (int polls = 0; polls < (1 << 14) && !all_in; polls++)
            {
                // (read with an addition of zero: a read-modify-write is carried out where all XCDs agree, whatever a plain load
                // with device scope may find in this XCD's L2)
                wa = __hip_atomic_fetch_add(panel_a, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                wb = __hip_atomic_fetch_add(panel_b, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                all_in = (wa & 0xFFFFu) >= (uint32_t) tiles_n && (wb & 0xFFFFu) >= (uint32_t) tiles_m;
                if (!all_in) __builtin_amdgcn_s_sleep(16);
            }
            again = !all_in || ((wa | wb) >> 16) != 0u;
        }
        if (__builtin_expect(__syncthreads_or(again) != 0, 0))
        {
            recompute_exactly();
            tile_exact = true;
            store_generic(); // (writes the whole tile again)
        }
    }
    (void) esz;
    (void) tile_exact;
    if (!PERSIST || !has_next) break;
    } // walk over tiles
}

// GemmProblem::clock_probe (diagnostics, normally NULL): the first lane of a workgroup notes the shader clock counter and
// the constant 100 MHz counter when the workgroup starts (cells 0, 1 of its four) and when its first wavefront ends (2, 3);
// the host derives the clock the kernel really ran at and the time a workgroup took from them.
__device__ __forceinline__ void clock_probe_stamp(KARG GemmProblem& g, int at_end)
{
    uint64_t* probe = g.clock_probe;
    if (!probe || threadIdx.x != 0) return;
    const unsigned wg = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    if (wg >= (unsigned) CLOCK_PROBE_WORKGROUPS) return;
    probe[4 * wg + 2 * at_end] = clock64();
    probe[4 * wg + 2 * at_end + 1] = wall_clock64();
}

template<int ES, int FMT, bool B_KC, int AMODE = 0, int TM = FBM, bool RG = false, bool PERSIST = false, bool CHK = false, int NST = FNST, int NW = 8>
__device__ __forceinline__ void gemm_fast_body(KARG GemmProblem& g)
{
    // (a launch that its predicate skips leaves the cells to the launch that ran)
    const bool probe = g.clock_probe && !(!CHK && g.skip_flag && ((*g.skip_flag == g.skip_epoch) == (g.skip_if != 0)));
    if (probe) clock_probe_stamp(g, 0);
    gemm_fast_body_impl<ES, FMT, B_KC, AMODE, TM, RG, PERSIST, CHK, NST, NW>(g);
    if (probe) clock_probe_stamp(g, 1);
}


// sets the dynamic-LDS limit once per kernel, then launches
template<class K>
hipError_t launch_fast(K kernel, bool& attr_done, const GemmProblem& p, dim3 grid, hipStream_t s, int tile_m = FBM, int stages = FNST, int lanes = 512)
{
    const int lds_bytes = stages * (tile_m * FBK + FBK * FBN);
    if (!attr_done)
    {
        hipError_t e = hipFuncSetAttribute((const void*) kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess) return e;
        attr_done = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(lanes), lds_bytes, s, p);
    return hipGetLastError();
}
} // namespace
} // namespace mme
