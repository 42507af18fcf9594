// MFMA tile-GEMM kernel template for gfx950 (CDNA4, wave64).
//
// One source, instantiated by -D macros (one instance = one point of the tuner's search space):
//   HRN_DTYPE   0: fp16 x fp16 -> fp32 accumulate -> fp16 store      (ops/cuda/dense.py:4-54)
//               1: uint8 x int8 -> int32 accumulate -> int32 store   (ops/x86/dense.py:6-32)
//   HRN_OP      0: GEMM / batch_matmul   C[b,i,j] = sum_k A[b,i,k] * B[b,j,k]
//               1: conv2d NHWC x KRSC as implicit GEMM (M = n*ho*wo, N = co, K = kh*kw*ci)
//   HRN_BM/BN   workgroup tile, HRN_BKB bytes of K per LDS row, HRN_WM x HRN_WN wave grid,
//   HRN_MFMA    32 | 16 (MFMA tile edge), HRN_STAGES LDS stages, HRN_SWZ LDS chunk swizzle,
//   HRN_EPI     0 stores straight from the accumulator registers, 1 LDS-staged epilogue with 16-byte coalesced
//               stores, 2 the same with half-width staging strips, HRN_WPE waves-per-SIMD hint, HRN_CONVWIN conv input window in LDS, HRN_PERSIST persistent
//               launch, HRN_SPLITK K split over several workgroups with raw partial sums as output.
//
// Data movement: both operands are K-contiguous, so a tile is a set of rows of HRN_BKB bytes.
// Rows are cut into 16-byte chunks; every lane moves one chunk per load straight from HBM/L2
// into LDS (buffer_load_dwordx4 ... lds), one wave instruction filling 1 KiB of consecutive LDS.
// The chunk a lane fetches is XOR-swizzled so that the MFMA operand reads (ds_read_b128, one
// 16-byte chunk per lane) spread over all LDS banks.  A lane's byte offset inside its row never
// changes; the k-tile is selected by the scalar offset operand of the load, so the k-loop spends
// no vector instruction on addresses.  Out-of-range rows and conv halo taps are fetched with an
// out-of-range lane offset, the dummy tiles past the end of K through a zero-length buffer
// descriptor: the buffer unit turns both into zeros.
//
// Pipeline: HRN_STAGES tiles are in flight.  The barrier that publishes tile t+1 sits before the
// last k-step of tile t, so operand fragments of the next tile are already being read while the
// last MFMAs of the current tile run; fragments are double-buffered in registers and read in the
// order the MFMAs of the next step consume them (all of B, then A row-tile by row-tile).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#ifndef HRN_DTYPE
#error "instantiate with -DHRN_DTYPE=... (see hrn_api.cpp)"
#endif

#ifndef HRN_KARGS_DEFINED
#define HRN_KARGS_DEFINED
struct HrnKArgs {
    const void* A;
    const void* B;
    void* C;
    int32_t M, N, K;            // K in elements
    int32_t lda, ldb, ldc;      // elements
    int64_t sA, sB, sC;         // batch strides, elements
    int32_t tiles_m, tiles_n, group_m, batch;
    // conv
    int32_t H, W, CI, HO, WO, KH, KW, cstride, cpad, cdil;
    int32_t cstride_w, cpad_w, cdil_w;   // conv: the width-direction values (cstride/cpad/cdil are the height ones)
    int32_t split, kt_per_slice;         // split-K: number of K slices and k-tiles per slice
    const void* bsum;                    // uint8 path: per batch entry N column sums of B (sum_k B[n,k], int32), or null
};
#endif

namespace {

constexpr int DT = HRN_DTYPE;
constexpr int OP = HRN_OP;
constexpr int BM = HRN_BM, BN = HRN_BN, BKB = HRN_BKB;
constexpr int WM = HRN_WM, WN = HRN_WN, MT = HRN_MFMA, NS = HRN_STAGES, SWZ = HRN_SWZ;
constexpr int EPI = HRN_EPI;
// Conv window mode (HRN_OP=1, stride 1, dilation 1, 'same' padding): instead of fetching an im2col tile of A for every
// filter tap, the workgroup loads ONCE the window of input pixels its BM output pixels can reach (a contiguous range
// of BM + 2*(pad_h*W + pad_w) pixels, all channels) and every tap reads its operand fragments from that window at a row offset
// of r*W + s pixels; taps that fall into the padding are masked to zero in registers.  Only B (the filter) streams
// through the LDS stages.  The window lives in dynamic LDS; the staged epilogue reuses it once the last tap is read.
#ifndef HRN_CONVWIN
#define HRN_CONVWIN 0
#endif
constexpr bool CW = (HRN_CONVWIN != 0);
// Persistent mode: the launch has fewer workgroups than output tiles and every workgroup walks tiles
// blockIdx.x, blockIdx.x + gridDim.x, ...  The k-tiles of all its output tiles form ONE stream through the LDS
// stages, so the first k-tiles of the next output tile are already being fetched while the current tile's result is
// stored.  The stores are buffer stores issued unconditionally (masked lanes get an out-of-range offset), so every
// wave has a known number of them in the vector-memory counter and the waits on the following tile fetches can
// allow for them instead of draining them.
#ifndef HRN_PERSIST
#define HRN_PERSIST 0
#endif
constexpr bool PERS = (HRN_PERSIST != 0);
// Split-K: the grid holds `split` copies of the tile grid; copy z multiplies k-tiles [z*kt_per_slice, (z+1)*kt_per_slice)
// and stores its raw fp32 / int32 partial sums to slice z of the output buffer (a workspace); a second kernel adds the slices.
#ifndef HRN_SPLITK
#define HRN_SPLITK 0
#endif
constexpr bool SPLITK = (HRN_SPLITK != 0);
// uint8 path: 1 = the column sums of B (sum_k B[n,k], what the (u8 - 128) x s8 product is short of, times 128) come
// from the caller (HrnKArgs.bsum: one int32 per column and batch entry, a property of the weights alone) instead of
// being added up in the k-loop from the B fragments.
#ifndef HRN_COLSUM
#define HRN_COLSUM 0
#endif
constexpr bool COLSUM = (HRN_DTYPE == 1) && (HRN_COLSUM != 0);
// the results leave with the non-temporal hint: C is written once and not read by this kernel, and a round's 8 MiB of it
// per XCD would otherwise push the operand slabs of the next round out of the 4 MiB L2 (split-K partial sums, which the
// reduction reads right away, keep the default policy)
#ifndef HRN_NTSTORE
#define HRN_NTSTORE 0
#endif
constexpr bool NTS = (HRN_NTSTORE != 0) && (HRN_SPLITK == 0);
// Issue order of a k-step: 1 = the source order of the row groups is pinned (a scheduling fence after every row of
// MFMAs), 0 = the compiler interleaves on its own, guided by group hints (one LDS read per few MFMAs), 2 = the two
// wave groups of an 8-wave workgroup alternate between a memory phase and a matrix phase (see "SCHED 2" below).
#ifndef HRN_SCHED
#define HRN_SCHED 1
#endif
constexpr int SCHED = HRN_SCHED;
#ifndef HRN_LSPREAD
#define HRN_LSPREAD 2
#endif
constexpr int LSPREAD = HRN_LSPREAD;
static_assert(LSPREAD >= 0 && LSPREAD <= 3, "load spread");
constexpr int ES = (DT == 0) ? 2 : 1;                  // input element bytes
constexpr int OES = (DT == 0 && !SPLITK) ? 2 : 4;      // output element bytes
constexpr int NW = WM * WN, NT = NW * 64;
constexpr int CPR = BKB / 16;               // 16-byte chunks per tile row
constexpr int RPI = 64 / CPR;               // tile rows one wave load instruction covers
constexpr int A_LPW = CW ? 0 : (BM / RPI) / NW;   // load instructions per wave per tile
constexpr int B_LPW = (BN / RPI) / NW;
constexpr int LPT = A_LPW + B_LPW;          // vector memory ops per lane per tile
constexpr int KSB = (MT == 32) ? 32 : 64;   // bytes of K one MFMA consumes
constexpr int KS = BKB / KSB;               // MFMA k-steps per tile
constexpr int CPS = KSB / 16;               // chunks per k-step (= 64 / MT)
constexpr int WTM = BM / WM, WTN = BN / WN;
constexpr int TM = WTM / MT, TN = WTN / MT;
constexpr int A_BYTES = CW ? 0 : BM * BKB, B_BYTES = BN * BKB, STAGE_BYTES = A_BYTES + B_BYTES;
constexpr int ACC_N = (MT == 32) ? 16 : 4;
constexpr uint32_t OOB = 0x80000000u;

static_assert(BKB == 64 || BKB == 128 || BKB == 256, "BKB");
static_assert(MT == 32 || MT == 16, "MFMA");
static_assert(KS >= 1, "k-steps per tile");
static_assert((WM & (WM - 1)) == 0, "wave rows must be a power of two");
static_assert((CW || ((BM / RPI) % NW == 0 && A_LPW >= 1)) && (BN / RPI) % NW == 0 && B_LPW >= 1, "loads per wave");
static_assert(!CW || OP == 1, "window mode is a conv2d load path");
static_assert(BM % (WM * MT) == 0 && BN % (WN * MT) == 0, "wave tile");
static_assert(NS >= 2 && NS <= 5, "stages");
// LDS-staged epilogue: per wave a strip of MT rows x WTN outputs, rows padded by 16 bytes; in front of the strips the
// uint8 path keeps the column sums of B, one row of BN sums per wave row (each wave row sums its share of the k-steps)
// (HRN_EPI = 2: strips of half the wave tile's width, filled and written out twice per row-tile - half the LDS)
constexpr int ESPLIT = (EPI == 2) ? 2 : 1;
constexpr int SW = WTN / ESPLIT;            // outputs per strip row
constexpr int EPI_PITCH = SW * OES + 16;
constexpr int EPI_BASE = (DT == 1) ? ((WM * BN * 4 + 1023) / 1024) * 1024 : 0;
constexpr int EPI_BYTES = (EPI >= 1) ? EPI_BASE + NW * MT * EPI_PITCH : 0;
// the epilogue region (column sums + strips) reuses the stages (window mode: the window), except in persistent mode
// where the stages stay live
constexpr int EPI_OFF = PERS ? NS * STAGE_BYTES : 0;
constexpr int LDS_BYTES = PERS ? NS * STAGE_BYTES + EPI_BYTES
                               : ((CW || NS * STAGE_BYTES > EPI_BYTES) ? NS * STAGE_BYTES : EPI_BYTES);
constexpr int STORES_PER_TILE = (EPI >= 1) ? TM * ESPLIT * (MT * (SW * OES / 16) / 64) : 0;   // store instructions per wave per output tile
static_assert(EPI >= 0 && EPI <= 2 && TN % ESPLIT == 0, "epilogue kind");
static_assert(!PERS || (EPI >= 1 && !CW && !SPLITK && KS % 2 == 0), "persistent mode: staged epilogue, even k-steps");
static_assert(!PERS || (NS - 2) * LPT + STORES_PER_TILE <= 63, "persistent mode: vmcnt range");
static_assert(!SPLITK || !CW, "split-K uses the im2col load path");
static_assert(LDS_BYTES <= 163840, "LDS");
static_assert(EPI == 0 || (MT * (SW * OES / 16)) % 64 == 0, "staged epilogue: a strip must split into whole wave stores");
static_assert(SWZ == 0 || (CPR << (SWZ - 1)) <= MT, "swizzle period must fit in one MFMA tile");
static_assert((NS - 1) * LPT <= 63, "vmcnt range");
static_assert(NT <= 1024, "threads");
static_assert(DT == 0 || NS * STAGE_BYTES >= WM * BN * 4, "column sums must fit the stages");

typedef int v4i __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

template <int N> struct AccT;
template <> struct AccT<16> { using F = v16f; using I = v16i; };
template <> struct AccT<4> { using F = v4f; using I = v4i; };
using acc_t = typename std::conditional<DT == 0, typename AccT<ACC_N>::F, typename AccT<ACC_N>::I>::type;

__device__ __forceinline__ int swz_of_row(int row) {
    if (SWZ == 0) return 0;
    return (row >> (SWZ - 1)) & (CPR - 1);
}

// s_waitcnt encodings for gfx9: vmcnt[3:0]|[15:14], expcnt[6:4], lgkmcnt[11:8]
template <int VM, int LGKM>
__device__ __forceinline__ void wait_and_barrier() {
    constexpr int vm = VM > 63 ? 63 : VM;
    constexpr int imm = (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((LGKM & 15) << 8);
    asm volatile("s_waitcnt %0\n\ts_barrier" ::"n"(imm) : "memory");
}

template <int VM, int LGKM>
__device__ __forceinline__ void wait_only() {
    constexpr int vm = VM > 63 ? 63 : VM;
    constexpr int imm = (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((LGKM & 15) << 8);
    asm volatile("s_waitcnt %0" ::"n"(imm) : "memory");
}

typedef __amdgpu_buffer_rsrc_t rsrc_t;

// raw buffer (stride 0): a lane offset >= `bytes` reads as zero instead of touching memory (the scalar offset of a
// load is not part of that check)
__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ void load_chunk_to_lds(rsrc_t rsrc, char* lds_wave_base, uint32_t voff, uint32_t soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds_wave_base,
                                             16, (int)voff, (int)soff, 0, 0);
}

__device__ __forceinline__ v16f mfma(v4i x, v4i y, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, x), __builtin_bit_cast(v8h, y), c, 0, 0, 0);
}
__device__ __forceinline__ v4f mfma(v4i x, v4i y, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, x), __builtin_bit_cast(v8h, y), c, 0, 0, 0);
}
__device__ __forceinline__ v16i mfma(v4i x, v4i y, v16i c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(x, y, c, 0, 0, 0);
}
__device__ __forceinline__ v4i mfma(v4i x, v4i y, v4i c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(x, y, c, 0, 0, 0);
}

// In-place form for the two-group schedule: the accumulator is both source and destination, so its registers stay
// where they are for the whole k-loop (with the intrinsic the register allocator is free to move them from step to
// step, and with the single fragment buffer of that schedule it does, at the price of spills).  The compiler does not
// know this instruction's latency: code that reads the accumulators afterwards starts with mfma_drain().
__device__ __forceinline__ void mfma_inplace(v4i x, v4i y, v16f& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(x), "v"(y));
}
__device__ __forceinline__ void mfma_inplace(v4i x, v4i y, v4f& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(x), "v"(y));
}
__device__ __forceinline__ void mfma_inplace(v4i x, v4i y, v16i& c) {
    asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(c) : "v"(x), "v"(y));
}
__device__ __forceinline__ void mfma_inplace(v4i x, v4i y, v4i& c) {
    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(c) : "v"(x), "v"(y));
}
__device__ __forceinline__ void mfma_drain() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

// Scheduling hints of one k-step (HRN_SCHED = 0): NR groups of {1 LDS read, NV/NR buffer loads, NMM/NR MFMAs}.
template <int R, int NR, int NMM, int NV>
__device__ __forceinline__ void sched_hint() {
    if constexpr (R < NR) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        constexpr int v = (NV * (R + 1)) / NR - (NV * R) / NR;
        if constexpr (v > 0) __builtin_amdgcn_sched_group_barrier(0x020, v, 0);
        constexpr int mm = (NMM * (R + 1)) / NR - (NMM * R) / NR;
        if constexpr (mm > 0) __builtin_amdgcn_sched_group_barrier(0x008, mm, 0);
        sched_hint<R + 1, NR, NMM, NV>();
    }
}

}  // namespace

extern "C" __global__ void __launch_bounds__(NT)
#if HRN_WPE > 0
__attribute__((amdgpu_waves_per_eu(HRN_WPE, HRN_WPE)))
#endif
hrn_mfma_kernel(const HrnKArgs a) {
    __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];
    extern __shared__ __attribute__((aligned(1024))) char win[];   // window mode: input window, later the epilogue region

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm_idx = wave / WN, wn_idx = wave % WN;

    const int tiles_mn = a.tiles_m * a.tiles_n;
    const int total = tiles_mn * a.batch;             // output tiles (of one K slice)
    const uint32_t Kb = (uint32_t)a.K * ES;           // bytes of K
    const int KT_all = (Kb + BKB - 1) / BKB;
    int first_pid = blockIdx.x, slice = 0;
    if constexpr (SPLITK) { slice = first_pid / total; first_pid -= slice * total; }
    const int kt0 = SPLITK ? slice * a.kt_per_slice : 0;                                   // first k-tile of this workgroup
    const int KT = SPLITK ? min(a.kt_per_slice, KT_all - kt0) : KT_all;                    // k-tiles of this workgroup

    // ---- tile raster: spread over the 8 XCDs so that each XCD's L2 sees a compact block ----
    auto tile_coords = [&](int pid, int& bz, int& tile_m, int& tile_n) {
        if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
        bz = pid / tiles_mn;
        const int t = pid - bz * tiles_mn;
        const int group_sz = a.group_m * a.tiles_n;
        const int gid = t / group_sz;
        const int first_m = gid * a.group_m;
        const int gsz = min(a.tiles_m - first_m, a.group_m);
        const int tin = t - gid * group_sz;
        // (the divisions run on the vector ALU; everything here is wave-uniform, and saying so keeps what is derived
        // from it - descriptors, scalar offsets - in scalar registers)
        tile_m = __builtin_amdgcn_readfirstlane(first_m + tin % gsz);
        tile_n = __builtin_amdgcn_readfirstlane(tin / gsz);
        bz = __builtin_amdgcn_readfirstlane(bz);
    };

    // ---- compute side: the output tile whose accumulators this workgroup holds ----
    int c_bz, c_tile_m, c_tile_n;
    tile_coords(first_pid, c_bz, c_tile_m, c_tile_n);
    int m0 = c_tile_m * BM, n0 = c_tile_n * BN;

    // ---- issue side: the tile whose k-tiles are being fetched (the same tile unless the launch is persistent) ----
    uint32_t a_bytes;
    const uint32_t b_bytes = (uint32_t)a.N * (uint32_t)a.ldb * ES;
    if constexpr (OP == 0) a_bytes = (uint32_t)a.M * (uint32_t)a.lda * ES;
    else a_bytes = (uint32_t)(a.M / (a.HO * a.WO)) * (uint32_t)(a.H * a.W * a.CI) * ES;
    const char* baseA = (const char*)a.A;
    const char* baseB = (const char*)a.B;
    bool issue_alive = true;

    const int lrow = lane / CPR, lpos = lane % CPR;
    // When the rows that successive load instructions of a wave cover (NW*RPI apart) share their swizzle phase, a
    // lane's byte offset inside "its" row block is the same for every load and every tile: lane_off.  The row block
    // itself - tile origin, wave, load index - is a scalar and goes into the buffer descriptor (base advanced by the
    // block's byte offset, size reduced by it, so that rows past the end of the matrix still read as zeros).  The
    // issue side then holds two vector registers instead of one per load and spends no vector ALU work per tile.
    constexpr bool UNI = (SWZ == 0) || ((NW * RPI) % (CPR << (SWZ > 0 ? SWZ - 1 : 0))) == 0;
    constexpr bool UNI_A = UNI && OP == 0;
    const uint32_t lane_chunk = (uint32_t)((lpos ^ swz_of_row(wave * RPI + lrow)) * 16);
    const uint32_t lane_offB = (uint32_t)lrow * (uint32_t)a.ldb * ES + lane_chunk;
    const uint32_t lane_offA = (uint32_t)lrow * (uint32_t)a.lda * ES + lane_chunk;
    uint32_t blkA = 0, blkB = 0;                 // byte offset of the wave's first row block of the issue-side tile
    uint32_t voffB[B_LPW];
    // GEMM: byte offset of the lane's chunk in k-tile 0.  Conv: pixel bookkeeping.
    uint32_t voffA[(A_LPW > 0 ? A_LPW : 1)];
    int iy0[OP == 1 ? (A_LPW > 0 ? A_LPW : 1) : 1], ix0[OP == 1 ? (A_LPW > 0 ? A_LPW : 1) : 1];
    int cc = 0, cs = 0, cr = 0;  // conv: channel / kw / kh position of the lane's chunk
    int itile = first_pid;
    int issue_kt = 0;            // next k-tile (relative to kt0) of tile `itile` to fetch

    auto setup_issue = [&](int t) {
        issue_alive = t < total;                      // past the last tile every fetch reads zeros
        int bz, tile_m, tile_n;
        tile_coords(issue_alive ? t : 0, bz, tile_m, tile_n);
        const int im0 = tile_m * BM, in0 = tile_n * BN;
        baseA = (const char*)a.A + (int64_t)bz * a.sA * ES;
        baseB = (const char*)a.B + (int64_t)bz * a.sB * ES;
        if constexpr (UNI) {
            blkB = (uint32_t)(in0 + wave * RPI) * (uint32_t)a.ldb * ES;
        } else {
#pragma unroll
            for (int i = 0; i < B_LPW; ++i) {
                const int row = (i * NW + wave) * RPI + lrow;
                const int chunk = lpos ^ swz_of_row(row);
                const int n = in0 + row;
                voffB[i] = (n < a.N) ? (uint32_t)n * (uint32_t)a.ldb * ES + chunk * 16 : OOB;
            }
        }
        if constexpr (UNI_A) {
            blkA = (uint32_t)(im0 + wave * RPI) * (uint32_t)a.lda * ES;
        } else if constexpr (OP == 0) {
#pragma unroll
            for (int i = 0; i < A_LPW; ++i) {
                const int row = (i * NW + wave) * RPI + lrow;
                const int chunk = lpos ^ swz_of_row(row);
                const int m = im0 + row;
                voffA[i] = (m < a.M) ? (uint32_t)m * (uint32_t)a.lda * ES + chunk * 16 : OOB;
            }
        } else if constexpr (!CW) {
            static_assert(OP == 0 || CW || SWZ == 0 || ((NW * RPI) % (CPR << (SWZ > 0 ? SWZ - 1 : 0))) == 0,
                          "conv: the lane's chunk column must not depend on the load index");
            const int chunk = lpos ^ swz_of_row(wave * RPI + lrow);
            int ke = chunk * (16 / ES) + kt0 * (BKB / ES);      // element index inside K of this workgroup's first k-tile
            cr = ke / (a.KW * a.CI); ke -= cr * (a.KW * a.CI);
            cs = ke / a.CI; cc = ke - cs * a.CI;
            // output pixel of the lane's first row by division, of the following rows (NW*RPI further each) by carry
            const int hw = a.HO * a.WO;
            int m = im0 + wave * RPI + lrow;
            int img = m / hw;
            int rem = m - img * hw;
            int oy = rem / a.WO, ox = rem - oy * a.WO;
#pragma unroll
            for (int i = 0; i < A_LPW; ++i) {
                const bool ok = m < a.M;
                voffA[i] = (uint32_t)img * (uint32_t)(a.H * a.W * a.CI) * ES;
                iy0[i] = ok ? oy * a.cstride - a.cpad : -(1 << 28);
                ix0[i] = ox * a.cstride_w - a.cpad_w;
                m += NW * RPI;
                ox += NW * RPI;
                while (ox >= a.WO) { ox -= a.WO; if (++oy == a.HO) { oy = 0; ++img; } }
            }
        }
    };
    setup_issue(itile);

    // the stream moves on: next k-tile of this tile, or (persistent) k-tile 0 of the workgroup's next tile
    auto advance_issue = [&]() {
        ++issue_kt;
        if constexpr (PERS) {
            if (issue_kt == KT) { issue_kt = 0; itile += gridDim.x; setup_issue(itile); }
        }
    };

    // Fetch k-tile `issue_kt` of the issue-side tile straight into LDS stage `stage`: begin_issue() fixes the tile's
    // descriptors and scalar offset, issue_loads(first, count) emits a part of its LPT wave loads (A first, then B), so
    // that the caller can spread them between MFMAs, end_issue() moves the stream on.  RAG = the tile may be the last,
    // partly filled one (its chunks past the end of K are masked per lane); the plain form spends no vector ALU work.
    rsrc_t rA_cur, rB_cur;
    uint32_t ks_cur = 0, koff_cur = 0;
    bool live_cur = false;
    // descriptor of row block `i` of an operand: base advanced by the block's offset, size reduced by it
    auto block_rsrc = [&](const char* base, uint32_t bytes, uint32_t blk0, uint32_t ld_bytes, int i) {
        // (wave-uniform by construction; said explicitly, or the descriptor is treated as a per-lane value)
        const uint32_t off = (uint32_t)__builtin_amdgcn_readfirstlane((int)(blk0 + (uint32_t)(i * NW * RPI) * ld_bytes));
        const uint32_t left = (uint32_t)__builtin_amdgcn_readfirstlane((int)((live_cur && bytes > off) ? bytes - off : 0u));
        return make_rsrc(base + off, left);
    };
    auto begin_issue = [&]() {
        const bool live = issue_alive && issue_kt < KT;                          // wave-uniform
        live_cur = live;
        koff_cur = (uint32_t)(kt0 + issue_kt) * BKB;                             // byte offset of the k-tile in a row
        // a dead tile (past the end of K, or past the workgroup's last output tile) reads zeros through empty descriptors
        rB_cur = make_rsrc(baseB, live ? b_bytes : 0u);
        rA_cur = make_rsrc(baseA, live ? a_bytes : 0u);
        ks_cur = live ? koff_cur : 0u;
        return live && koff_cur + BKB > Kb;                                      // ragged: the last tile is not full
    };
    [[maybe_unused]] int conv_iyr = 0, conv_ixs = 0;
    [[maybe_unused]] bool conv_kvalid = false;
    auto conv_tap = [&]() {
        if constexpr (OP == 1 && !CW) { conv_iyr = cr * a.cdil; conv_ixs = cs * a.cdil_w; conv_kvalid = cr < a.KH; }
    };
    auto issue_loads = [&](auto ragc, int stage, auto firstc, auto countc) {
        constexpr bool RAG = decltype(ragc)::value;
        constexpr int FIRST = decltype(firstc)::value, COUNT = decltype(countc)::value;
        char* sbase = lds + stage * STAGE_BYTES;
        [[maybe_unused]] uint32_t koff_rag = koff_cur;
        // the masks of the ragged form are computed inside its (rarely taken) branch, not hoisted in front of it
        if constexpr (RAG) asm volatile("" : "+v"(koff_rag));
#pragma unroll
        for (int q = FIRST; q < FIRST + COUNT; ++q) {
            if (q < A_LPW) {
                const int i = q;
                if constexpr (UNI_A) {
                    uint32_t v = lane_offA;
                    if constexpr (RAG) { if (koff_rag + lane_chunk >= Kb) v = OOB; }
                    load_chunk_to_lds(block_rsrc(baseA, a_bytes, blkA, (uint32_t)a.lda * ES, i), sbase + (i * NW + wave) * 1024, v, ks_cur);
                } else if constexpr (OP == 0) {
                    uint32_t v = voffA[i];
                    if constexpr (RAG) {
                        const int row = (i * NW + wave) * RPI + lrow;
                        if (koff_rag + (uint32_t)((lpos ^ swz_of_row(row)) * 16) >= Kb) v = OOB;
                    }
                    load_chunk_to_lds(rA_cur, sbase + (i * NW + wave) * 1024, v, ks_cur);
                } else if constexpr (!CW) {
                    const int iy = iy0[i] + conv_iyr, ix = ix0[i] + conv_ixs;
                    const bool ok = conv_kvalid && (unsigned)iy < (unsigned)a.H && (unsigned)ix < (unsigned)a.W;
                    const uint32_t v = ok ? voffA[i] + (uint32_t)((iy * a.W + ix) * a.CI + cc) * ES : OOB;
                    load_chunk_to_lds(rA_cur, sbase + (i * NW + wave) * 1024, v, 0u);
                }
            } else {
                const int i = q - A_LPW;
                if constexpr (UNI) {
                    uint32_t v = lane_offB;
                    if constexpr (RAG) { if (koff_rag + lane_chunk >= Kb) v = OOB; }
                    load_chunk_to_lds(block_rsrc(baseB, b_bytes, blkB, (uint32_t)a.ldb * ES, i), sbase + A_BYTES + (i * NW + wave) * 1024, v, ks_cur);
                } else {
                    uint32_t v = voffB[i];
                    if constexpr (RAG) {
                        const int row = (i * NW + wave) * RPI + lrow;
                        if (koff_rag + (uint32_t)((lpos ^ swz_of_row(row)) * 16) >= Kb) v = OOB;
                    }
                    load_chunk_to_lds(rB_cur, sbase + A_BYTES + (i * NW + wave) * 1024, v, ks_cur);
                }
            }
        }
    };
    auto end_issue = [&]() {
        if constexpr (OP == 1 && !CW) {
            // advance the lane's (kh, kw, ci) position by one k-tile
            cc += BKB / ES;
            while (cc >= a.CI) { cc -= a.CI; if (++cs == a.KW) { cs = 0; ++cr; } }
        }
        advance_issue();
    };
    using TrueC = std::integral_constant<bool, true>;
    using FalseC = std::integral_constant<bool, false>;
    auto issue_tile = [&](int stage) {          // the whole tile at once (prologue)
        const bool rag = begin_issue();
        conv_tap();
        if (rag) issue_loads(TrueC{}, stage, std::integral_constant<int, 0>{}, std::integral_constant<int, LPT>{});
        else issue_loads(FalseC{}, stage, std::integral_constant<int, 0>{}, std::integral_constant<int, LPT>{});
        end_issue();
    };

    // ---- per-lane MFMA operand addresses ----
    const int lr = lane % MT, lq = lane / MT;

    // ---- conv window mode: the window itself (dynamic LDS) and the per-row tap masks ----
    const int w_pitch = a.CI * ES;                       // bytes of one pixel (all channels)
    const int w_cch = CW ? w_pitch / BKB : 1;            // k-tiles per tap
    uint32_t tapmask[CW ? TM : 1];                       // bit t: tap t of this lane's pixel i is inside the image
    if constexpr (CW) {
        const rsrc_t rA = make_rsrc(baseA, a_bytes);
        const int w_rows = BM + 2 * (a.cpad * a.W + a.cpad_w);  // pixels the BM outputs can reach
        const int cpp = w_pitch / 16;                    // 16-byte chunks per pixel
        const int n_instr = (w_rows * cpp + 63) / 64;    // 1 KiB wave loads that cover the window
        const int gp0 = m0 - (a.cpad * a.W + a.cpad_w);  // input pixel index of window row 0
        for (int q = wave; q < n_instr; q += NW) {
            const int L = q * 64 + lane;
            const int wrow = L / cpp, pos = L - wrow * cpp;
            const int src = (pos & ~(CPR - 1)) | ((pos & (CPR - 1)) ^ swz_of_row(wrow));
            const int gp = gp0 + wrow;
            const uint32_t v = (wrow < w_rows && gp >= 0) ? (uint32_t)gp * (uint32_t)w_pitch + src * 16 : OOB;
            load_chunk_to_lds(rA, win + q * 1024, v, 0u);
        }
        // masks: pixel of fragment row i by one division, the following rows (MT further each) by carry
        const int hw = a.H * a.W;
        int m = m0 + wm_idx * WTM + lr;
        int img = m / hw;
        int rem = m - img * hw;
        int oy = rem / a.W, ox = rem - oy * a.W;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            uint32_t bits = 0;
            if (m < a.M) {
                for (int r = 0; r < a.KH; ++r)
                    for (int s2 = 0; s2 < a.KW; ++s2) {
                        const int iy = oy + r - a.cpad, ix = ox + s2 - a.cpad_w;
                        if ((unsigned)iy < (unsigned)a.H && (unsigned)ix < (unsigned)a.W) bits |= 1u << (r * a.KW + s2);
                    }
            }
            tapmask[i] = bits;
            m += MT;
            ox += MT;
            while (ox >= a.W) { ox -= a.W; if (++oy == a.H) { oy = 0; ++img; } }
        }
    }
    const int w_lane = (wm_idx * WTM + lr);              // window mode: tile row of fragment 0
    int rd_tap = 0, rd_cch = 0, rd_r = 0, rd_s = 0;      // window mode: tap / channel chunk of the k-tile being READ
    const int g16 = (lq ^ swz_of_row(lr)) << 4;      // swizzle period <= MT, so only lr matters
    const int a_lane = (wm_idx * WTM + lr) * BKB;
    const int b_lane = A_BYTES + (wn_idx * WTN + lr) * BKB;

    acc_t acc[TM][TN];
    int bsum[TN];
    auto clear_acc = [&]() {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < ACC_N; ++r) acc[i][j][r] = 0;
#pragma unroll
        for (int j = 0; j < TN; ++j) bsum[j] = 0;
    };
    clear_acc();

    // Operand fragments, double-buffered in registers.  Read slot r of a step: r < TN is B fragment r, the others are
    // the A fragments in row-tile order - the order in which the MFMAs of the step consume them (the first row of
    // MFMAs needs every B fragment).
    v4i fa[2][TM], fb[2][TN];
    constexpr int NRD = TM + TN;
    auto read_slot = [&](int buf, int stage_off, int kk, int r) {
        if (r < TN) {
            fb[buf][r] = *(const v4i*)(lds + stage_off + b_lane + r * MT * BKB + (g16 ^ (kk * KSB)));
        } else {
            const int i = r - TN;
            if constexpr (CW) {
                const int tapoff = (rd_r < a.KH) ? rd_r * a.W + rd_s : 0;    // r*W + s pixels; 0 past the last tap
                const int wrow = w_lane + i * MT + tapoff;
                const int kc = (kk * CPS + lq) ^ swz_of_row(wrow);
                fa[buf][i] = *(const v4i*)(win + wrow * w_pitch + rd_cch * BKB + kc * 16);
            } else {
                fa[buf][i] = *(const v4i*)(lds + stage_off + a_lane + i * MT * BKB + (g16 ^ (kk * KSB)));
            }
        }
    };
    auto read_frags = [&](int buf, int stage_off, int kk) {
#pragma unroll
        for (int r = 0; r < NRD; ++r) read_slot(buf, stage_off, kk, r);
    };
    // window mode: move the reader to the next k-tile (channel chunks inside a tap first, then kw, then kh)
    auto advance_reader = [&]() {
        if constexpr (CW) {
            if (++rd_cch == w_cch) { rd_cch = 0; ++rd_tap; if (++rd_s == a.KW) { rd_s = 0; ++rd_r; } }
        }
    };
    int mm_tap = 0, mm_cch = 0;                           // window mode: tap of the k-tile being MULTIPLIED
    uint32_t tap_bit = 0;
    auto set_masks = [&]() {
        if constexpr (CW) {
            tap_bit = mm_tap;
            if (++mm_cch == w_cch) { mm_cch = 0; ++mm_tap; }
        }
    };
    // the A fragment of row-tile i as the MFMA takes it: window taps in the padding contribute zero, uint8 becomes
    // int8 by subtracting 128 (the sign-bit flip; the epilogue adds 128 * sum_k B back)
    auto a_operand = [&](int buf, int i) {
        v4i av = fa[buf][i];
        if constexpr (CW) {
            const int on = -(int)((tapmask[i] >> tap_bit) & 1u);
            av = av & (v4i){on, on, on, on};
        }
        if constexpr (DT == 1) av = av ^ (int)0x80808080;
        return av;
    };
    // uint8 path: sum_k B[n,k] of the step's B fragments.  The WM waves of one column hold the same fragments, so
    // they take turns: wave row w sums the steps with step % WM == w, the epilogue adds the WM partial sums.
    auto bsum_step = [&](int buf, int step) {
        if constexpr (DT == 1 && !COLSUM) {
            if (WM == 1 || (step & (WM - 1)) == wm_idx) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    int s = bsum[j];
                    s = __builtin_amdgcn_sdot4(fb[buf][j].x, 0x01010101, s, false);
                    s = __builtin_amdgcn_sdot4(fb[buf][j].y, 0x01010101, s, false);
                    s = __builtin_amdgcn_sdot4(fb[buf][j].z, 0x01010101, s, false);
                    s = __builtin_amdgcn_sdot4(fb[buf][j].w, 0x01010101, s, false);
                    bsum[j] = s;
                }
            }
        }
    };

    // ---- epilogue of the compute-side tile (c_bz, m0, n0) ----
    // MFMA was issued as (B fragment, A fragment), so a lane holds 4 consecutive n for one m:
    //   m = lr, n = (r/4)*8 + lq*4 + r%4   (32x32)     m = lr, n = lq*4 + r   (16x16)
    auto store_tile = [&]() __attribute__((always_inline)) {
        // the lane's coordinates, re-derived from values the compiler cannot trace back past this point: otherwise it
        // computes the epilogue's addresses in front of the k-loop and keeps them in registers all the way through it
        int lane_e = lane, lr_e, lq_e;
        asm volatile("" : "+v"(lane_e));
        lr_e = lane_e % MT; lq_e = lane_e / MT;
        char* const epi = CW ? win : lds + EPI_OFF;
        int* bs_lds = (int*)epi;
        if constexpr (DT == 1) {
            // 128 * sum_k B[n,k] completes the u8 x s8 product computed as (u8-128) x s8
            if constexpr (PERS) wait_and_barrier<63, 0>();     // the stages stay live: LDS traffic only, no drain
            else wait_and_barrier<0, 0>();
            if constexpr (COLSUM) {
                // the caller's sums of this tile's BN columns, 16 bytes per lane (N is a multiple of 4); a split-K
                // slice other than the first adds nothing (the sums cover all of K)
                for (int q = tid; q < BN / 4; q += NT) {
                    const int n = n0 + q * 4;
                    v4i v = {0, 0, 0, 0};
                    if (slice == 0 && n + 4 <= a.N) v = *(const v4i*)((const int*)a.bsum + (int64_t)c_bz * a.N + n);
                    *(v4i*)(bs_lds + q * 4) = v;
                }
            } else {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    int s = bsum[j];
#pragma unroll
                    for (int d = MT; d < 64; d <<= 1) s += __shfl_xor(s, d, 64);
                    if (lq_e == 0) bs_lds[wm_idx * BN + wn_idx * WTN + j * MT + lr_e] = s;
                }
            }
            if constexpr (PERS) wait_and_barrier<63, 0>();
            else __syncthreads();
        }
        // column sums of the 4 consecutive outputs a lane_e holds, all wave rows added
        auto colsum4 = [&](int nl) {
            v4i bs = *(const v4i*)(bs_lds + nl);
            if constexpr (!COLSUM) {
#pragma unroll
                for (int w = 1; w < WM; ++w) bs += *(const v4i*)(bs_lds + w * BN + nl);
            }
            return bs;
        };

        char* Cb = (char*)a.C + ((int64_t)slice * a.batch + c_bz) * a.sC * OES;
        auto put = [&](auto* ptr, auto val) __attribute__((always_inline)) {
            if constexpr (NTS) __builtin_nontemporal_store(val, ptr);
            else *ptr = val;
        };
        if constexpr (EPI >= 1) {
            // LDS-staged epilogue: a wave parks one MFMA row-tile (MT rows x SW columns) of its result in a private,
            // padded LDS strip, then streams it out with 16 bytes per lane_e, whole row segments per store instruction.
            if constexpr (DT == 0 && !PERS) wait_and_barrier<0, 0>();   // (the int8 path has synchronised above) stages are dead now
            [[maybe_unused]] const rsrc_t rsrcC = make_rsrc(Cb, (uint32_t)a.M * (uint32_t)a.ldc * OES);
            char* strip = epi + EPI_BASE + wave * (MT * EPI_PITCH);
            constexpr int CPRW = SW * OES / 16;                // 16-byte chunks per strip row
            constexpr int EPC = 16 / OES;                      // output elements per chunk
            constexpr int TNS = TN / ESPLIT;                   // MFMA column tiles per strip
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int h = 0; h < ESPLIT; ++h) {
#pragma unroll
                    for (int js = 0; js < TNS; ++js) {
                        const int j = h * TNS + js;
#pragma unroll
                        for (int g = 0; g < ACC_N / 4; ++g) {
                            const int cl = js * MT + g * 8 + lq_e * 4;         // column inside the strip
                            char* dst = strip + lr_e * EPI_PITCH + cl * OES;
                            if constexpr (DT == 0 && !SPLITK) {
                                v4h o;
#pragma unroll
                                for (int r = 0; r < 4; ++r) o[r] = (_Float16)acc[i][j][g * 4 + r];
                                *(v4h*)dst = o;
                            } else if constexpr (DT == 0) {
                                v4f o;
#pragma unroll
                                for (int r = 0; r < 4; ++r) o[r] = acc[i][j][g * 4 + r];
                                *(v4f*)dst = o;
                            } else {
                                const v4i bs = colsum4(wn_idx * WTN + h * SW + cl);
                                v4i o;
#pragma unroll
                                for (int r = 0; r < 4; ++r) o[r] = acc[i][j][g * 4 + r] + 128 * bs[r];
                                *(v4i*)dst = o;
                            }
                        }
                    }
                    asm volatile("" ::: "memory");     // LDS serves one wave's requests in order: the reads below see the writes
#pragma unroll
                    for (int it = 0; it < MT * CPRW / 64; ++it) {
                        const int c = it * 64 + lane_e;
                        const int row = c / CPRW, cc2 = c % CPRW;
                        const v4i val = *(const v4i*)(strip + row * EPI_PITCH + cc2 * 16);
                        const int m = m0 + wm_idx * WTM + i * MT + row;
                        const int n = n0 + wn_idx * WTN + h * SW + cc2 * EPC;
                        if constexpr (PERS) {
                            // always issued, so that every wave has exactly STORES_PER_TILE stores per tile in flight
                            const uint32_t off = (m < a.M && n + EPC <= a.N) ? (uint32_t)(m * a.ldc + n) * OES : OOB;
                            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(unsigned int __attribute__((ext_vector_type(4))), val), rsrcC, (int)off, 0, NTS ? 2 : 0);
                        } else {
                            char* dst = Cb + ((int64_t)m * a.ldc + n) * OES;
                            if (m < a.M) {
                                if (n + EPC <= a.N) put((v4i*)dst, val);
                                else if (OES == 2 && n + 4 <= a.N) put((long*)dst, (long)(((long)(uint32_t)val.y << 32) | (uint32_t)val.x));
                            }
                        }
                    }
                    asm volatile("" ::: "memory");
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int m = m0 + wm_idx * WTM + i * MT + lr_e;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
#pragma unroll
                    for (int g = 0; g < ACC_N / 4; ++g) {
                        const int nl = wn_idx * WTN + j * MT + g * 8 + lq_e * 4;
                        const int n = n0 + nl;
                        if (m < a.M && n < a.N) {
                            char* dst = Cb + ((int64_t)m * a.ldc + n) * OES;
                            if constexpr (DT == 0 && !SPLITK) {
                                v4h o;
#pragma unroll
                                for (int r = 0; r < 4; ++r) o[r] = (_Float16)acc[i][j][g * 4 + r];
                                put((v4h*)dst, o);
                            } else if constexpr (DT == 0) {
                                v4f o;
#pragma unroll
                                for (int r = 0; r < 4; ++r) o[r] = acc[i][j][g * 4 + r];
                                put((v4f*)dst, o);
                            } else {
                                const v4i bs = colsum4(nl);
                                v4i o;
#pragma unroll
                                for (int r = 0; r < 4; ++r) o[r] = acc[i][j][g * 4 + r] + 128 * bs[r];
                                put((v4i*)dst, o);
                            }
                        }
                    }
                }
            }
        }
    };

    // ---- prologue: fill all stages, wait for tile 0 ----
#pragma unroll
    for (int s = 0; s < NS; ++s) issue_tile(s);
    wait_and_barrier<(NS - 1) * LPT, 0>();
    if constexpr (SCHED != 2) read_frags(0, 0, 0);

    int stage = 0;
    // One k-step: the MFMAs of register buffer `cur`, row-tile by row-tile, with the fragment reads of the next step
    // (into the other buffer) and - in the last step of a k-tile - the wave loads of the tile that recycles this stage
    // issued between the rows.  The source order IS the issue order: every row ends in a scheduling fence.  Loads
    // come first (the next tile's fragment reads may not pass them: both touch LDS), over the first rows of the last
    // step; reads fill the remaining rows but leave the final row free, so that the barrier of the next tile does
    // not wait for a read that was just issued.
    auto kstep = [&](auto lastc, auto mayragc, const bool rag, const int cur, const int rd_stage_off, const int rd_kk,
                     const int kt, const int step) __attribute__((always_inline)) {
        constexpr bool LAST = decltype(lastc)::value;
        constexpr bool MAYRAG = decltype(mayragc)::value;
        constexpr int NLD = LAST ? LPT : 0;
        // rows of the last step that carry the tile's loads: HRN_LSPREAD 0 = none (all loads right behind the barrier),
        // 1 = the first quarter of the rows, 2 = half, 3 = all but the last two; spreading the requests smooths the
        // demand on the L2 (every workgroup of an XCD reaches its barrier at about the same time), at the price of a
        // later arrival of the tile.  The reads of the next step follow, the final row stays free (so that the barrier
        // of the next tile does not wait for a read that was just issued).
        constexpr int LWANT = LSPREAD == 0 ? 0 : (LSPREAD == 1 ? TM / 4 : (LSPREAD == 2 ? TM / 2 : TM - 2));
        constexpr int LROWS = NLD == 0 ? 0 : (LWANT < 1 ? ((LSPREAD > 0 && TM >= 2) ? 1 : 0) : (LWANT > TM - 1 ? TM - 1 : LWANT));
        constexpr int LFIRST = 0;                                                     // first load row
        constexpr int RFIRST_ROW = LROWS;                                             // first read row
        constexpr int RROWS_ALL = TM - LROWS;                                         // rows left for the reads
        constexpr int RROWS = RROWS_ALL >= 2 ? RROWS_ALL - 1 : RROWS_ALL;             // ... minus the free final row
        // the ragged form differs in the loads only, so the branch (wave-uniform) goes around just these
        auto loads = [&](auto firstc, auto countc) {
            if constexpr (MAYRAG) {
                if (rag) issue_loads(TrueC{}, stage, firstc, countc);
                else issue_loads(FalseC{}, stage, firstc, countc);
            } else {
                issue_loads(FalseC{}, stage, firstc, countc);
            }
        };
        if constexpr (LROWS == 0 && NLD > 0) loads(std::integral_constant<int, 0>{}, std::integral_constant<int, NLD>{});
        v4i av = a_operand(cur, 0);
        auto row = [&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if constexpr (i >= RFIRST_ROW && i - RFIRST_ROW < RROWS) {
                constexpr int f = NRD * (i - RFIRST_ROW) / RROWS, n = NRD * (i - RFIRST_ROW + 1) / RROWS - f;
#pragma unroll
                for (int r = f; r < f + n; ++r) read_slot(cur ^ 1, rd_stage_off, rd_kk, r);
            }
            if constexpr (LROWS > 0 && i >= LFIRST && i - LFIRST < LROWS) {
                constexpr int f = NLD * (i - LFIRST) / LROWS, n = NLD * (i - LFIRST + 1) / LROWS - f;
                loads(std::integral_constant<int, f>{}, std::integral_constant<int, n>{});
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = mfma(fb[cur][j], av, acc[i][j]);
            if constexpr (i + 1 < TM) av = a_operand(cur, i + 1);      // ready before the next row's MFMAs ask for it
            if constexpr (SCHED >= 1) __builtin_amdgcn_sched_barrier(0);
        };
        auto rows = [&](auto self, auto ic) -> void {
            row(ic);
            if constexpr (decltype(ic)::value + 1 < TM) self(self, std::integral_constant<int, decltype(ic)::value + 1>{});
        };
        rows(rows, std::integral_constant<int, 0>{});
        if constexpr (SCHED == 0) sched_hint<0, TM + TN, TM * TN, NLD>();
        bsum_step(cur, step);
    };
    // One k-tile.  P = register buffer that holds the fragments of its first k-step (the buffers alternate per
    // k-step, so with an odd number of k-steps per tile P alternates per tile).
    // MAYRAG: the k-tile this iteration fetches may be the partly filled last one of K (only then is the per-lane
    // masking of the loads compiled in; every other iteration runs the branch-free form).
    auto tile_body = [&](auto pc, auto mayragc, const int kt, const bool stores_between) __attribute__((always_inline)) {
        constexpr int P = decltype(pc)::value;
        const int stage_off = stage * STAGE_BYTES;
        const int next_stage = (stage + 1 == NS) ? 0 : stage + 1;
        set_masks();
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            const int cur = (kk + P) & 1;
            if (kk == KS - 1) {
                // every fragment of tile kt is in registers: publish tile kt+1, recycle this stage
                if constexpr (PERS) {
                    if (stores_between && kt <= NS - 2) wait_and_barrier<(NS - 2) * LPT + STORES_PER_TILE, 0>();
                    else wait_and_barrier<(NS - 2) * LPT, 0>();
                } else {
                    wait_and_barrier<(NS - 2) * LPT, 0>();
                }
                const bool rag = begin_issue();
                conv_tap();
                advance_reader();
                kstep(TrueC{}, mayragc, rag, cur, next_stage * STAGE_BYTES, 0, kt, kt * KS + kk);
                end_issue();
            } else {
                kstep(FalseC{}, FalseC{}, false, cur, stage_off, kk + 1, kt, kt * KS + kk);
            }
        }
        stage = next_stage;
    };
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    // Iteration kt fetches k-tile kt + NS of the stream, so only iteration KT - 1 - NS can meet the partly filled last
    // k-tile (a persistent stream shorter than NS + 1 k-tiles wraps more than once: every iteration may then).
    const bool k_ragged = (Kb % BKB) != 0;
    const int kt_rag = k_ragged ? KT - 1 - NS : -1;
    const bool rag_any = k_ragged && PERS && kt_rag < 0;
    // the k-tiles [from, to) of the compute-side tile; P0/P1 alternate when a k-tile holds an odd number of k-steps
    auto tiles = [&](auto mayragc, const int from, const int to, const bool stores_between) __attribute__((always_inline)) {
        if constexpr (KS % 2 == 0) {
            for (int kt = from; kt < to; ++kt) tile_body(P0{}, mayragc, kt, stores_between);
        } else {
            int kt = from;
            if (kt < to && (kt & 1)) { tile_body(P1{}, mayragc, kt, stores_between); ++kt; }
            for (; kt < to; kt += 2) {
                tile_body(P0{}, mayragc, kt, stores_between);
                if (kt + 1 < to) tile_body(P1{}, mayragc, kt + 1, stores_between);
            }
        }
    };
    auto run_tile = [&](const bool stores_between) __attribute__((always_inline)) {
        if (rag_any) {
            tiles(TrueC{}, 0, KT, stores_between);
        } else {
            // three loops in a row instead of a test inside one: the hot loops carry no ragged-tile code at all
            const int cut = min(max(kt_rag, 0), KT);
            tiles(FalseC{}, 0, cut, stores_between);
            if (kt_rag >= 0) tiles(TrueC{}, cut, min(cut + 1, KT), stores_between);
            tiles(FalseC{}, kt_rag >= 0 ? min(cut + 1, KT) : cut, KT, stores_between);
        }
        store_tile();
    };
    // ---- SCHED 2: two wave groups half a k-step apart ("ping-pong") ----
    // Waves w and w + 4 run on the same SIMD.  Group 0 (waves 0-3) and group 1 (waves 4-7) alternate between two kinds
    // of phase, one barrier apart: a memory phase (read the fragments of one k-step from LDS into the single register
    // buffer, flip the uint8 sign bits, add up the column sums) and a matrix phase (nothing but that step's MFMAs).
    // While one wave of a SIMD multiplies, the other waits for LDS and for a slot in the vector-memory queue, so those
    // waits never hold back an MFMA.  Phase 2s: group 0 multiplies step s, group 1 reads step s; phase 2s+1: group 0
    // reads step s+1, group 1 multiplies step s.  The stage of k-tile t is free once group 1 has read its last step;
    // in the phase after that every wave issues its share of the loads of k-tile t + NS, and every wave waits for its
    // own loads of k-tile t + 1 at the end of the phase in which group 1 reads the last step of k-tile t.
    // fragment reads of the step whose k-offset inside the stage row is `koff` bytes (a runtime value here: the
    // k-loop of this schedule is not unrolled over the k-steps of a tile, so that every fragment register has one
    // definition per iteration and stays where it is)
    auto pp_mem = [&](const int stage_off, const int koff) __attribute__((always_inline)) {
        const int gk = g16 ^ koff;
        const char* pb = lds + stage_off + b_lane + gk;
        const char* pa = lds + stage_off + a_lane + gk;
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[0][j] = *(const v4i*)(pb + j * MT * BKB);
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[0][i] = *(const v4i*)(pa + i * MT * BKB);
    };
    auto pp_ready = [&](const int step) __attribute__((always_inline)) {      // after the reads have landed
        if constexpr (DT == 1) {
            // (as volatile statements, so that the sign flips stay in this phase: plain code may be moved past
            // the barrier into the matrix phase)
            const int flip = (int)0x80808080;
#pragma unroll
            for (int i = 0; i < TM; ++i)
                asm volatile("v_xor_b32 %0, %4, %0\n\tv_xor_b32 %1, %4, %1\n\tv_xor_b32 %2, %4, %2\n\tv_xor_b32 %3, %4, %3"
                             : "+v"(fa[0][i].x), "+v"(fa[0][i].y), "+v"(fa[0][i].z), "+v"(fa[0][i].w) : "s"(flip));
        }
        bsum_step(0, step);
    };
    auto pp_mfma = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) mfma_inplace(fb[0][j], fa[0][i], acc[i][j]);
        __builtin_amdgcn_s_setprio(0);
    };
    auto pp_fence = [&]() __attribute__((always_inline)) { __builtin_amdgcn_sched_barrier(0); };
    const bool grp1 = wave >= NW / 2;                     // wave-uniform: the group that runs one phase behind
    // Both groups run the SAME instruction stream - read step s, barrier, multiply step s, barrier, read step s+1 ... -
    // and group 1 enters it one barrier later, so the two are always in opposite kinds of phase.  Only the fetches of
    // the next k-tile and the waits for them sit at group-dependent places of the stream (uniform branches around
    // nothing but those), because they are tied to the moment at which a stage becomes free for BOTH groups.
    auto pp_loads = [&]() __attribute__((always_inline)) {
        const bool rag = begin_issue();
        conv_tap();
        if (rag) issue_loads(TrueC{}, stage, std::integral_constant<int, 0>{}, std::integral_constant<int, LPT>{});
        else issue_loads(FalseC{}, stage, std::integral_constant<int, 0>{}, std::integral_constant<int, LPT>{});
        end_issue();
    };
    auto pp_run = [&]() __attribute__((always_inline)) {
        if (grp1) wait_and_barrier<63, 15>();            // group 1 enters the stream one phase later
        pp_fence();
        pp_mem(0, 0);
        pp_fence();
        wait_only<63, 0>();
        pp_ready(0);
        pp_fence();
        if (KS == 1 && grp1) wait_only<(NS - 2) * LPT, 15>();
        wait_and_barrier<63, 15>();
        pp_fence();
        int kk = 0;                                      // k-step inside the k-tile
        const int steps = KT * KS;
        for (int step = 0; step < steps; ++step) {
            const bool last = (kk == KS - 1);
            const int nkk = last ? 0 : kk + 1;
            const bool next_last = (nkk == KS - 1);
            const int next_stage = (stage + 1 == NS) ? 0 : stage + 1;
            // ---- multiply step `step` (group 0: phase 2*step, group 1: one phase later) ----
            if (last && grp1) pp_loads();                // the stage of this k-tile is free for both groups now
            pp_fence();
            pp_mfma();
            pp_fence();
            // before the next k-tile is published every wave's share of it has landed (group 0 waits here ...)
            if (last && !grp1) wait_only<(NS - 2) * LPT, 15>();
            wait_and_barrier<63, 15>();
            pp_fence();
            // ---- read step `step + 1` ----
            pp_mem((last ? next_stage : stage) * STAGE_BYTES, nkk * KSB);
            pp_fence();
            if (last && !grp1) pp_loads();               // group 0 is one phase ahead: the stage is free only now
            pp_fence();
            wait_only<63, 0>();
            pp_ready(step + 1);
            pp_fence();
            if (next_last && grp1) wait_only<(NS - 2) * LPT, 15>();      // (... group 1 here)
            wait_and_barrier<63, 15>();
            pp_fence();
            kk = nkk;
            if (last) stage = next_stage;
        }
        if (!grp1) wait_and_barrier<63, 15>();           // ... and group 0 leaves it one phase earlier
    };
    if constexpr (SCHED == 2) {
        static_assert(SCHED != 2 || (NW == 8 && !CW && !PERS && !SPLITK), "the two-group schedule: 8 waves, plain launch");
        pp_run();
        mfma_drain();
        store_tile();
    } else if constexpr (PERS) {
        for (int ct = blockIdx.x; ct < total; ct += (int)gridDim.x) {
            tile_coords(ct, c_bz, c_tile_m, c_tile_n);
            m0 = c_tile_m * BM; n0 = c_tile_n * BN;
            // the stores of the previous tile's epilogue sit between the fetches that were issued before it and
            // the ones issued after it; while such a fetch is the one waited for, the wait allows for them
            run_tile(ct != (int)blockIdx.x && KT >= NS - 1);
            clear_acc();
        }
    } else {
        run_tile(false);
    }
}
