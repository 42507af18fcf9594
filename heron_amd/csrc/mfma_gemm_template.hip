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
//               stores, HRN_WPE waves-per-SIMD hint, HRN_PF L2 prefetch distance, HRN_LOAD load path.
//
// Data movement: both operands are K-contiguous, so a tile is a set of rows of HRN_BKB bytes.
// Rows are cut into 16-byte chunks; every lane moves one chunk per load straight from HBM/L2
// into LDS (buffer_load_dwordx4 ... lds), one wave instruction filling 1 KiB of consecutive LDS.
// The chunk a lane fetches is XOR-swizzled so that the MFMA operand reads (ds_read_b128, one
// 16-byte chunk per lane) spread over all LDS banks.  Out-of-range rows, conv halo taps and the
// dummy tiles past the end of K are fetched with an out-of-range buffer offset, which the
// buffer unit turns into zeros.
//
// Pipeline: HRN_STAGES tiles are in flight.  The barrier that publishes tile t+1 sits before the
// last k-step of tile t, so operand fragments of the next tile are already being read while the
// last MFMAs of the current tile run; fragments are double-buffered in registers.
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
    int32_t pf_sa, pf_sb;       // L2 prefetch: column-tiles / row-tiles of the block one XCD runs concurrently
    int32_t cstride_w, cpad_w, cdil_w;   // conv: the width-direction values (cstride/cpad/cdil are the height ones)
};
#endif

namespace {

constexpr int DT = HRN_DTYPE;
constexpr int OP = HRN_OP;
constexpr int BM = HRN_BM, BN = HRN_BN, BKB = HRN_BKB;
constexpr int WM = HRN_WM, WN = HRN_WN, MT = HRN_MFMA, NS = HRN_STAGES, SWZ = HRN_SWZ;
constexpr int EPI = HRN_EPI;
// Diagnostic switches for bottleneck analysis (results are WRONG when non-zero; 0 in every shipped
// instance): 1 skip LDS fragment reads after the first tile, 2 skip global->LDS loads after the
// prologue, 4 drop the per-tile barrier, 8 skip the MFMAs, 16 skip the stores of C.
#ifndef HRN_ABLATE
#define HRN_ABLATE 0
#endif
constexpr int ABL = HRN_ABLATE;
// L2 prefetch: with HRN_PF = d > 0 every tile fetch is preceded by 4-byte "touch" loads of the k-tile d tiles
// further on (this workgroup's share of the rows, see the kernel).  The data is discarded; the point is that
// the sectors are in L2 (not HBM) when the real fetch arrives, because a tile is only usable when its slowest
// load has landed.
#ifndef HRN_PF
#define HRN_PF 0
#endif
constexpr int PF = HRN_PF;
// Load path: 0 = global -> LDS directly (LDS-DMA), HRN_STAGES tiles in LDS.
//            1 = global -> registers -> LDS: two register sets hold the two tiles in flight, LDS holds the tile
//                being multiplied and the next one (HRN_STAGES must be 2); a tile then has two tile-times to land.
#ifndef HRN_LOAD
#define HRN_LOAD 0
#endif

constexpr int LOADM = HRN_LOAD;
// Conv window mode (HRN_OP=1, stride 1, dilation 1, 'same' padding): instead of fetching an im2col tile of A for every
// filter tap, the workgroup loads ONCE the window of input pixels its BM output pixels can reach (a contiguous range
// of BM + 2*(pad_h*W + pad_w) pixels, all channels) and every tap reads its operand fragments from that window at a row offset
// of r*W + s pixels; taps that fall into the padding are masked to zero in registers.  Only B (the filter) streams
// through the LDS stages.
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
constexpr int ES = (DT == 0) ? 2 : 1;       // input element bytes
constexpr int OES = (DT == 0) ? 2 : 4;      // output element bytes
constexpr int NW = WM * WN, NT = NW * 64;
constexpr int CPR = BKB / 16;               // 16-byte chunks per tile row
constexpr int RPI = 64 / CPR;               // tile rows one wave load instruction covers
constexpr int A_LPW = CW ? 0 : (BM / RPI) / NW;   // load instructions per wave per tile
constexpr int B_LPW = (BN / RPI) / NW;
constexpr int LPR = (BKB + 127) / 128;                         // 128-byte lines per tile row
constexpr int PF_N = PF ? 1 : 0;                                // prefetch touches per lane per tile
constexpr int LPT = A_LPW + B_LPW + PF_N;                       // vector memory ops per lane per tile
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
static_assert(KS >= 2 && (KS % 2) == 0, "need an even number of k-steps per tile");
static_assert((CW || ((BM / RPI) % NW == 0 && A_LPW >= 1)) && (BN / RPI) % NW == 0 && B_LPW >= 1, "loads per wave");
static_assert(!CW || (OP == 1 && LOADM == 0 && PF == 0), "window mode is a conv2d load path");
static_assert(OP == 0 || PF == 0, "L2 prefetch is implemented for the GEMM address pattern only");
static_assert(PF == 0 || NW >= 2, "L2 prefetch needs one wave for each operand");
static_assert(BM % (WM * MT) == 0 && BN % (WN * MT) == 0, "wave tile");
static_assert(NS >= 2 && NS <= 5, "stages");
static_assert(LOADM == 0 || (NS == 2 && PF == 0), "register-staged loads use exactly two LDS stages");
constexpr int PF_SCRATCH = PF ? NW * 256 : 0;                   // LDS corner the prefetch touches land in
// LDS-staged epilogue: per wave a strip of MT rows x WTN outputs, rows padded by 16 bytes; after the int8 column sums
constexpr int EPI_PITCH = WTN * OES + 16;
constexpr int EPI_BASE = (DT == 1) ? ((BN * 4 + 1023) / 1024) * 1024 : 0;
constexpr int EPI_BYTES = (EPI == 1) ? EPI_BASE + NW * MT * EPI_PITCH : 0;
// the epilogue region (column sums + strips) reuses the stages, except in persistent mode where the stages stay live
constexpr int EPI_OFF = PERS ? NS * STAGE_BYTES : 0;
constexpr int LDS_BYTES = PERS ? NS * STAGE_BYTES + EPI_BYTES
                               : ((NS * STAGE_BYTES + PF_SCRATCH > EPI_BYTES) ? NS * STAGE_BYTES + PF_SCRATCH : EPI_BYTES);
constexpr int STORES_PER_TILE = (EPI == 1) ? TM * (MT * (WTN * OES / 16) / 64) : 0;   // store instructions per wave per output tile
static_assert(!PERS || (EPI == 1 && LOADM == 0 && PF == 0 && !CW && HRN_ABLATE == 0), "persistent mode: staged epilogue, direct loads");
static_assert(!PERS || (NS - 2) * (A_LPW + B_LPW) + STORES_PER_TILE <= 63, "persistent mode: vmcnt range");
static_assert(LDS_BYTES <= 163840, "LDS");
static_assert(EPI == 0 || (MT * (WTN * OES / 16)) % 64 == 0, "staged epilogue: a strip must split into whole wave stores");
static_assert(SWZ == 0 || (CPR << (SWZ - 1)) <= MT, "swizzle period must fit in one MFMA tile");
static_assert((NS - 1) * LPT <= 63, "vmcnt range");
static_assert(NT <= 1024, "threads");

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

// raw buffer (stride 0): an offset >= `bytes` reads as zero instead of touching memory
__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ void load_chunk_to_lds(rsrc_t rsrc, char* lds_wave_base, uint32_t voff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds_wave_base,
                                             16, (int)voff, 0, 0, 0);
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

// Scheduling pattern of one k-step: NR groups of {1 LDS read, NV/NR buffer loads, NDW/NR LDS writes, NMM/NR MFMAs}.
template <int R, int NR, int NMM, int NV, int NDW = 0>
__device__ __forceinline__ void sched_pattern() {
    if constexpr (R < NR) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        constexpr int v = (NV * (R + 1)) / NR - (NV * R) / NR;
        if constexpr (v > 0) __builtin_amdgcn_sched_group_barrier(0x020, v, 0);
        constexpr int w = (NDW * (R + 1)) / NR - (NDW * R) / NR;
        if constexpr (w > 0) __builtin_amdgcn_sched_group_barrier(0x200, w, 0);
        constexpr int mm = (NMM * (R + 1)) / NR - (NMM * R) / NR;
        if constexpr (mm > 0) __builtin_amdgcn_sched_group_barrier(0x008, mm, 0);
        sched_pattern<R + 1, NR, NMM, NV, NDW>();
    }
}

}  // namespace

extern "C" __global__ void __launch_bounds__(NT)
#if HRN_WPE > 0
__attribute__((amdgpu_waves_per_eu(HRN_WPE, HRN_WPE)))
#endif
hrn_mfma_kernel(const HrnKArgs a) {
    __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm_idx = wave / WN, wn_idx = wave % WN;

    const int tiles_mn = a.tiles_m * a.tiles_n;
    const int total = tiles_mn * a.batch;
    const uint32_t Kb = (uint32_t)a.K * ES;           // bytes of K
    const int KT = (Kb + BKB - 1) / BKB;

    // ---- tile raster: spread over the 8 XCDs so that each XCD's L2 sees a compact block ----
    auto tile_coords = [&](int pid, int& bz, int& tile_m, int& tile_n, int& tin, int& gsz) {
        if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
        bz = pid / tiles_mn;
        const int t = pid - bz * tiles_mn;
        const int group_sz = a.group_m * a.tiles_n;
        const int gid = t / group_sz;
        const int first_m = gid * a.group_m;
        gsz = min(a.tiles_m - first_m, a.group_m);
        tin = t - gid * group_sz;
        tile_m = first_m + tin % gsz;
        tile_n = tin / gsz;
    };

    // ---- compute side: the output tile whose accumulators this workgroup holds ----
    int c_bz, c_tile_m, c_tile_n, c_tin, c_gsz;
    tile_coords(blockIdx.x, c_bz, c_tile_m, c_tile_n, c_tin, c_gsz);
    int m0 = c_tile_m * BM, n0 = c_tile_n * BN;

    // ---- issue side: the tile whose k-tiles are being fetched (the same tile unless the launch is persistent) ----
    uint32_t a_bytes;
    const uint32_t b_bytes = (uint32_t)a.N * (uint32_t)a.ldb * ES;
    if constexpr (OP == 0) a_bytes = (uint32_t)a.M * (uint32_t)a.lda * ES;
    else a_bytes = (uint32_t)(a.M / (a.HO * a.WO)) * (uint32_t)(a.H * a.W * a.CI) * ES;
    rsrc_t rsrcA = make_rsrc(a.A, a_bytes);
    rsrc_t rsrcB = make_rsrc(a.B, b_bytes);

    const int lrow = lane / CPR, lpos = lane % CPR;
    uint32_t voffB[B_LPW];
    // GEMM: byte offset of the lane's chunk in k-tile 0.  Conv: pixel bookkeeping.
    uint32_t voffA[(A_LPW > 0 ? A_LPW : 1)];
    int iy0[OP == 1 ? (A_LPW > 0 ? A_LPW : 1) : 1], ix0[OP == 1 ? (A_LPW > 0 ? A_LPW : 1) : 1];
    int cc = 0, cs = 0, cr = 0;  // conv: channel / kw / kh position of the lane's chunk
    int itile = blockIdx.x;
    int issue_kt = 0;            // next k-tile of tile `itile` to fetch

    auto setup_issue = [&](int t) {
        const bool alive = t < total;                 // past the last tile every fetch reads zeros
        int bz, tile_m, tile_n, tin, gsz;
        tile_coords(alive ? t : 0, bz, tile_m, tile_n, tin, gsz);
        const int im0 = tile_m * BM, in0 = tile_n * BN;
        rsrcA = make_rsrc((const char*)a.A + (int64_t)bz * a.sA * ES, a_bytes);
        rsrcB = make_rsrc((const char*)a.B + (int64_t)bz * a.sB * ES, b_bytes);
#pragma unroll
        for (int i = 0; i < B_LPW; ++i) {
            const int row = (i * NW + wave) * RPI + lrow;
            const int chunk = lpos ^ swz_of_row(row);
            const int n = in0 + row;
            voffB[i] = (alive && n < a.N) ? (uint32_t)n * (uint32_t)a.ldb * ES + chunk * 16 : OOB;
        }
        if constexpr (OP == 0) {
#pragma unroll
            for (int i = 0; i < A_LPW; ++i) {
                const int row = (i * NW + wave) * RPI + lrow;
                const int chunk = lpos ^ swz_of_row(row);
                const int m = im0 + row;
                voffA[i] = (alive && m < a.M) ? (uint32_t)m * (uint32_t)a.lda * ES + chunk * 16 : OOB;
            }
        } else if constexpr (!CW) {
            static_assert(OP == 0 || SWZ == 0 || ((NW * RPI) % (CPR << (SWZ > 0 ? SWZ - 1 : 0))) == 0,
                          "conv: the lane's chunk column must not depend on the load index");
            const int chunk = lpos ^ swz_of_row(wave * RPI + lrow);
            int ke = chunk * (16 / ES);                 // element index inside K of tile 0
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
                const bool ok = alive && m < a.M;
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

    // L2 prefetch duty of this workgroup.  The tiles that run on one XCD at the same time form a block of
    // a.pf_sb row-tiles x a.pf_sa column-tiles; the pf_sa tiles of one block row read the same rows of A and the
    // pf_sb tiles of one block column the same rows of B, so each tile touches only its 1/pf_sa share of the A rows
    // and 1/pf_sb share of the B rows (every 64-byte sector of them) of the k-tile PF tiles past the one being
    // fetched.  Waves of the lower half touch A, waves of the upper half B, one touch per lane per tile.
    uint32_t pf_off[PF_N > 0 ? PF_N : 1];
    const bool pf_isb = wave >= (NW + 1) / 2;
    if constexpr (PF > 0) {
        constexpr int SEC = BKB >= 64 ? BKB / 64 : 1;
        const int share = pf_isb ? a.pf_sb : a.pf_sa;
        const int duty = pf_isb ? (c_tin % c_gsz) % share : c_tile_n % share;
        const int q = (pf_isb ? tid - ((NW + 1) / 2) * 64 : tid);      // touch slot inside the operand's waves
        const int row = duty + share * (q / SEC), sec = q % SEC;
        const int g = (pf_isb ? n0 : m0) + row;
        const bool ok = row < (pf_isb ? BN : BM) && g < (pf_isb ? a.N : a.M);
        pf_off[0] = ok ? (uint32_t)g * (uint32_t)(pf_isb ? a.ldb : a.lda) * ES + sec * 64 : OOB;
    }

    // Byte offsets of this lane's chunks in k-tile `issue_kt` (out-of-range offset = zeros), shared by both load paths.
    uint32_t offA[(A_LPW > 0 ? A_LPW : 1)], offB[B_LPW];
    auto tile_offsets = [&]() {
        const bool live = issue_kt < KT;
        const bool ragged = (uint32_t)(issue_kt + 1) * BKB > Kb;   // last tile not full (wave-uniform)
        const uint32_t koff = live ? (uint32_t)issue_kt * BKB : OOB;
        if constexpr (OP == 0) {
#pragma unroll
            for (int i = 0; i < A_LPW; ++i) {
                uint32_t v = voffA[i] + koff;
                if (ragged && live) {
                    const int row = (i * NW + wave) * RPI + lrow;
                    const uint32_t kb = koff + (uint32_t)((lpos ^ swz_of_row(row)) * 16);
                    if (kb >= Kb) v = OOB;
                }
                offA[i] = v;
            }
        } else if constexpr (!CW) {
            const int iyr = cr * a.cdil, ixs = cs * a.cdil_w;
            const bool kvalid = live && cr < a.KH;
#pragma unroll
            for (int i = 0; i < A_LPW; ++i) {
                const int iy = iy0[i] + iyr, ix = ix0[i] + ixs;
                const bool ok = kvalid && (unsigned)iy < (unsigned)a.H && (unsigned)ix < (unsigned)a.W;
                offA[i] = ok ? voffA[i] + (uint32_t)((iy * a.W + ix) * a.CI + cc) * ES : OOB;
            }
            // advance the lane's (kh, kw, ci) position by one k-tile
            cc += BKB / ES;
            while (cc >= a.CI) { cc -= a.CI; if (++cs == a.KW) { cs = 0; ++cr; } }
        }
#pragma unroll
        for (int i = 0; i < B_LPW; ++i) {
            uint32_t v = voffB[i] + koff;
            if (ragged && live) {
                const int row = (i * NW + wave) * RPI + lrow;
                const uint32_t kb = koff + (uint32_t)((lpos ^ swz_of_row(row)) * 16);
                if (kb >= Kb) v = OOB;
            }
            offB[i] = v;
        }
    };
    // the stream moves on: next k-tile of this tile, or (persistent) k-tile 0 of the workgroup's next tile
    auto advance_issue = [&]() {
        ++issue_kt;
        if constexpr (PERS) {
            if (issue_kt == KT) { issue_kt = 0; itile += gridDim.x; setup_issue(itile); }
        }
    };

    // path 0: fetch k-tile `issue_kt` straight into LDS stage `stage`
    auto issue_tile = [&](int stage) {
        char* sbase = lds + stage * STAGE_BYTES;
        if constexpr (PF > 0) {
            // the touched dwords are dropped into a scratch corner of LDS: no register is tied up and
            // the loads are counted by vmcnt like the tile fetches that follow them
            const uint32_t pk = (uint32_t)(issue_kt + PF) * BKB;
            const bool pf_live = pk < Kb;
            auto* scratch = (__attribute__((address_space(3))) void*)(lds + NS * STAGE_BYTES + wave * 256);
            const uint32_t v = pf_live ? pf_off[0] + pk : OOB;
            if (pf_isb) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcB, scratch, 4, (int)v, 0, 0, 0);
            else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, scratch, 4, (int)v, 0, 0, 0);
        }
        tile_offsets();
#pragma unroll
        for (int i = 0; i < A_LPW; ++i) load_chunk_to_lds(rsrcA, sbase + (i * NW + wave) * 1024, offA[i]);
#pragma unroll
        for (int i = 0; i < B_LPW; ++i) load_chunk_to_lds(rsrcB, sbase + A_BYTES + (i * NW + wave) * 1024, offB[i]);
        advance_issue();
    };

    // path 1: fetch k-tile `issue_kt` into register set SET; later copy a set into an LDS stage
    v4i regA[LOADM ? 2 : 1][LOADM ? (A_LPW > 0 ? A_LPW : 1) : 1], regB[LOADM ? 2 : 1][LOADM ? B_LPW : 1];
    auto issue_regs = [&](auto setc) {
        constexpr int SET = decltype(setc)::value;
        tile_offsets();
#pragma unroll
        for (int i = 0; i < A_LPW; ++i) regA[SET][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrcA, (int)offA[i], 0, 0);
#pragma unroll
        for (int i = 0; i < B_LPW; ++i) regB[SET][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrcB, (int)offB[i], 0, 0);
        ++issue_kt;
    };
    auto write_lds = [&](auto setc, int stage) {
        constexpr int SET = decltype(setc)::value;
        char* sbase = lds + stage * STAGE_BYTES + lane * 16;
#pragma unroll
        for (int i = 0; i < A_LPW; ++i) *(v4i*)(sbase + (i * NW + wave) * 1024) = regA[SET][i];
#pragma unroll
        for (int i = 0; i < B_LPW; ++i) *(v4i*)(sbase + A_BYTES + (i * NW + wave) * 1024) = regB[SET][i];
    };

    // ---- per-lane MFMA operand addresses ----
    const int lr = lane % MT, lq = lane / MT;

    // ---- conv window mode: the window itself (dynamic LDS) and the per-row tap masks ----
    extern __shared__ __attribute__((aligned(1024))) char win[];
    const int w_pitch = a.CI * ES;                       // bytes of one pixel (all channels)
    const int w_cch = CW ? w_pitch / BKB : 1;            // k-tiles per tap
    uint32_t tapmask[CW ? TM : 1];                       // bit t: tap t of this lane's pixel i is inside the image
    if constexpr (CW) {
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
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, (__attribute__((address_space(3))) void*)(win + q * 1024),
                                                     16, (int)v, 0, 0, 0);
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

    v4i fa[2][TM], fb[2][TN];
    auto read_frags = [&](int buf, int stage_off, int kk) {
        const int ko = g16 ^ (kk * KSB);
        if constexpr (CW) {
            const int tapoff = (rd_r < a.KH) ? rd_r * a.W + rd_s : 0;    // r*W + s pixels; 0 past the last tap
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int wrow = w_lane + i * MT + tapoff;
                const int kc = (kk * CPS + lq) ^ swz_of_row(wrow);
                fa[buf][i] = *(const v4i*)(win + wrow * w_pitch + rd_cch * BKB + kc * 16);
            }
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i)
                fa[buf][i] = *(const v4i*)(lds + stage_off + a_lane + i * MT * BKB + ko);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j)
            fb[buf][j] = *(const v4i*)(lds + stage_off + b_lane + j * MT * BKB + ko);
    };
    // window mode: move the reader to the next k-tile (channel chunks inside a tap first, then kw, then kh)
    auto advance_reader = [&]() {
        if constexpr (CW) {
            if (++rd_cch == w_cch) { rd_cch = 0; ++rd_tap; if (++rd_s == a.KW) { rd_s = 0; ++rd_r; } }
        }
    };
    int mm_tap = 0, mm_cch = 0;                           // window mode: tap of the k-tile being MULTIPLIED
    v4i amask[CW ? TM : 1];
    auto set_masks = [&]() {
        if constexpr (CW) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int on = -(int)((tapmask[i] >> mm_tap) & 1u);
                amask[i] = (v4i){on, on, on, on};
            }
            if (++mm_cch == w_cch) { mm_cch = 0; ++mm_tap; }
        }
    };
    auto mfma_step = [&](int buf) {
        if constexpr (DT == 1) {
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
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            v4i av = fa[buf][i];
            if constexpr (CW) av = av & amask[i];               // taps in the padding contribute zero
            if constexpr (DT == 1) av = av ^ (int)0x80808080;   // u8 -> s8 by subtracting 128
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = mfma(fb[buf][j], av, acc[i][j]);
        }
    };

    // ---- epilogue of the compute-side tile (c_bz, m0, n0) ----
    // MFMA was issued as (B fragment, A fragment), so a lane holds 4 consecutive n for one m:
    //   m = lr, n = (r/4)*8 + lq*4 + r%4   (32x32)     m = lr, n = lq*4 + r   (16x16)
    auto store_tile = [&]() {
        int* bs_lds = (int*)(lds + EPI_OFF);
        if constexpr (DT == 1) {
            // 128 * sum_k B[n,k] completes the u8 x s8 product computed as (u8-128) x s8
            if constexpr (PERS) wait_and_barrier<63, 0>();     // the stages stay live: LDS traffic only, no drain
            else wait_and_barrier<0, 0>();
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                int s = bsum[j];
#pragma unroll
                for (int d = MT; d < 64; d <<= 1) s += __shfl_xor(s, d, 64);
                if (wm_idx == 0 && lq == 0) bs_lds[wn_idx * WTN + j * MT + lr] = s;
            }
            if constexpr (PERS) wait_and_barrier<63, 0>();
            else __syncthreads();
        }

        char* Cb = (char*)a.C + (int64_t)c_bz * a.sC * OES;
        const bool do_store = !(ABL & 16) || a.K == 0x7fffffff;   // the ablation keeps the stores reachable but never takes them
        if constexpr (EPI == 1) {
            // LDS-staged epilogue: a wave parks one MFMA row-tile (MT rows x WTN columns) of its result in a private,
            // padded LDS strip, then streams it out with 16 bytes per lane, whole row segments per store instruction.
            if constexpr (DT == 0 && !PERS) wait_and_barrier<0, 0>();   // (the int8 path has synchronised above) stages are dead now
            [[maybe_unused]] const rsrc_t rsrcC = make_rsrc(Cb, (uint32_t)a.M * (uint32_t)a.ldc * OES);
            char* strip = lds + EPI_OFF + EPI_BASE + wave * (MT * EPI_PITCH);
            constexpr int CPRW = WTN * OES / 16;               // 16-byte chunks per strip row
            constexpr int EPC = 16 / OES;                      // output elements per chunk
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
#pragma unroll
                    for (int g = 0; g < ACC_N / 4; ++g) {
                        const int cl = j * MT + g * 8 + lq * 4;          // column inside the wave tile
                        char* dst = strip + lr * EPI_PITCH + cl * OES;
                        if constexpr (DT == 0) {
                            v4h o;
#pragma unroll
                            for (int r = 0; r < 4; ++r) o[r] = (_Float16)acc[i][j][g * 4 + r];
                            *(v4h*)dst = o;
                        } else {
                            const v4i bs = *(const v4i*)(bs_lds + wn_idx * WTN + cl);
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
                    const int c = it * 64 + lane;
                    const int row = c / CPRW, cc2 = c % CPRW;
                    const v4i val = *(const v4i*)(strip + row * EPI_PITCH + cc2 * 16);
                    const int m = m0 + wm_idx * WTM + i * MT + row;
                    const int n = n0 + wn_idx * WTN + cc2 * EPC;
                    if constexpr (PERS) {
                        // always issued, so that every wave has exactly STORES_PER_TILE stores per tile in flight
                        const uint32_t off = (m < a.M && n + EPC <= a.N) ? (uint32_t)(m * a.ldc + n) * OES : OOB;
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(unsigned int __attribute__((ext_vector_type(4))), val), rsrcC, (int)off, 0, 0);
                    } else {
                        char* dst = Cb + ((int64_t)m * a.ldc + n) * OES;
                        if (do_store && m < a.M) {
                            if (n + EPC <= a.N) *(v4i*)dst = val;
                            else if (DT == 0 && n + 4 <= a.N) *(long*)dst = ((long)(uint32_t)val.y << 32) | (uint32_t)val.x;
                        }
                    }
                }
                asm volatile("" ::: "memory");
            }
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int m = m0 + wm_idx * WTM + i * MT + lr;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
#pragma unroll
                    for (int g = 0; g < ACC_N / 4; ++g) {
                        const int nl = wn_idx * WTN + j * MT + g * 8 + lq * 4;
                        const int n = n0 + nl;
                        if (do_store && m < a.M && n < a.N) {
                            char* dst = Cb + ((int64_t)m * a.ldc + n) * OES;
                            if constexpr (DT == 0) {
                                v4h o;
#pragma unroll
                                for (int r = 0; r < 4; ++r) o[r] = (_Float16)acc[i][j][g * 4 + r];
                                *(v4h*)dst = o;
                            } else {
                                const v4i bs = *(const v4i*)(bs_lds + nl);
                                v4i o;
#pragma unroll
                                for (int r = 0; r < 4; ++r) o[r] = acc[i][j][g * 4 + r] + 128 * bs[r];
                                *(v4i*)dst = o;
                            }
                        }
                    }
                }
            }
        }
    };

    if constexpr (LOADM == 0) {
        // ---- prologue: fill all stages, wait for tile 0 ----
    #pragma unroll
        for (int s = 0; s < NS; ++s) issue_tile(s);
        wait_and_barrier<(NS - 1) * LPT, 0>();
        read_frags(0, 0, 0);

        int stage = 0;
        auto run_tile = [&](const bool stores_between) {
            for (int kt = 0; kt < KT; ++kt) {
                const int stage_off = stage * STAGE_BYTES;
                const int next_stage = (stage + 1 == NS) ? 0 : stage + 1;
                set_masks();
    #pragma unroll
                for (int kk = 0; kk < KS; ++kk) {
                    const int cur = kk & 1;
                    if (kk == KS - 1) {
                        // every fragment of tile kt is in registers: publish tile kt+1, recycle this stage
                        if constexpr (PERS) {
                            if (stores_between && kt <= NS - 2) wait_and_barrier<(NS - 2) * LPT + STORES_PER_TILE, 0>();
                            else wait_and_barrier<(NS - 2) * LPT, 0>();
                        } else if constexpr (ABL & 4) {
                            wait_only<(NS - 2) * LPT, 0>();
                        } else {
                            wait_and_barrier<(NS - 2) * LPT, 0>();
                        }
                        if (!(ABL & 2)) issue_tile(stage);
                        advance_reader();
                        if (!(ABL & 1) || kt == 0) read_frags(cur ^ 1, next_stage * STAGE_BYTES, 0);
                    } else {
                        if (!(ABL & 1) || kt == 0) read_frags(cur ^ 1, stage_off, kk + 1);
                    }
                    if (!(ABL & 8)) mfma_step(cur);
                    // pin the issue order: fragment reads (and, in the last step, the tile fetch) are
                    // spread between the MFMAs of this step instead of being sunk behind them
                    if (kk == KS - 1) sched_pattern<0, TM + TN, TM * TN, LPT>();
                    else sched_pattern<0, TM + TN, TM * TN, 0>();
                }
                stage = next_stage;
            }
            store_tile();
        };
        if constexpr (PERS) {
            for (int ct = blockIdx.x; ct < total; ct += (int)gridDim.x) {
                tile_coords(ct, c_bz, c_tile_m, c_tile_n, c_tin, c_gsz);
                m0 = c_tile_m * BM; n0 = c_tile_n * BN;
                // the stores of the previous tile's epilogue sit between the fetches that were issued before it and
                // the ones issued after it; while such a fetch is the one waited for, the wait allows for them
                run_tile(ct != (int)blockIdx.x && KT >= NS - 1);
                clear_acc();
            }
        } else {
            run_tile(false);
        }
    } else {
        // ---- register-staged pipeline: tile t is requested during tile t-3's last k-step, copied into LDS
        // during tile t-1 and multiplied as tile t: two tile-times for the data to arrive ----
        using S0 = std::integral_constant<int, 0>;
        using S1 = std::integral_constant<int, 1>;
        issue_regs(S0{});
        issue_regs(S1{});
        write_lds(S0{}, 0);
        wait_and_barrier<63, 0>();
        issue_regs(S0{});
        read_frags(0, 0, 0);
        auto body = [&](auto parity) {
            constexpr int P = decltype(parity)::value;      // LDS stage of the tile being multiplied
            using Other = std::integral_constant<int, 1 - P>;
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) {
                const int cur = kk & 1;
                if (kk == KS - 2) write_lds(Other{}, 1 - P);       // next tile: registers -> the free LDS stage
                if (kk == KS - 1) {
                    wait_and_barrier<63, 0>();                      // LDS writes visible, old stage drained
                    issue_regs(Other{});                            // request the tile three ahead
                    read_frags(cur ^ 1, (1 - P) * STAGE_BYTES, 0);
                } else {
                    read_frags(cur ^ 1, P * STAGE_BYTES, kk + 1);
                }
                if (!(ABL & 8)) mfma_step(cur);
                if (kk == KS - 1) sched_pattern<0, TM + TN, TM * TN, A_LPW + B_LPW, 0>();
                else if (kk == KS - 2) sched_pattern<0, TM + TN, TM * TN, 0, A_LPW + B_LPW>();
                else sched_pattern<0, TM + TN, TM * TN, 0, 0>();
            }
        };
        for (int kt = 0; kt < KT; kt += 2) {
            body(S0{});
            if (kt + 1 < KT) body(S1{});
        }
        store_tile();
    }
}
