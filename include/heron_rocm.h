/*
 * heron_rocm.h - C ABI of the MI355X (gfx950) backend for the tensor programs Heron tunes.
 *
 * The reference has no FFI of its own for this path: its kernels are generated, built and
 * timed through TVM from Python.  Each entry point below names the reference interface it
 * stands in for (paths relative to the reference checkout).  All pointers named A, B, C
 * are DEVICE pointers owned by the caller; the library never allocates persistent device
 * memory and never frees caller memory.  Every function returns HRN_OK (0) or a negative
 * HRN_E_* code; hrn_last_error() gives the message of the last failure on the calling thread.
 *
 * Launches are asynchronous on the given stream and may be issued from several host
 * threads.  The library is NOT fork-safe once a HIP call has been made: processes forked
 * for sampling must not call into it (hrn_compile is the exception: it never touches HIP).
 */
#ifndef HERON_ROCM_H
#define HERON_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HRN_OK 0
#define HRN_E_BADPARAM (-1)   /* descriptor/problem violates a template constraint */
#define HRN_E_BUILD (-2)      /* hipcc failed or timed out */
#define HRN_E_LOAD (-3)       /* code object could not be loaded */
#define HRN_E_LAUNCH (-4)     /* HIP reported a launch/runtime error */
#define HRN_E_TIMEOUT (-5)    /* build exceeded the time limit */
#define HRN_E_NODEVICE (-6)   /* no HIP device */

/* element types of a template */
#define HRN_DT_F16 0   /* fp16 x fp16 -> fp32 accumulate -> fp16 store */
#define HRN_DT_U8S8 1  /* uint8 x int8 -> int32 accumulate -> int32 store */

/* operators */
#define HRN_OP_GEMM 0    /* C[b,i,j] = sum_k A[b,i,k] * B[b,j,k]  (batch may be 1) */
#define HRN_OP_CONV2D 1  /* NHWC input, KRSC filter, implicit GEMM */

/*
 * Device limits the schedule context reads.  Replaces the `check_gpu` dictionary that
 * the reference's runner hands to its builder (environment.py:110-120, consumed at
 * schedule/context/cuda_context.py:49-51,74-78).
 */
typedef struct hrn_devinfo {
    char arch[64];            /* e.g. "gfx950:sramecc+:xnack-" */
    char name[128];
    int32_t cu_count;
    int32_t wave_size;
    int32_t lds_bytes_per_wg;
    int32_t max_threads_per_wg;
    int32_t clock_khz;        /* peak engine clock */
    int32_t mem_clock_khz;
    int32_t mem_bus_bits;
    int32_t l2_bytes;
    int32_t regs_per_simd_lane; /* unified VGPR+AGPR file per lane of one SIMD */
    int32_t simd_per_cu;
    uint64_t hbm_bytes;
} hrn_devinfo;

/*
 * One instance of the MFMA kernel template = one point of the tuner's search space.
 * Replaces the (schedule, args) pair the reference gets from Task.instantiate
 * (task/task.py:76-89) and passes to tvm.build (tests/quick_start/dlboost/run.py:44-46).
 */
typedef struct hrn_kernel_desc {
    int32_t dtype;      /* HRN_DT_* */
    int32_t op;         /* HRN_OP_* */
    int32_t bm, bn;     /* workgroup tile (rows of A / rows of B) */
    int32_t bkb;        /* bytes of K per LDS stage row: 64, 128 or 256 */
    int32_t wm, wn;     /* wave grid inside the workgroup; waves = wm*wn, 64 lanes each */
    int32_t mfma;       /* 32 -> 32x32x(16 f16|32 i8), 16 -> 16x16x(32 f16|64 i8) */
    int32_t stages;     /* LDS stages of the A/B tiles, 2..5 (2 = double buffer) */
    int32_t swizzle;    /* LDS 16-byte-chunk XOR swizzle: 0 none, 1 row, 2 row/2, 3 row/4 */
    int32_t epilogue;   /* 0 = store accumulators straight from registers, 1 = stage C through LDS strips as wide as
                           the wave tile, 2 = through strips of half that width (half the LDS) */
    int32_t waves_per_eu; /* 0 = let the compiler pick, else occupancy hint 1..4 */
    int32_t conv_window;  /* conv2d only: 1 = keep the reachable input window in LDS and read every filter tap from it
                             (needs stride 1, dilation 1, 'same' padding, CI*2 a multiple of bkb) instead of im2col tiles */
    int32_t persistent;   /* 1 = launch only as many workgroups as fit the device and let each walk several output tiles,
                             fetching the next tile's operands while the current result is stored (needs epilogue 1 and
                             N*out_bytes a multiple of 16) */
    int32_t split_k;      /* 1 = K is cut into hrn_problem.split_k slices that run as separate workgroups; the kernel
                             stores raw fp32 / int32 partial sums per slice into hrn_problem.workspace and a second
                             pass of the library adds them into C (for small M*N with long K: more workgroups than
                             output tiles).  Not with persistent or conv_window. */
    int32_t sched;        /* issue order of a k-step: 1 = the template's own interleaving of fragment reads, tile loads
                             and MFMAs is pinned with scheduling fences, 0 = left to the compiler under group hints,
                             2 = two-group schedule (8 waves, no conv_window / persistent / split_k): waves 0-3 and
                             4-7 alternate, one barrier apart, between a phase that only reads fragments and one that
                             only multiplies, with a single fragment register buffer */
    int32_t load_spread;  /* with sched = 1: how far the wave loads of the next k-tile are spread over the MFMA rows of the
                             step that issues them: 0 = all right behind the barrier, 1 = over a quarter of the rows,
                             2 = half, 3 = all but the last two (smoother demand on the L2, later arrival) */
    int32_t colsum;       /* u8s8 only: the kernel computes (u8 - 128) x s8 on the signed MFMA and adds 128 * sum_k B[n,k];
                             0 = it adds those column sums up itself from the B fragments in its k-loop, 1 = it takes
                             them from hrn_problem.bsum (they depend on the weights alone: hrn_colsum_s8 makes them) */
    int32_t nt_store;     /* 1 = the results are stored with the non-temporal hint, so that C (written once, never read
                             by the kernel) does not push the operand slabs of the next round of tiles out of L2;
                             0 = default cache policy (a consumer that reads C right away finds more of it in L2).
                             Split-K partial sums always take the default policy */
} hrn_kernel_desc;

/* Resource usage of a built instance, for cross-checks of the constraint set. */
typedef struct hrn_kernel_info {
    int32_t vgprs;       /* architectural VGPRs per lane */
    int32_t agprs;       /* accumulation VGPRs per lane */
    int32_t sgprs;
    int32_t lds_bytes;   /* static LDS of the kernel; a conv_window instance adds its window at launch */
    int32_t scratch_bytes;
    int32_t occupancy;   /* waves per SIMD the compiler reports */
    int32_t threads;     /* workgroup size */
    int32_t reserved;
} hrn_kernel_info;

/*
 * Shapes.  GEMM/bmm: A (batch,M,K), B (batch,N,K), C (batch,M,N), all row-major with the
 * given leading dimensions (elements) and batch strides (elements).  ops/cuda/dense.py:5-7,
 * ops/cuda/batch_matmul.py:7-9, ops/x86/dense.py:7-9.
 * Conv: input (n,h,w,ci), filter (co,kh,kw,ci), output (n,ho,wo,co);
 * argument order of ops/cuda/conv2d.py:137-139.
 */
typedef struct hrn_problem {
    int32_t op;         /* HRN_OP_* */
    int32_t batch;
    int32_t m, n, k;
    int32_t lda, ldb, ldc;
    int64_t stride_a, stride_b, stride_c;
    /* conv only; cstride/cpad/cdil act on the height, the *_w fields on the width (the reference's operators take
     * an int or an (h, w) pair for each, ops/cuda/conv2d.py:143-153); padding is symmetric per direction */
    int32_t cn, ch, cw, ci, co, kh, kw, cstride, cpad, cdil;
    /* launch-time raster knob: tiles are walked in column groups of this many row-tiles */
    int32_t group_m;
    int32_t cstride_w, cpad_w, cdil_w;
    /* split-K instances only (hrn_kernel_desc.split_k = 1): number of K slices wanted (>= 1; slices never get less
     * than one k-tile, so fewer may run) and the caller-owned device workspace for the partial sums, at least
     * hrn_splitk_workspace_bytes() large and 16-byte aligned.  Launches that share a workspace must not overlap. */
    int32_t split_k;
    void* workspace;
    size_t workspace_bytes;
    /* colsum instances only (hrn_kernel_desc.colsum = 1): device pointer to batch x n int32 column sums of B,
     * bsum[b*n + j] = sum_k B[b][j][k] (conv: over the whole filter of output channel j), 16-byte aligned */
    const void* bsum;
} hrn_problem;

typedef struct hrn_module hrn_module;

/* Device query.  Stands in for runner.get_build_kwargs() (environment.py:110-120). */
int hrn_device_info(int device, hrn_devinfo* out);

/*
 * Checks a descriptor against the template's structural constraints without building
 * (tile divisibility, LDS ceiling, wave count).  Stands in for the feasibility check the
 * reference leaves to tvm.build failing (runner/measure_methods.py:178-185).
 */
int hrn_check_desc(const hrn_kernel_desc* desc);

/*
 * Compiles one template instance with hipcc into the on-disk cache and returns the path of
 * the code object.  Touches no GPU (safe in forked/pooled builder processes).  Stands in for
 * autotvm.LocalBuilder -> tvm.build (tests/quick_start/dlboost/run.py:89-96), including its
 * `build_timeout` (config.py:48): timeout_s <= 0 means no limit.  path_out may be NULL; a buffer
 * that cannot hold the path and its terminator is HRN_E_BADPARAM.
 */
int hrn_compile(const hrn_kernel_desc* desc, double timeout_s, char* path_out, size_t path_cap);

/* hrn_compile + load on the current device.  Stands in for the module loader of
 * runner/measure_methods.py:129-130. */
int hrn_build(const hrn_kernel_desc* desc, double timeout_s, hrn_module** out);
int hrn_module_info(const hrn_module* mod, hrn_kernel_info* out);
void hrn_module_free(hrn_module* mod);

/* LDS bytes an instance needs (pure arithmetic; mirrors the constraint of
 * schedule/context/cuda_context.py:45-63 for this template). */
int hrn_lds_bytes(const hrn_kernel_desc* desc);

/*
 * Launchers.  Each replaces the packed function TVM builds for the named operator and that
 * run.py:60-62 / measure_methods.py:138-145 call with device arrays.
 *   hrn_launch_gemm_f16        ops/cuda/dense.py:4-54          (fp16 in, fp32 accumulate, fp16 out)
 *   hrn_launch_gemm_u8s8       ops/x86/dense.py:6-32           (uint8 x int8 -> int32)
 *   hrn_launch_bmm_f16         ops/cuda/batch_matmul.py:5-56
 *   hrn_launch_conv2d_nhwc_f16 ops/cuda/conv2d.py:137-232      (filter KRSC)
 *   hrn_launch_bmm_u8s8        ops/x86/batch_matmul.py:6-34    (uint8 x int8 -> int32 per batch entry)
 *   hrn_launch_conv2d_nhwc_u8s8 ops/x86/conv2d_int8.py:31-109  (uint8 NHWC input, int8 filter -> int32; the filter is
 *                              taken KRSC (co,kh,kw,ci), not in the reference's blocked (co/b,kh,kw,ci/4,b,4) order;
 *                              the output (n,ho,wo,co) is the reference's (n,ho,wo,co/b,b) seen flat)
 */
int hrn_launch_gemm_f16(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream);
int hrn_launch_gemm_u8s8(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream);
int hrn_launch_bmm_f16(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream);
int hrn_launch_conv2d_nhwc_f16(const hrn_module* mod, const hrn_problem* p, const void* In, const void* Filter, void* Out, void* stream);
int hrn_launch_bmm_u8s8(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream);
int hrn_launch_conv2d_nhwc_u8s8(const hrn_module* mod, const hrn_problem* p, const void* In, const void* Filter, void* Out, void* stream);

/*
 * Split-K launch that allocates nothing.  No counterpart in the reference; it is for callers that cannot allocate
 * device memory around a launch (code under HIP graph capture, tight serving loops, harnesses that forbid it).  Same as
 * launching a split_k instance through the entry points above, except that the partial sums go to a workspace that
 * is part of the library's own device image (HRN_STATIC_WORKSPACE_BYTES per GPU, held until the process ends) instead
 * of hrn_problem.workspace, which is ignored.  A problem whose partial sums (slices * batch * m * n * 4 bytes) exceed
 * that size is refused with HRN_E_BADPARAM.  Every call on a GPU uses that GPU's one workspace: a call on another
 * stream than the previous one first waits (on the device) for that previous call, so calls from several streams or
 * host threads are serialised rather than racing; nothing in the workspace needs to be zero between calls.  Calls no
 * hipMalloc / hipFree; the workspace's address and the ordering event are set up by hrn_build of a split_k instance.
 * The cross-stream wait is an event wait, which a stream under graph capture cannot take from a stream outside the
 * capture: inside a capture keep to one stream.
 */
#define HRN_STATIC_WORKSPACE_BYTES (32u << 20)
int hrn_launch_splitk_static(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream);

/* `count` back-to-back launches of the same problem from one host call (the inner loop of a time_evaluator
 * repeat, runner/measure_methods.py:138-145, without the events). */
int hrn_launch_repeat(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C,
                      int count, void* stream);

/*
 * Event-timed measurement with the semantics of TVM's time_evaluator as the reference uses
 * it (runner/measure_methods.py:138-145): `repeat` results, each the mean seconds of `number`
 * back-to-back launches; `number` is raised until one repeat lasts at least min_repeat_ms.
 * costs_out must hold `repeat` doubles.
 */
int hrn_time(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C,
             int number, int repeat, double min_repeat_ms, double* costs_out, void* stream);

/*
 * Cold-cache variant: before each of the `repeat` single launches, `flush_bytes` of caller-owned device memory at
 * flush_buf (use at least twice the last-level cache: 1 GiB covers the 256 MiB memory-side cache) are streamed through
 * the caches, so the launch finds its operands in HBM only.  The GPU-side counterpart of the reference runner's
 * `enable_cpu_cache_flush` (tests/quick_start/dlboost/run.py:89-96, runner/measure_methods.py:138-145).
 */
int hrn_time_cold(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C,
                  void* flush_buf, size_t flush_bytes, int repeat, double* costs_out, void* stream);

/*
 * Column sums of an int8 operand: bsum[b*n + j] = sum_k B[b][j][k] for B (batch, n, k) with leading dimension ldb and
 * batch stride stride_b (elements = bytes); k and ldb multiples of 16.  This is the weight-side preparation of the
 * colsum instances, the counterpart of the reference's pre-packed weight operand: ops/x86/dense.py:7-9 takes the
 * weights already blocked as (N/16, K/4, 16, 4), so what depends on the weights alone is done once, outside the
 * operator.  Both buffers are caller-owned device memory; bsum holds batch * n int32.
 */
int hrn_colsum_s8(const void* B, void* bsum, int batch, int n, int k, int ldb, int64_t stride_b, void* stream);

/*
 * Channel padding pre-stage: copies `rows` rows of `c` elements (1 or 2 bytes each) from `src` to rows of `cp`
 * elements in `dst`, zero-filling the tail; cp * elem_bytes must be a multiple of 16.  Replaces the `pad` /
 * layout stages the reference inlines in front of its tensorized conv (ops/cuda/conv2d.py:160-170) for inputs whose
 * channel count is short of a 16-byte chunk (the 3-channel stem).  Both buffers are caller-owned device memory.
 */
int hrn_pad_rows(const void* src, void* dst, size_t rows, int c, int cp, int elem_bytes, void* stream);

/*
 * Layout pre-stage / post-stage: batched transpose src[batch][rows][cols] -> dst[batch][cols][rows_padded], the tail of
 * every output row (rows..rows_padded) zero-filled; elements of 1, 2 or 4 bytes.  Channels-first activations
 * (N,C,H*W) become channels-last with padded channels in one pass, and a channels-last result goes back to
 * channels-first: the layout stages the reference inlines around its tensorized product for the NCHW / NCW
 * operators (ops/cuda/conv2d.py:9-135, ops/cuda/conv1d.py).  Both buffers are caller-owned device memory.
 */
int hrn_transpose_pad(const void* src, void* dst, int batch, int rows, int cols, int rows_padded, int elem_bytes, void* stream);

/*
 * Injective pre-stage as one pass: dst = f(gather(src)).  The reference declares such stages as tensor expressions in
 * front of its tensorized product and inlines them into the shared-memory load (utils.py:290-303 traverse_inline,
 * schedule/sched_op/sched_common.py:198-202): zero padding and depth unfolding of conv3d (ops/cuda/conv3d.py), the
 * stride expansion of the transposed conv (ops/cuda/conv2d_transposed.py:93-104), the 3x3 window gathering of the
 * depthwise conv (ops/cuda/dep.py), the channel-major view of mean (ops/cuda/mean.py) and (x - mean)^2 of var
 * (ops/cuda/var.py:9-14).  Here the stage is described by an affine index map and runs as a kernel of the library in
 * front of hrn_mfma_kernel.
 *
 * dst has `ndim` dimensions (outermost first) with extents dst_dim and element strides dst_stride (innermost 1).  For
 * the element at index (i_0 .. i_{ndim-1}) source coordinate s (0 <= s < nsrc) is
 *     c_s = (add[s] + sum_d mul[s][d] * i_d) / div[s]
 * and the element is src[sum_s c_s * src_stride[s]] when every i_d < dst_live[d], every numerator is non-negative and
 * divisible by div[s] and every c_s < src_dim[s]; otherwise it is zero.  op HRN_GATHER_CENTER_SQUARE (fp16 only) stores
 * (x - y)^2, both steps rounded to fp16, where a plain copy stores x; y is the element of `aux` at x's offset (aux has
 * the layout of src: var's Mean operand, ops/cuda/var.py:7-13).  When the innermost dimension
 * moves whole, aligned 16-byte pieces (the library checks the map, the extents and both pointers) every lane moves 16
 * bytes, otherwise one element.  All buffers are caller-owned device memory; elements not covered by dst_dim /
 * dst_stride (row padding) are left alone.
 */
#define HRN_GATHER_DIMS 6
#define HRN_GATHER_COPY 0
#define HRN_GATHER_CENTER_SQUARE 1
typedef struct hrn_gather {
    int32_t ndim;
    int32_t nsrc;
    int32_t elem_bytes;       /* 1, 2 or 4 */
    int32_t op;
    int32_t reserved[2];
    int64_t dst_dim[HRN_GATHER_DIMS];
    int64_t dst_stride[HRN_GATHER_DIMS];
    int64_t dst_live[HRN_GATHER_DIMS];
    int64_t src_dim[HRN_GATHER_DIMS];
    int64_t src_stride[HRN_GATHER_DIMS];
    int64_t add[HRN_GATHER_DIMS];
    int64_t div[HRN_GATHER_DIMS];
    int64_t mul[HRN_GATHER_DIMS][HRN_GATHER_DIMS];   /* mul[s][d] */
} hrn_gather;
int hrn_gather_nd(const hrn_gather* g, const void* src, const void* aux, void* dst, void* stream);

/*
 * Roofline probes (no counterpart in the reference, which never relates a timing to a hardware
 * limit).  hrn_probe_mfma times a register-resident loop of independent MFMAs of the given
 * dtype/shape on every CU and returns dense T(FL)OP/s (random_operands != 0 feeds operands with the
 * bit statistics of real data instead of small constants: switching power lowers the sustained
 * clock); hrn_probe_copy times a 16-byte-per-lane
 * copy kernel over `bytes` of caller-owned device memory and returns GB/s counting read + write.
 * The copy kernel is also the known-size reference for scaling FETCH_SIZE / WRITE_SIZE counters.
 * hrn_probe_launch times `repeat` back-to-back dispatches of a kernel that does nothing (`grid` workgroups of 256
 * lanes) and returns microseconds per dispatch: the floor under every small layer's latency.
 */
int hrn_probe_launch(int grid, int repeat, double* us_out, void* stream);
/* hrn_probe_read streams `bytes` of caller-owned device memory through the lanes without storing (GB/s read): what
 * a kernel that only reads, like the P x V batch_matmul, can draw from HBM when the buffer exceeds the caches. */
int hrn_probe_read(const void* src, size_t bytes, int repeat, double* gbs_out, void* stream);
int hrn_probe_mfma(int dtype, int mfma, int random_operands, double* tops_out, void* stream);
/* hrn_probe_traffic_cold times, `repeat` times, ONE launch of a kernel that reads read_bytes from src and writes
 * write_bytes to dst (16-byte words, 16 bytes per lane) right after the caches were flushed with flush_buf exactly as
 * hrn_time_cold does; us_out holds `repeat` microsecond values.  With a workload's algorithmic byte counts this is the
 * like-for-like floor of its cold launch: same flush, same single dispatch, nothing but the traffic. */
int hrn_probe_traffic_cold(const void* src, size_t read_bytes, void* dst, size_t write_bytes, void* flush_buf,
                           size_t flush_bytes, int repeat, double* us_out, void* stream);
int hrn_probe_copy(const void* src, void* dst, size_t bytes, int repeat, double* gbs_out, void* stream);

/*
 * Bytes of workspace a launch of `desc` on problem `p` (with p->split_k set) needs: slices * batch * m * n * 4, or 0
 * when the instance is not a split-K one; negative HRN_E_* on bad arguments.  The reference has no counterpart: its
 * TensorCore schedules never split the reduction over thread blocks (ops/cuda/dense.py:18-26 binds only the
 * spatial axes to blockIdx).
 */
int64_t hrn_splitk_workspace_bytes(const hrn_kernel_desc* desc, const hrn_problem* p);

/* Fills an hrn_problem for the plain cases (packed row-major operands). */
void hrn_problem_gemm(hrn_problem* p, int batch, int m, int n, int k);
void hrn_problem_conv2d(hrn_problem* p, int n, int h, int w, int ci, int co, int kh, int kw,
                        int stride, int pad, int dil);
void hrn_problem_conv2d_hw(hrn_problem* p, int n, int h, int w, int ci, int co, int kh, int kw,
                           int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w);

const char* hrn_last_error(void);
const char* hrn_version(void);

#ifdef __cplusplus
}
#endif
#endif /* HERON_ROCM_H */
