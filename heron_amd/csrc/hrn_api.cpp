// C ABI of the gfx950 backend: template instantiation (hipcc -> code object cache), module
// loading, launchers and event timing.  Declarations and the reference interfaces each entry
// point stands in for are in include/heron_rocm.h.
#include "../../include/heron_rocm.h"

#include <hip/hip_runtime.h>

#include <dlfcn.h>
#include <fcntl.h>
#include <signal.h>
#include <sys/stat.h>
#include <sys/types.h>
#include <spawn.h>
#include <sys/wait.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <mutex>
#include <sstream>
#include <string>
#include <thread>
#include <type_traits>
#include <vector>

#define HRN_KARGS_DEFINED
struct HrnKArgs {  // must match mfma_gemm_template.hip
    const void* A;
    const void* B;
    void* C;
    int32_t M, N, K;
    int32_t lda, ldb, ldc;
    int64_t sA, sB, sC;
    int32_t tiles_m, tiles_n, group_m, batch;
    int32_t H, W, CI, HO, WO, KH, KW, cstride, cpad, cdil;
    int32_t cstride_w, cpad_w, cdil_w;
    int32_t split, kt_per_slice;
    const void* bsum;
};

struct hrn_module {
    hrn_kernel_desc desc;
    hrn_kernel_info info;
    hipModule_t mod;
    hipFunction_t fn;
    std::string path;
    int persist_grid;   // persistent instances: workgroups that fit the device at once (multiple of 8 when >= 8)
    int epi_bytes;      // LDS bytes of the epilogue region (column sums + strips)
};

extern char** environ;

namespace {

thread_local std::string g_err;

int fail(int code, const char* fmt, ...) {
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}

#define HIP_TRY(expr)                                                                         \
    do {                                                                                      \
        hipError_t e_ = (expr);                                                               \
        if (e_ != hipSuccess) return fail(HRN_E_LAUNCH, "%s: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

// two timing events that are destroyed on every exit path
struct EventPair {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t create() {
        hipError_t e = hipEventCreate(&e0);
        return e != hipSuccess ? e : hipEventCreate(&e1);
    }
    ~EventPair() {
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
    }
};

std::string lib_dir() {
    Dl_info di;
    if (dladdr((void*)&hrn_last_error, &di) && di.dli_fname) {
        std::string p = di.dli_fname;
        size_t s = p.rfind('/');
        return s == std::string::npos ? "." : p.substr(0, s);
    }
    return ".";
}

std::string env_or(const char* name, const std::string& dflt) {
    const char* v = getenv(name);
    return (v && *v) ? std::string(v) : dflt;
}

std::string kernel_source() { return env_or("HRN_KERNEL_DIR", lib_dir()) + "/mfma_gemm_template.hip"; }
std::string cache_dir() { return env_or("HRN_CACHE_DIR", lib_dir() + "/cache"); }

bool file_exists(const std::string& p) {
    struct stat st;
    return stat(p.c_str(), &st) == 0 && st.st_size > 0;
}

uint64_t fnv1a_file(const std::string& p) {
    std::ifstream f(p, std::ios::binary);
    uint64_t h = 1469598103934665603ull;
    char buf[4096];
    while (f) {
        f.read(buf, sizeof buf);
        for (std::streamsize i = 0; i < f.gcount(); ++i) { h ^= (unsigned char)buf[i]; h *= 1099511628211ull; }
    }
    return h;
}

struct Derived {
    int es, oes, nw, cpr, rpi, a_lpw, b_lpw, lpt, ksb, ks, tm, tn, stage_bytes, lds, epi_bytes;
};

// Structural constraints of the template; the same conditions are static_asserts in the kernel.
int derive(const hrn_kernel_desc* d, Derived* o) {
    if (!d) return fail(HRN_E_BADPARAM, "null descriptor");
    if (d->dtype != HRN_DT_F16 && d->dtype != HRN_DT_U8S8) return fail(HRN_E_BADPARAM, "dtype %d", d->dtype);
    if (d->op != HRN_OP_GEMM && d->op != HRN_OP_CONV2D) return fail(HRN_E_BADPARAM, "op %d", d->op);
    if (d->bkb != 64 && d->bkb != 128 && d->bkb != 256) return fail(HRN_E_BADPARAM, "bkb %d not in {64,128,256}", d->bkb);
    if (d->mfma != 32 && d->mfma != 16) return fail(HRN_E_BADPARAM, "mfma %d not in {16,32}", d->mfma);
    if (d->wm < 1 || d->wn < 1 || d->wm * d->wn > 16) return fail(HRN_E_BADPARAM, "wave grid %dx%d", d->wm, d->wn);
    if (d->wm & (d->wm - 1)) return fail(HRN_E_BADPARAM, "wave rows %d must be a power of two", d->wm);
    if (d->bm < 16 || d->bn < 16 || d->bm > 512 || d->bn > 512) return fail(HRN_E_BADPARAM, "tile %dx%d", d->bm, d->bn);
    if (d->stages < 2 || d->stages > 5) return fail(HRN_E_BADPARAM, "stages %d not in 2..5", d->stages);
    if (d->swizzle < 0 || d->swizzle > 3) return fail(HRN_E_BADPARAM, "swizzle %d", d->swizzle);
    if (d->epilogue < 0 || d->epilogue > 2) return fail(HRN_E_BADPARAM, "epilogue %d", d->epilogue);
    if (d->sched < 0 || d->sched > 2) return fail(HRN_E_BADPARAM, "sched %d", d->sched);
    if (d->load_spread < 0 || d->load_spread > 3) return fail(HRN_E_BADPARAM, "load_spread %d", d->load_spread);
    if (d->waves_per_eu < 0 || d->waves_per_eu > 8) return fail(HRN_E_BADPARAM, "waves_per_eu %d", d->waves_per_eu);
    if (d->conv_window < 0 || d->conv_window > 1) return fail(HRN_E_BADPARAM, "conv_window %d", d->conv_window);
    if (d->conv_window && d->op != HRN_OP_CONV2D) return fail(HRN_E_BADPARAM, "conv_window is a conv2d option");
    if (d->persistent < 0 || d->persistent > 1) return fail(HRN_E_BADPARAM, "persistent %d", d->persistent);
    if (d->split_k < 0 || d->split_k > 1) return fail(HRN_E_BADPARAM, "split_k %d", d->split_k);
    if (d->persistent && (d->epilogue < 1 || d->conv_window || d->split_k))
        return fail(HRN_E_BADPARAM, "persistent needs the LDS-staged epilogue and neither conv_window nor split_k");
    if (d->split_k && d->conv_window) return fail(HRN_E_BADPARAM, "split_k uses the im2col load path, not conv_window");
    if (d->colsum < 0 || d->colsum > 1 || (d->colsum && d->dtype != HRN_DT_U8S8))
        return fail(HRN_E_BADPARAM, "colsum %d (caller-supplied column sums are an option of the u8s8 instances)", d->colsum);
    if (d->nt_store < 0 || d->nt_store > 1) return fail(HRN_E_BADPARAM, "nt_store %d (0 or 1)", d->nt_store);
    if (d->sched == 2 && (d->wm * d->wn != 8 || d->conv_window || d->persistent || d->split_k))
        return fail(HRN_E_BADPARAM, "sched 2 (two wave groups) needs 8 waves and neither conv_window, persistent nor split_k");
    Derived r;
    r.es = d->dtype == HRN_DT_F16 ? 2 : 1;
    r.oes = (d->dtype == HRN_DT_F16 && !d->split_k) ? 2 : 4;
    r.nw = d->wm * d->wn;
    r.cpr = d->bkb / 16;
    r.rpi = 64 / r.cpr;
    if ((!d->conv_window && (d->bm % r.rpi || (d->bm / r.rpi) % r.nw)) || d->bn % r.rpi || (d->bn / r.rpi) % r.nw)
        return fail(HRN_E_BADPARAM, "tile rows must split evenly into 1 KiB wave loads (bm %d bn %d, %d rows/load, %d waves)",
                    d->bm, d->bn, r.rpi, r.nw);
    r.a_lpw = d->conv_window ? 0 : d->bm / r.rpi / r.nw;
    r.b_lpw = d->bn / r.rpi / r.nw;
    r.lpt = r.a_lpw + r.b_lpw;
    r.ksb = d->mfma == 32 ? 32 : 64;
    r.ks = d->bkb / r.ksb;
    if (r.ks < 1) return fail(HRN_E_BADPARAM, "bkb %d is less than one k-step of mfma %d", d->bkb, d->mfma);
    if (d->persistent && r.ks % 2) return fail(HRN_E_BADPARAM, "persistent needs an even number of k-steps per tile (bkb %d, mfma %d)", d->bkb, d->mfma);
    if (d->bm % (d->wm * d->mfma) || d->bn % (d->wn * d->mfma))
        return fail(HRN_E_BADPARAM, "tile %dx%d not divisible by wave grid %dx%d x mfma %d", d->bm, d->bn, d->wm, d->wn, d->mfma);
    r.tm = d->bm / d->wm / d->mfma;
    r.tn = d->bn / d->wn / d->mfma;
    r.stage_bytes = ((d->conv_window ? 0 : d->bm) + d->bn) * d->bkb;
    r.lds = d->stages * r.stage_bytes;
    // epilogue region: the uint8 path's column sums (one row of bn sums per wave row) and, for the staged epilogue, the strips
    const int base = d->dtype == HRN_DT_U8S8 ? ((d->wm * d->bn * 4 + 1023) / 1024) * 1024 : 0;
    r.epi_bytes = base;
    if (d->epilogue >= 1) {
        const int esplit = d->epilogue == 2 ? 2 : 1;
        if (r.tn % esplit) return fail(HRN_E_BADPARAM, "epilogue 2 needs an even number of MFMA column tiles per wave (%d)", r.tn);
        const int sw = d->bn / d->wn / esplit;              // outputs per strip row
        r.epi_bytes = base + r.nw * d->mfma * (sw * r.oes + 16);
        if ((d->mfma * (sw * r.oes / 16)) % 64) return fail(HRN_E_BADPARAM, "staged epilogue needs mfma*strip_width*out_bytes/16 %% 64 == 0");
        if (d->persistent) {
            // the stages stay live during the epilogue, and its stores share the 6-bit vector-memory counter with the fetches
            r.lds += r.epi_bytes;
            const int stores = r.tm * esplit * (d->mfma * (sw * r.oes / 16) / 64);
            if ((d->stages - 2) * r.lpt + stores > 63)
                return fail(HRN_E_BADPARAM, "persistent: %d fetches + %d stores in flight exceed 63", (d->stages - 2) * r.lpt, stores);
        } else if (!d->conv_window) {
            r.lds = std::max(r.lds, r.epi_bytes);
        }
    }
    // (a conv_window instance keeps the epilogue region in its dynamic LDS, where the window was)
    if (r.lds > 163840) return fail(HRN_E_BADPARAM, "LDS %d > 163840", r.lds);
    if (d->swizzle && (r.cpr << (d->swizzle - 1)) > d->mfma)
        return fail(HRN_E_BADPARAM, "swizzle %d period %d exceeds mfma %d", d->swizzle, r.cpr << (d->swizzle - 1), d->mfma);
    if (d->op == HRN_OP_CONV2D && !d->conv_window && d->swizzle && (r.nw * r.rpi) % (r.cpr << (d->swizzle - 1)))
        return fail(HRN_E_BADPARAM, "conv: swizzle period must divide rows per load round");
    if ((d->stages - 1) * r.lpt > 63) return fail(HRN_E_BADPARAM, "too many loads in flight (%d)", (d->stages - 1) * r.lpt);
    const int acc = r.tm * r.tn * (d->mfma == 32 ? 16 : 4);
    if (acc > 256) return fail(HRN_E_BADPARAM, "accumulators %d > 256 registers per lane", acc);
    if (d->dtype == HRN_DT_U8S8 && !d->conv_window && d->wm * d->bn * 4 > d->stages * r.stage_bytes)
        return fail(HRN_E_BADPARAM, "LDS stages too small for the column sums");
    if (o) *o = r;
    return HRN_OK;
}

std::string desc_key(const hrn_kernel_desc* d, uint64_t srch) {
    char b[256];
    snprintf(b, sizeof b, "hrn_d%d_o%d_m%dn%dk%d_w%dx%d_t%d_s%d_z%d_e%d_p%d_c%d_r%d_k%d_i%d_l%d_b%d_n%d_%08x", d->dtype, d->op, d->bm, d->bn,
             d->bkb, d->wm, d->wn, d->mfma, d->stages, d->swizzle, d->epilogue, d->waves_per_eu, d->conv_window,
             d->persistent, d->split_k, d->sched, d->load_spread, d->colsum, d->nt_store, (unsigned)(srch ^ (srch >> 32)));
    return b;
}

int parse_remark(const std::string& log, const char* tag) {
    size_t p = log.find(tag);
    if (p == std::string::npos) return -1;
    return atoi(log.c_str() + p + strlen(tag));
}

int run_hipcc(const std::vector<std::string>& args, const std::string& log_path, double timeout_s) {
    // posix_spawn, not fork: the calling process may own a multi-threaded HIP runtime, whose address space (device
    // mappings included) a forked child would duplicate; the spawned compiler starts from a clean image in its own
    // process group, with the log file as stdout and stderr
    std::vector<char*> argv;
    for (auto& a : args) argv.push_back(const_cast<char*>(a.c_str()));
    argv.push_back(nullptr);
    const int fd = open(log_path.c_str(), O_WRONLY | O_CREAT | O_TRUNC | O_CLOEXEC, 0644);
    posix_spawn_file_actions_t fa;
    posix_spawnattr_t at;
    posix_spawn_file_actions_init(&fa);
    posix_spawnattr_init(&at);
    if (fd >= 0) {
        posix_spawn_file_actions_adddup2(&fa, fd, 1);
        posix_spawn_file_actions_adddup2(&fa, fd, 2);
    }
    posix_spawnattr_setflags(&at, POSIX_SPAWN_SETPGROUP);
    posix_spawnattr_setpgroup(&at, 0);
    pid_t pid = -1;
    const int sp = posix_spawnp(&pid, argv[0], &fa, &at, argv.data(), environ);
    posix_spawn_file_actions_destroy(&fa);
    posix_spawnattr_destroy(&at);
    if (sp != 0) { if (fd >= 0) close(fd); return fail(HRN_E_BUILD, "cannot start %s: %s", argv[0], strerror(sp)); }
    if (fd >= 0) close(fd);
    auto t0 = std::chrono::steady_clock::now();
    int status = 0;
    for (;;) {
        pid_t r = waitpid(pid, &status, WNOHANG);
        if (r == pid) break;
        if (r < 0) return fail(HRN_E_BUILD, "waitpid failed");
        double el = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        if (timeout_s > 0 && el > timeout_s) {
            kill(-pid, SIGKILL);
            kill(pid, SIGKILL);
            waitpid(pid, &status, 0);
            return fail(HRN_E_TIMEOUT, "hipcc exceeded %.1f s", timeout_s);
        }
        std::this_thread::sleep_for(std::chrono::milliseconds(20));
    }
    if (!WIFEXITED(status) || WEXITSTATUS(status) != 0) {
        std::ifstream f(log_path);
        std::stringstream ss;
        ss << f.rdbuf();
        std::string s = ss.str();
        if (s.size() > 1500) s = s.substr(0, 1500);
        return fail(HRN_E_BUILD, "hipcc failed (status %d): %s", status, s.c_str());
    }
    return HRN_OK;
}

int compile_desc(const hrn_kernel_desc* d, double timeout_s, std::string* out_path) {
    Derived dv;
    int rc = derive(d, &dv);
    if (rc) return rc;
    const std::string src = kernel_source();
    if (!file_exists(src)) return fail(HRN_E_BUILD, "kernel template not found: %s", src.c_str());
    const std::string dir = cache_dir();
    mkdir(dir.c_str(), 0755);
    // extra compiler flags (e.g. -D switches of the template under study) are part of the instance's identity
    const std::string extra = env_or("HRN_HIPCC_FLAGS", "");
    uint64_t srch = fnv1a_file(src);
    for (unsigned char ch : extra) { srch ^= ch; srch *= 1099511628211ull; }
    const std::string key = desc_key(d, srch);
    const std::string co = dir + "/" + key + ".hsaco";
    const std::string info = dir + "/" + key + ".info";
    *out_path = co;
    if (file_exists(co) && file_exists(info)) return HRN_OK;

    char tmp[64];
    snprintf(tmp, sizeof tmp, ".tmp%d_%lx", (int)getpid(), (unsigned long)pthread_self());
    const std::string co_tmp = co + tmp, log = dir + "/" + key + tmp + ".log";
    std::vector<std::string> args = {env_or("HRN_HIPCC", "/opt/rocm/bin/hipcc"),
                                     "--offload-arch=gfx950", "-O3", "--genco", "-std=c++17",
                                     "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                                     "-Rpass-analysis=kernel-resource-usage"};
    auto def = [&](const char* n, int v) { args.push_back(std::string("-D") + n + "=" + std::to_string(v)); };
    def("HRN_DTYPE", d->dtype); def("HRN_OP", d->op); def("HRN_BM", d->bm); def("HRN_BN", d->bn);
    def("HRN_BKB", d->bkb); def("HRN_WM", d->wm); def("HRN_WN", d->wn); def("HRN_MFMA", d->mfma);
    def("HRN_STAGES", d->stages); def("HRN_SWZ", d->swizzle); def("HRN_EPI", d->epilogue);
    def("HRN_WPE", d->waves_per_eu);
    def("HRN_CONVWIN", d->conv_window);
    def("HRN_PERSIST", d->persistent);
    def("HRN_SPLITK", d->split_k);
    def("HRN_SCHED", d->sched);
    def("HRN_LSPREAD", d->load_spread);
    def("HRN_COLSUM", d->colsum);
    def("HRN_NTSTORE", d->nt_store);
    {
        std::stringstream es(extra);
        std::string tok;
        while (es >> tok) args.push_back(tok);
    }
    args.push_back(src);
    args.push_back("-o");
    args.push_back(co_tmp);
    rc = run_hipcc(args, log, timeout_s);
    if (rc) { unlink(co_tmp.c_str()); unlink(log.c_str()); return rc; }

    std::ifstream lf(log);
    std::stringstream ss;
    ss << lf.rdbuf();
    const std::string ls = ss.str();
    const std::string info_tmp = info + tmp;
    {
        std::ofstream o(info_tmp);
        o << "vgprs " << parse_remark(ls, " VGPRs: ") << "\n"
          << "agprs " << parse_remark(ls, "AGPRs: ") << "\n"
          << "sgprs " << parse_remark(ls, "TotalSGPRs: ") << "\n"
          << "scratch " << parse_remark(ls, "ScratchSize [bytes/lane]: ") << "\n"
          << "occupancy " << parse_remark(ls, "Occupancy [waves/SIMD]: ") << "\n"
          << "lds " << parse_remark(ls, "LDS Size [bytes/block]: ") << "\n";
    }
    unlink(log.c_str());
    if (rename(co_tmp.c_str(), co.c_str()) != 0) return fail(HRN_E_BUILD, "rename %s failed", co.c_str());
    rename(info_tmp.c_str(), info.c_str());
    return HRN_OK;
}

void read_info(const std::string& path, hrn_kernel_info* o) {
    std::ifstream f(path);
    std::string k;
    int v;
    while (f >> k >> v) {
        if (k == "vgprs") o->vgprs = v;
        else if (k == "agprs") o->agprs = v;
        else if (k == "sgprs") o->sgprs = v;
        else if (k == "scratch") o->scratch_bytes = v;
        else if (k == "occupancy") o->occupancy = v;
        else if (k == "lds") o->lds_bytes = v;
    }
}

// What one launch consists of: the template kernel and, for a split-K instance, the pass that adds the K slices.
struct LaunchPlan {
    HrnKArgs k;
    unsigned grid, dyn_lds;
    int split;                 // K slices the grid covers (1 = the kernel writes C itself)
    void* C;                   // the caller's output
    int32_t ldc;
    int64_t stride_c;
};

int64_t splitk_bytes(const hrn_problem* p, int split) { return (int64_t)split * p->batch * p->m * p->n * 4; }

// k-tiles per slice and the number of non-empty slices for a requested split
void split_shape(const hrn_kernel_desc& d, const hrn_problem* p, int* kt_per_slice, int* split) {
    const int es = d.dtype == HRN_DT_F16 ? 2 : 1;
    const int kt_all = (int)(((int64_t)p->k * es + d.bkb - 1) / d.bkb);
    const int want = std::max(1, std::min(p->split_k, kt_all));
    *kt_per_slice = (kt_all + want - 1) / want;
    *split = (kt_all + *kt_per_slice - 1) / *kt_per_slice;
}

int fill_args(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* workspace,
              size_t workspace_bytes, LaunchPlan* plan) {
    HrnKArgs* k = &plan->k;
    plan->dyn_lds = 0;
    plan->split = 1;
    if (!mod || !p || !A || !B || !C) return fail(HRN_E_BADPARAM, "null argument");
    const hrn_kernel_desc& d = mod->desc;
    if (p->op != d.op) return fail(HRN_E_BADPARAM, "problem op %d does not match module op %d", p->op, d.op);
    const int es = d.dtype == HRN_DT_F16 ? 2 : 1;
    const int oes = d.dtype == HRN_DT_F16 ? 2 : 4;     // bytes of an element of the caller's C
    memset(k, 0, sizeof *k);
    k->A = A; k->B = B; k->C = C;
    if (p->m <= 0 || p->n <= 0 || p->k <= 0 || p->batch <= 0) return fail(HRN_E_BADPARAM, "empty problem");
    if ((int64_t)p->k * es % 16) return fail(HRN_E_BADPARAM, "K*%d must be a multiple of 16 bytes", es);
    if (p->n % 4) return fail(HRN_E_BADPARAM, "N must be a multiple of 4");
    k->M = p->m; k->N = p->n; k->K = p->k;
    k->lda = p->lda; k->ldb = p->ldb; k->ldc = p->ldc;
    k->sA = p->stride_a; k->sB = p->stride_b; k->sC = p->stride_c;
    k->batch = p->batch;
    k->split = 1;
    if (d.colsum) {
        if (!p->bsum || ((uintptr_t)p->bsum % 16))
            return fail(HRN_E_BADPARAM, "a colsum instance needs hrn_problem.bsum: batch x n int32 column sums of B (hrn_colsum_s8), 16-byte aligned");
        k->bsum = p->bsum;
    }
    if ((int64_t)p->ldb * es % 16 || p->ldb < p->k) return fail(HRN_E_BADPARAM, "ldb %d", p->ldb);
    if (p->ldc % 4 || p->ldc < p->n) return fail(HRN_E_BADPARAM, "ldc %d", p->ldc);
    if (d.epilogue >= 1 && !d.split_k && (((int64_t)p->ldc * oes) % 16 || ((uintptr_t)C % 16) || ((int64_t)p->stride_c * oes) % 16))
        return fail(HRN_E_BADPARAM, "the LDS-staged epilogue stores 16 bytes per lane: C, ldc and stride_c must be 16-byte aligned");
    if ((int64_t)p->n * p->ldb * es >= (1ll << 31)) return fail(HRN_E_BADPARAM, "B operand exceeds 2 GiB per batch entry");
    if (d.op == HRN_OP_GEMM) {
        if ((int64_t)p->lda * es % 16 || p->lda < p->k) return fail(HRN_E_BADPARAM, "lda %d", p->lda);
        if ((int64_t)p->m * p->lda * es >= (1ll << 31)) return fail(HRN_E_BADPARAM, "A operand exceeds 2 GiB per batch entry");
    } else {
        if (p->batch != 1) return fail(HRN_E_BADPARAM, "conv batch is the image count");
        if (p->cstride < 1 || p->cdil < 1 || p->cpad < 0 || p->cstride_w < 1 || p->cdil_w < 1 || p->cpad_w < 0)
            return fail(HRN_E_BADPARAM, "conv stride/pad/dilation (height %d/%d/%d, width %d/%d/%d)", p->cstride, p->cpad,
                        p->cdil, p->cstride_w, p->cpad_w, p->cdil_w);
        const int ho = (p->ch - ((p->kh - 1) * p->cdil + 1) + 2 * p->cpad) / p->cstride + 1;
        const int wo = (p->cw - ((p->kw - 1) * p->cdil_w + 1) + 2 * p->cpad_w) / p->cstride_w + 1;
        if (ho <= 0 || wo <= 0) return fail(HRN_E_BADPARAM, "conv output is empty");
        if (p->m != p->cn * ho * wo || p->n != p->co || p->k != p->kh * p->kw * p->ci)
            return fail(HRN_E_BADPARAM, "conv GEMM view (m,n,k)=(%d,%d,%d) inconsistent with the image shape", p->m, p->n, p->k);
        if ((p->ci * es) % 16) return fail(HRN_E_BADPARAM, "CI*%d must be a multiple of 16 bytes", es);
        if ((int64_t)p->cn * p->ch * p->cw * p->ci * es >= (1ll << 31)) return fail(HRN_E_BADPARAM, "input exceeds 2 GiB");
        k->H = p->ch; k->W = p->cw; k->CI = p->ci; k->HO = ho; k->WO = wo; k->KH = p->kh; k->KW = p->kw;
        k->cstride = p->cstride; k->cpad = p->cpad; k->cdil = p->cdil;
        k->cstride_w = p->cstride_w; k->cpad_w = p->cpad_w; k->cdil_w = p->cdil_w;
        if (d.conv_window) {
            if (p->cstride != 1 || p->cdil != 1 || p->cstride_w != 1 || p->cdil_w != 1 || ho != p->ch || wo != p->cw)
                return fail(HRN_E_BADPARAM, "conv_window needs stride 1, dilation 1 and 'same' padding");
            if ((p->ci * es) % d.bkb) return fail(HRN_E_BADPARAM, "conv_window needs CI*%d to be a multiple of bkb %d", es, d.bkb);
            if (p->kh * p->kw > 32) return fail(HRN_E_BADPARAM, "conv_window supports at most 32 filter taps");
            const int64_t rows = d.bm + 2 * ((int64_t)p->cpad * p->cw + p->cpad_w);
            const int64_t instr = (rows * (p->ci * es / 16) + 63) / 64;
            // dynamic LDS: the window, reused by the epilogue region (column sums, strips) once the last tap is read
            const int64_t dyn = std::max<int64_t>(instr * 1024, mod->epi_bytes);
            if (dyn + mod->info.lds_bytes > 163840)
                return fail(HRN_E_BADPARAM, "conv_window: window of %lld bytes + %d static LDS exceeds 163840", (long long)dyn, mod->info.lds_bytes);
            plan->dyn_lds = (unsigned)dyn;
        }
    }
    k->tiles_m = (p->m + d.bm - 1) / d.bm;
    k->tiles_n = (p->n + d.bn - 1) / d.bn;
    k->group_m = p->group_m > 0 ? p->group_m : 8;
    int64_t total = (int64_t)k->tiles_m * k->tiles_n * p->batch;
    plan->C = C; plan->ldc = p->ldc; plan->stride_c = p->stride_c;
    if (d.split_k) {
        // the kernel writes raw partial sums, slice by slice, into the workspace; hrn's reduction pass writes C
        if (p->split_k < 1) return fail(HRN_E_BADPARAM, "a split_k instance needs problem.split_k >= 1 (got %d)", p->split_k);
        int kps, split;
        split_shape(d, p, &kps, &split);
        const int64_t need = splitk_bytes(p, split);
        if (!workspace || ((uintptr_t)workspace % 16)) return fail(HRN_E_BADPARAM, "split_k needs a 16-byte aligned device workspace");
        if ((int64_t)workspace_bytes < need)
            return fail(HRN_E_BADPARAM, "split_k workspace of %zu bytes is too small: %d slices x %d x %d x %d x 4 = %lld", workspace_bytes,
                        split, p->batch, p->m, p->n, (long long)need);
        if ((int64_t)p->m * p->n * 4 >= (1ll << 31)) return fail(HRN_E_BADPARAM, "split_k: one slice of C exceeds 2 GiB");
        k->C = workspace; k->ldc = p->n; k->sC = (int64_t)p->m * p->n;
        k->split = split; k->kt_per_slice = kps;
        plan->split = split;
        total *= split;
    } else if (p->split_k > 1) {
        return fail(HRN_E_BADPARAM, "problem.split_k = %d but the instance was not built with split_k", p->split_k);
    }
    if (total <= 0 || total >= (1ll << 31)) return fail(HRN_E_BADPARAM, "grid size");
    plan->grid = (unsigned)total;
    if (d.persistent) {
        if ((int64_t)p->n * oes % 16) return fail(HRN_E_BADPARAM, "persistent instances store whole 16-byte chunks: N*%d must be a multiple of 16", oes);
        if ((int64_t)p->m * p->ldc * oes >= (1ll << 31)) return fail(HRN_E_BADPARAM, "persistent: C exceeds 2 GiB per batch entry");
        int64_t g = std::min<int64_t>(total, mod->persist_grid);
        if (const char* e = getenv("HRN_PERSIST_GRID")) {      // override of the number of workgroups (tuning / tests)
            const long v = atol(e);
            if (v >= 1) g = std::min<int64_t>(total, v);
        }
        if (g >= 8) g &= ~7ll;          // workgroup i runs on XCD i % 8: keep tile t on XCD t % 8 in every round
        plan->grid = (unsigned)g;
    }
    return HRN_OK;
}

// Adds the K slices of a split-K launch: C[b,m,n] = sum_z ws[z,b,m,n], converted to the output type.  One lane per
// 4 consecutive n (N is a multiple of 4): 16-byte reads, 8- or 16-byte writes.
typedef float rv4f __attribute__((ext_vector_type(4)));
typedef int rv4i __attribute__((ext_vector_type(4)));
typedef _Float16 rv4h __attribute__((ext_vector_type(4)));

template <bool F16>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const void* __restrict__ ws, void* __restrict__ C, int split,
                                                            int batch, int M, int N, int ldc, int64_t stride_c) {
    const int64_t n4 = N / 4;
    const int64_t count = (int64_t)batch * M * n4;
    const int64_t slice = (int64_t)batch * M * N;           // elements of one slice
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t bm = i / n4;
        const int q = (int)(i - bm * n4);
        const int b = (int)(bm / M), m = (int)(bm - (int64_t)b * M);
        const int64_t src = bm * N + (int64_t)q * 4;
        const int64_t dst = (int64_t)b * stride_c + (int64_t)m * ldc + (int64_t)q * 4;
        if constexpr (F16) {
            rv4f acc = *(const rv4f*)((const float*)ws + src);
            for (int z = 1; z < split; ++z) acc += *(const rv4f*)((const float*)ws + z * slice + src);
            rv4h o;
            for (int r = 0; r < 4; ++r) o[r] = (_Float16)acc[r];
            *(rv4h*)((_Float16*)C + dst) = o;
        } else {
            rv4i acc = *(const rv4i*)((const int*)ws + src);
            for (int z = 1; z < split; ++z) acc += *(const rv4i*)((const int*)ws + z * slice + src);
            *(rv4i*)((int*)C + dst) = acc;
        }
    }
}

int run_plan(const hrn_module* mod, const hrn_problem* p, const LaunchPlan& plan, void* workspace, hipStream_t st) {
    size_t sz = sizeof plan.k;
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, (void*)&plan.k, HIP_LAUNCH_PARAM_BUFFER_SIZE, &sz, HIP_LAUNCH_PARAM_END};
    HIP_TRY(hipModuleLaunchKernel(mod->fn, plan.grid, 1, 1, (unsigned)mod->info.threads, 1, 1, plan.dyn_lds, st, nullptr, extra));
    if (mod->desc.split_k) {
        const int64_t count = (int64_t)p->batch * p->m * (p->n / 4);
        const unsigned blocks = (unsigned)std::min<int64_t>((count + 255) / 256, 256 * 32);
        if (mod->desc.dtype == HRN_DT_F16)
            splitk_reduce_kernel<true><<<blocks, 256, 0, st>>>(workspace, plan.C, plan.split, p->batch, p->m, p->n, plan.ldc, plan.stride_c);
        else
            splitk_reduce_kernel<false><<<blocks, 256, 0, st>>>(workspace, plan.C, plan.split, p->batch, p->m, p->n, plan.ldc, plan.stride_c);
        HIP_TRY(hipGetLastError());
    }
    return HRN_OK;
}

// ---- split-K workspace that needs no allocation --------------------------------------------------------------
// Device memory every GPU the library runs on holds until the process ends; hrn_launch_splitk_static keeps the
// partial sums of a split-K launch here instead of in a caller-owned workspace.  In host code the array's name is
// only a stand-in: its device address is looked up once per device and that pointer is what kernels get.
static __device__ __align__(256) unsigned char scratch[HRN_STATIC_WORKSPACE_BYTES];

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];
bool g_scratch_known[kMaxDevices];
hipEvent_t g_scratch_done[kMaxDevices];      // recorded behind the last launch that used the device's workspace ...
hipStream_t g_scratch_stream[kMaxDevices];   // ... on this stream
bool g_scratch_used[kMaxDevices];
std::mutex g_scratch_mutex;

// Address of `scratch` on the current device and the event that orders its users: set up on the first call per
// device (hrn_build does it for split-K instances, so that a launch - possibly under graph capture - finds it done).
int static_scratch(void** out, int* dev_out = nullptr) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(HRN_E_BADPARAM, "device index %d", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_known[dev]) {
        void* ptr = nullptr;
        HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fail(HRN_E_LAUNCH, "hipGetSymbolAddress returned a null address");
        HIP_TRY(hipEventCreateWithFlags(&g_scratch_done[dev], hipEventDisableTiming));
        g_scratch_ptr[dev] = ptr;
        g_scratch_known[dev] = true;
    }
    *out = g_scratch_ptr[dev];
    if (dev_out) *dev_out = dev;
    return HRN_OK;
}

int launch(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream) {
    LaunchPlan plan;
    int rc = fill_args(mod, p, A, B, C, p ? p->workspace : nullptr, p ? p->workspace_bytes : 0, &plan);
    if (rc) return rc;
    return run_plan(mod, p, plan, p->workspace, (hipStream_t)stream);
}

// ---- column sums of an int8 matrix ------------------------------------------------------------
// out[b][n] = sum_k B[b][n][k]: one wave per row, 16 bytes per lane and step, v_dot4 against ones, wave reduction.
__global__ void __launch_bounds__(256) colsum_s8_kernel(const signed char* __restrict__ B, int* __restrict__ out, int batch, int N,
                                                        int K, int ldb, int64_t stride_b) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (int64_t)batch * N) return;
    const int b = (int)(row / N), n = (int)(row - (int64_t)b * N);
    const signed char* src = B + (int64_t)b * stride_b + (int64_t)n * ldb;
    int s = 0;
    for (int k = lane * 16; k < K; k += 64 * 16) {          // K is a multiple of 16
        const rv4i v = *(const rv4i*)(src + k);
        s = __builtin_amdgcn_sdot4(v.x, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(v.y, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(v.z, 0x01010101, s, false);
        s = __builtin_amdgcn_sdot4(v.w, 0x01010101, s, false);
    }
    for (int d = 1; d < 64; d <<= 1) s += __shfl_xor(s, d, 64);
    if (lane == 0) out[row] = s;
}

// ---- roofline probes -----------------------------------------------------------------------
typedef int pv4i __attribute__((ext_vector_type(4)));
typedef _Float16 pv8h __attribute__((ext_vector_type(8)));
typedef float pv16f __attribute__((ext_vector_type(16)));
typedef float pv4f __attribute__((ext_vector_type(4)));
typedef int pv16i __attribute__((ext_vector_type(16)));

// KIND 0: f16 32x32x16, 1: f16 16x16x32, 2: i8 32x32x32, 3: i8 16x16x64; 4 independent accumulators
template <int KIND>
__global__ void __launch_bounds__(256) probe_mfma_kernel(float* sink, int iters, int random_operands) {
    pv4i a = {(int)threadIdx.x, 1, 2, 3}, b = {4, 5, 6, (int)blockIdx.x};
    if (random_operands) {
        // operands with the bit statistics of real data: fp16 values of magnitude ~2^-3..2^0 with random
        // sign and mantissa, or uniformly random bytes (data-dependent switching power is part of the roofline)
        uint32_t h = (threadIdx.x * 2654435761u) ^ (blockIdx.x * 40503u + 0x9e3779b9u);
        for (int r = 0; r < 4; ++r) {
            uint32_t w[2];
            for (int q = 0; q < 2; ++q) {
                h = h * 1664525u + 1013904223u;
                uint32_t x = h ^ (h >> 15);
                if (KIND < 2) {   // two halves: sign(1) exp in {12,13,14,15} mantissa(10)
                    uint32_t lo = (x & 0x83ffu) | ((12u + ((x >> 10) & 3u)) << 10);
                    uint32_t hi = ((x >> 16) & 0x83ffu) | ((12u + ((x >> 26) & 3u)) << 10);
                    w[q] = lo | (hi << 16);
                } else {
                    w[q] = x;
                }
            }
            a[r] = (int)w[0];
            b[r] = (int)w[1];
        }
    }
    if constexpr (KIND == 0 || KIND == 2) {
        using acc_t = typename std::conditional<KIND == 0, pv16f, pv16i>::type;
        acc_t c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
        for (int i = 0; i < iters; ++i) {
            if constexpr (KIND == 0) {
                c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pv8h, a), __builtin_bit_cast(pv8h, b), c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pv8h, a), __builtin_bit_cast(pv8h, b), c1, 0, 0, 0);
                c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pv8h, a), __builtin_bit_cast(pv8h, b), c2, 0, 0, 0);
                c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pv8h, a), __builtin_bit_cast(pv8h, b), c3, 0, 0, 0);
            } else {
                c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c1, 0, 0, 0);
                c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c2, 0, 0, 0);
                c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c3, 0, 0, 0);
            }
        }
        float s = 0;
        for (int r = 0; r < 16; ++r) s += (float)(c0[r] + c1[r] + c2[r] + c3[r]);
        asm volatile("" ::"v"(s));   // keeps the accumulators live; nothing is stored
        (void)sink;
    } else {
        using acc_t = typename std::conditional<KIND == 1, pv4f, pv4i>::type;
        acc_t c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
        for (int i = 0; i < iters; ++i) {
            if constexpr (KIND == 1) {
                c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pv8h, a), __builtin_bit_cast(pv8h, b), c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pv8h, a), __builtin_bit_cast(pv8h, b), c1, 0, 0, 0);
                c2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pv8h, a), __builtin_bit_cast(pv8h, b), c2, 0, 0, 0);
                c3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pv8h, a), __builtin_bit_cast(pv8h, b), c3, 0, 0, 0);
            } else {
                c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c1, 0, 0, 0);
                c2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c2, 0, 0, 0);
                c3 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c3, 0, 0, 0);
            }
        }
        float s = 0;
        for (int r = 0; r < 4; ++r) s += (float)(c0[r] + c1[r] + c2[r] + c3[r]);
        asm volatile("" ::"v"(s));   // keeps the accumulators live; nothing is stored
        (void)sink;
    }
}

__global__ void __launch_bounds__(256) probe_copy_kernel(const pv4i* __restrict__ src, pv4i* __restrict__ dst, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + 3 * stride < n16; i += 4 * stride) {      // four independent 16-byte loads in flight per lane
        const pv4i v0 = src[i], v1 = src[i + stride], v2 = src[i + 2 * stride], v3 = src[i + 3 * stride];
        dst[i] = v0; dst[i + stride] = v1; dst[i + 2 * stride] = v2; dst[i + 3 * stride] = v3;
    }
    for (; i < n16; i += stride) dst[i] = src[i];
}

// One lane per row: copies `c` elements of ES bytes and zero-fills up to `cp` elements, writing whole 16-byte words.
template <int ES>
__global__ void __launch_bounds__(256) pad_rows_kernel(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst,
                                                       size_t rows, int c, int cp) {
    const size_t row = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows) return;
    const unsigned char* in = src + row * (size_t)c * ES;
    pv4i* out = (pv4i*)(dst + row * (size_t)cp * ES);
    const int words = cp * ES / 16, live = c * ES;
    for (int w = 0; w < words; ++w) {
        unsigned int q[4] = {0u, 0u, 0u, 0u};
        for (int b = 0; b < 16; b += ES) {
            const int at = w * 16 + b;
            if (at < live) {
                const unsigned int v = ES == 2 ? (unsigned int)*(const unsigned short*)(in + at) : (unsigned int)in[at];
                q[b / 4] |= v << (8 * (b % 4));
            }
        }
        out[w] = pv4i{(int)q[0], (int)q[1], (int)q[2], (int)q[3]};
    }
}

// Affine gather (hrn_gather_nd): one lane per 16-byte piece of the innermost dst dimension (VEC) or per element.
template <int ES, bool VEC, typename IDX>
__global__ void __launch_bounds__(256) gather_nd_kernel(const hrn_gather g, const char* __restrict__ src,
                                                        const _Float16* __restrict__ aux, char* __restrict__ dst, IDX total) {
    const IDX t = (IDX)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    constexpr int V = VEC ? 16 / ES : 1;
    // 32-bit index arithmetic when the launch is small enough for it (IDX = uint32_t: the host has checked that every
    // extent, numerator and coordinate fits), 64-bit otherwise; the element offsets are 64-bit in both cases
    using CO = typename std::conditional<sizeof(IDX) == 4, int32_t, int64_t>::type;
    CO idx[HRN_GATHER_DIMS];
    IDX rem = t;
#pragma unroll
    for (int d = HRN_GATHER_DIMS - 1; d >= 0; --d) {
        idx[d] = 0;
        if (d < g.ndim) {
            const IDX ext = (IDX)(d == g.ndim - 1 ? g.dst_dim[d] / V : g.dst_dim[d]);
            const IDX q = rem / ext;
            idx[d] = (CO)(rem - q * ext) * (d == g.ndim - 1 ? V : 1);
            rem = q;
        }
    }
    int64_t doff = 0;
    bool live = true;
#pragma unroll
    for (int d = 0; d < HRN_GATHER_DIMS; ++d)
        if (d < g.ndim) {
            doff += (int64_t)idx[d] * g.dst_stride[d];
            live = live && idx[d] < (CO)g.dst_live[d];
        }
    int64_t soff = 0;
#pragma unroll
    for (int s = 0; s < HRN_GATHER_DIMS; ++s)
        if (s < g.nsrc) {
            CO num = (CO)g.add[s];
#pragma unroll
            for (int d = 0; d < HRN_GATHER_DIMS; ++d)
                if (d < g.ndim) num += (CO)g.mul[s][d] * idx[d];
            const CO dv = (CO)g.div[s];
            const CO q = dv == 1 ? num : num / dv;
            live = live && num >= 0 && q * dv == num && q < (CO)g.src_dim[s];
            soff += (int64_t)q * g.src_stride[s];
        }
    if constexpr (VEC) {
        pv4i v = {0, 0, 0, 0};
        if (live) {
            v = *(const pv4i*)(src + soff * ES);
            if (g.op == HRN_GATHER_CENTER_SQUARE) {
                const pv4i y = *(const pv4i*)((const char*)aux + soff * ES);
                _Float16 h[8], m[8];
                __builtin_memcpy(h, &v, 16);
                __builtin_memcpy(m, &y, 16);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const _Float16 dlt = h[e] - m[e];
                    h[e] = dlt * dlt;
                }
                __builtin_memcpy(&v, h, 16);
            }
        }
        *(pv4i*)(dst + doff * ES) = v;
    } else if constexpr (ES == 2) {
        unsigned short v = 0;
        if (live) {
            v = *(const unsigned short*)(src + soff * 2);
            if (g.op == HRN_GATHER_CENTER_SQUARE) {
                const _Float16 dlt = __builtin_bit_cast(_Float16, v) - aux[soff];
                v = __builtin_bit_cast(unsigned short, (_Float16)(dlt * dlt));
            }
        }
        *(unsigned short*)(dst + doff * 2) = v;
    } else if constexpr (ES == 1) {
        dst[doff] = live ? src[soff] : (char)0;
    } else {
        *(unsigned int*)(dst + doff * 4) = live ? *(const unsigned int*)(src + soff * 4) : 0u;
    }
}

// Batched transpose src[b][r][c] -> dst[b][c][r'] with r' padded to rp >= rows (zeros), through a 64x64 LDS tile so that
// both the reads (along c) and the writes (along r) are contiguous.  blockDim = (64, 4).
template <typename T>
__global__ void __launch_bounds__(256) transpose_pad_kernel(const T* __restrict__ src, T* __restrict__ dst,
                                                            int rows, int cols, int rp) {
    __shared__ T tile[64][65];
    const size_t b = blockIdx.z;
    const T* in = src + b * (size_t)rows * cols;
    T* out = dst + b * (size_t)cols * rp;
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    for (int i = threadIdx.y; i < 64; i += 4) {
        const int r = r0 + i, c = c0 + threadIdx.x;
        tile[i][threadIdx.x] = (r < rows && c < cols) ? in[(size_t)r * cols + c] : (T)0;
    }
    __syncthreads();
    for (int i = threadIdx.y; i < 64; i += 4) {
        const int c = c0 + i, r = r0 + threadIdx.x;
        if (c < cols && r < rp) out[(size_t)c * rp + r] = tile[threadIdx.x][i];
    }
}

// streams `n16` 16-byte words through every lane without storing anything: the read-only counterpart of the copy probe
__global__ void __launch_bounds__(256) probe_read_kernel(const pv4i* __restrict__ src, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    pv4i acc = {0, 0, 0, 0};
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const pv4i v0 = src[i], v1 = src[i + stride], v2 = src[i + 2 * stride], v3 = src[i + 3 * stride];
        acc |= v0 | v1 | v2 | v3;
    }
    for (; i < n16; i += stride) acc |= src[i];
    const int keep = acc.x | acc.y | acc.z | acc.w;
    asm volatile("" ::"v"(keep));   // keeps the loads live; nothing is stored
}

// reads `r16` 16-byte words and writes `w16` of them (the words it read, as far as they go): the plainest kernel that
// moves a workload's algorithmic bytes
__global__ void __launch_bounds__(256) probe_traffic_kernel(const pv4i* __restrict__ src, size_t r16, pv4i* __restrict__ dst, size_t w16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t n = r16 > w16 ? r16 : w16;
    pv4i acc = {0, 0, 0, 0};
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += 2 * stride) {
        const size_t j = i + stride;
        pv4i v0 = {0, 0, 0, 0}, v1 = {0, 0, 0, 0};
        if (i < r16) v0 = src[i];
        if (j < r16) v1 = src[j];
        if (i < w16) dst[i] = v0; else acc |= v0;
        if (j < w16) dst[j] = v1; else acc |= v1;
    }
    const int keep = acc.x | acc.y | acc.z | acc.w;
    asm volatile("" ::"v"(keep));
}

// does nothing: what the device needs to start and retire one dispatch of `grid` workgroups
__global__ void __launch_bounds__(256) probe_empty_kernel(int* sink) {
    if (sink && threadIdx.x == 0x7fffffff) *sink = 0;
}

}  // namespace

extern "C" {

int hrn_colsum_s8(const void* B, void* bsum, int batch, int n, int k, int ldb, int64_t stride_b, void* stream) {
    if (!B || !bsum || batch < 1 || n < 1 || k < 16 || k % 16 || ldb < k || ldb % 16 || ((uintptr_t)B % 16) || stride_b % 16)
        return fail(HRN_E_BADPARAM, "colsum_s8: batch %d, n %d, k %d, ldb %d (k and ldb multiples of 16, B 16-byte aligned)", batch, n, k, ldb);
    const int64_t rows = (int64_t)batch * n;
    if ((rows + 3) / 4 >= (1ll << 31)) return fail(HRN_E_BADPARAM, "colsum_s8: too many rows");
    colsum_s8_kernel<<<(unsigned)((rows + 3) / 4), 256, 0, (hipStream_t)stream>>>((const signed char*)B, (int*)bsum, batch, n, k, ldb, stride_b);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HRN_E_LAUNCH, "colsum_s8: %s", hipGetErrorString(e));
    return HRN_OK;
}

int hrn_pad_rows(const void* src, void* dst, size_t rows, int c, int cp, int elem_bytes, void* stream) {
    if (!src || !dst || c < 1 || cp < c || (elem_bytes != 1 && elem_bytes != 2) || (cp * elem_bytes) % 16 || rows > ((size_t)1 << 40))
        return fail(HRN_E_BADPARAM, "pad_rows: %d -> %d elements of %d bytes (the padded row must be whole 16-byte words)", c, cp, elem_bytes);
    if (rows == 0) return HRN_OK;
    const unsigned grid = (unsigned)((rows + 255) / 256);
    hipStream_t st = (hipStream_t)stream;
    if (elem_bytes == 2) pad_rows_kernel<2><<<grid, 256, 0, st>>>((const unsigned char*)src, (unsigned char*)dst, rows, c, cp);
    else pad_rows_kernel<1><<<grid, 256, 0, st>>>((const unsigned char*)src, (unsigned char*)dst, rows, c, cp);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HRN_E_LAUNCH, "pad_rows: %s", hipGetErrorString(e));
    return HRN_OK;
}

int hrn_transpose_pad(const void* src, void* dst, int batch, int rows, int cols, int rows_padded, int elem_bytes, void* stream) {
    if (!src || !dst || batch < 0 || rows < 1 || cols < 1 || rows_padded < rows || batch > 65535 ||
        (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4))
        return fail(HRN_E_BADPARAM, "transpose_pad: batch %d, %d x %d -> %d x %d, %d-byte elements", batch, rows, cols, cols, rows_padded, elem_bytes);
    if (batch == 0) return HRN_OK;
    const dim3 grid((cols + 63) / 64, (rows_padded + 63) / 64, batch), block(64, 4);
    if (grid.y > 65535) return fail(HRN_E_BADPARAM, "transpose_pad: %d rows are more than 65535 tiles", rows_padded);
    hipStream_t st = (hipStream_t)stream;
    if (elem_bytes == 1) transpose_pad_kernel<unsigned char><<<grid, block, 0, st>>>((const unsigned char*)src, (unsigned char*)dst, rows, cols, rows_padded);
    else if (elem_bytes == 2) transpose_pad_kernel<unsigned short><<<grid, block, 0, st>>>((const unsigned short*)src, (unsigned short*)dst, rows, cols, rows_padded);
    else transpose_pad_kernel<unsigned int><<<grid, block, 0, st>>>((const unsigned int*)src, (unsigned int*)dst, rows, cols, rows_padded);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HRN_E_LAUNCH, "transpose_pad: %s", hipGetErrorString(e));
    return HRN_OK;
}

int hrn_gather_nd(const hrn_gather* g, const void* src, const void* aux, void* dst, void* stream) {
    if (!g || !src || !dst) return fail(HRN_E_BADPARAM, "gather: null argument");
    const int nd = g->ndim, ns = g->nsrc, es = g->elem_bytes;
    if (nd < 1 || nd > HRN_GATHER_DIMS || ns < 1 || ns > HRN_GATHER_DIMS || (es != 1 && es != 2 && es != 4))
        return fail(HRN_E_BADPARAM, "gather: %d dst dimensions, %d source coordinates, %d-byte elements", nd, ns, es);
    if (g->op != HRN_GATHER_COPY && g->op != HRN_GATHER_CENTER_SQUARE)
        return fail(HRN_E_BADPARAM, "gather: unknown op %d", g->op);
    if (g->op == HRN_GATHER_CENTER_SQUARE && (es != 2 || !aux))
        return fail(HRN_E_BADPARAM, "gather: center-square takes fp16 elements and an aux tensor laid out like src");
    if (g->dst_stride[nd - 1] != 1) return fail(HRN_E_BADPARAM, "gather: the innermost dst dimension must have stride 1");
    // the largest dst and src offsets any index can reach; totals that overflow are refused
    long double total_ld = 1, dmax = 0, smax = 0;
    for (int d = 0; d < nd; ++d) {
        if (g->dst_dim[d] < 0 || g->dst_stride[d] < 0 || g->dst_live[d] < 0 || g->dst_live[d] > g->dst_dim[d])
            return fail(HRN_E_BADPARAM, "gather: dst dimension %d: extent %lld, stride %lld, live %lld", d, (long long)g->dst_dim[d],
                        (long long)g->dst_stride[d], (long long)g->dst_live[d]);
        total_ld *= (long double)g->dst_dim[d];
        dmax += (long double)(g->dst_dim[d] ? g->dst_dim[d] - 1 : 0) * (long double)g->dst_stride[d];
    }
    for (int s = 0; s < ns; ++s) {
        if (g->src_dim[s] < 1 || g->src_stride[s] < 0 || g->div[s] < 1)
            return fail(HRN_E_BADPARAM, "gather: source coordinate %d: extent %lld, stride %lld, divisor %lld", s, (long long)g->src_dim[s],
                        (long long)g->src_stride[s], (long long)g->div[s]);
        smax += (long double)(g->src_dim[s] - 1) * (long double)g->src_stride[s];
    }
    if (total_ld > 9.0e15L || dmax > 9.0e15L || smax > 9.0e15L) return fail(HRN_E_BADPARAM, "gather: extents too large");
    const int64_t total = (int64_t)total_ld;
    if (total == 0) return HRN_OK;
    // 16 bytes per lane when whole aligned pieces move along the innermost dimension
    const int V = 16 / es, d0 = nd - 1;
    bool vec = g->dst_dim[d0] % V == 0 && g->dst_live[d0] % V == 0 && ((uintptr_t)src % 16) == 0 && ((uintptr_t)dst % 16) == 0 &&
               (g->op != HRN_GATHER_CENTER_SQUARE || ((uintptr_t)aux % 16) == 0);
    for (int d = 0; d < d0 && vec; ++d) vec = g->dst_stride[d] % V == 0;
    int s0 = -1;
    for (int s = 0; s < ns && vec; ++s) {
        if (g->mul[s][d0] == 0) {
            vec = g->src_stride[s] % V == 0;
            continue;
        }
        vec = s0 < 0 && g->mul[s][d0] == 1 && g->div[s] == 1 && g->src_stride[s] == 1 && g->src_dim[s] % V == 0 && g->add[s] % V == 0;
        for (int d = 0; d < d0 && vec; ++d) vec = g->mul[s][d] % V == 0;
        s0 = s;
    }
    vec = vec && s0 >= 0;
    const int64_t lanes = vec ? total / V : total;
    const int64_t blocks = (lanes + 255) / 256;
    if (blocks > 0x7fffffffLL) return fail(HRN_E_BADPARAM, "gather: %lld elements are more than one launch covers", (long long)total);
    hipStream_t st = (hipStream_t)stream;
    const char* sp = (const char*)src;
    const _Float16* ap = (const _Float16*)aux;
    char* dp = (char*)dst;
    // 32-bit index arithmetic in the kernel needs every extent, divisor and reachable numerator below 2^31
    long double reach = 0;
    for (int sidx = 0; sidx < ns; ++sidx) {
        long double r = g->add[sidx] < 0 ? -(long double)g->add[sidx] : (long double)g->add[sidx];
        for (int d = 0; d < nd; ++d) {
            const long double m = g->mul[sidx][d] < 0 ? -(long double)g->mul[sidx][d] : (long double)g->mul[sidx][d];
            r += m * (long double)(g->dst_dim[d] ? g->dst_dim[d] - 1 : 0);
        }
        if (r > reach) reach = r;
        if ((long double)g->src_dim[sidx] > reach) reach = (long double)g->src_dim[sidx];
        if ((long double)g->div[sidx] > reach) reach = (long double)g->div[sidx];
    }
    const bool small = lanes < (1LL << 31) && total < (1LL << 31) && reach < 2.0e9L;
#define HRN_GATHER_LAUNCH(ES_, VEC_)                                                                                          \
    do {                                                                                                                      \
        if (small) gather_nd_kernel<ES_, VEC_, uint32_t><<<(unsigned)blocks, 256, 0, st>>>(*g, sp, ap, dp, (uint32_t)lanes);   \
        else gather_nd_kernel<ES_, VEC_, uint64_t><<<(unsigned)blocks, 256, 0, st>>>(*g, sp, ap, dp, (uint64_t)lanes);         \
    } while (0)
    if (es == 1) { if (vec) HRN_GATHER_LAUNCH(1, true); else HRN_GATHER_LAUNCH(1, false); }
    else if (es == 2) { if (vec) HRN_GATHER_LAUNCH(2, true); else HRN_GATHER_LAUNCH(2, false); }
    else { if (vec) HRN_GATHER_LAUNCH(4, true); else HRN_GATHER_LAUNCH(4, false); }
#undef HRN_GATHER_LAUNCH
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HRN_E_LAUNCH, "gather: %s", hipGetErrorString(e));
    return HRN_OK;
}

int hrn_probe_read(const void* src, size_t bytes, int repeat, double* gbs_out, void* stream) {
    if (!src || !gbs_out || bytes < 16 || bytes % 16 || repeat < 1) return fail(HRN_E_BADPARAM, "probe arguments");
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t pr;
    HIP_TRY(hipGetDeviceProperties(&pr, dev));
    hipStream_t st = (hipStream_t)stream;
    EventPair ev;
    HIP_TRY(ev.create());
    hipEvent_t e0 = ev.e0, e1 = ev.e1;
    const int grid = pr.multiProcessorCount * 16;
    probe_read_kernel<<<grid, 256, 0, st>>>((const pv4i*)src, bytes / 16);
    (void)hipEventRecord(e0, st);
    for (int i = 0; i < repeat; ++i) probe_read_kernel<<<grid, 256, 0, st>>>((const pv4i*)src, bytes / 16);
    (void)hipEventRecord(e1, st);
    hipError_t e = hipEventSynchronize(e1);
    float ms = 0;
    (void)hipEventElapsedTime(&ms, e0, e1);
    if (e != hipSuccess) return fail(HRN_E_LAUNCH, "probe: %s", hipGetErrorString(e));
    *gbs_out = (double)bytes * repeat / (ms * 1e-3) / 1e9;
    return HRN_OK;
}

int hrn_probe_traffic_cold(const void* src, size_t read_bytes, void* dst, size_t write_bytes, void* flush_buf,
                           size_t flush_bytes, int repeat, double* us_out, void* stream) {
    if (!src || !dst || !us_out || !flush_buf || read_bytes % 16 || write_bytes % 16 || (read_bytes == 0 && write_bytes == 0) ||
        repeat < 1 || flush_bytes < (64u << 20))
        return fail(HRN_E_BADPARAM, "probe arguments (16-byte multiples, flush buffer >= 64 MiB)");
    int dev = 0;
    hipDeviceProp_t pr;
    HIP_TRY(hipGetDevice(&dev));
    HIP_TRY(hipGetDeviceProperties(&pr, dev));
    hipStream_t st = (hipStream_t)stream;
    EventPair ev;
    HIP_TRY(ev.create());
    const size_t half16 = flush_bytes / 32;
    const int grid = pr.multiProcessorCount * 8;
    for (int r = 0; r < repeat; ++r) {
        // the same flush as hrn_time_cold: one half of the buffer streamed into the other
        probe_copy_kernel<<<pr.multiProcessorCount * 16, 256, 0, st>>>((const pv4i*)flush_buf, (pv4i*)flush_buf + half16, half16);
        (void)hipEventRecord(ev.e0, st);
        probe_traffic_kernel<<<grid, 256, 0, st>>>((const pv4i*)src, read_bytes / 16, (pv4i*)dst, write_bytes / 16);
        (void)hipEventRecord(ev.e1, st);
        if (hipEventSynchronize(ev.e1) != hipSuccess) return fail(HRN_E_LAUNCH, "probe: %s", hipGetErrorString(hipGetLastError()));
        float ms = 0;
        (void)hipEventElapsedTime(&ms, ev.e0, ev.e1);
        us_out[r] = (double)ms * 1e3;
    }
    return HRN_OK;
}

int hrn_probe_launch(int grid, int repeat, double* us_out, void* stream) {
    if (!us_out || grid < 1 || grid > (1 << 20) || repeat < 1) return fail(HRN_E_BADPARAM, "probe arguments");
    hipStream_t st = (hipStream_t)stream;
    EventPair ev;
    HIP_TRY(ev.create());
    hipEvent_t e0 = ev.e0, e1 = ev.e1;
    for (int i = 0; i < 20; ++i) probe_empty_kernel<<<grid, 256, 0, st>>>(nullptr);
    (void)hipEventRecord(e0, st);
    for (int i = 0; i < repeat; ++i) probe_empty_kernel<<<grid, 256, 0, st>>>(nullptr);
    (void)hipEventRecord(e1, st);
    hipError_t e = hipEventSynchronize(e1);
    float ms = 0;
    (void)hipEventElapsedTime(&ms, e0, e1);
    if (e != hipSuccess) return fail(HRN_E_LAUNCH, "probe: %s", hipGetErrorString(e));
    *us_out = ms * 1e3 / repeat;
    return HRN_OK;
}

int hrn_probe_mfma(int dtype, int mfma, int random_operands, double* tops_out, void* stream) {
    if (!tops_out || (mfma != 32 && mfma != 16) || (dtype != HRN_DT_F16 && dtype != HRN_DT_U8S8))
        return fail(HRN_E_BADPARAM, "probe arguments");
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t pr;
    HIP_TRY(hipGetDeviceProperties(&pr, dev));
    hipStream_t st = (hipStream_t)stream;
    const int iters = 20000, grid = pr.multiProcessorCount * 2;   // 2 workgroups x 4 waves per CU: 2 waves per SIMD
    const int kind = (dtype == HRN_DT_F16 ? 0 : 2) + (mfma == 32 ? 0 : 1);
    EventPair ev;
    HIP_TRY(ev.create());
    hipEvent_t e0 = ev.e0, e1 = ev.e1;
    float ms = 0;
    for (int rep = 0; rep < 2; ++rep) {   // first pass warms up
        (void)hipEventRecord(e0, st);
        switch (kind) {
            case 0: probe_mfma_kernel<0><<<grid, 256, 0, st>>>(nullptr, iters, random_operands); break;
            case 1: probe_mfma_kernel<1><<<grid, 256, 0, st>>>(nullptr, iters, random_operands); break;
            case 2: probe_mfma_kernel<2><<<grid, 256, 0, st>>>(nullptr, iters, random_operands); break;
            default: probe_mfma_kernel<3><<<grid, 256, 0, st>>>(nullptr, iters, random_operands); break;
        }
        (void)hipEventRecord(e1, st);
        hipError_t e = hipEventSynchronize(e1);
        if (e != hipSuccess) return fail(HRN_E_LAUNCH, "probe: %s", hipGetErrorString(e));
        (void)hipEventElapsedTime(&ms, e0, e1);
    }
    const double ops_per_mfma = (dtype == HRN_DT_F16) ? 32768.0 : 65536.0;   // 2*m*n*k for either shape
    const double total = ops_per_mfma * (mfma == 32 ? 1.0 : 0.5) * 4.0 * iters * 4.0 * grid;  // 4 accumulators, 4 waves
    *tops_out = total / (ms * 1e-3) / 1e12;
    return HRN_OK;
}

int hrn_probe_copy(const void* src, void* dst, size_t bytes, int repeat, double* gbs_out, void* stream) {
    if (!src || !dst || !gbs_out || bytes < 16 || bytes % 16 || repeat < 1) return fail(HRN_E_BADPARAM, "probe arguments");
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t pr;
    HIP_TRY(hipGetDeviceProperties(&pr, dev));
    hipStream_t st = (hipStream_t)stream;
    EventPair ev;
    HIP_TRY(ev.create());
    hipEvent_t e0 = ev.e0, e1 = ev.e1;
    const int grid = pr.multiProcessorCount * 16;
    probe_copy_kernel<<<grid, 256, 0, st>>>((const pv4i*)src, (pv4i*)dst, bytes / 16);
    (void)hipEventRecord(e0, st);
    for (int i = 0; i < repeat; ++i) probe_copy_kernel<<<grid, 256, 0, st>>>((const pv4i*)src, (pv4i*)dst, bytes / 16);
    (void)hipEventRecord(e1, st);
    hipError_t e = hipEventSynchronize(e1);
    float ms = 0;
    (void)hipEventElapsedTime(&ms, e0, e1);
    if (e != hipSuccess) return fail(HRN_E_LAUNCH, "probe: %s", hipGetErrorString(e));
    *gbs_out = 2.0 * bytes * repeat / (ms * 1e-3) / 1e9;
    return HRN_OK;
}

const char* hrn_last_error(void) { return g_err.c_str(); }
const char* hrn_version(void) { return "heron-rocm 0.1 (gfx950)"; }

int hrn_device_info(int device, hrn_devinfo* out) {
    if (!out) return fail(HRN_E_BADPARAM, "null out");
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return fail(HRN_E_NODEVICE, "no HIP device");
    if (device < 0 || device >= n) return fail(HRN_E_BADPARAM, "device %d of %d", device, n);
    hipDeviceProp_t pr;
    HIP_TRY(hipGetDeviceProperties(&pr, device));
    memset(out, 0, sizeof *out);
    snprintf(out->arch, sizeof out->arch, "%s", pr.gcnArchName);
    snprintf(out->name, sizeof out->name, "%s", pr.name);
    out->cu_count = pr.multiProcessorCount;
    out->wave_size = pr.warpSize;
    out->lds_bytes_per_wg = (int32_t)pr.sharedMemPerBlock;
    out->max_threads_per_wg = pr.maxThreadsPerBlock;
    out->clock_khz = pr.clockRate;
    out->mem_clock_khz = pr.memoryClockRate;
    out->mem_bus_bits = pr.memoryBusWidth;
    out->l2_bytes = pr.l2CacheSize;
    out->regs_per_simd_lane = 512;
    out->simd_per_cu = 4;
    out->hbm_bytes = pr.totalGlobalMem;
    return HRN_OK;
}

int hrn_check_desc(const hrn_kernel_desc* desc) { return derive(desc, nullptr); }

int hrn_lds_bytes(const hrn_kernel_desc* desc) {
    Derived d;
    int rc = derive(desc, &d);
    return rc ? rc : d.lds;
}

int hrn_compile(const hrn_kernel_desc* desc, double timeout_s, char* path_out, size_t path_cap) {
    std::string path;
    int rc = compile_desc(desc, timeout_s, &path);
    if (rc) return rc;
    if (path_out) {
        if (path.size() + 1 > path_cap)
            return fail(HRN_E_BADPARAM, "path buffer of %zu bytes is too small for %zu", path_cap, path.size() + 1);
        memcpy(path_out, path.c_str(), path.size() + 1);
    }
    return HRN_OK;
}

int hrn_build(const hrn_kernel_desc* desc, double timeout_s, hrn_module** out) {
    if (!out) return fail(HRN_E_BADPARAM, "null out");
    *out = nullptr;
    std::string path;
    int rc = compile_desc(desc, timeout_s, &path);
    if (rc) return rc;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return fail(HRN_E_NODEVICE, "no HIP device");
    hrn_module* m = new hrn_module();
    m->desc = *desc;
    m->path = path;
    memset(&m->info, 0, sizeof m->info);
    read_info(path.substr(0, path.size() - 6) + ".info", &m->info);
    m->info.threads = desc->wm * desc->wn * 64;
    {
        Derived dv;
        (void)derive(desc, &dv);        // compile_desc has validated the descriptor
        m->epi_bytes = dv.epi_bytes;
    }
    hipError_t e = hipModuleLoad(&m->mod, path.c_str());
    if (e != hipSuccess) {
        delete m;
        return fail(HRN_E_LOAD, "hipModuleLoad(%s): %s", path.c_str(), hipGetErrorString(e));
    }
    e = hipModuleGetFunction(&m->fn, m->mod, "hrn_mfma_kernel");
    if (e != hipSuccess) {
        (void)hipModuleUnload(m->mod);
        delete m;
        return fail(HRN_E_LOAD, "hipModuleGetFunction: %s", hipGetErrorString(e));
    }
    if (desc->split_k) {
        // hrn_launch_splitk_static finds the library's workspace of this device looked up already
        void* ws = nullptr;
        rc = static_scratch(&ws);
        if (rc) { (void)hipModuleUnload(m->mod); delete m; return rc; }
    }
    m->persist_grid = 0;
    if (desc->persistent) {
        int per_cu = 0, dev = 0;
        hipDeviceProp_t pr;
        if (hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, m->fn, m->info.threads, 0) != hipSuccess || per_cu < 1 ||
            hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&pr, dev) != hipSuccess) {
            (void)hipModuleUnload(m->mod);
            delete m;
            return fail(HRN_E_LOAD, "occupancy query failed: %s", hipGetErrorString(hipGetLastError()));
        }
        m->persist_grid = per_cu * pr.multiProcessorCount;
    }
    *out = m;
    return HRN_OK;
}

int hrn_module_info(const hrn_module* mod, hrn_kernel_info* out) {
    if (!mod || !out) return fail(HRN_E_BADPARAM, "null argument");
    *out = mod->info;
    return HRN_OK;
}

void hrn_module_free(hrn_module* mod) {
    if (!mod) return;
    (void)hipModuleUnload(mod->mod);
    delete mod;
}

int hrn_launch_gemm_f16(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream) {
    if (mod && (mod->desc.dtype != HRN_DT_F16 || mod->desc.op != HRN_OP_GEMM)) return fail(HRN_E_BADPARAM, "module is not an fp16 GEMM");
    if (p && p->batch != 1) return fail(HRN_E_BADPARAM, "gemm takes batch 1 (use hrn_launch_bmm_f16)");
    return launch(mod, p, A, B, C, stream);
}

int hrn_launch_gemm_u8s8(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream) {
    if (mod && (mod->desc.dtype != HRN_DT_U8S8 || mod->desc.op != HRN_OP_GEMM)) return fail(HRN_E_BADPARAM, "module is not a u8s8 GEMM");
    if (p && p->batch != 1) return fail(HRN_E_BADPARAM, "gemm takes batch 1 (use hrn_launch_bmm_u8s8)");
    return launch(mod, p, A, B, C, stream);
}

int hrn_launch_bmm_f16(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream) {
    if (mod && (mod->desc.dtype != HRN_DT_F16 || mod->desc.op != HRN_OP_GEMM)) return fail(HRN_E_BADPARAM, "module is not an fp16 GEMM");
    return launch(mod, p, A, B, C, stream);
}

int hrn_launch_conv2d_nhwc_f16(const hrn_module* mod, const hrn_problem* p, const void* In, const void* Filter, void* Out, void* stream) {
    if (mod && (mod->desc.dtype != HRN_DT_F16 || mod->desc.op != HRN_OP_CONV2D)) return fail(HRN_E_BADPARAM, "module is not an fp16 conv2d");
    return launch(mod, p, In, Filter, Out, stream);
}

int hrn_launch_bmm_u8s8(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream) {
    if (mod && (mod->desc.dtype != HRN_DT_U8S8 || mod->desc.op != HRN_OP_GEMM)) return fail(HRN_E_BADPARAM, "module is not a u8s8 GEMM");
    return launch(mod, p, A, B, C, stream);
}

int hrn_launch_conv2d_nhwc_u8s8(const hrn_module* mod, const hrn_problem* p, const void* In, const void* Filter, void* Out, void* stream) {
    if (mod && (mod->desc.dtype != HRN_DT_U8S8 || mod->desc.op != HRN_OP_CONV2D)) return fail(HRN_E_BADPARAM, "module is not a u8s8 conv2d");
    return launch(mod, p, In, Filter, Out, stream);
}

int hrn_launch_repeat(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, int count,
                      void* stream) {
    if (count < 1) return fail(HRN_E_BADPARAM, "count %d", count);
    LaunchPlan plan;
    int rc = fill_args(mod, p, A, B, C, p ? p->workspace : nullptr, p ? p->workspace_bytes : 0, &plan);
    if (rc) return rc;
    for (int i = 0; i < count; ++i) {
        rc = run_plan(mod, p, plan, p->workspace, (hipStream_t)stream);
        if (rc) return rc;
    }
    return HRN_OK;
}

int hrn_launch_splitk_static(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* stream) {
    if (!mod || !p) return fail(HRN_E_BADPARAM, "null argument");
    if (!mod->desc.split_k) return fail(HRN_E_BADPARAM, "hrn_launch_splitk_static needs an instance built with split_k");
    if (p->m <= 0 || p->n <= 0 || p->k <= 0 || p->batch <= 0 || p->split_k < 1) return fail(HRN_E_BADPARAM, "empty problem or split_k < 1");
    int kps, split;
    split_shape(mod->desc, p, &kps, &split);
    const int64_t need = splitk_bytes(p, split);
    if (need > (int64_t)HRN_STATIC_WORKSPACE_BYTES)
        return fail(HRN_E_BADPARAM, "split-K partial sums of %lld bytes (%d slices x %d x %d x %d x 4) exceed the library's static workspace of %lld bytes",
                    (long long)need, split, p->batch, p->m, p->n, (long long)HRN_STATIC_WORKSPACE_BYTES);
    void* ws = nullptr;
    int dev = 0;
    int rc = static_scratch(&ws, &dev);
    if (rc) return rc;
    LaunchPlan plan;
    rc = fill_args(mod, p, A, B, C, ws, (size_t)HRN_STATIC_WORKSPACE_BYTES, &plan);
    if (rc) return rc;
    // Every call on a GPU shares that GPU's one workspace.  Calls on one stream are ordered by the stream; a call on
    // another stream is made to wait for the previous user (an event recorded behind each call), so calls from several
    // streams or threads are serialised on the device instead of racing.
    hipStream_t st = (hipStream_t)stream;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_used[dev] && g_scratch_stream[dev] != st) HIP_TRY(hipStreamWaitEvent(st, g_scratch_done[dev], 0));
    rc = run_plan(mod, p, plan, ws, st);
    if (rc) return rc;
    HIP_TRY(hipEventRecord(g_scratch_done[dev], st));
    g_scratch_stream[dev] = st;
    g_scratch_used[dev] = true;
    return HRN_OK;
}

int hrn_time(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, int number, int repeat,
             double min_repeat_ms, double* costs_out, void* stream) {
    if (!costs_out || number < 1 || repeat < 1) return fail(HRN_E_BADPARAM, "number/repeat/costs_out");
    LaunchPlan plan;
    int rc = fill_args(mod, p, A, B, C, p ? p->workspace : nullptr, p ? p->workspace_bytes : 0, &plan);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    EventPair ev;
    HIP_TRY(ev.create());
    hipEvent_t e0 = ev.e0, e1 = ev.e1;
    rc = launch(mod, p, A, B, C, stream);  // warm-up, also surfaces launch errors
    if (rc) return rc;
    if (hipStreamSynchronize(st) != hipSuccess) { return fail(HRN_E_LAUNCH, "warm-up failed: %s", hipGetErrorString(hipGetLastError())); }
    for (int r = 0; r < repeat; ++r) {
        int num = number;
        for (;;) {
            (void)hipEventRecord(e0, st);
            for (int i = 0; i < num; ++i) {
                rc = launch(mod, p, A, B, C, stream);
                if (rc) return rc;
            }
            (void)hipEventRecord(e1, st);
            if (hipEventSynchronize(e1) != hipSuccess) { return fail(HRN_E_LAUNCH, "kernel failed: %s", hipGetErrorString(hipGetLastError())); }
            float ms = 0;
            (void)hipEventElapsedTime(&ms, e0, e1);
            if (ms >= min_repeat_ms || num >= (1 << 20)) {
                costs_out[r] = (double)ms * 1e-3 / num;
                number = num;  // keep the grown count for the next repeats
                break;
            }
            // grow like time_evaluator: aim past min_repeat_ms with some margin
            const double per = std::max((double)ms / num, 1e-4);
            num = std::max(num + 1, (int)std::min(1048576.0, min_repeat_ms * 1.2 / per + 1));
        }
    }
    return HRN_OK;
}

int hrn_time_cold(const hrn_module* mod, const hrn_problem* p, const void* A, const void* B, void* C, void* flush_buf,
                  size_t flush_bytes, int repeat, double* costs_out, void* stream) {
    if (!costs_out || repeat < 1 || !flush_buf || flush_bytes < (64u << 20)) return fail(HRN_E_BADPARAM, "repeat/costs_out/flush buffer (>= 64 MiB)");
    LaunchPlan plan;
    int rc = fill_args(mod, p, A, B, C, p ? p->workspace : nullptr, p ? p->workspace_bytes : 0, &plan);
    if (rc) return rc;
    int dev = 0;
    hipDeviceProp_t pr;
    HIP_TRY(hipGetDevice(&dev));
    HIP_TRY(hipGetDeviceProperties(&pr, dev));
    hipStream_t st = (hipStream_t)stream;
    EventPair ev;
    HIP_TRY(ev.create());
    hipEvent_t e0 = ev.e0, e1 = ev.e1;
    rc = launch(mod, p, A, B, C, stream);  // surfaces launch errors before anything is timed
    if (rc) return rc;
    const size_t half16 = flush_bytes / 32;   // 16-byte elements in each half of the flush buffer
    for (int r = 0; r < repeat; ++r) {
        // stream one half of the flush buffer into the other: every L2 and the memory-side cache are refilled with it
        probe_copy_kernel<<<pr.multiProcessorCount * 16, 256, 0, st>>>((const pv4i*)flush_buf, (pv4i*)flush_buf + half16, half16);
        (void)hipEventRecord(e0, st);
        rc = launch(mod, p, A, B, C, stream);
        if (rc) return rc;
        (void)hipEventRecord(e1, st);
        if (hipEventSynchronize(e1) != hipSuccess) { return fail(HRN_E_LAUNCH, "kernel failed: %s", hipGetErrorString(hipGetLastError())); }
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        costs_out[r] = (double)ms * 1e-3;
    }
    return HRN_OK;
}

int64_t hrn_splitk_workspace_bytes(const hrn_kernel_desc* desc, const hrn_problem* p) {
    if (!desc || !p) return fail(HRN_E_BADPARAM, "null argument");
    if (!desc->split_k) return 0;
    if (p->m <= 0 || p->n <= 0 || p->k <= 0 || p->batch <= 0 || p->split_k < 1) return fail(HRN_E_BADPARAM, "empty problem or split_k < 1");
    if (desc->bkb != 64 && desc->bkb != 128 && desc->bkb != 256) return fail(HRN_E_BADPARAM, "bkb %d", desc->bkb);
    int kps, split;
    split_shape(*desc, p, &kps, &split);
    return splitk_bytes(p, split);
}

void hrn_problem_gemm(hrn_problem* p, int batch, int m, int n, int k) {
    memset(p, 0, sizeof *p);
    p->op = HRN_OP_GEMM;
    p->batch = batch; p->m = m; p->n = n; p->k = k;
    p->lda = k; p->ldb = k; p->ldc = n;
    p->stride_a = (int64_t)m * k; p->stride_b = (int64_t)n * k; p->stride_c = (int64_t)m * n;
    p->group_m = 8;
}

void hrn_problem_conv2d_hw(hrn_problem* p, int n, int h, int w, int ci, int co, int kh, int kw, int stride_h, int stride_w,
                           int pad_h, int pad_w, int dil_h, int dil_w) {
    memset(p, 0, sizeof *p);
    p->op = HRN_OP_CONV2D;
    p->batch = 1;
    p->cn = n; p->ch = h; p->cw = w; p->ci = ci; p->co = co; p->kh = kh; p->kw = kw;
    p->cstride = stride_h; p->cpad = pad_h; p->cdil = dil_h;
    p->cstride_w = stride_w; p->cpad_w = pad_w; p->cdil_w = dil_w;
    const int ho = (stride_h > 0) ? (h - ((kh - 1) * dil_h + 1) + 2 * pad_h) / stride_h + 1 : 0;
    const int wo = (stride_w > 0) ? (w - ((kw - 1) * dil_w + 1) + 2 * pad_w) / stride_w + 1 : 0;
    p->m = n * ho * wo; p->n = co; p->k = kh * kw * ci;
    p->lda = ci; p->ldb = p->k; p->ldc = co;
    p->group_m = 8;
}

void hrn_problem_conv2d(hrn_problem* p, int n, int h, int w, int ci, int co, int kh, int kw, int stride, int pad, int dil) {
    hrn_problem_conv2d_hw(p, n, h, w, ci, co, kh, kw, stride, stride, pad, pad, dil, dil);
}

}  // extern "C"
