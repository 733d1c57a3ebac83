// Run-time side of the compiled fused-row programs: finds the kernel of a program among those built into the
// library, compiles it through hipRTC when it is not there, and launches it as a persistent grid.
#include "rows_prog.hpp"

#include <hip/hiprtc.h>

#include <sys/stat.h>
#include <sys/types.h>
#include <unistd.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "rows_prog_body.h" // kRowsProgBody: the text of rows_prog.inc, written by the build

namespace axhip {
namespace {

// A program with everything a kernel does not depend on taken out (addresses, extents along rows, immediate
// values): two programs with equal keys run the same kernel under the same plan.
struct StructKey {
    AxhipRowsProgram p;
};

void make_struct_key(const AxhipRowsProgram &P, StructKey *k) {
    memset(k, 0, sizeof(*k));
    AxhipRowsProgram &q = k->p;
    // (the address modulo 16 decides between the aligned, the grid and the unaligned form of a kernel)
    auto align_tag = [](const void *p) { return reinterpret_cast<const void *>(static_cast<uintptr_t>(reinterpret_cast<uintptr_t>(p) & 15u) + 16u); };
    q.cols = P.cols;
    // (arrays of many short rows have a plan of their own; elementwise chains are compiled from a size on)
    q.rows = (P.rows >= kRowsProgLaneMinRows ? 1 : 0) | (P.row_op == AXHIP_ROWOP_NONE && P.reduce == AXHIP_RED_NONE && rows_prog_flat_large(P) ? 2 : 0);
    q.input = align_tag(P.input);
    q.input_dtype = P.input_dtype;
    q.n_operands = P.n_operands;
    for (int i = 0; i < P.n_operands && i < AXHIP_MAX_OPERANDS; ++i) {
        q.operands[i].ptr = align_tag(P.operands[i].ptr);
        q.operands[i].dtype = P.operands[i].dtype;
        q.operands[i].kind = P.operands[i].kind;
    }
    auto copy_chain = [](const AxhipChainOp *src, int n, AxhipChainOp *dst) {
        for (int i = 0; i < n && i < AXHIP_MAX_CHAIN; ++i) {
            dst[i].op = src[i].op;
            dst[i].imm_kind = src[i].imm_kind;
            dst[i].operand = src[i].imm_kind == AXHIP_BK_IMM ? -1 : src[i].operand;
        }
    };
    q.n_pre = P.n_pre;
    copy_chain(P.pre, P.n_pre, q.pre);
    q.row_op = P.row_op;
    q.norm_weight = P.norm_weight;
    q.norm_bias = P.norm_bias;
    q.n_post = P.n_post;
    copy_chain(P.post, P.n_post, q.post);
    q.reduce = P.reduce == AXHIP_RED_MEAN ? AXHIP_RED_SUM : P.reduce;
    q.output = const_cast<void *>(align_tag(P.output));
    q.output_dtype = P.output_dtype;
}

uint64_t hash_bytes(const void *p, size_t n) {
    const unsigned char *b = static_cast<const unsigned char *>(p);
    uint64_t h = 14695981039346656037ull;
    for (size_t i = 0; i < n; ++i) {
        h ^= b[i];
        h *= 1099511628211ull;
    }
    return h;
}

struct Kernel {
    const void *builtin = nullptr; // address of a kernel compiled into the library, or
    hipModule_t module = nullptr;  // a module compiled at run time
    hipFunction_t function = nullptr;
    int blocks_per_cu = 0;         // resident blocks per compute unit (0: not yet asked)
};

struct Entry {
    StructKey key;
    bool eligible = false;
    RowsProgSpec spec;
    std::shared_ptr<Kernel> kernel; // null until the program is first launched (a name query compiles nothing)
    bool is_builtin = false;
    bool jit_failed = false;
    bool has_builtin_alternative = false; // a built-in kernel under a looser plan exists next to the tight plan's spec
    RowsProgSpec builtin_spec;
    std::shared_ptr<Kernel> alt_kernel;
};

std::mutex g_mutex;
std::unordered_multimap<uint64_t, std::unique_ptr<Entry>> g_entries;      // by structure
std::unordered_map<std::string, std::shared_ptr<Kernel>> g_kernels;      // by configuration text
int g_num_cus = 0;

// read at every dispatch (a getenv is cheap against a launch), so that a test can switch within one process
bool jit_enabled() {
    const char *e = getenv("AXHIP_JIT");
    return !(e && e[0] == '0');
}

Entry *find_or_make_entry(const AxhipRowsProgram &P) {
    StructKey k;
    make_struct_key(P, &k);
    const uint64_t h = hash_bytes(&k, sizeof(k));
    auto range = g_entries.equal_range(h);
    for (auto it = range.first; it != range.second; ++it)
        if (memcmp(&it->second->key, &k, sizeof(k)) == 0) return it->second.get();
    // (one entry per row length and program structure: a loop over ever-changing row lengths must not grow this
    // without bound; compiled kernels live in g_kernels and are found again by their configuration text)
    if (g_entries.size() >= 4096) g_entries.clear();
    auto e = std::make_unique<Entry>();
    e->key = k;
    // Two candidate plans: the tightest fit for this row length, and the nearest of the shapes the build compiles.
    // The built-in kernel wins when it exists and its idle lanes cost at most 15 % more chunk slots; otherwise the
    // tight plan's kernel is compiled at first launch.
    RowsProgPlan tight, stock;
    RowsProgSpec stock_spec;
    const bool has_tight = rows_prog_plan(P, true, &tight) && rows_prog_spec(P, tight, &e->spec);
    const bool has_stock = rows_prog_plan(P, false, &stock) && rows_prog_spec(P, stock, &stock_spec) &&
                           rows_prog_find_builtin(stock_spec.config + stock_spec.chains) != nullptr;
    e->eligible = has_tight || has_stock;
    e->has_builtin_alternative = false;
    static const bool forced_group = getenv("AXHIP_ROWS_GROUP") != nullptr; // (the tuning switch of the tight plan wins over the built-in shapes)
    if (has_stock && (!has_tight || (!forced_group && !tight.lane && stock.slots() * 100 <= tight.slots() * 115))) {
        e->spec = stock_spec;
        e->is_builtin = true;
    } else if (has_tight) {
        e->is_builtin = rows_prog_find_builtin(e->spec.config + e->spec.chains) != nullptr;
        if (!e->is_builtin && has_stock) { // kept for when run-time compilation is off or fails
            e->has_builtin_alternative = true;
            e->builtin_spec = stock_spec;
        }
    }
    Entry *raw = e.get();
    g_entries.emplace(h, std::move(e));
    return raw;
}

// ---- on-disk cache of run-time compiled kernels.  A code object is stored under the hash of everything it depends
// on (generated source, compiler options, hipRTC version), so a new process loads it instead of compiling again
// (0.5 s for the first compile of a process, 10-35 ms for later ones).  AXHIP_CACHE_DIR names the folder (default
// $XDG_CACHE_HOME/axhip, else $HOME/.cache/axhip); AXHIP_DISK_CACHE=0 turns it off.
const char *const kCompileOptions[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
constexpr int kNumCompileOptions = static_cast<int>(sizeof(kCompileOptions) / sizeof(kCompileOptions[0]));

std::string cache_dir() {
    const char *off = getenv("AXHIP_DISK_CACHE");
    if (off && off[0] == '0') return "";
    if (const char *d = getenv("AXHIP_CACHE_DIR")) return d[0] ? std::string(d) : "";
    if (const char *x = getenv("XDG_CACHE_HOME")) if (x[0]) return std::string(x) + "/axhip";
    if (const char *h = getenv("HOME")) if (h[0]) return std::string(h) + "/.cache/axhip";
    return "";
}

bool make_dirs(const std::string &path) {
    for (size_t i = 1; i <= path.size(); ++i)
        if (i == path.size() || path[i] == '/') {
            const std::string part = path.substr(0, i);
            if (mkdir(part.c_str(), 0777) != 0 && errno != EEXIST) return false;
        }
    return true;
}

std::string cache_path(const RowsProgSpec &spec, const std::string &src) {
    const std::string dir = cache_dir();
    if (dir.empty()) return "";
    int major = 0, minor = 0;
    (void)hiprtcVersion(&major, &minor);
    std::string what = src;
    for (const char *o : kCompileOptions) what += std::string("\n") + o;
    what += "\nhiprtc " + std::to_string(major) + "." + std::to_string(minor);
    char name[32];
    snprintf(name, sizeof(name), "%016llx", static_cast<unsigned long long>(hash_bytes(what.data(), what.size())));
    return dir + "/" + spec.symbol + "_" + name + ".hsaco";
}

bool read_file(const std::string &path, std::vector<char> *out) {
    FILE *f = fopen(path.c_str(), "rb");
    if (!f) return false;
    bool ok = fseek(f, 0, SEEK_END) == 0;
    const long n = ok ? ftell(f) : -1;
    ok = ok && n > 0 && fseek(f, 0, SEEK_SET) == 0;
    if (ok) {
        out->resize(static_cast<size_t>(n));
        ok = fread(out->data(), 1, out->size(), f) == out->size();
    }
    fclose(f);
    return ok;
}

void write_file_atomically(const std::string &path, const std::vector<char> &data) {
    const size_t slash = path.rfind('/');
    if (slash == std::string::npos || !make_dirs(path.substr(0, slash))) return;
    const std::string tmp = path + ".tmp." + std::to_string(static_cast<long long>(getpid()));
    FILE *f = fopen(tmp.c_str(), "wb");
    if (!f) return;
    const bool ok = fwrite(data.data(), 1, data.size(), f) == data.size();
    if (fclose(f) != 0 || !ok || rename(tmp.c_str(), path.c_str()) != 0) (void)remove(tmp.c_str());
}

std::shared_ptr<Kernel> load_code(const std::vector<char> &code, const RowsProgSpec &spec, bool report) {
    auto k = std::make_shared<Kernel>();
    hipError_t e = hipModuleLoadData(&k->module, code.data());
    if (e == hipSuccess) e = hipModuleGetFunction(&k->function, k->module, spec.symbol.c_str());
    if (e != hipSuccess) {
        if (report) set_last_error("fused rows: loading the compiled %s failed: %s", spec.label.c_str(), hipGetErrorString(e));
        (void)hipGetLastError();
        return nullptr;
    }
    return k;
}

int g_disk_hits = 0, g_compiles = 0; // (under g_mutex)

// the program's kernel from the on-disk cache, else compiled through hipRTC (and stored); on failure the reason goes
// to the library's error text.  Called WITHOUT g_mutex: other threads keep dispatching while this one compiles.
std::shared_ptr<Kernel> compile(const RowsProgSpec &spec, bool *from_disk) {
    *from_disk = false;
    const std::string src = rows_prog_source(spec, kRowsProgBody);
    const std::string path = cache_path(spec, src);
    if (!path.empty()) {
        std::vector<char> code;
        if (read_file(path, &code)) {
            if (auto k = load_code(code, spec, false)) {
                *from_disk = true;
                return k;
            } // (an unreadable or stale file is compiled again and replaced)
        }
    }
    hiprtcProgram prog = nullptr;
    if (hiprtcCreateProgram(&prog, src.c_str(), (spec.symbol + ".hip").c_str(), 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
        set_last_error("fused rows: hiprtcCreateProgram failed for %s", spec.label.c_str());
        return nullptr;
    }
    const hiprtcResult r = hiprtcCompileProgram(prog, kNumCompileOptions, const_cast<const char **>(kCompileOptions));
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, '\0');
        if (n) hiprtcGetProgramLog(prog, log.data());
        set_last_error("fused rows: run-time compilation of %s failed: %s: %.300s", spec.label.c_str(), hiprtcGetErrorString(r), log.c_str());
        hiprtcDestroyProgram(&prog);
        return nullptr;
    }
    size_t size = 0;
    hiprtcGetCodeSize(prog, &size);
    std::vector<char> code(size);
    hiprtcGetCode(prog, code.data());
    hiprtcDestroyProgram(&prog);
    auto k = load_code(code, spec, true);
    if (k && !path.empty()) write_file_atomically(path, code);
    return k;
}

} // namespace

bool rows_prog_compile_only(const AxhipRowsProgram &P, std::string *label, std::string *error) {
    RowsProgPlan plan;
    RowsProgSpec spec;
    if (!rows_prog_plan(P, true, &plan) || !rows_prog_spec(P, plan, &spec)) {
        if (error) *error = "the program does not qualify for a compiled kernel";
        return false;
    }
    if (label) *label = spec.label;
    const std::string src = rows_prog_source(spec, kRowsProgBody);
    hiprtcProgram prog = nullptr;
    if (hiprtcCreateProgram(&prog, src.c_str(), "probe.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
        if (error) *error = "hiprtcCreateProgram failed";
        return false;
    }
    const hiprtcResult r = hiprtcCompileProgram(prog, kNumCompileOptions, const_cast<const char **>(kCompileOptions));
    if (r != HIPRTC_SUCCESS && error) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, '\0');
        if (n) hiprtcGetProgramLog(prog, log.data());
        *error = std::string(hiprtcGetErrorString(r)) + ": " + log;
    }
    hiprtcDestroyProgram(&prog);
    return r == HIPRTC_SUCCESS;
}

bool rows_prog_dispatch(const AxhipRowsProgram &P, hipStream_t s, bool launch, char *name, size_t name_len, int *rc, bool builtin_only) {
    if (rc) *rc = AXHIP_OK;
    if (P.rows <= 0 || P.cols <= 0 || P.rows >= (int64_t(1) << 31)) return false;
    std::shared_ptr<Kernel> kernel;
    RowsProgArgs args;
    int threads = 0, rows_per_block = 1;
    // A kernel that has to be compiled is compiled with g_mutex released (hundreds of milliseconds during which
    // other threads' dispatches go on); the loop then takes the lock again and publishes it.
    std::shared_ptr<Kernel> compiled;
    bool compile_done = false, compiled_from_disk = false;
    RowsProgSpec to_compile;
    for (;;) {
        bool need_compile = false;
        {
        std::lock_guard<std::mutex> lock(g_mutex);
        Entry *e = find_or_make_entry(P);
        if (!e->eligible) return false;
        if (builtin_only && !e->is_builtin) return false; // (a caller that must not compile: the no-allocation reduction)
        // the tight plan's kernel, compiled on first launch -- or, with run-time compilation off or failed, the
        // looser built-in plan when there is one, else the interpreter
        bool use_alt = false;
        if (!e->is_builtin && (!jit_enabled() || e->jit_failed)) {
            if (!e->has_builtin_alternative) return false;
            use_alt = true;
        }
        if (!use_alt && !e->kernel && launch) {
            const std::string key = e->spec.config + e->spec.chains;
            auto it = g_kernels.find(key);
            if (it != g_kernels.end()) {
                e->kernel = it->second;
            } else {
                std::shared_ptr<Kernel> k;
                if (e->is_builtin) {
                    k = std::make_shared<Kernel>();
                    k->builtin = rows_prog_find_builtin(key);
                } else if (!compile_done) {
                    need_compile = true;
                    to_compile = e->spec;
                } else {
                    k = compiled;
                    if (k) {
                        ++(compiled_from_disk ? g_disk_hits : g_compiles);
                    } else {
                        e->jit_failed = true;
                        if (!e->has_builtin_alternative) return false;
                        use_alt = true;
                    }
                }
                if (k) {
                    g_kernels.emplace(key, k); // (another thread may have published the same kernel meanwhile: its copy stays)
                    e->kernel = g_kernels.find(key)->second;
                }
            }
        }
        if (!need_compile) {
        if (use_alt && !e->alt_kernel) {
            e->alt_kernel = std::make_shared<Kernel>();
            e->alt_kernel->builtin = rows_prog_find_builtin(e->builtin_spec.config + e->builtin_spec.chains);
        }
        const RowsProgSpec &spec = use_alt ? e->builtin_spec : e->spec;
        if (name) snprintf(name, name_len, "%s%s", (use_alt || e->is_builtin) ? "rows_static_" : "rows_jit_", spec.label.c_str());
        if (!launch) return true;
        kernel = use_alt ? e->alt_kernel : e->kernel;
        if (kernel->blocks_per_cu == 0) {
            int n = 0;
            hipError_t err = kernel->builtin ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel->builtin, spec.threads, 0)
                                             : hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel->function, spec.threads, 0);
            if (err != hipSuccess) (void)hipGetLastError();
            kernel->blocks_per_cu = err == hipSuccess && n > 0 ? n : 2;
            // Fewer resident blocks than fit, where a block keeps much of its input requested at a time: with inputs
            // that come from HBM aligned rows run faster with about 128 KiB of requests per CU (two blocks of four
            // wavefront rows of 4096 16-bit columns, pipelined) than with every wave slot filled -- softmax bf16
            // [16384,4096] 67.9 -> 69.7 % of the HBM peak, fp32 [8192,8192] 65.9 -> 69.1 %, RMS norm [32768,2048]
            // 67.7 -> 72.2 %, row sums 68.2 -> 71.4 %; unchanged back to back on one buffer pair.  Never fewer than two
            // blocks (with one, 64 KiB, chains that are heavy on arithmetic lose: softmax(exp(x)) 70 -> 64 %), four
            // where the output pass carries a chain of its own (gelu(layer norm) back to back: 77.8 % with four or
            // more, 75.9 % with two).
            // AXHIP_ROWS_INFLIGHT_KB=<n> (read once) sets the figure, 0 fills the CU.
            static const int inflight_kb = [] { const char *v = getenv("AXHIP_ROWS_INFLIGHT_KB"); return v ? atoi(v) : 128; }();
            if (inflight_kb > 0 && spec.inflight_bytes > 0) {
                const int64_t want = std::max<int64_t>(spec.post_ops > 0 ? 4 : 2, (static_cast<int64_t>(inflight_kb) * 1024 + spec.inflight_bytes / 2) / spec.inflight_bytes);
                if (kernel->blocks_per_cu > want) kernel->blocks_per_cu = static_cast<int>(want);
            }
        }
        if (g_num_cus == 0) {
            int dev = 0, n = 0;
            if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
                (void)hipGetLastError();
                n = 256;
            }
            g_num_cus = n;
        }
        rows_prog_bind(P, spec, &args);
        threads = spec.threads;
        rows_per_block = spec.rows_per_block;
        }
        }
        if (!need_compile) break;
        compiled = compile(to_compile, &compiled_from_disk);
        compile_done = true;
    }
    const int64_t row_groups = (P.rows + rows_per_block - 1) / rows_per_block;
    // As many blocks as fit on the device at once, then fewer, so that every block walks the same number of rows
    // (4096 row groups on 1280 resident blocks would leave most blocks idle during a fourth pass: 1024 blocks of 4).
    const int64_t resident = static_cast<int64_t>(kernel->blocks_per_cu) * g_num_cus;
    const int64_t passes = (row_groups + resident - 1) / resident;
    const unsigned grid = static_cast<unsigned>((row_groups + passes - 1) / passes);
    void *params[] = {&args};
    hipError_t err = kernel->builtin ? hipLaunchKernel(kernel->builtin, dim3(grid), dim3(threads), params, 0, s)
                                     : hipModuleLaunchKernel(kernel->function, grid, 1, 1, threads, 1, 1, 0, s, params, nullptr);
    if (err != hipSuccess) {
        set_last_error("fused rows: launch failed: %s", hipGetErrorString(err));
        if (rc) *rc = static_cast<int>(err);
    }
    return true;
}

// how many run-time kernels this process loaded from the on-disk cache / compiled (diagnostic)
void rows_prog_jit_counters(int *from_disk, int *compiled) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (from_disk) *from_disk = g_disk_hits;
    if (compiled) *compiled = g_compiles;
}

} // namespace axhip
