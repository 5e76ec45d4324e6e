// HIP runtime side: context, hipRTC kernel cache, device buffers, plan executor, C ABI.
//
// What it replaces in the reference: src/devices/opencl/device.rs (execute / proc_exec / get_tensor)
// and src/devices/opencl/context.rs (buffers, program build, kernel cache).  Differences that matter:
// one stream and no wait after each kernel (the reference waits on every launch, e.g.
// kernels/binary.rs:51); the program runs once (the reference runs it twice, device.rs:68-74);
// CreateMat payloads are uploaded once, not on every execution of their Alloc (kernels/alloc.rs:5-12);
// counted loops cost one host synchronisation in total, not one per iteration (device.rs:133).
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hiprtc.h>

#include <dirent.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <thread>
#include <atomic>
#include <cerrno>
#include <cmath>
#include <cstring>
#include <map>
#include <set>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/adhip.h"
#include "ir.hpp"
#include "lower.hpp"
#include "plan.hpp"

using namespace adhip;

// Scratch memory of adhip_program_enqueue_noalloc: the temporaries of a program (partial sums, slices of split
// products, intermediate tensors) and its control-flow flags live here instead of in allocations of the program's
// own.  Every GPU the library runs on holds its own copy of the array, at its own address, until the process ends;
// host code never uses the array's name as an address, only what hipGetSymbolAddress returned for the current device.
static __device__ __align__(256) unsigned char adhip_static_scratch[ADHIP_STATIC_SCRATCH_BYTES];

namespace {

thread_local std::string g_tls_error;

#define HIP_OK(expr)                                                                                     \
    do {                                                                                                 \
        hipError_t e_ = (expr);                                                                          \
        if (e_ != hipSuccess) throw Error(strf("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__)); \
    } while (0)

struct Module {
    hipModule_t mod = nullptr;
    std::map<std::string, hipFunction_t> fns;
    ~Module() {
        if (mod) (void)hipModuleUnload(mod);
    }
};

// A kept tensor on the host.  Small ones live in a vector and arrive through the staging area; large ones live in
// pinned memory of their own, which the copy engine writes directly (about five times the rate of a copy into
// pageable memory) and which is kept for the next read-back of the same id.
struct HostResult {
    std::vector<float> data;
    float* pinned = nullptr;
    size_t pinned_elems = 0;
    std::vector<uint64_t> dims;
    const float* ptr() const { return pinned ? pinned : data.data(); }
    HostResult() = default;
    HostResult(const HostResult&) = delete;
    HostResult& operator=(const HostResult&) = delete;
    HostResult(HostResult&& o) noexcept { *this = std::move(o); }
    HostResult& operator=(HostResult&& o) noexcept {
        if (this != &o) {
            release();
            data = std::move(o.data);
            dims = std::move(o.dims);
            pinned = o.pinned;
            pinned_elems = o.pinned_elems;
            o.pinned = nullptr;
            o.pinned_elems = 0;
        }
        return *this;
    }
    void release() {
        if (pinned) (void)hipHostFree(pinned);
        pinned = nullptr;
        pinned_elems = 0;
    }
    ~HostResult() { release(); }
};
constexpr size_t kPinnedResultBytes = size_t(1) << 20;  // results at least this large get pinned memory

}  // namespace

struct adhip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    std::string arch;
    std::string last_error;
    std::map<std::string, std::shared_ptr<Module>> modules;  // by source text
    std::map<std::string, HostResult> results;
    float* pinned = nullptr;  // small pinned area for predicate read-back
    char* stage = nullptr;    // pinned staging area for small uploads and read-backs
    unsigned char* static_scratch = nullptr;  // this device's copy of adhip_static_scratch (device address)
    std::string static_scratch_error;         // why it could not be located, if so
    double compile_ms = 0;
    // Programs kept from earlier adhip_execute calls, most recently used first: a caller that executes the same
    // program again (a training loop) skips lowering, module loading and allocation.
    struct CachedExec { std::string key; adhip_program* prog; size_t bytes; };
    std::vector<CachedExec> exec_cache;
};
constexpr size_t kStageBytes = 1 << 20;        // pinned staging area
constexpr size_t kStageMaxItem = 64 << 10;     // larger transfers go directly
constexpr size_t kExecCacheEntries = 4;        // programs kept per context
constexpr size_t kExecCacheBytes = size_t(4) << 30;  // device memory the kept programs may hold together

struct adhip_program {
    adhip_ctx* ctx = nullptr;
    std::unique_ptr<Proc> ir;
    std::unique_ptr<Plan> plan;
    std::vector<void*> buf_ptr;   // per plan buffer
    std::vector<void*> owned;     // allocations to free
    // Small home / constant buffers share one allocation, uploaded ones first: their payloads go up in one copy and
    // the small results come back in one, instead of a copy per buffer (a few microseconds each, and they queue up).
    char* arena = nullptr;
    std::vector<size_t> arena_off;   // per plan buffer: offset in the arena, or SIZE_MAX
    size_t arena_upload_bytes = 0;   // the uploaded buffers occupy [0, arena_upload_bytes)
    std::vector<hipFunction_t> fn;  // per plan kernel
    std::vector<std::shared_ptr<Module>> mods;
    bool profiling = false;
    bool exited = false;
    // runs of consecutive launches replayed as one hipGraph: key = (step list, index of the first launch)
    std::map<std::pair<const void*, size_t>, hipGraphExec_t> graphs;
    std::vector<hipGraph_t> graph_objs;
    bool use_graphs = true;
    std::set<std::pair<const void*, size_t>> seen_runs;  // launch runs executed once already
    std::vector<const float*> payloads;  // CreateMat host pointers in stream order (programs made by adhip_execute)
    std::vector<int> payload_of;         // per plan buffer: index into `payloads`, -1 if none
    size_t device_bytes = 0;
    int* flags = nullptr;            // device flags of predicated blocks
    // the same buffer table with every temporary, and the flags, placed in the device's static scratch area
    // (adhip_program_enqueue_noalloc); static_need is what the program takes of it
    std::vector<void*> static_buf_ptr;
    int* static_flags = nullptr;
    size_t static_need = 0;
    bool use_static = false;         // set for the duration of a run that uses the static area
    hipFunction_t flag_fn = nullptr;
    uint64_t flag_launches = 0;
    std::vector<std::pair<int, std::pair<hipEvent_t, hipEvent_t>>> pending;  // stat index, (start, stop)
    std::vector<hipEvent_t> event_pool;
    std::string description;
};

namespace {

// Code objects are cached on disk, keyed by a hash of (arch, options, source), so that a process that
// runs a program it has seen before does not pay for hipRTC again.  ADHIP_CACHE_DIR overrides the
// location; ADHIP_CACHE_DIR=off disables the cache.
const char* kCompileOptionsTag = "O3;fp-contract=off;correctly-rounded-divide-sqrt;no-packed-fp32;v1";

uint64_t fnv1a(const std::string& s, uint64_t h = 1469598103934665603ull) {
    for (unsigned char c : s) { h ^= c; h *= 1099511628211ull; }
    return h;
}

std::string cache_path(const std::string& source, const std::string& arch_name) {
    const char* dir = getenv("ADHIP_CACHE_DIR");
    std::string d;
    if (dir && *dir) {
        if (std::string(dir) == "off") return "";
        d = dir;
    } else {
        const char* home = getenv("HOME");
        d = std::string(home && *home ? home : "/tmp") + "/.cache/adhip";
    }
    std::string cmd_dir = d;
    // create the directory (two levels at most); failures just disable the cache
    for (size_t i = 1; i <= cmd_dir.size(); ++i)
        if (i == cmd_dir.size() || cmd_dir[i] == '/') {
            std::string sub = cmd_dir.substr(0, i);
            if (mkdir(sub.c_str(), 0755) != 0 && errno != EEXIST) { /* keep going: a parent may be read-only but exist */ }
        }
    uint64_t h = fnv1a(source, fnv1a(arch_name + ";" + kCompileOptionsTag));
    return d + "/" + strf("%016llx_%zu.hsaco", (unsigned long long)h, source.size());
}

std::vector<char> compile_code_object_uncached(const std::string& source, const std::string& arch_name);

// Once per process, when the cache directory holds more than `limit` entries, the older half (by modification
// time) is removed: a cache nobody ever empties would otherwise grow with every program the machine has seen.
void prune_cache_dir(const std::string& file_in_dir, size_t limit = 8192) {
    static std::atomic<bool> done{false};
    if (done.exchange(true)) return;
    const size_t slash = file_in_dir.rfind('/');
    if (slash == std::string::npos) return;
    const std::string dir = file_in_dir.substr(0, slash);
    DIR* d = opendir(dir.c_str());
    if (!d) return;
    std::vector<std::pair<time_t, std::string>> entries;
    while (dirent* e = readdir(d)) {
        const std::string name = e->d_name;
        if (name.size() < 7 || name.compare(name.size() - 6, 6, ".hsaco") != 0) continue;
        struct stat st;
        const std::string path = dir + "/" + name;
        if (stat(path.c_str(), &st) == 0) entries.push_back({st.st_mtime, path});
    }
    closedir(d);
    if (entries.size() <= limit) return;
    std::sort(entries.begin(), entries.end());
    for (size_t i = 0; i < entries.size() / 2; ++i) remove(entries[i].second.c_str());
}

// Cache file: "ADHC1\n", the source length, the source text, then the code object.  The source is stored so that a
// hit is only taken when the text matches: the file name is a 64-bit hash, and a collision must not load the wrong
// kernel.
std::vector<char> compile_code_object(const std::string& source, const std::string& arch_name) {
    const std::string path = cache_path(source, arch_name);
    static const char kMagic[6] = {'A', 'D', 'H', 'C', '1', '\n'};
    if (!path.empty()) {
        if (FILE* f = fopen(path.c_str(), "rb")) {
            std::vector<char> blob;
            char buf[65536];
            size_t n;
            while ((n = fread(buf, 1, sizeof buf, f)) > 0) blob.insert(blob.end(), buf, buf + n);
            fclose(f);
            const size_t head = sizeof kMagic + sizeof(uint64_t);
            if (blob.size() > head && memcmp(blob.data(), kMagic, sizeof kMagic) == 0) {
                uint64_t sl = 0;
                memcpy(&sl, blob.data() + sizeof kMagic, sizeof sl);
                if (sl == source.size() && blob.size() > head + sl + 64 && memcmp(blob.data() + head, source.data(), sl) == 0)
                    return std::vector<char>(blob.begin() + (long)(head + sl), blob.end());
            }
        }
    }
    std::vector<char> code = compile_code_object_uncached(source, arch_name);
    if (!path.empty()) {
        prune_cache_dir(path);
        std::string tmp = path + strf(".tmp%d", (int)getpid());
        if (FILE* f = fopen(tmp.c_str(), "wb")) {
            const uint64_t sl = source.size();
            bool ok = fwrite(kMagic, 1, sizeof kMagic, f) == sizeof kMagic && fwrite(&sl, 1, sizeof sl, f) == sizeof sl &&
                      fwrite(source.data(), 1, source.size(), f) == source.size() &&
                      fwrite(code.data(), 1, code.size(), f) == code.size();
            fclose(f);
            if (ok) rename(tmp.c_str(), path.c_str());
            else remove(tmp.c_str());
        }
    }
    return code;
}

std::vector<char> compile_code_object_uncached(const std::string& source, const std::string& arch_name) {
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, source.c_str(), "adhip_kernel.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS)
        throw Error("hiprtcCreateProgram failed");
    std::string arch = "--offload-arch=" + arch_name;
    // Element-wise chains keep multiply and add separate (no contraction) so that they round like
    // the unfused operations they replace; packed-FP32 code generation is switched off.
    const char* opts[] = {arch.c_str(), "-O3", "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt",
                          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    hiprtcResult r = hiprtcCompileProgram(prog, (int)(sizeof opts / sizeof opts[0]), opts);
    if (r != HIPRTC_SUCCESS) {
        size_t ls = 0;
        hiprtcGetProgramLogSize(prog, &ls);
        std::string log(ls, '\0');
        if (ls) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        throw Error("hipRTC compilation failed:\n" + log + "\n--- source ---\n" + source);
    }
    size_t cs = 0;
    hiprtcGetCodeSize(prog, &cs);
    std::vector<char> code(cs);
    hiprtcGetCode(prog, code.data());
    hiprtcDestroyProgram(&prog);
    return code;
}

// Code objects of several sources at once: hipRTC takes a few hundred milliseconds per kernel and a program can
// have dozens of them, so the ones that are not cached are compiled on several host threads
// (ADHIP_COMPILE_THREADS, default 8; 1 compiles one after the other).
std::map<std::string, std::vector<char>> compile_code_objects(const std::vector<std::string>& sources, const std::string& arch) {
    std::map<std::string, std::vector<char>> out;
    std::vector<const std::string*> todo;
    for (const std::string& src : sources)
        if (out.emplace(src, std::vector<char>()).second) todo.push_back(&out.find(src)->first);
    int threads = 8;
    if (const char* e = getenv("ADHIP_COMPILE_THREADS")) threads = std::max(1, atoi(e));
    threads = (int)std::min<size_t>((size_t)threads, todo.size());
    if (threads <= 1) {
        for (const std::string* src : todo) out[*src] = compile_code_object(*src, arch);
        return out;
    }
    std::atomic<size_t> next{0};
    std::vector<std::string> errors((size_t)threads);
    std::vector<std::thread> pool;
    for (int t = 0; t < threads; ++t)
        pool.emplace_back([&, t] {
            try {
                for (size_t i = next.fetch_add(1); i < todo.size(); i = next.fetch_add(1)) {
                    std::vector<char> code = compile_code_object(*todo[i], arch);
                    out.find(*todo[i])->second = std::move(code);   // distinct keys: no two threads touch one entry
                }
            } catch (const std::exception& e) {
                errors[(size_t)t] = e.what();
                next.store(todo.size());
            }
        });
    for (auto& th : pool) th.join();
    for (auto& e : errors)
        if (!e.empty()) throw Error(e);
    return out;
}

// What the compiler wrote into a code object's metadata note (msgpack) about each kernel's register spills: a kernel
// with more pointers and values in flight than the 102 scalar / 512 vector registers of a lane hold keeps the rest in
// lanes of spare vector registers and in scratch memory.  The lowering bounds the pointers of a kernel so that vector
// registers are not spilled: three generated kernels with 512 vector registers, some 200 spilled scalar registers and
// spilled vector registers on top computed wrong elements, and none without vector spills did.  The keys of a kernel's map
// are sorted: .name < .private_segment_fixed_size < .sgpr_spill_count < .vgpr_spill_count.
struct KernelSpills {
    std::string name;
    long scalar = 0, vector = 0, scratch_bytes = 0;
};

std::vector<KernelSpills> code_object_spills(const std::vector<char>& code) {
    const std::string blob(code.begin(), code.end());
    auto key = [](const std::string& k) { return std::string(1, (char)(0xa0 + k.size())) + k; };  // fixstr: all < 32 bytes
    auto uint_at = [&](size_t p) -> long {
        if (p >= blob.size()) return -1;
        const unsigned char b = (unsigned char)blob[p];
        auto be = [&](size_t n) -> long {
            if (p + n >= blob.size()) return -1;
            long v = 0;
            for (size_t i = 1; i <= n; ++i) v = (v << 8) | (unsigned char)blob[p + i];
            return v;
        };
        if (b < 0x80) return b;
        if (b == 0xcc) return be(1);
        if (b == 0xcd) return be(2);
        if (b == 0xce) return be(4);
        return -1;
    };
    auto str_at = [&](size_t p) -> std::string {
        if (p >= blob.size()) return "";
        const unsigned char b = (unsigned char)blob[p];
        size_t len = 0, at = p + 1;
        if (b >= 0xa0 && b <= 0xbf) len = b - 0xa0;
        else if (b == 0xd9 && p + 1 < blob.size()) { len = (unsigned char)blob[p + 1]; at = p + 2; }
        else if (b == 0xda && p + 2 < blob.size()) { len = ((size_t)(unsigned char)blob[p + 1] << 8) | (unsigned char)blob[p + 2]; at = p + 3; }
        else return "";
        return at + len <= blob.size() ? blob.substr(at, len) : "";
    };
    const std::string k_name = key(".name"), k_priv = key(".private_segment_fixed_size"), k_s = key(".sgpr_spill_count"),
                      k_v = key(".vgpr_spill_count");
    std::vector<KernelSpills> out;
    for (size_t p = blob.find(k_s); p != std::string::npos; p = blob.find(k_s, p + 1)) {
        KernelSpills ks;
        ks.scalar = uint_at(p + k_s.size());
        const size_t nm = blob.rfind(k_name, p), pv = blob.rfind(k_priv, p), vp = blob.find(k_v, p);
        if (nm != std::string::npos) ks.name = str_at(nm + k_name.size());
        if (pv != std::string::npos && (nm == std::string::npos || pv > nm)) ks.scratch_bytes = uint_at(pv + k_priv.size());
        if (vp != std::string::npos) ks.vector = uint_at(vp + k_v.size());
        out.push_back(ks);
    }
    return out;
}

// everything: also list kernels that only keep scalar registers in lanes of spare vector registers (the compiler's
// ordinary answer to many lane masks in flight; costs a few instructions) or use scratch memory without spilling
// (the library sine's reduction of huge arguments does)
std::string describe_spills(const std::vector<char>& code, bool everything) {
    std::string text;
    for (auto& ks : code_object_spills(code))
        if (ks.vector > 0 || (everything && (ks.scalar > 0 || ks.scratch_bytes > 0)))
            text += strf("%s%s (%ld scalar, %ld vector registers spilled, %ld bytes of scratch per lane)", text.empty() ? "" : "; ",
                         ks.name.c_str(), ks.scalar, ks.vector, ks.scratch_bytes);
    return text;
}

// Lowers a program and compiles the kernels that `have` does not know yet into `objects` (by source text).  A kernel
// that the compiler could only build by spilling vector registers to scratch memory is never accepted: the regions
// it belongs to are lowered again with their kernel-size bounds halved (LowerOptions::region_shift), up to four
// times, and if a kernel still spills then -- or is not one the lowering can cut: a hand-written one -- the program
// is refused.  `relowered` receives the number of extra lowerings.
template <class Have>
std::unique_ptr<Plan> lower_and_compile(const Proc& ir, const std::vector<std::string>& deps, const std::string& arch, Have&& have,
                                        std::map<std::string, std::vector<char>>& objects, int* relowered = nullptr) {
    LowerOptions opt;
    for (int attempt = 0;; ++attempt) {
        std::unique_ptr<Plan> plan = lower_program(ir, deps, opt);
        std::vector<std::string> missing;
        for (const KernelDef& k : plan->kernels)
            if (!objects.count(k.source) && !have(k.source)) missing.push_back(k.source);
        for (auto& kv : compile_code_objects(missing, arch)) objects[kv.first] = std::move(kv.second);
        std::set<int> regions;
        std::string report;
        for (const KernelDef& k : plan->kernels) {
            auto it = objects.find(k.source);
            if (it == objects.end()) continue;  // loaded before, so accepted before
            for (const KernelSpills& ks : code_object_spills(it->second)) {
                if (ks.vector <= 0) continue;
                report += strf("%s%s [%s] (%ld vector, %ld scalar registers spilled, %ld bytes of scratch per lane)", report.empty() ? "" : "; ",
                               ks.name.c_str(), k.kind.c_str(), ks.vector, ks.scalar, ks.scratch_bytes);
                for (int r : k.regions)
                    if (r >= 0) regions.insert(r);
            }
        }
        if (relowered) *relowered = attempt;
        if (report.empty()) return plan;
        bool tighter = false;
        for (int r : regions) {
            int& sh = opt.region_shift[r];
            if (sh < 4) { ++sh; tighter = true; }
        }
        ADHIP_CHECK(tighter && attempt < 4,
                    "refusing to run kernels that spill vector registers to scratch memory (after %d lowerings with tighter bounds): %s",
                    attempt, report.c_str());
    }
}

std::shared_ptr<Module> compile_module(adhip_ctx* ctx, const std::string& source, const std::vector<char>* code_in = nullptr) {
    auto it = ctx->modules.find(source);
    if (it != ctx->modules.end()) return it->second;
    std::vector<char> code = code_in ? *code_in : compile_code_object(source, ctx->arch);
    auto m = std::make_shared<Module>();
    HIP_OK(hipModuleLoadData(&m->mod, code.data()));
    // a long-lived context that keeps seeing new programs does not keep every module it ever loaded: beyond a
    // bound, the ones no live program refers to are unloaded (their code objects stay in the on-disk cache)
    if (ctx->modules.size() >= 1024) {
        for (auto it2 = ctx->modules.begin(); it2 != ctx->modules.end();) {
            if (it2->second.use_count() == 1) it2 = ctx->modules.erase(it2);
            else ++it2;
        }
    }
    ctx->modules[source] = m;
    return m;
}

hipFunction_t get_function(Module& m, const std::string& entry) {
    auto it = m.fns.find(entry);
    if (it != m.fns.end()) return it->second;
    hipFunction_t f;
    HIP_OK(hipModuleGetFunction(&f, m.mod, entry.c_str()));
    m.fns[entry] = f;
    return f;
}

void program_free(adhip_program* p) {
    if (!p) return;
    if (p->ctx) (void)hipSetDevice(p->ctx->device);
    for (auto& pe : p->pending) { (void)hipEventDestroy(pe.second.first); (void)hipEventDestroy(pe.second.second); }
    for (auto e : p->event_pool) (void)hipEventDestroy(e);
    for (auto& g : p->graphs) (void)hipGraphExecDestroy(g.second);
    for (auto g : p->graph_objs) (void)hipGraphDestroy(g);
    for (void* q : p->owned) (void)hipFree(q);
    delete p;
}

std::vector<std::string> dep_vector(const char* const* dep_ids, size_t n) {
    std::vector<std::string> d;
    for (size_t i = 0; i < n; ++i)
        if (dep_ids && dep_ids[i]) d.emplace_back(dep_ids[i]);
    return d;
}

adhip_program* program_create(adhip_ctx* ctx, const uint8_t* program, size_t len, const char* const* dep_ids, size_t n,
                              std::vector<size_t>* payload_offsets = nullptr) {
    HIP_OK(hipSetDevice(ctx->device));
    std::unique_ptr<adhip_program> p(new adhip_program());
    p->ctx = ctx;
    const char* genv = getenv("ADHIP_GRAPHS");
    if (genv && *genv == '0') p->use_graphs = false;
    p->ir = parse_program(program, len, payload_offsets);
    std::map<std::string, std::vector<char>> fresh;
    // kernels: what the context has not loaded yet is compiled (or fetched from the disk cache) in parallel
    p->plan = lower_and_compile(*p->ir, dep_vector(dep_ids, n), ctx->arch, [&](const std::string& src) { return ctx->modules.count(src) != 0; }, fresh);
    Plan& plan = *p->plan;
    try {
        for (const KernelDef& k : plan.kernels) {
            auto f = fresh.find(k.source);
            auto m = compile_module(ctx, k.source, f != fresh.end() ? &f->second : nullptr);
            p->mods.push_back(m);
            p->fn.push_back(get_function(*m, k.entry));
        }
        // buffers: one allocation per home / constant buffer, one per temp slot
        std::vector<void*> slot_ptr(plan.slot_elems.size(), nullptr);
        for (size_t s = 0; s < plan.slot_elems.size(); ++s) {
            void* q = nullptr;
            HIP_OK(hipMalloc(&q, (size_t)std::max<int64_t>(plan.slot_elems[s], 1) * sizeof(float)));
            p->owned.push_back(q);
            p->device_bytes += (size_t)std::max<int64_t>(plan.slot_elems[s], 1) * sizeof(float);
            slot_ptr[s] = q;
        }
        if (plan.n_flags > 0) {
            void* q = nullptr;
            HIP_OK(hipMalloc(&q, (size_t)plan.n_flags * sizeof(int)));
            p->owned.push_back(q);
            p->flags = (int*)q;
            auto m = compile_module(ctx, fixed_kernels_source());
            p->mods.push_back(m);
            p->flag_fn = get_function(*m, "adhip_flag");
        }
        p->buf_ptr.resize(plan.buffers.size(), nullptr);
        p->arena_off.assign(plan.buffers.size(), SIZE_MAX);
        {
            // the arena: uploaded small buffers, then small results, then the other small ones, 256-byte aligned each,
            // as long as everything fits half the staging area
            std::set<int> result_bufs;
            for (auto& kv : plan.results) result_bufs.insert(kv.second.buf);
            size_t total = 0;
            for (int pass = 0; pass < 3; ++pass) {
                for (size_t i = 0; i < plan.buffers.size(); ++i) {
                    const PlanBuffer& b = plan.buffers[i];
                    if (b.kind == PlanBuffer::TEMP || p->arena_off[i] != SIZE_MAX) continue;
                    const size_t nb = (size_t)std::max<int64_t>(b.elems, 1) * sizeof(float);
                    const bool uploaded = b.host && b.host_elems > 0;
                    const int cls = uploaded ? 0 : (result_bufs.count((int)i) ? 1 : 2);
                    if (cls != pass || nb > kStageMaxItem || total + nb > kStageBytes / 2) continue;  // half: the rest stages what is not in the arena
                    p->arena_off[i] = total;
                    total += (nb + 255) & ~size_t(255);
                }
                if (pass == 0) p->arena_upload_bytes = total;
            }
            if (total > 0) {
                void* q = nullptr;
                HIP_OK(hipMalloc(&q, total));
                p->owned.push_back(q);
                p->device_bytes += total;
                p->arena = (char*)q;
            }
        }
        for (size_t i = 0; i < plan.buffers.size(); ++i) {
            const PlanBuffer& b = plan.buffers[i];
            if (b.kind == PlanBuffer::TEMP) { p->buf_ptr[i] = slot_ptr[b.slot]; continue; }
            if (p->arena_off[i] != SIZE_MAX) { p->buf_ptr[i] = p->arena + p->arena_off[i]; continue; }
            void* q = nullptr;
            HIP_OK(hipMalloc(&q, (size_t)std::max<int64_t>(b.elems, 1) * sizeof(float)));
            p->owned.push_back(q);
            p->device_bytes += (size_t)std::max<int64_t>(b.elems, 1) * sizeof(float);
            p->buf_ptr[i] = q;
        }
        // where the temporaries and the flags would sit in the static scratch area (256-byte aligned slots)
        {
            std::vector<size_t> slot_off(plan.slot_elems.size(), 0);
            size_t need = 0;
            for (size_t s = 0; s < plan.slot_elems.size(); ++s) {
                slot_off[s] = need;
                need += (((size_t)std::max<int64_t>(plan.slot_elems[s], 1) * sizeof(float)) + 255) & ~size_t(255);
            }
            const size_t flags_off = need;
            need += (((size_t)plan.n_flags * sizeof(int)) + 255) & ~size_t(255);
            p->static_need = need;
            if (ctx->static_scratch && need <= (size_t)ADHIP_STATIC_SCRATCH_BYTES) {
                p->static_buf_ptr = p->buf_ptr;
                for (size_t i = 0; i < plan.buffers.size(); ++i)
                    if (plan.buffers[i].kind == PlanBuffer::TEMP) p->static_buf_ptr[i] = ctx->static_scratch + slot_off[(size_t)plan.buffers[i].slot];
                p->static_flags = (int*)(ctx->static_scratch + flags_off);
            }
        }
    } catch (...) {
        program_free(p.release());
        throw;
    }
    return p.release();
}

// `wait`: return only when the copies are done (a caller of adhip_program_upload may reuse its payload memory then)
void program_upload(adhip_program* p, bool wait = true) {
    adhip_ctx* ctx = p->ctx;
    HIP_OK(hipSetDevice(ctx->device));
    Plan& plan = *p->plan;
    size_t staged = 0;
    if (p->arena_upload_bytes > 0) {
        // the small payloads, laid out as they sit in the arena, in one copy
        memset(ctx->stage, 0, p->arena_upload_bytes);
        for (size_t i = 0; i < plan.buffers.size(); ++i) {
            const PlanBuffer& b = plan.buffers[i];
            if (p->arena_off[i] < p->arena_upload_bytes && b.host && b.host_elems > 0)
                memcpy(ctx->stage + p->arena_off[i], b.host, (size_t)b.host_elems * sizeof(float));
        }
        HIP_OK(hipMemcpyAsync(p->arena, ctx->stage, p->arena_upload_bytes, hipMemcpyHostToDevice, ctx->stream));
        staged = p->arena_upload_bytes;
    }
    for (size_t i = 0; i < plan.buffers.size(); ++i) {
        const PlanBuffer& b = plan.buffers[i];
        if (b.kind == PlanBuffer::TEMP) continue;
        if (p->arena_off[i] < p->arena_upload_bytes && b.host && b.host_elems > 0) continue;  // went up with the arena
        if (b.host && b.host_elems > 0) {
            const size_t nb = (size_t)b.host_elems * sizeof(float);
            const void* src = b.host;
            if (nb <= kStageMaxItem) {
                // small payloads go through pinned memory, so that the copies queue up instead of each one waiting
                if (staged + nb > kStageBytes) {
                    HIP_OK(hipStreamSynchronize(ctx->stream));
                    staged = 0;
                }
                memcpy(ctx->stage + staged, b.host, nb);
                src = ctx->stage + staged;
                staged += (nb + 255) & ~size_t(255);
            }
            HIP_OK(hipMemcpyAsync(p->buf_ptr[i], src, nb, hipMemcpyHostToDevice, ctx->stream));
        } else if (b.kind == PlanBuffer::HOME && b.zero_init) {
            HIP_OK(hipMemsetAsync(p->buf_ptr[i], 0, (size_t)std::max<int64_t>(b.elems, 1) * sizeof(float), ctx->stream));
        }
    }
    if (wait) HIP_OK(hipStreamSynchronize(ctx->stream));
}

hipEvent_t get_event(adhip_program* p) {
    if (!p->event_pool.empty()) {
        hipEvent_t e = p->event_pool.back();
        p->event_pool.pop_back();
        return e;
    }
    hipEvent_t e;
    HIP_OK(hipEventCreate(&e));
    return e;
}

void drain_events(adhip_program* p) {
    for (auto& pe : p->pending) {
        float ms = 0;
        HIP_OK(hipEventSynchronize(pe.second.second));
        HIP_OK(hipEventElapsedTime(&ms, pe.second.first, pe.second.second));
        KernelStat& st = p->plan->stats[pe.first];
        st.total_ms += ms;
        p->event_pool.push_back(pe.second.first);
        p->event_pool.push_back(pe.second.second);
    }
    p->pending.clear();
}

int* cur_flags(adhip_program* p) { return p->use_static ? p->static_flags : p->flags; }
void* cur_buf(adhip_program* p, int buf) { return p->use_static ? p->static_buf_ptr[(size_t)buf] : p->buf_ptr[(size_t)buf]; }

void launch(adhip_program* p, const Launch& l) {
    adhip_ctx* ctx = p->ctx;
    // argument block: guard pointer, then the plan's arguments; on the stack, so that a run allocates nothing on the
    // host either
    const void* guard = l.guard >= 0 ? (const void*)(cur_flags(p) + l.guard) : nullptr;
    constexpr size_t kStackArgs = 192;  // merged launches take at most 160 arguments, shared ones 96 pointers
    void* ptrs[kStackArgs + 1];
    uint64_t vals[kStackArgs];
    ADHIP_CHECK(l.args.size() <= kStackArgs, "internal: launch '%s' takes %zu arguments", l.label.c_str(), l.args.size());
    ptrs[0] = (void*)&guard;
    for (size_t i = 0; i < l.args.size(); ++i) {
        const Arg& a = l.args[i];
        switch (a.kind) {
        case Arg::BUF: {
            char* base = (char*)cur_buf(p, a.buf);
            void* q = base + a.off * (int64_t)sizeof(float);
            memcpy(&vals[i], &q, sizeof q);
            break;
        }
        case Arg::I32: { int v = (int)a.iv; memcpy(&vals[i], &v, sizeof v); break; }
        case Arg::I64: { long long v = a.iv; memcpy(&vals[i], &v, sizeof v); break; }
        case Arg::F32: { memcpy(&vals[i], &a.fv, sizeof a.fv); break; }
        case Arg::FLAG: { int* q = cur_flags(p) + a.iv; memcpy(&vals[i], &q, sizeof q); break; }
        }
        ptrs[i + 1] = &vals[i];
    }
    if (p->profiling && !p->use_static) {
        // the launch carries its own start and stop events, which take the kernel's begin and end on the device
        // (events recorded around the launch would include the dispatch gap before it)
        hipEvent_t e0 = get_event(p), e1 = get_event(p);
        const uint64_t gx = (uint64_t)l.grid[0] * l.block[0], gy = (uint64_t)l.grid[1] * l.block[1],
                       gz = (uint64_t)l.grid[2] * l.block[2];
        if (gx <= 0xffffffffull && gy <= 0xffffffffull && gz <= 0xffffffffull) {
            HIP_OK(hipExtModuleLaunchKernel(p->fn[l.kernel], (uint32_t)gx, (uint32_t)gy, (uint32_t)gz, l.block[0], l.block[1],
                                            l.block[2], l.lds_bytes, ctx->stream, ptrs, nullptr, e0, e1, 0));
        } else {
            HIP_OK(hipEventRecord(e0, ctx->stream));
            HIP_OK(hipModuleLaunchKernel(p->fn[l.kernel], l.grid[0], l.grid[1], l.grid[2], l.block[0], l.block[1], l.block[2],
                                         l.lds_bytes, ctx->stream, ptrs, nullptr));
            HIP_OK(hipEventRecord(e1, ctx->stream));
        }
        p->pending.push_back({l.stat, {e0, e1}});
        if (p->pending.size() > 4096) drain_events(p);
    } else {
        HIP_OK(hipModuleLaunchKernel(p->fn[l.kernel], l.grid[0], l.grid[1], l.grid[2], l.block[0], l.block[1], l.block[2],
                                     l.lds_bytes, ctx->stream, ptrs, nullptr));
    }
    p->plan->stats[l.stat].launches++;
}

void launch_flag(adhip_program* p, int slot, int parent, int cond_buf, int mode, int taken) {
    int* flags = cur_flags(p);
    const float* cond = cond_buf >= 0 ? (const float*)cur_buf(p, cond_buf) : nullptr;
    void* args[] = {&flags, &slot, &parent, &cond, &mode, &taken};
    HIP_OK(hipModuleLaunchKernel(p->flag_fn, 1, 1, 1, 64, 1, 1, 0, p->ctx->stream, args, nullptr));
    p->flag_launches++;
}

float read_scalar(adhip_program* p, int buf, int slot) {
    adhip_ctx* ctx = p->ctx;
    HIP_OK(hipMemcpyAsync(ctx->pinned + slot, cur_buf(p, buf), sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    return 0.f;
}

// A run of at least eight consecutive kernel launches is captured once into a hipGraph and replayed with a
// single submission afterwards (kernel arguments are fixed device pointers and constants, so the captured
// nodes never need updating).  Per-kernel profiling and ADHIP_GRAPHS=0 bypass this.
bool replay_run(adhip_program* p, const std::vector<Step>& steps, size_t first, size_t last) {
    if (!p->use_graphs || p->profiling || p->use_static || last - first < 8) return false;
    adhip_ctx* ctx = p->ctx;
    auto key = std::make_pair((const void*)&steps, first);
    auto it = p->graphs.find(key);
    // the first time a run is met it is launched directly: a program that runs once never pays for a capture
    if (it == p->graphs.end() && p->seen_runs.insert(key).second) return false;
    if (it == p->graphs.end()) {
        hipGraph_t graph = nullptr;
        HIP_OK(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
        try {
            for (size_t i = first; i < last; ++i) launch(p, steps[i].launch);
        } catch (...) {
            (void)hipStreamEndCapture(ctx->stream, &graph);
            if (graph) (void)hipGraphDestroy(graph);
            throw;
        }
        HIP_OK(hipStreamEndCapture(ctx->stream, &graph));
        hipGraphExec_t exec = nullptr;
        HIP_OK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        p->graph_objs.push_back(graph);
        it = p->graphs.emplace(key, exec).first;
    } else {
        for (size_t i = first; i < last; ++i) p->plan->stats[steps[i].launch.stat].launches++;
    }
    HIP_OK(hipGraphLaunch(it->second, ctx->stream));
    return true;
}

void exec_steps(adhip_program* p, const std::vector<Step>& steps) {
    adhip_ctx* ctx = p->ctx;
    for (size_t si = 0; si < steps.size(); ++si) {
        const Step& s = steps[si];
        if (p->exited) return;
        switch (s.kind) {
        case Step::LAUNCH: {
            size_t last = si;
            while (last < steps.size() && steps[last].kind == Step::LAUNCH) ++last;
            if (replay_run(p, steps, si, last)) si = last - 1;
            else launch(p, s.launch);
            break;
        }
        case Step::EXIT: p->exited = true; return;
        case Step::LOOP: {
            if (s.counter_buf >= 0) {
                // counted loop: one read of (cond, x) at entry decides the trip count
                read_scalar(p, s.cond_buf, 0);
                read_scalar(p, s.counter_buf, 1);
                HIP_OK(hipStreamSynchronize(ctx->stream));
                float cond = ctx->pinned[0], x = ctx->pinned[1];
                int64_t n = 0;
                while (cond != 0.0f) {
                    ++n;
                    x = x + s.counter_inc;
                    float t = x + s.counter_add;
                    cond = (t < 0.0f) ? 1.0f : 0.0f;
                    if (n > (int64_t(1) << 40)) throw Error("counted loop does not terminate");
                    if (x + s.counter_inc == x && cond != 0.0f) throw Error("counted loop does not terminate (counter saturated)");
                }
                for (int64_t i = 0; i < n && !p->exited; ++i) exec_steps(p, s.body);
            } else if (s.flag_slot >= 0) {
                // device-predicated: enqueue a batch of iterations, then look at the predicate once
                // (when the body's last kernel latches the flag for the next iteration itself, the one-thread kernel
                // that does so runs before the first iteration only)
                int batch = 4;
                bool first = true;
                while (true) {
                    for (int b = 0; b < batch; ++b) {
                        if (first || !s.latch_in_body) launch_flag(p, s.flag_slot, s.parent_guard, s.cond_buf, 0, -1);
                        first = false;
                        exec_steps(p, s.body);
                    }
                    read_scalar(p, s.cond_buf, 0);
                    HIP_OK(hipMemcpyAsync(ctx->pinned + 1, cur_flags(p) + s.flag_slot, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
                    HIP_OK(hipStreamSynchronize(ctx->stream));
                    int flag;
                    memcpy(&flag, ctx->pinned + 1, sizeof flag);
                    if (flag == 0 || ctx->pinned[0] == 0.0f) break;
                    if (batch < 32) batch *= 2;
                }
            } else {
                while (!p->exited) {
                    read_scalar(p, s.cond_buf, 0);
                    HIP_OK(hipStreamSynchronize(ctx->stream));
                    if (ctx->pinned[0] == 0.0f) break;
                    exec_steps(p, s.body);
                }
            }
            break;
        }
        case Step::BRANCH: {
            if (s.taken_slot >= 0) {
                // inside a predicated loop: every arm is enqueued under its own device flag
                launch_flag(p, s.taken_slot, -1, -1, 3, -1);
                for (size_t i = 0; i < s.arms.size(); ++i) {
                    launch_flag(p, s.arm_slots[i], s.parent_guard, s.arms[i].first, 1, s.taken_slot);
                    exec_steps(p, s.arms[i].second);
                }
                if (s.else_slot >= 0) {
                    launch_flag(p, s.else_slot, s.parent_guard, -1, 2, s.taken_slot);
                    exec_steps(p, s.else_body);
                }
                break;
            }
            // the predicates are read 64 at a time (the size of the pinned area); the first arm whose predicate is 1 runs
            bool ran = false;
            for (size_t i0 = 0; i0 < s.arms.size() && !ran; i0 += 64) {
                const size_t i1 = std::min(s.arms.size(), i0 + 64);
                for (size_t i = i0; i < i1; ++i) read_scalar(p, s.arms[i].first, (int)(i - i0));
                HIP_OK(hipStreamSynchronize(ctx->stream));
                for (size_t i = i0; i < i1; ++i) {
                    if (ctx->pinned[i - i0] == 1.0f) {
                        exec_steps(p, s.arms[i].second);
                        ran = true;
                        break;
                    }
                }
            }
            if (!ran) exec_steps(p, s.else_body);
            break;
        }
        }
    }
}

void program_run(adhip_program* p, bool wait = true) {
    adhip_ctx* ctx = p->ctx;
    HIP_OK(hipSetDevice(ctx->device));
    p->exited = false;
    exec_steps(p, p->plan->steps);
    if (!wait) return;
    HIP_OK(hipStreamSynchronize(ctx->stream));
    if (p->profiling) drain_events(p);
}

void program_readback(adhip_program* p) {
    adhip_ctx* ctx = p->ctx;
    HIP_OK(hipSetDevice(ctx->device));
    // host buffers of the previous read-back are reused where an id comes back again: fresh pages of a large
    // result cost more than the copy itself
    std::map<std::string, HostResult> previous;
    previous.swap(ctx->results);
    struct Staged { HostResult* r; size_t off, nb; };
    std::vector<Staged> staged;
    size_t used = 0;
    size_t reserved = 0;  // the head of the staging area that holds the arena's stretch until the last result is out
    auto drain = [&] {
        HIP_OK(hipStreamSynchronize(ctx->stream));
        for (auto& st : staged) memcpy(st.r->data.data(), ctx->stage + st.off, st.nb);
        staged.clear();
        used = reserved;
    };
    // the small results that live in the arena come back in one copy of the stretch they span
    size_t span_lo = SIZE_MAX, span_hi = 0;
    for (auto& kv : p->plan->results) {
        const size_t off = p->arena_off[(size_t)kv.second.buf];
        const int64_t ne = numel(kv.second.shape);
        if (off == SIZE_MAX || ne <= 0) continue;
        span_lo = std::min(span_lo, off);
        span_hi = std::max(span_hi, off + (size_t)ne * sizeof(float));
    }
    const bool span = span_lo < span_hi && span_hi - span_lo <= kStageBytes;
    if (span) {
        HIP_OK(hipMemcpyAsync(ctx->stage, p->arena + span_lo, span_hi - span_lo, hipMemcpyDeviceToHost, ctx->stream));
        reserved = used = (span_hi - span_lo + 255) & ~size_t(255);
    }
    for (auto& kv : p->plan->results) {
        HostResult& r = ctx->results[kv.first];
        auto prev = previous.find(kv.first);
        if (prev != previous.end()) r = std::move(prev->second);
        r.dims.clear();
        for (auto d : kv.second.shape) r.dims.push_back((uint64_t)d);
        const int64_t ne = numel(kv.second.shape);
        const size_t nb = (size_t)std::max<int64_t>(ne, 0) * sizeof(float);
        if (nb >= kPinnedResultBytes) {
            if (r.pinned_elems < (size_t)ne) {
                r.release();
                HIP_OK(hipHostMalloc((void**)&r.pinned, nb, hipHostMallocDefault));
                r.pinned_elems = (size_t)ne;
            }
            r.data.clear();
            HIP_OK(hipMemcpyAsync(r.pinned, p->buf_ptr[kv.second.buf], nb, hipMemcpyDeviceToHost, ctx->stream));
            continue;
        }
        r.release();
        r.data.resize((size_t)std::max<int64_t>(ne, 0));
        if (ne <= 0) continue;
        if (span && p->arena_off[(size_t)kv.second.buf] != SIZE_MAX) {
            staged.push_back({&r, p->arena_off[(size_t)kv.second.buf] - span_lo, nb});
            continue;
        }
        if (nb <= kStageMaxItem) {
            if (used + nb > kStageBytes) drain();
            HIP_OK(hipMemcpyAsync(ctx->stage + used, p->buf_ptr[kv.second.buf], nb, hipMemcpyDeviceToHost, ctx->stream));
            staged.push_back({&r, used, nb});
            used += (nb + 255) & ~size_t(255);
        } else {
            HIP_OK(hipMemcpyAsync(r.data.data(), p->buf_ptr[kv.second.buf], nb, hipMemcpyDeviceToHost, ctx->stream));
        }
    }
    drain();
}

template <class F>
int guarded(adhip_ctx* ctx, F&& f) {
    try {
        f();
        return 0;
    } catch (const std::exception& e) {
        if (ctx) ctx->last_error = e.what();
        g_tls_error = e.what();
        return 2;
    } catch (...) {
        if (ctx) ctx->last_error = "unknown error";
        g_tls_error = "unknown error";
        return 2;
    }
}

}  // namespace

extern "C" {

const char* adhip_version(void) { return "adhip 0.1 (gfx950)"; }

int adhip_create(int device_ordinal, adhip_ctx** out) {
    if (!out) return 2;
    *out = nullptr;
    return guarded(nullptr, [&] {
        int n = 0;
        HIP_OK(hipGetDeviceCount(&n));
        ADHIP_CHECK(device_ordinal >= 0 && device_ordinal < n, "HIP device %d not available (%d devices)", device_ordinal, n);
        HIP_OK(hipSetDevice(device_ordinal));
        std::unique_ptr<adhip_ctx> ctx(new adhip_ctx());
        ctx->device = device_ordinal;
        hipDeviceProp_t prop;
        HIP_OK(hipGetDeviceProperties(&prop, device_ordinal));
        std::string arch = prop.gcnArchName;
        size_t colon = arch.find(':');
        if (colon != std::string::npos) arch = arch.substr(0, colon);
        ctx->arch = arch;
        HIP_OK(hipStreamCreate(&ctx->stream));
        HIP_OK(hipHostMalloc((void**)&ctx->pinned, 64 * sizeof(float), hipHostMallocDefault));
        HIP_OK(hipHostMalloc((void**)&ctx->stage, kStageBytes, hipHostMallocDefault));
        // this device's copy of the static scratch area (the device is current, see hipSetDevice above)
        void* sp = nullptr;
        const hipError_t se = hipGetSymbolAddress(&sp, HIP_SYMBOL(adhip_static_scratch));
        if (se == hipSuccess && sp) ctx->static_scratch = (unsigned char*)sp;
        else {
            ctx->static_scratch_error = strf("hipGetSymbolAddress(adhip_static_scratch) failed: %s", hipGetErrorString(se));
            (void)hipGetLastError();  // the failure concerns adhip_program_enqueue_noalloc only; do not leave it pending
        }
        *out = ctx.release();
    });
}

void adhip_destroy(adhip_ctx* ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    for (auto& e : ctx->exec_cache) program_free(e.prog);
    ctx->exec_cache.clear();
    ctx->modules.clear();
    if (ctx->pinned) (void)hipHostFree(ctx->pinned);
    if (ctx->stage) (void)hipHostFree(ctx->stage);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

const char* adhip_last_error(adhip_ctx* ctx) { return ctx ? ctx->last_error.c_str() : g_tls_error.c_str(); }

int adhip_execute(adhip_ctx* ctx, const uint8_t* program, size_t program_len, const char* const* dep_ids, size_t n_dep_ids) {
    if (!ctx) return 2;
    return guarded(ctx, [&] {
        // results of an earlier call stay in place until the read-back replaces them (it reuses their host
        // buffers); a call that fails leaves none visible
        struct ClearOnFailure {
            adhip_ctx* c;
            bool ok = false;
            ~ClearOnFailure() { if (!ok) c->results.clear(); }
        } results_guard{ctx};
        const char* cenv = getenv("ADHIP_EXEC_CACHE");
        const bool caching = !(cenv && *cenv == '0');
        adhip_program* p = nullptr;
        std::string key;
        std::vector<size_t> offs;
        std::vector<const float*> ptrs;
        if (caching && program && program_len >= 8) {
            // key: the stream with every payload pointer blanked, plus the keep list
            parse_program(program, program_len, &offs);
            key.assign((const char*)program, program_len);
            for (size_t o : offs) {
                uint64_t v;
                memcpy(&v, program + o, 8);
                ptrs.push_back((const float*)(uintptr_t)v);
                memset(&key[o], 0, 8);
            }
            for (const std::string& d : dep_vector(dep_ids, n_dep_ids)) { key.push_back('\0'); key += d; }
            key.push_back('\0');
            key += lowering_switches();  // a plan made under other switches is another program
            for (size_t i = 0; i < ctx->exec_cache.size(); ++i) {
                if (ctx->exec_cache[i].key != key) continue;
                adhip_program* q = ctx->exec_cache[i].prog;
                // the kept program can be re-bound if payloads that shared a pointer before still share one
                bool ok = q->payloads.size() == ptrs.size();
                for (size_t a = 0; ok && a < ptrs.size(); ++a)
                    for (size_t b = a + 1; ok && b < ptrs.size(); ++b)
                        if (q->payloads[a] == q->payloads[b] && ptrs[a] != ptrs[b]) ok = false;
                auto entry = std::move(ctx->exec_cache[i]);
                ctx->exec_cache.erase(ctx->exec_cache.begin() + (long)i);
                if (ok) {
                    for (size_t bi = 0; bi < q->plan->buffers.size(); ++bi)
                        if (q->payload_of[bi] >= 0) q->plan->buffers[bi].host = ptrs[(size_t)q->payload_of[bi]];
                    q->payloads = ptrs;
                    ctx->exec_cache.insert(ctx->exec_cache.begin(), std::move(entry));
                    p = q;
                } else {
                    program_free(q);
                }
                break;
            }
        }
        const bool reused = p != nullptr;
        if (!p) {
            offs.clear();
            p = program_create(ctx, program, program_len, dep_ids, n_dep_ids, &offs);
        }
        bool keep = reused;
        try {
            if (!reused && caching && p->device_bytes <= kExecCacheBytes) {
                p->payloads = ptrs;
                p->payload_of.assign(p->plan->buffers.size(), -1);
                keep = true;
                for (size_t bi = 0; bi < p->plan->buffers.size() && keep; ++bi) {
                    const float* h = p->plan->buffers[bi].host;
                    if (!h) continue;
                    for (size_t a = 0; a < ptrs.size(); ++a)
                        if (ptrs[a] == h) { p->payload_of[bi] = (int)a; break; }
                    if (p->payload_of[bi] < 0) keep = false;  // a payload the stream does not name: cannot be re-bound
                }
                if (keep) {
                    ctx->exec_cache.insert(ctx->exec_cache.begin(), {key, p, p->device_bytes});
                    size_t total = 0, n_keep = 0;
                    for (; n_keep < ctx->exec_cache.size() && n_keep < kExecCacheEntries; ++n_keep) {
                        if (total + ctx->exec_cache[n_keep].bytes > kExecCacheBytes && n_keep > 0) break;
                        total += ctx->exec_cache[n_keep].bytes;
                    }
                    while (ctx->exec_cache.size() > n_keep) {
                        program_free(ctx->exec_cache.back().prog);
                        ctx->exec_cache.pop_back();
                    }
                }
            }
            // one wait for the whole call: uploads, kernels and read-back copies are ordered by the stream, and the
            // read-back ends with the wait that also covers the staging area both ends use
            program_upload(p, false);
            program_run(p, p->profiling);
            program_readback(p);
        } catch (...) {
            // a program that failed is not kept
            for (size_t i = 0; i < ctx->exec_cache.size(); ++i)
                if (ctx->exec_cache[i].prog == p) { ctx->exec_cache.erase(ctx->exec_cache.begin() + (long)i); break; }
            program_free(p);
            throw;
        }
        if (!keep) program_free(p);
        results_guard.ok = true;
    });
}

int adhip_get_tensor(adhip_ctx* ctx, const char* id, const float** data, const uint64_t** dims, size_t* ndim) {
    if (!ctx || !id || !data || !dims || !ndim) return 2;
    auto it = ctx->results.find(id);
    if (it == ctx->results.end()) return 1;
    *data = it->second.ptr();
    *dims = it->second.dims.data();
    *ndim = it->second.dims.size();
    return 0;
}

int adhip_dot_prod_shape(const uint64_t* a_dims, size_t a_ndim, const uint64_t* b_dims, size_t b_ndim, uint64_t out[2]) {
    if (!a_dims || !b_dims || !out || a_ndim == 0 || b_ndim == 0) return 2;
    out[0] = a_dims[0];
    out[1] = b_dims[b_ndim - 1];
    return 0;
}

int adhip_program_create(adhip_ctx* ctx, const uint8_t* program, size_t program_len, const char* const* dep_ids,
                         size_t n_dep_ids, adhip_program** out) {
    if (!ctx || !out) return 2;
    *out = nullptr;
    return guarded(ctx, [&] { *out = program_create(ctx, program, program_len, dep_ids, n_dep_ids); });
}

int adhip_program_upload(adhip_program* p) {
    if (!p) return 2;
    return guarded(p->ctx, [&] { program_upload(p); });
}

int adhip_program_run(adhip_program* p) {
    if (!p) return 2;
    return guarded(p->ctx, [&] { program_run(p); });
}

int adhip_program_enqueue(adhip_program* p) {
    if (!p) return 2;
    return guarded(p->ctx, [&] { program_run(p, false); });
}

int adhip_program_enqueue_noalloc(adhip_program* p) {
    if (!p) return 2;
    return guarded(p->ctx, [&] {
        adhip_ctx* ctx = p->ctx;
        ADHIP_CHECK(ctx->static_scratch, "adhip_program_enqueue_noalloc: the static scratch area is not available on this device (%s)",
                    ctx->static_scratch_error.c_str());
        ADHIP_CHECK(p->static_need <= (size_t)ADHIP_STATIC_SCRATCH_BYTES && !p->static_buf_ptr.empty(),
                    "adhip_program_enqueue_noalloc: the program needs %zu bytes of scratch memory, the static area holds %zu",
                    p->static_need, (size_t)ADHIP_STATIC_SCRATCH_BYTES);
        struct Restore {
            adhip_program* q;
            ~Restore() { q->use_static = false; }
        } restore{p};
        p->use_static = true;
        program_run(p, false);
    });
}

int adhip_program_sync(adhip_program* p) {
    if (!p) return 2;
    return guarded(p->ctx, [&] {
        HIP_OK(hipSetDevice(p->ctx->device));
        HIP_OK(hipStreamSynchronize(p->ctx->stream));
        if (p->profiling) drain_events(p);
    });
}

int adhip_program_readback(adhip_program* p) {
    if (!p) return 2;
    return guarded(p->ctx, [&] { program_readback(p); });
}

void adhip_program_destroy(adhip_program* p) { program_free(p); }

int adhip_program_set_profiling(adhip_program* p, int enabled) {
    if (!p) return 2;
    p->profiling = enabled != 0;
    return 0;
}

int adhip_program_kernel_count(adhip_program* p) { return p ? (int)p->plan->stats.size() : 0; }

int adhip_program_kernel_stat(adhip_program* p, int i, char* label, size_t label_cap, uint64_t* launches, double* total_ms,
                              double* bytes_per_launch, double* flops_per_launch) {
    if (!p || i < 0 || i >= (int)p->plan->stats.size()) return 2;
    const KernelStat& s = p->plan->stats[i];
    if (label && label_cap) {
        std::string l = s.kind + ":" + s.label;
        snprintf(label, label_cap, "%s", l.c_str());
    }
    if (launches) *launches = s.launches;
    if (total_ms) *total_ms = s.total_ms;
    if (bytes_per_launch) *bytes_per_launch = s.bytes;
    if (flops_per_launch) *flops_per_launch = s.flops;
    return 0;
}

const char* adhip_program_kernel_source(adhip_program* p, int i) {
    if (!p || i < 0 || i >= (int)p->plan->stats.size()) return "";
    return p->plan->kernels[p->plan->stats[i].kernel].source.c_str();
}

const char* adhip_program_describe(adhip_program* p) {
    if (!p) return "";
    p->description = p->plan->describe();
    return p->description.c_str();
}

int adhip_lower_describe(const uint8_t* program, size_t program_len, const char* const* dep_ids, size_t n_dep_ids, char* out,
                         size_t out_cap) {
    if (!out || out_cap == 0) return 2;
    std::string text;
    int rc = guarded(nullptr, [&] {
        auto ir = parse_program(program, program_len);
        auto plan = lower_program(*ir, dep_vector(dep_ids, n_dep_ids));
        text = plan->describe();
        const char* dump = getenv("ADHIP_DUMP_SOURCE");
        if (dump && *dump == '1')
            for (auto& k : plan->kernels) text += "\n// ===== " + k.entry + " [" + k.kind + "] =====\n" + k.source;
    });
    if (rc != 0) text = g_tls_error;
    snprintf(out, out_cap, "%s", text.c_str());
    return rc;
}

int adhip_compile_check(const uint8_t* program, size_t program_len, const char* const* dep_ids, size_t n_dep_ids,
                        const char* arch, char* out, size_t out_cap) {
    if (!out || out_cap == 0) return 2;
    std::string text;
    int rc = guarded(nullptr, [&] {
        auto ir = parse_program(program, program_len);
        size_t bytes = 0;
        const char* dump_dir = getenv("ADHIP_DUMP_CODE_DIR");
        std::map<std::string, std::vector<char>> objects;
        int relowered = 0;
        auto plan = lower_and_compile(*ir, dep_vector(dep_ids, n_dep_ids), arch && *arch ? arch : "gfx950", [](const std::string&) { return false; }, objects, &relowered);
        for (auto& k : plan->kernels) {
            const std::vector<char>& code = objects[k.source];
            bytes += code.size();
            if (dump_dir && *dump_dir) {
                std::string base = std::string(dump_dir) + "/" + k.entry;
                if (FILE* f = fopen((base + ".hsaco").c_str(), "wb")) { fwrite(code.data(), 1, code.size(), f); fclose(f); }
                if (FILE* f = fopen((base + ".hip").c_str(), "wb")) { fwrite(k.source.data(), 1, k.source.size(), f); fclose(f); }
            }
        }
        text = strf("%zu kernels compiled, %zu bytes of code objects", plan->kernels.size(), bytes);
        if (relowered) text += strf("; lowered %d more times with tighter kernel bounds", relowered);
        std::string spills;
        for (auto& k : plan->kernels) {
            const std::string one = describe_spills(objects[k.source], true);
            if (!one.empty()) spills += (spills.empty() ? "" : "; ") + one;
        }
        if (!spills.empty()) text += "; spilling kernels: " + spills;
    });
    if (rc != 0) text = g_tls_error;
    snprintf(out, out_cap, "%s", text.c_str());
    return rc;
}

}  // extern "C"
