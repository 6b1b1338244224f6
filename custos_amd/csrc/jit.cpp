// Run-time compilation of kernels (hiprtc), the kernel caches in memory and on
// disk, and the host-only expression helpers of the C ABI (include/custos_hip.h).
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>

#include "runtime.hpp"

namespace custos_hip {

namespace {

// ---- code objects on disk ----
//
// With CUSTOS_HIP_KERNEL_CACHE_DIR set, every compiled code object is stored as
// <dir>/<key>[_batched|_ragged]-<arch>-<hiprtc version>.co together with the source it was built
// from; a later process loads it instead of compiling when the stored source is
// identical (the 64-bit key alone is not trusted).

std::string cache_file(const KernelSpec& spec, const std::string& arch, EntrySet which) {
    const char* dir = std::getenv("CUSTOS_HIP_KERNEL_CACHE_DIR");
    if (!dir || !*dir) return "";
    int major = 0, minor = 0;
    (void)hiprtcVersion(&major, &minor);
    std::string a = arch;
    for (char& c : a)
        if (c == ':' || c == '/' || c == '+') c = '_';
    char key[17];
    std::snprintf(key, sizeof key, "%016llx", static_cast<unsigned long long>(spec.hash));
    return std::string(dir) + "/" + key + entry_suffix(which) + "-" + a + "-" + std::to_string(major) + "." + std::to_string(minor) + ".co";
}

// the text hiprtc compiles: generated kernels start with a comment line that
// spells the expression as the caller wrote it; it is not part of the identity
std::string source_identity(const KernelSpec& spec, EntrySet which) {
    const std::string& text = spec.source[static_cast<int>(which)];
    if (spec.kind == Kind::Source) return spec.name + "\n" + text;
    return text.substr(text.find('\n') + 1);
}

bool load_cached_code(const KernelSpec& spec, const std::string& arch, EntrySet which, std::vector<char>* code) {
    const std::string path = cache_file(spec, arch, which);
    if (path.empty()) return false;
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    char magic[8] = {0};
    uint64_t src_len = 0, code_len = 0;
    f.read(magic, 8);
    f.read(reinterpret_cast<char*>(&src_len), 8);
    if (!f || std::memcmp(magic, "CUSTOSC1", 8) != 0 || src_len > (1u << 26)) return false;
    std::string src(src_len, '\0');
    f.read(&src[0], static_cast<std::streamsize>(src_len));
    f.read(reinterpret_cast<char*>(&code_len), 8);
    if (!f || src != source_identity(spec, which) || code_len == 0 || code_len > (1u << 28)) return false;
    code->resize(code_len);
    f.read(code->data(), static_cast<std::streamsize>(code_len));
    return static_cast<bool>(f);
}

void store_cached_code(const KernelSpec& spec, const std::string& arch, EntrySet which, const std::vector<char>& code) {
    const std::string path = cache_file(spec, arch, which);
    if (path.empty()) return;
    (void)mkdir(std::getenv("CUSTOS_HIP_KERNEL_CACHE_DIR"), 0777);
    const std::string tmp = path + ".tmp" + std::to_string(static_cast<long>(getpid()));
    {
        std::ofstream f(tmp, std::ios::binary | std::ios::trunc);
        if (!f) return;
        const std::string src = source_identity(spec, which);
        const uint64_t src_len = src.size(), code_len = code.size();
        f.write("CUSTOSC1", 8);
        f.write(reinterpret_cast<const char*>(&src_len), 8);
        f.write(src.data(), static_cast<std::streamsize>(src_len));
        f.write(reinterpret_cast<const char*>(&code_len), 8);
        f.write(code.data(), static_cast<std::streamsize>(code_len));
        if (!f) {
            std::remove(tmp.c_str());
            return;
        }
    }
    if (std::rename(tmp.c_str(), path.c_str()) != 0) std::remove(tmp.c_str());
}

bool markers_from_c(const char* const* markers, int32_t n, std::vector<std::string>* out) {
    if (!markers || n < 1 || n > 4) return false;
    for (int i = 0; i < n; i++) {
        if (!markers[i] || !markers[i][0]) return false;
        out->push_back(markers[i]);
    }
    return true;
}

int32_t spec_from_c(custos_hip_device* dev, int32_t kind, int32_t dtype, const char* src,
                    const char* const* markers, int32_t n_markers, const Tuning& tuning,
                    bool literals_in_code, KernelSpec* spec, bool with_source = true) {
    if (!src) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "expression source is null");
    if (kind != CUSTOS_HIP_KIND_APPLY && kind != CUSTOS_HIP_KIND_UNARY_GRAD)
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "unknown kernel kind");
    if (!dtype_valid(dtype)) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "unknown element type");
    std::vector<std::string> m;
    if (!markers_from_c(markers, n_markers, &m))
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "1 to 4 non-empty markers are required");
    ParseError err;
    if (!build_kernel_spec(static_cast<Kind>(kind), static_cast<DType>(dtype), src, m, tuning, literals_in_code, spec, &err,
                           with_source))
        return set_error(dev, err.code ? err.code : CUSTOS_HIP_ERR_EXPR_SYNTAX, err.message);
    return CUSTOS_HIP_OK;
}

// The three translation units of a generated kernel, one after the other (generated on the way).
std::string all_units(KernelSpec* spec) {
    std::string text;
    for (int w = 0; w < kEntrySets; w++) {
        ParseError err;
        if (spec->source[w].empty()) (void)emit_kernel_source(spec, &err, static_cast<EntrySet>(w));
        // (every unit starts with a line that spells the expression: once is enough here)
        if (w) text += "\n// ---- translation unit of the entry point " + spec->name + entry_suffix(static_cast<EntrySet>(w)) + " ----\n";
        text += w ? spec->source[w].substr(spec->source[w].find('\n') + 1) : spec->source[w];
    }
    return text;
}

int32_t copy_out_string(const std::string& s, char* buf, size_t cap, size_t* needed) {
    if (needed) *needed = s.size() + 1;
    if (buf && cap) {
        size_t n = std::min(cap - 1, s.size());
        std::memcpy(buf, s.data(), n);
        buf[n] = '\0';
    }
    return CUSTOS_HIP_OK;
}

}  // namespace

// ---- hiprtc ----

int32_t compile_to_code_object(custos_hip_device* dev, const KernelSpec& spec,
                               const std::string& arch, std::vector<char>* code, EntrySet which) {
    const std::string& text = spec.source[static_cast<int>(which)];
    // A switch for tests of the error paths: kernels whose entry name contains the value fail to
    // compile (what a compiler defect or an exhausted machine would do, neither of which a test can call up).
    if (const char* fail = std::getenv("CUSTOS_HIP_FAIL_COMPILE_OF"))
        if (*fail && spec.name.find(fail) != std::string::npos)
            return set_error(dev, CUSTOS_HIP_ERR_COMPILE, "hiprtcCompileProgram: refused, CUSTOS_HIP_FAIL_COMPILE_OF names " + spec.name);
    hiprtcProgram prog = nullptr;
    hiprtcResult r = hiprtcCreateProgram(&prog, text.c_str(), "custos_kernel.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS)
        return set_error(dev, CUSTOS_HIP_ERR_COMPILE, std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r));
    std::vector<std::string> opts = hiprtc_options(arch);
    std::vector<const char*> copts;
    for (const std::string& o : opts) copts.push_back(o.c_str());
    r = hiprtcCompileProgram(prog, static_cast<int>(copts.size()), copts.data());
    if (r != HIPRTC_SUCCESS) {
        size_t log_size = 0;
        hiprtcGetProgramLogSize(prog, &log_size);
        std::string log(log_size, '\0');
        if (log_size) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        return set_error(dev, CUSTOS_HIP_ERR_COMPILE,
                         std::string("hiprtcCompileProgram: ") + hiprtcGetErrorString(r) + "\n" + log +
                             "\n--- source ---\n" + text);
    }
    size_t size = 0;
    hiprtcGetCodeSize(prog, &size);
    code->resize(size);
    hiprtcGetCode(prog, code->data());
    hiprtcDestroyProgram(&prog);
    return CUSTOS_HIP_OK;
}

// The translation unit `which` of `k`: code object from the disk cache or from hiprtc, loaded as
// a module, entry point looked up.  `k` owns its code.
static int32_t build_module(custos_hip_device* dev, custos_hip_kernel* k, EntrySet which) {
    const int w = static_cast<int>(which);
    if (k->spec.source[w].empty()) {
        ParseError err;
        if (k->spec.kind == Kind::Source || !emit_kernel_source(&k->spec, &err, which))
            return set_error(dev, err.code ? err.code : CUSTOS_HIP_ERR_EXPR_SYNTAX, err.message);
    }
    std::vector<char> code;
    hipModule_t module = nullptr;
    bool from_disk = load_cached_code(k->spec, dev->arch, which, &code);
    if (from_disk && hipModuleLoadData(&module, code.data()) != hipSuccess) {
        (void)hipGetLastError();  // a stale or damaged file: compile instead
        module = nullptr;
        from_disk = false;
    }
    if (!from_disk) {
        const auto t0 = std::chrono::steady_clock::now();
        int32_t rc = compile_to_code_object(dev, k->spec, dev->arch, &code, which);
        dev->compile_ns += static_cast<uint64_t>(
            std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t0).count());
        if (rc != CUSTOS_HIP_OK) return rc;
        HIP_TRY(dev, hipModuleLoadData(&module, code.data()));
        store_cached_code(k->spec, dev->arch, which, code);
        dev->compiles++;
    } else {
        dev->disk_hits++;
    }
    hipFunction_t fn = nullptr;
    hipError_t e = hipModuleGetFunction(&fn, module, (k->spec.name + entry_suffix(which)).c_str());
    if (e != hipSuccess) {
        (void)hipModuleUnload(module);
        return hip_fail(dev, e, "hipModuleGetFunction");
    }
    k->modules[w] = module;
    k->fns[w] = fn;
    return CUSTOS_HIP_OK;
}

int32_t entry_point(custos_hip_device* dev, custos_hip_kernel* k, EntrySet which, hipFunction_t* fn) {
    const int w = static_cast<int>(which);
    if (!k->fns[w]) {
        custos_hip_kernel* owner = k->code ? k->code : k;
        if (!owner->fns[w]) {
            if (owner->spec.kind == Kind::Source && which != EntrySet::Single)
                return set_error(dev, CUSTOS_HIP_ERR_KIND_MISMATCH, "a caller-written kernel has no entry point for merged launches");
            int32_t rc = build_module(dev, owner, which);
            if (rc != CUSTOS_HIP_OK) return rc;
        }
        k->fns[w] = owner->fns[w];
    }
    *fn = k->fns[w];
    return CUSTOS_HIP_OK;
}

// The cached kernel for the same translation unit as `spec` (compared by structure: `spec`
// need not have its text yet).
static custos_hip_kernel* find_code(custos_hip_device* dev, const KernelSpec& spec) {
    auto bucket = dev->cache.find(spec.hash);
    if (bucket == dev->cache.end()) return nullptr;
    for (auto& cached : bucket->second)
        if (cached->spec.kind != Kind::Source && same_code(cached->spec, spec)) return cached.get();
    return nullptr;
}

// The handle on `owner`'s code that carries the literal values of `k`: the owner itself if
// they are its own, else a handle that shares the owner's module (made on first use).
static custos_hip_kernel* handle_for_values(custos_hip_kernel* owner, std::unique_ptr<custos_hip_kernel> k,
                                            const char* src, const char* const* markers, int32_t n_markers) {
    if (owner->spec.consts.bytes == k->spec.consts.bytes) return owner;
    const std::string values(k->spec.consts.bytes.begin(), k->spec.consts.bytes.end());
    auto sibling = owner->siblings.find(values);
    if (sibling == owner->siblings.end()) {
        k->code = owner;  // (which also holds the text, the modules and the entry points)
        k->expr_src = src;
        for (int i = 0; i < n_markers; i++) k->markers.push_back(markers[i]);
        sibling = owner->siblings.emplace(values, std::move(k)).first;
    }
    return sibling->second.get();
}

// Parses, looks the key up in the cache, compiles on a miss.
//
// Literal values: the first set of values an expression is seen with is compiled into the
// code (the compiler folds them: a fused chain that sits at the edge of being ALU-bound
// runs 4 % faster than with the values in registers).  When the same expression arrives
// with other values, the form that takes them as launch parameters is compiled once, and
// every further set of values is a handle on that code.  custos_hip_set_literal_policy pins
// either behaviour.
static int32_t compile_expr(custos_hip_device* dev, int32_t kind, int32_t dtype, const char* src,
                            const char* const* markers, int32_t n_markers, const Tuning& tuning,
                            custos_hip_kernel** out) {
    std::unique_ptr<custos_hip_kernel> k(new custos_hip_kernel);
    // (specs without their text: it is generated only for what is compiled)
    int32_t rc = spec_from_c(dev, kind, dtype, src, markers, n_markers, tuning, /*literals_in_code=*/true, &k->spec, false);
    if (rc != CUSTOS_HIP_OK) return rc;
    if (custos_hip_kernel* known = find_code(dev, k->spec)) {
        dev->hits++;
        *out = known;
        return CUSTOS_HIP_OK;
    }
    if (k->spec.n_literals > 0 && dev->literal_policy != CUSTOS_HIP_LITERALS_IN_CODE) {
        std::unique_ptr<custos_hip_kernel> shared(new custos_hip_kernel);
        rc = spec_from_c(dev, kind, dtype, src, markers, n_markers, tuning, /*literals_in_code=*/false, &shared->spec, false);
        if (rc != CUSTOS_HIP_OK) return rc;
        if (shared->spec.consts.n_params > 0) {
            custos_hip_kernel* owner = find_code(dev, shared->spec);
            uint32_t& value_sets = dev->value_sets_seen[shared->spec.hash];
            const bool first_values = value_sets++ == 0;
            if (owner || dev->literal_policy == CUSTOS_HIP_LITERALS_AS_PARAMETERS || !first_values)
                k = std::move(shared);
            if (owner) {
                dev->hits++;
                *out = handle_for_values(owner, std::move(k), src, markers, n_markers);
                return CUSTOS_HIP_OK;
            }
        }
    }
    // The text also finds what cannot be compiled (a transcendental node over integers, say).
    ParseError err;
    if (!emit_kernel_source(&k->spec, &err)) return set_error(dev, err.code ? err.code : CUSTOS_HIP_ERR_EXPR_SYNTAX, err.message);
    k->code = k.get();
    // The entry point for single launches is compiled now, so that no launch compiles anything --
    // unless the device is recording: nothing is launched then, and the graph build compiles the
    // entry point each kernel is replayed through (for launches that are joined or merged that
    // is not this one).
    if (!dev->capturing) {
        hipFunction_t unused = nullptr;
        rc = entry_point(dev, k.get(), EntrySet::Single, &unused);
        if (rc != CUSTOS_HIP_OK) return rc;
    }
    k->expr_src = src;
    for (int i = 0; i < n_markers; i++) k->markers.push_back(markers[i]);
    *out = k.get();
    dev->cache[k->spec.hash].push_back(std::move(k));
    return CUSTOS_HIP_OK;
}

int32_t chain_kernel(custos_hip_device* dev, DType dtype, std::vector<ChainStage> stages, int n_ext, int n_outs,
                     const Tuning& tuning, custos_hip_kernel** out) {
    std::unique_ptr<custos_hip_kernel> k(new custos_hip_kernel);
    ParseError err;
    if (!build_chain_spec(dtype, std::move(stages), n_ext, n_outs, tuning, &k->spec, &err, /*with_source=*/false))
        return set_error(dev, err.code ? err.code : CUSTOS_HIP_ERR_EXPR_SYNTAX, err.message);
    if (custos_hip_kernel* known = find_code(dev, k->spec)) {
        dev->hits++;
        *out = known;
        return CUSTOS_HIP_OK;
    }
    // (nothing is compiled here: the graph build asks for the entry point it replays the chain through)
    if (!emit_kernel_source(&k->spec, &err)) return set_error(dev, err.code ? err.code : CUSTOS_HIP_ERR_EXPR_SYNTAX, err.message);
    k->expr_src = k->spec.chain_text;
    k->code = k.get();
    *out = k.get();
    dev->cache[k->spec.hash].push_back(std::move(k));
    return CUSTOS_HIP_OK;
}

int32_t identity_kernel(custos_hip_device* dev, DType dtype, custos_hip_kernel** out) {
    custos_hip_kernel*& slot = dtype == DType::U32 ? dev->identity_u32 : dev->identity_u8;
    if (!slot) {
        const char* markers[] = {"x"};
        int32_t rc = compile_expr(dev, CUSTOS_HIP_KIND_APPLY, static_cast<int32_t>(dtype), "x", markers, 1, dev->tuning, &slot);
        if (rc != CUSTOS_HIP_OK) return rc;
    }
    *out = slot;
    return CUSTOS_HIP_OK;
}

ResolvedShape resolve_shape(const custos_hip_device* dev, const custos_hip_kernel* k, unsigned long long footprint_bytes,
                            CacheHint hint, unsigned long long working_set_bytes, bool revisits, int keep_inputs) {
    const int n_operands = kernel_pointers(k->spec);
    const int n_written = k->spec.kind == Kind::Chain ? k->spec.n_outs : 1;
    const LaunchShape shape = preferred_shape(footprint_bytes, n_operands, hint, working_set_bytes, revisits, n_written, keep_inputs);
    ResolvedShape r;
    const int direction = dev->tuning.direction;
    r.alternate = direction == 2 || (direction == 0 && shape.alternate);
    // a kernel whose shape the caller left open runs as the launch says; a pinned one as it was compiled
    r.unroll = k->spec.auto_unroll ? shape.unroll : k->spec.tuning.unroll;
    r.block = k->spec.auto_unroll && shape.block > 0 ? std::min(shape.block, k->spec.tuning.block_threads) : k->spec.tuning.block_threads;
    r.nontemporal = dev->tuning.nontemporal >= 0
                        ? dev->tuning.nontemporal & (3 | kStoresWriteThrough)
                        : shape.nontemporal;
    return r;
}

}  // namespace custos_hip

using namespace custos_hip;

extern "C" {

// ---- expression kernels ----

int32_t custos_hip_expr_compile(custos_hip_device* dev, int32_t kind, int32_t dtype, const char* src,
                                const char* const* markers, int32_t n_markers,
                                custos_hip_kernel** kernel) {
    // A recording that repeats the one before (custos_hip_device::matching) asks for the kernel of its
    // next launch again, under the same settings: the handle that launch was recorded with answers,
    // by a comparison of the text alone.
    if (dev && kernel && src && markers && dev->capturing && dev->matching && dev->matched < dev->previous_recorded.size()) {
        custos_hip_kernel* expected = dev->previous_recorded[dev->matched].k;
        if (expected && expected->request_epoch == dev->compile_epoch && expected->request_kind == kind &&
            expected->request_dtype == dtype && expected->markers.size() == static_cast<size_t>(n_markers) &&
            std::strcmp(expected->expr_src.c_str(), src) == 0) {
            bool same = true;
            for (int i = 0; same && i < n_markers; i++) same = markers[i] && expected->markers[static_cast<size_t>(i)] == markers[i];
            if (same) {
                dev->hits++;
                *kernel = expected;
                return CUSTOS_HIP_OK;
            }
        }
    }
    REQUIRE_DEV(dev);
    if (!kernel) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "kernel out pointer is null");
    *kernel = nullptr;
    std::string text_key;
    if (src && markers && n_markers >= 1 && n_markers <= 4) {
        const Tuning& t = dev->tuning;
        // (the settings as raw bytes, then the markers and the text: one allocation)
        size_t length = 6 * sizeof(int32_t) + 2 + std::strlen(src);
        for (int i = 0; i < n_markers; i++) length += 1 + (markers[i] ? std::strlen(markers[i]) : 0);
        text_key.reserve(length);
        for (int32_t v : {kind, dtype, static_cast<int32_t>(t.block_threads), static_cast<int32_t>(t.unroll),
                          static_cast<int32_t>(t.blocks_per_cu), static_cast<int32_t>(t.nontemporal)})
            text_key.append(reinterpret_cast<const char*>(&v), sizeof v);
        text_key.push_back(dev->eq_as_cpu_eval ? 'l' : 'e');
        for (int i = 0; i < n_markers; i++) text_key.append(1, '\x1f').append(markers[i] ? markers[i] : "");
        text_key.append(1, '\x1e').append(src);
        auto known = dev->by_text.find(text_key);
        if (known != dev->by_text.end()) {
            dev->hits++;
            *kernel = known->second;
            known->second->request_kind = kind, known->second->request_dtype = dtype, known->second->request_epoch = dev->compile_epoch;
            return CUSTOS_HIP_OK;
        }
    }
    custos_hip_kernel* k = nullptr;
    Tuning tuning = dev->tuning;
    tuning.eq_as_leq = dev->eq_as_cpu_eval;
    int32_t rc = compile_expr(dev, kind, dtype, src, markers, n_markers, tuning, &k);
    if (rc != CUSTOS_HIP_OK) return rc;
    *kernel = k;
    k->request_kind = kind, k->request_dtype = dtype, k->request_epoch = dev->compile_epoch;
    dev->by_text.emplace(std::move(text_key), k);
    return CUSTOS_HIP_OK;
}

// ---- caller-written kernels (src/devices/cuda/kernel_cache.rs:39-61, kernel_launch.rs:81-163) ----

int32_t custos_hip_source_compile(custos_hip_device* dev, const char* src, const char* fn_name,
                                  custos_hip_kernel** kernel) {
    REQUIRE_DEV(dev);
    if (!kernel) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "kernel out pointer is null");
    *kernel = nullptr;
    if (!src || !fn_name || !*fn_name) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "source or function name is null");
    std::unique_ptr<custos_hip_kernel> k(new custos_hip_kernel);
    k->spec.kind = Kind::Source;
    k->spec.name = fn_name;
    k->spec.source[0] = src;
    k->spec.hash = fnv1a64(fn_name, std::strlen(fn_name), fnv1a64(src, std::strlen(src), fnv1a64("custos-source-v1", 16)));
    auto& bucket = dev->cache[k->spec.hash];
    for (auto& cached : bucket) {
        if (cached->spec.kind == Kind::Source && cached->spec.name == k->spec.name && cached->spec.source[0] == k->spec.source[0]) {
            dev->hits++;
            *kernel = cached.get();
            return CUSTOS_HIP_OK;
        }
    }
    int32_t rc = build_module(dev, k.get(), EntrySet::Single);
    if (rc != CUSTOS_HIP_OK) return rc;
    *kernel = k.get();
    bucket.push_back(std::move(k));
    return CUSTOS_HIP_OK;
}

const char* custos_hip_kernel_source(const custos_hip_kernel* kernel) {
    if (!kernel) return "";
    return (kernel->code ? kernel->code : kernel)->spec.source[0].c_str();
}

const char* custos_hip_kernel_name(const custos_hip_kernel* kernel) {
    return kernel ? kernel->spec.name.c_str() : "";
}

uint64_t custos_hip_kernel_hash(const custos_hip_kernel* kernel) { return kernel ? kernel->spec.hash : 0; }

int32_t custos_hip_kernel_arity(const custos_hip_kernel* kernel) {
    return kernel ? kernel->spec.expr.n_vars : 0;
}

int32_t custos_hip_kernel_launched_as(custos_hip_device* dev, custos_hip_kernel* kernel, size_t n,
                                      custos_hip_kernel** variant) {
    REQUIRE_DEV(dev);
    if (!kernel || !variant) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null argument");
    (void)n;
    *variant = kernel;  // one kernel per expression: the launch shape is an argument of the launch
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_cache_stats(custos_hip_device* dev, uint64_t* compiles, uint64_t* hits) {
    REQUIRE_DEV(dev);
    if (compiles) *compiles = dev->compiles;
    if (hits) *hits = dev->hits;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_compile_stats(custos_hip_device* dev, uint64_t* units, double* milliseconds) {
    REQUIRE_DEV(dev);
    if (units) *units = dev->compiles;
    if (milliseconds) *milliseconds = static_cast<double>(dev->compile_ns) * 1e-6;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_cache_disk_hits(custos_hip_device* dev, uint64_t* disk_hits) {
    REQUIRE_DEV(dev);
    if (disk_hits) *disk_hits = dev->disk_hits;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_expr_emit(int32_t kind, int32_t dtype, const char* src, const char* const* markers,
                             int32_t n_markers, const custos_hip_tuning* tuning, char* buf, size_t cap,
                             size_t* needed, uint64_t* hash) {
    KernelSpec spec;
    int32_t rc = spec_from_c(nullptr, kind, dtype, src, markers, n_markers, tuning_from_c(tuning), true, &spec);
    if (rc != CUSTOS_HIP_OK) return rc;
    if (hash) *hash = spec.hash;
    return copy_out_string(all_units(&spec), buf, cap, needed);
}

int32_t custos_hip_expr_emit_shared(int32_t kind, int32_t dtype, const char* src, const char* const* markers,
                                    int32_t n_markers, const custos_hip_tuning* tuning, char* buf, size_t cap,
                                    size_t* needed, uint64_t* hash) {
    KernelSpec spec;
    int32_t rc = spec_from_c(nullptr, kind, dtype, src, markers, n_markers, tuning_from_c(tuning), false, &spec);
    if (rc != CUSTOS_HIP_OK) return rc;
    if (hash) *hash = spec.hash;
    return copy_out_string(all_units(&spec), buf, cap, needed);
}

int32_t custos_hip_set_eq_policy(custos_hip_device* dev, int32_t policy) {
    REQUIRE_DEV(dev);
    if (policy != CUSTOS_HIP_EQ_EXACT && policy != CUSTOS_HIP_EQ_AS_CPU_EVAL)
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "unknown eq policy");
    dev->eq_as_cpu_eval = policy == CUSTOS_HIP_EQ_AS_CPU_EVAL;
    dev->compile_epoch++;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_literal_policy(custos_hip_device* dev, int32_t policy) {
    REQUIRE_DEV(dev);
    if (policy != CUSTOS_HIP_LITERALS_ADAPTIVE && policy != CUSTOS_HIP_LITERALS_IN_CODE &&
        policy != CUSTOS_HIP_LITERALS_AS_PARAMETERS)
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "unknown literal policy");
    dev->literal_policy = policy;
    dev->by_text.clear();  // the same text may now map to another kernel
    dev->compile_epoch++;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_expr_build_code_object(int32_t kind, int32_t dtype, const char* src,
                                          const char* const* markers, int32_t n_markers,
                                          const custos_hip_tuning* tuning, size_t* code_size) {
    KernelSpec spec;
    int32_t rc = spec_from_c(nullptr, kind, dtype, src, markers, n_markers, tuning_from_c(tuning), true, &spec);
    if (rc != CUSTOS_HIP_OK) return rc;
    (void)all_units(&spec);
    size_t total = 0;
    for (int w = 0; w < kEntrySets; w++) {
        std::vector<char> code;
        rc = compile_to_code_object(nullptr, spec, "gfx950", &code, static_cast<EntrySet>(w));
        if (rc != CUSTOS_HIP_OK) return rc;
        total += code.size();
    }
    if (code_size) *code_size = total;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_chain_emit(int32_t dtype, const char* const* stage_srcs, const int32_t* stage_vars, int32_t n_stages,
                              const int32_t* sources, const int32_t* stage_outs, int32_t n_inputs, int32_t n_outputs,
                              int32_t literals_as_parameters, char* buf, size_t cap, size_t* needed, size_t* code_size) {
    if (!dtype_valid(dtype)) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "unknown element type");
    if (!stage_srcs || !stage_vars || !sources || !stage_outs || n_stages < 1 || n_stages > kMaxChainStages)
        return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "1 to 8 stages are required");
    std::vector<ChainStage> stages;
    const int32_t* from = sources;
    for (int32_t s = 0; s < n_stages; s++) {
        if (!stage_srcs[s] || stage_vars[s] < 1 || stage_vars[s] > 4)
            return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "a stage takes 1 to 4 variables");
        std::vector<std::string> names;
        for (int32_t v = 0; v < stage_vars[s]; v++) names.push_back("v" + std::to_string(v));
        ChainStage stage;
        ParseError err;
        if (!parse_expr(stage_srcs[s], names, &stage.expr, &err))
            return set_error(nullptr, err.code ? err.code : CUSTOS_HIP_ERR_EXPR_SYNTAX, err.message);
        // (an expression need not use every variable: the stage still takes stage_vars[s] of them)
        stage.expr.n_vars = stage_vars[s];
        stage.source.assign(from, from + stage_vars[s]);
        from += stage_vars[s];
        stage.out = stage_outs[s];
        if (literals_as_parameters) {
            ConstPlan plan;
            if (!plan_constants(stage.expr, static_cast<DType>(dtype), /*all_in_code=*/false, &plan, &err))
                return set_error(nullptr, err.code ? err.code : CUSTOS_HIP_ERR_EXPR_SYNTAX, err.message);
            if (plan.n_params > 0) {
                stage.slot = plan.slot;
                stage.n_params = plan.n_params;
                stage.param_bytes = plan.bytes.size();
            }
        }
        stages.push_back(std::move(stage));
    }
    KernelSpec spec;
    ParseError err;
    if (!build_chain_spec(static_cast<DType>(dtype), std::move(stages), n_inputs, n_outputs, Tuning{}, &spec, &err))
        return set_error(nullptr, err.code ? err.code : CUSTOS_HIP_ERR_EXPR_SYNTAX, err.message);
    const std::string text = all_units(&spec);
    if (code_size) {
        *code_size = 0;
        for (int w = 0; w < kEntrySets; w++) {
            std::vector<char> code;
            const int32_t rc = compile_to_code_object(nullptr, spec, "gfx950", &code, static_cast<EntrySet>(w));
            if (rc != CUSTOS_HIP_OK) return rc;
            *code_size += code.size();
        }
    }
    return copy_out_string(text, buf, cap, needed);
}

int32_t custos_hip_preferred_shape(uint64_t footprint_bytes, int32_t n_operands, int32_t* unroll,
                                   int32_t* nontemporal, int32_t* alternate) {
    if (n_operands < 1) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "n_operands must be positive");
    const LaunchShape s = preferred_shape(footprint_bytes, n_operands);
    if (unroll) *unroll = s.unroll;
    if (nontemporal) *nontemporal = s.nontemporal;
    if (alternate) *alternate = s.alternate ? 1 : 0;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_preferred_shape_of(uint64_t footprint_bytes, int32_t n_operands, int32_t n_written,
                                      uint64_t working_set_bytes, int32_t revisits, int32_t* unroll, int32_t* nontemporal,
                                      int32_t* alternate, int32_t* block_threads) {
    if (n_operands < 1 || n_written < 0 || n_written > n_operands)
        return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "n_operands must be positive and n_written within it");
    const LaunchShape s = preferred_shape(footprint_bytes, n_operands, CacheHint::Unknown, working_set_bytes, revisits == 1, n_written,
                                          revisits == 2 ? 1 : 0);
    if (unroll) *unroll = s.unroll;
    if (nontemporal) *nontemporal = s.nontemporal;
    if (alternate) *alternate = s.alternate ? 1 : 0;
    if (block_threads) *block_threads = s.block;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_expr_canonical(const char* src, const char* const* markers, int32_t n_markers,
                                  char* buf, size_t cap, size_t* needed) {
    if (!src) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "expression source is null");
    std::vector<std::string> m;
    if (!markers_from_c(markers, n_markers, &m))
        return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "1 to 4 non-empty markers are required");
    Expr e;
    ParseError err;
    if (!parse_expr(src, m, &e, &err)) return set_error(nullptr, err.code, err.message);
    return copy_out_string(to_cl_source(e, m), buf, cap, needed);
}

int32_t custos_hip_expr_constants(int32_t dtype, const char* src, const char* const* markers, int32_t n_markers,
                                  void* buf, size_t cap, size_t* needed, int32_t* n_params) {
    if (!src) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "expression source is null");
    if (!dtype_valid(dtype)) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "unknown element type");
    std::vector<std::string> m;
    if (!markers_from_c(markers, n_markers, &m))
        return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "1 to 4 non-empty markers are required");
    Expr e;
    ParseError err;
    ConstPlan plan;
    if (!parse_expr(src, m, &e, &err) || !plan_constants(e, static_cast<DType>(dtype), false, &plan, &err))
        return set_error(nullptr, err.code, err.message);
    if (needed) *needed = plan.bytes.size();
    if (n_params) *n_params = plan.n_params;
    if (buf && cap >= plan.bytes.size() && !plan.bytes.empty()) std::memcpy(buf, plan.bytes.data(), plan.bytes.size());
    return CUSTOS_HIP_OK;
}

}  // extern "C"
