#include "rtc.h"

#include <dlfcn.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdlib>
#include <fstream>
#include <unordered_map>

namespace kn {

namespace {

// Options are part of the cache key. Packed f32 instructions are kept off and contraction into FMA is disabled so
// that elementwise arithmetic rounds exactly like the scalar host semantics.
const std::vector<const char *> &compile_options() {
    static const std::vector<const char *> opts = {
        "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    };
    return opts;
}

std::mutex g_mutex;
std::unordered_map<uint64_t, std::shared_ptr<const CodeObject>> g_cache;
CompileStats g_stats;

uint64_t source_key(const std::string &source) {
    uint64_t h = fnv1a(source.data(), source.size());
    for (const char *o : compile_options()) h = fnv1a(o, strlen(o) + 1, h);
    return hash_combine(h, source.size());
}

std::string cache_dir() {
    const char *env = getenv("KNHIP_CACHE_DIR");
    if (env) return env;  // may be empty: disabled
    return library_dir() + "/_kcache";
}

std::string cache_path(const std::string &dir, uint64_t key) {
    char buf[32];
    snprintf(buf, sizeof buf, "%016llx", (unsigned long long) key);
    return dir + "/" + buf + ".hsaco";
}

}  // namespace

std::string library_dir() {
    Dl_info info;
    if (dladdr((void *) &library_dir, &info) && info.dli_fname) {
        std::string path = info.dli_fname;
        size_t slash = path.find_last_of('/');
        if (slash != std::string::npos) return path.substr(0, slash);
    }
    return ".";
}

CompileStats compile_stats() {
    std::lock_guard<std::mutex> lock(g_mutex);
    return g_stats;
}

std::shared_ptr<const CodeObject> compile_kernel(const std::string &source) {
    uint64_t key = source_key(source);
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g_cache.find(key);
    if (it != g_cache.end()) {
        g_stats.memory_hits++;
        return it->second;
    }

    auto obj = std::make_shared<CodeObject>();
    obj->key = key;
    std::string dir = cache_dir();
    if (!dir.empty()) {
        std::ifstream f(cache_path(dir, key), std::ios::binary);
        if (f) {
            obj->binary.assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
            if (!obj->binary.empty()) {
                g_stats.disk_hits++;
                g_cache[key] = obj;
                return obj;
            }
        }
    }

    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, source.c_str(), "kn_kernel.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS) fail("hiprtcCreateProgram failed: ", hiprtcGetErrorString(r));
    const auto &opts = compile_options();
    r = hiprtcCompileProgram(prog, (int) opts.size(), const_cast<const char **>(opts.data()));
    if (r != HIPRTC_SUCCESS) {
        size_t log_size = 0;
        hiprtcGetProgramLogSize(prog, &log_size);
        std::string log(log_size, '\0');
        if (log_size) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        fail("kernel compilation failed: ", hiprtcGetErrorString(r), "\n", log, "\n---- source ----\n", source);
    }
    size_t size = 0;
    hiprtcGetCodeSize(prog, &size);
    obj->binary.resize(size);
    hiprtcGetCode(prog, obj->binary.data());
    hiprtcDestroyProgram(&prog);
    g_stats.compiled++;

    if (!dir.empty()) {
        mkdir(dir.c_str(), 0755);
        std::string path = cache_path(dir, key);
        std::string tmp = path + ".tmp" + std::to_string((long) getpid());
        std::ofstream f(tmp, std::ios::binary);
        if (f) {
            f.write(obj->binary.data(), (std::streamsize) obj->binary.size());
            f.close();
            if (f) rename(tmp.c_str(), path.c_str());
            else unlink(tmp.c_str());
        }
    }
    g_cache[key] = obj;
    return obj;
}

}  // namespace kn
