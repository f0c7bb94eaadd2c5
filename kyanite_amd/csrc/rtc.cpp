#include "rtc.h"

#include <dlfcn.h>
#include <hip/hip_version.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdlib>
#include <cstring>
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

// The compiler's identity is part of the key too: a code object that another hipRTC release built is never picked up.
uint64_t toolchain_key() {
    static const uint64_t key = [] {
        int major = 0, minor = 0;
        (void) hiprtcVersion(&major, &minor);
        uint64_t h = hash_combine(hash_combine(0x6b6e68697063ull, (uint64_t) major), (uint64_t) minor);
        return hash_combine(h, (uint64_t) HIP_VERSION);  // the headers the generated sources are compiled against
    }();
    return key;
}

uint64_t source_key(const std::string &source) {
    uint64_t h = fnv1a(source.data(), source.size());
    for (const char *o : compile_options()) h = fnv1a(o, strlen(o) + 1, h);
    return hash_combine(hash_combine(h, source.size()), toolchain_key());
}

// a second hash of the source, independent of the first, stored inside the file: two sources whose keys collide
// are told apart by it
uint64_t source_check(const std::string &source) {
    return fnv1a(source.data(), source.size(), 0x9e3779b97f4a7c15ull ^ source.size());
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

// A cache file is this header followed by the code object. A file that is short, was written by another layout or
// toolchain, belongs to another source or whose bytes do not hash to what the header says is deleted and rebuilt.
struct CacheHeader {
    char magic[8];         // "KNHSACO\0"
    uint32_t layout;       // CACHE_LAYOUT
    uint32_t header_bytes; // sizeof(CacheHeader)
    uint64_t key;          // source_key
    uint64_t source_check; // source_check
    uint64_t code_bytes;
    uint64_t code_hash;    // fnv1a of the code object
};
constexpr uint32_t CACHE_LAYOUT = 2;
const char CACHE_MAGIC[8] = {'K', 'N', 'H', 'S', 'A', 'C', 'O', 0};

bool read_cache_file(const std::string &path, uint64_t key, uint64_t check, std::vector<char> &binary) {
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    std::vector<char> bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    CacheHeader h;
    bool ok = bytes.size() >= sizeof h;
    if (ok) {
        memcpy(&h, bytes.data(), sizeof h);
        ok = memcmp(h.magic, CACHE_MAGIC, 8) == 0 && h.layout == CACHE_LAYOUT && h.header_bytes == sizeof h && h.key == key &&
             h.source_check == check && h.code_bytes > 0 && h.code_bytes == bytes.size() - sizeof h &&
             h.code_hash == fnv1a(bytes.data() + sizeof h, (size_t) h.code_bytes);
    }
    if (!ok) {
        unlink(path.c_str());
        return false;
    }
    binary.assign(bytes.begin() + sizeof h, bytes.end());
    return true;
}

void write_cache_file(const std::string &dir, const std::string &path, uint64_t key, uint64_t check, const std::vector<char> &binary) {
    mkdir(dir.c_str(), 0755);
    CacheHeader h{};
    memcpy(h.magic, CACHE_MAGIC, 8);
    h.layout = CACHE_LAYOUT;
    h.header_bytes = sizeof h;
    h.key = key;
    h.source_check = check;
    h.code_bytes = binary.size();
    h.code_hash = fnv1a(binary.data(), binary.size());
    // written under a name of its own and renamed into place, so that a reader never sees half a file
    std::string tmp = path + ".tmp" + std::to_string((long) getpid());
    std::ofstream f(tmp, std::ios::binary);
    if (!f) return;
    f.write((const char *) &h, sizeof h);
    f.write(binary.data(), (std::streamsize) binary.size());
    f.close();
    if (f) rename(tmp.c_str(), path.c_str());
    else unlink(tmp.c_str());
}

std::shared_ptr<const CodeObject> compile_locked(const std::string &source, uint64_t key, bool use_disk_copy) {
    auto obj = std::make_shared<CodeObject>();
    obj->key = key;
    uint64_t check = source_check(source);
    std::string dir = cache_dir();
    std::string path = dir.empty() ? std::string() : cache_path(dir, key);
    if (!dir.empty()) {
        if (!use_disk_copy) unlink(path.c_str());
        else if (read_cache_file(path, key, check, obj->binary)) {
            obj->from_disk = true;
            g_stats.disk_hits++;
            g_cache[key] = obj;
            return obj;
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

    if (!dir.empty()) write_cache_file(dir, path, key, check, obj->binary);
    g_cache[key] = obj;
    return obj;
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

size_t kernarg_segment_bytes(const CodeObject &code) {
    // the metadata is a MessagePack map; the key is a string, the value behind it an unsigned integer
    static const char key[] = ".kernarg_segment_size";
    const size_t key_len = sizeof key - 1;
    const std::vector<char> &b = code.binary;
    size_t found = 0, value = 0;
    for (size_t i = 0; i + key_len < b.size(); i++) {
        if (memcmp(b.data() + i, key, key_len) != 0) continue;
        const unsigned char *p = (const unsigned char *) b.data() + i + key_len;
        const size_t left = b.size() - i - key_len;
        size_t v = 0;
        if (p[0] <= 0x7f) v = p[0];
        else if (p[0] == 0xcc && left >= 2) v = p[1];
        else if (p[0] == 0xcd && left >= 3) v = ((size_t) p[1] << 8) | p[2];
        else if (p[0] == 0xce && left >= 5) v = ((size_t) p[1] << 24) | ((size_t) p[2] << 16) | ((size_t) p[3] << 8) | p[4];
        else continue;
        found++;
        value = v;
    }
    return found == 1 ? value : 0;
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
    return compile_locked(source, key, true);
}

std::shared_ptr<const CodeObject> recompile_kernel(const std::string &source) {
    uint64_t key = source_key(source);
    std::lock_guard<std::mutex> lock(g_mutex);
    g_cache.erase(key);
    g_stats.discarded++;
    return compile_locked(source, key, false);
}

}  // namespace kn
