// Shared helpers: the error type that stands in for the reference's panics, and small utilities.
#pragma once

#include <cstdint>
#include <cstdio>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace kn {

// Every contract violation the reference reports with `panic!`/`assert!` becomes a KnError here.
// It never crosses the C ABI: the entry points catch it and turn it into a status + message.
struct KnError : std::runtime_error {
    explicit KnError(const std::string &msg) : std::runtime_error(msg) {}
};

template <typename... Args>
[[noreturn]] inline void fail(const Args &...args) {
    std::ostringstream ss;
    (ss << ... << args);
    throw KnError(ss.str());
}

#define KN_ASSERT(cond, ...)                                                                   \
    do {                                                                                       \
        if (!(cond)) ::kn::fail("assertion failed: " #cond " (", __FILE__, ":", __LINE__, ") ", ##__VA_ARGS__); \
    } while (0)

template <typename T>
inline std::string vec_str(const std::vector<T> &v) {
    std::ostringstream ss;
    ss << "[";
    for (size_t i = 0; i < v.size(); i++) {
        if (i) ss << ", ";
        ss << v[i];
    }
    ss << "]";
    return ss.str();
}

inline uint64_t hash_combine(uint64_t seed, uint64_t v) {
    // splitmix-style mixing
    v += 0x9e3779b97f4a7c15ull + (seed << 6) + (seed >> 2);
    v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ull;
    v = (v ^ (v >> 27)) * 0x94d049bb133111ebull;
    return seed ^ (v ^ (v >> 31));
}

inline uint64_t fnv1a(const void *data, size_t len, uint64_t h = 0xcbf29ce484222325ull) {
    const uint8_t *p = (const uint8_t *) data;
    for (size_t i = 0; i < len; i++) {
        h ^= p[i];
        h *= 0x100000001b3ull;
    }
    return h;
}

}  // namespace kn
