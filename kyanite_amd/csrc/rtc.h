// Run-time compilation of generated kernels for gfx950 through hipRTC, with an in-memory and an on-disk cache.
// Takes the role of kn-cuda-sys/src/wrapper/rtc/core.rs (compile, module load, launch) and of the process-wide
// kernel cache in kn-cuda-eval/src/autokernel/common.rs:14-46.
#pragma once

#include <memory>
#include <mutex>

#include "kernels.h"

namespace kn {

struct CodeObject {
    std::vector<char> binary;
    uint64_t key = 0;
    bool from_disk = false;  // read from the disk cache rather than compiled by this process
};

// Compile (or fetch from cache) the code object for a kernel source. Works without a GPU.
// The disk cache lives in $KNHIP_CACHE_DIR, or next to the library in `_kcache/` when that is unset;
// set KNHIP_CACHE_DIR to an empty string to disable it.
// A cache file carries a header (layout, key, a second hash of the source, length and hash of the code object); the
// key covers the source, the compile options and the hipRTC / HIP versions. A file that fails any of these checks is
// deleted and the kernel compiled again.
std::shared_ptr<const CodeObject> compile_kernel(const std::string &source);
// Forget the cached code object of `source` (memory and disk) and compile it again: for a code object from the disk
// cache that passed the checks above and still does not load.
std::shared_ptr<const CodeObject> recompile_kernel(const std::string &source);

// Bytes of launch arguments the (single) kernel of a code object expects, read from the code object's metadata note
// (the value behind the key ".kernarg_segment_size"); 0 when the note does not hold exactly one such key.
size_t kernarg_segment_bytes(const CodeObject &code);

struct CompileStats {
    size_t compiled = 0, memory_hits = 0, disk_hits = 0, discarded = 0;
};
CompileStats compile_stats();

// The directory of the shared library that contains this code.
std::string library_dir();

}  // namespace kn
