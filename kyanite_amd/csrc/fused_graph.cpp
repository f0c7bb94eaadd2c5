// One kernel for a whole small graph. A graph of a few tiny steps (an MLP at batch 8: two matmuls and a softmax,
// a few KB of data) spends its time in launches, not in arithmetic: three launches take about 12 us back to back
// where each kernel runs for one or two. When every step of a plan is small enough for a single workgroup, the
// generated sources of the steps become device functions of ONE kernel, executed by one workgroup of 256 threads in
// launch order with a barrier in between (which also orders the global memory traffic of the waves of a workgroup:
// they share the compute unit's cache); matmul steps of that size are written as plain dot products, one output
// element per thread at a time, summed over k in order like the reference's CPU path does.
#include "fused_graph.h"

#include <sstream>

namespace kn {

namespace {

void replace_all(std::string &s, const std::string &from, const std::string &to) {
    for (size_t pos = s.find(from); pos != std::string::npos; pos = s.find(from, pos + to.size())) s.replace(pos, from.size(), to);
}

// the generated translation unit of a step as a namespace of its own with the kernel as a device function
// `kn_step(KnPtrs, workgroup index)`; false when the source does not look like expected
bool emit_generated_part(std::ostringstream &ss, const KernelSpec &k, size_t index) {
    const std::string prelude = kernel_prelude();
    if (k.source.compare(0, prelude.size(), prelude) != 0) return false;
    std::string body = k.source.substr(prelude.size());
    const size_t entry = body.find("extern \"C\" __global__");
    const std::string tail = "(KnPtrs ptrs) {";
    const size_t open = entry == std::string::npos ? std::string::npos : body.find(tail, entry);
    if (open == std::string::npos) return false;
    body.replace(entry, open + tail.size() - entry, "KN_DEV void kn_step(KnPtrs ptrs, const unsigned kn_bid) {");
    replace_all(body, "blockIdx.x", "kn_bid");
    ss << "namespace kn_s" << index << " {\n" << body << "}\n";
    // macros do not stop at the end of a namespace
    for (size_t pos = body.find("#define "); pos != std::string::npos; pos = body.find("#define ", pos + 1)) {
        size_t begin = pos + 8, end = begin;
        while (end < body.size() && (isalnum((unsigned char) body[end]) || body[end] == '_')) end++;
        const std::string name = body.substr(begin, end - begin);
        if (name != "KN_DEV" && name != "KN_INF") ss << "#undef " << name << "\n";
    }
    return true;
}

void emit_matmul_part(std::ostringstream &ss, const FusedPart &part, size_t index) {
    const GemmParams &p = part.gemm;
    const char *t = part.f16 ? "_Float16" : "float";
    ss << "namespace kn_s" << index << " {\nstruct KnPtrs { void *p[" << part.n_ptrs << "]; };\n";
    ss << "KN_DEV void kn_step(KnPtrs ptrs, const unsigned kn_bid) {\n";
    ss << "    const " << t << " *a = (const " << t << " *) ptrs.p[0], *b = (const " << t << " *) ptrs.p[1];\n";
    ss << "    " << t << " *c = (" << t << " *) ptrs.p[2];\n";
    size_t next = 3;
    if (part.has_addend) ss << "    const " << t << " *d = (const " << t << " *) ptrs.p[" << next++ << "];\n";
    if (part.has_addend2) ss << "    const " << t << " *d2 = (const " << t << " *) ptrs.p[" << next++ << "];\n";
    const long long mn = (long long) p.m * p.n, total = mn * p.batch;
    ss << "    for (int e = (int) threadIdx.x; e < " << total << "; e += 256) {\n";
    ss << "        const long long z = e / " << mn << ", i = (e / " << p.n << ") % " << p.m << ", j = e % " << p.n << ";\n";
    ss << "        const " << t << " *ar = a + z * " << p.a_sb << "ll + i * " << p.a_sm << "ll, *bc = b + z * " << p.b_sb << "ll + j * " << p.b_sn << "ll;\n";
    ss << "        float acc = 0.0f;\n";
    ss << "        for (int k = 0; k < " << p.k << "; k++) acc += (float) ar[k * " << p.a_sk << "ll] * (float) bc[k * " << p.b_sk << "ll];\n";
    // one rounding to the element type at the store, then the addends and the relu on values of that type, exactly
    // like the epilogue of the matrix-core kernels
    ss << "        " << t << " r = (" << t << ") acc;\n";
    if (part.has_addend) ss << "        r = (" << t << ") ((float) r + (float) d[z * " << p.d_sb << "ll + i * " << p.d_sm << "ll + j * " << p.d_sn << "ll]);\n";
    if (part.has_addend2) ss << "        r = (" << t << ") ((float) r + (float) d2[z * " << p.d2_sb << "ll + i * " << p.d2_sm << "ll + j * " << p.d2_sn << "ll]);\n";
    if (p.relu) ss << "        r = r > (" << t << ") 0 ? r : (" << t << ") 0;\n";
    ss << "        c[z * " << p.c_sb << "ll + i * " << p.c_sm << "ll + j * " << p.c_sn << "ll] = r;\n";
    ss << "    }\n}\n}\n";
}

}  // namespace

std::optional<KernelSpec> make_fused_graph_kernel(const std::vector<FusedPart> &parts) {
    if (parts.empty() || parts.size() > FUSED_MAX_STEPS) return std::nullopt;
    size_t total_ptrs = 0;
    for (auto &part : parts) {
        total_ptrs += part.n_ptrs;
        if (part.kernel) {
            if (part.kernel->block != 256 || part.kernel->grid > FUSED_MAX_WORKGROUPS) return std::nullopt;
        } else {
            const GemmParams &p = part.gemm;
            if (p.groups > 1 || p.pair_op || p.batch <= 0 || p.m <= 0 || p.n <= 0 || p.k < 0) return std::nullopt;
            const long long outputs = (long long) p.batch * p.m * p.n;
            if (outputs > FUSED_MAX_MATMUL_OUTPUTS || outputs * (long long) p.k > FUSED_MAX_MATMUL_MACS) return std::nullopt;
        }
    }
    if (total_ptrs > 256) return std::nullopt;

    std::ostringstream ss;
    ss << kernel_prelude();
    for (size_t i = 0; i < parts.size(); i++) {
        if (parts[i].kernel) {
            if (parts[i].kernel->grid == 0) continue;
            if (!emit_generated_part(ss, *parts[i].kernel, i)) return std::nullopt;
        } else {
            emit_matmul_part(ss, parts[i], i);
        }
    }
    ss << "struct KnFusedPtrs { void *p[" << std::max<size_t>(total_ptrs, 1) << "]; };\n";
    ss << "extern \"C\" __global__ __launch_bounds__(256) void kn_fused(KnFusedPtrs all, unsigned *done, unsigned seq) {\n";
    size_t offset = 0;
    for (size_t i = 0; i < parts.size(); i++) {
        const size_t n = parts[i].n_ptrs;
        const uint32_t grid = parts[i].kernel ? parts[i].kernel->grid : 1;
        if (grid > 0) {
            ss << "    {\n        kn_s" << i << "::KnPtrs q;\n";
            for (size_t k = 0; k < n; k++) ss << "        q.p[" << k << "] = all.p[" << offset + k << "];\n";
            // A step body is written for a fresh workgroup: its LDS arrays are used once, behind one barrier. When one
            // workgroup plays several, a fast wave must not write the arrays for workgroup b + 1 while a slow one
            // still reads what workgroup b left there: a barrier between the turns.
            if (grid > 1)
                ss << "        for (unsigned b = 0; b < " << grid << "u; b++) {\n            kn_s" << i << "::kn_step(q, b);\n            __syncthreads();\n        }\n    }\n";
            else
                ss << "        kn_s" << i << "::kn_step(q, 0u);\n    }\n";
            if (i + 1 < parts.size()) ss << "    __syncthreads();\n";
        }
        offset += n;
    }
    // the launch reports its own completion to a host that polls `done`: every store of every thread first
    ss << "    __threadfence_system();\n    __syncthreads();\n    if (threadIdx.x == 0) __hip_atomic_store(done, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);\n";
    ss << "}\n";

    KernelSpec spec;
    spec.name = "kn_fused";
    spec.source = ss.str();
    spec.grid = 1;
    spec.block = 256;
    spec.n_ptrs = total_ptrs;
    spec.strategy = "whole graph in one workgroup, " + std::to_string(parts.size()) + " steps";
    return spec;
}

}  // namespace kn
