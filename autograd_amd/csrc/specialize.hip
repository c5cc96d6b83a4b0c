// Programs that recur get a kernel of their own.
//
// The interpreter (program.hip) pays, per instruction and wave, some thirty register moves and twenty scalar
// instructions of decode and dispatch around four arithmetic instructions: a chain of a dozen rules over a few
// million elements runs at a quarter of what its memory traffic allows.  A training loop or a solver evaluates the
// same few chains again and again, so a program that has been seen a few times is written out as straight-line HIP
// (the same functors of functors.h, one statement per instruction, each operation rounded on its own under
// -ffp-contract=off: the same bits), compiled for this GPU with the run-time compiler, and from then on launched
// in the interpreter's place with the very same argument block over the same tiling.  Everything that runs once or
// twice stays with the interpreter; a program whose compilation fails stays there too.
#include <hip/hiprtc.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iterator>
#include <mutex>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.h"

#include "functors.h"
#include "program_params.h"

namespace agmi {

// agmi.h, functors.h and program_params.h as text (written by the Makefile from the files themselves)
static const char *const kSpecHeaders[] = {
#include "specialize_headers.inc"
};

struct SpecKernel {
    int seen = 0;
    int state = 0;  // 0 not compiled, 1 ready, -1 failed
    hipModule_t module = nullptr;
    hipFunction_t function = nullptr;
    std::string name;
};

static std::mutex g_spec_mutex;
static std::unordered_map<std::string, SpecKernel> g_spec;
static int g_spec_after = -1;  // compile at this many sightings; 0: never; -1: read the environment first
static long long g_spec_launches = 0, g_spec_compiled = 0;
constexpr long long kSpecMaxKernels = 4096;  // compiled programs kept (each a loaded code object of some tens of KB)
constexpr size_t kSpecMaxSeen = 16384;        // programs remembered, compiled or only counted

static const char *functor_name(int op) {
#define AGMI_NAME_CASE(OP, FN) \
    case OP: return #FN;
    switch (op) {
        AGMI_FOR_EACH_PROGRAM_OP(AGMI_NAME_CASE)
        AGMI_FOR_EACH_CHAINED_OP(AGMI_NAME_CASE)
        default: return nullptr;
    }
#undef AGMI_NAME_CASE
}

static int functor_arity(int op) {
#define AGMI_ARITY_CASE(OP, FN) \
    case OP: return FN<float>::NIN;
    switch (op) {
        AGMI_FOR_EACH_PROGRAM_OP(AGMI_ARITY_CASE)
        AGMI_FOR_EACH_CHAINED_OP(AGMI_ARITY_CASE)
        default: return -1;
    }
#undef AGMI_ARITY_CASE
}

// The kernel's name in traces: precision, instruction count and a hash of the instruction words, so that one
// row of a kernel trace is one program.
static std::string spec_name(bool f32, const ProgParams &p) {
    uint32_t h = 2166136261u;
    for (int i = 0; i < p.n_instr; ++i)
        for (int b = 0; b < 4; ++b) h = (h ^ ((p.code[i] >> (8 * b)) & 0xffu)) * 16777619u;
    char text[64];
    std::snprintf(text, sizeof(text), "agmi_specialized_%s_%dinstr_%08x", f32 ? "f32" : "f64", p.n_instr, h);
    return text;
}

// The kernel's text.  Leaves are read with plain loads (chains read one array at several shifts: the second and third
// read of a line must find it in the cache, which the interpreter's non-temporal loads cost 20 us of a 95 us
// Hessian-vector product), results leave with non-temporal stores (nothing in the kernel reads them back: 81 -> 62 us).
//  Registers are plain local arrays with constant indices: the compiler keeps what is live.
static std::string spec_source(bool f32, int nreg, const ProgParams &p, const std::string &name) {
    std::ostringstream o;
    o << "typedef signed long long int64_t;\ntypedef unsigned long long uint64_t;\ntypedef int int32_t;\n"
         "typedef unsigned int uint32_t;\ntypedef unsigned char uint8_t;\ntypedef unsigned long size_t;\n";
    for (const char *h : kSpecHeaders) o << h << "\n";
    o << "using namespace agmi;\n"
         "extern \"C\" __global__ __launch_bounds__(256) void " << name << "(const agmi::ProgParams p) {\n"
      << "    typedef " << (f32 ? "float" : "double") << " T;\n"
      << R"SRC(    constexpr int U = 2, VL = 16 / sizeof(T), V = VL * U, TW = 64 * V;
    typedef T vec_t __attribute__((ext_vector_type(VL), aligned(sizeof(T))));
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t t = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    if (t >= p.n_tiles) return;
    const uint32_t tpr = p.tiles_per_row;
    uint32_t row = t / tpr, chunk = t - row * tpr;
    const int64_t cols = p.cols;
)SRC";
    if (p.row_group > 0) o << "    __shared__ __align__(16) T row_values[4][TW];\n";
    for (int k = 0; k < p.n_imm; ++k) o << "    const T imm" << k << " = static_cast<T>(p.imm[" << k << "]);\n";
    o << R"SRC(    for (;;) {
        const uint32_t cur_row = row;
        const int64_t tile_begin = static_cast<int64_t>(chunk) * TW, c0 = tile_begin + lane * VL;
        const bool interior = tile_begin + TW <= cols;
        const bool readable = interior && tile_begin >= p.safe_lo && tile_begin + TW <= p.safe_hi;
)SRC";
    for (int k = 0; k < nreg; ++k) o << "        T r" << k << "[V];\n";
    for (int k = 0; k < p.n_leaf; ++k) {
        o << "        {\n            const T *base = static_cast<const T *>(p.leaf[" << k << "]) + static_cast<int64_t>(cur_row) * p.leaf_rs["
          << k << "];\n            if (p.leaf_cs[" << k << "] == 0) {\n                const T s = *base;\n"
          << "                _Pragma(\"unroll\") for (int j = 0; j < V; ++j) r" << k << "[j] = s;\n"
          << "            } else if (readable) {\n                _Pragma(\"unroll\") for (int u = 0; u < U; ++u) {\n"
          << "                    const vec_t v = *reinterpret_cast<const vec_t *>(base + c0 + u * (64 * VL));\n"
          << "                    _Pragma(\"unroll\") for (int j = 0; j < VL; ++j) r" << k << "[u * VL + j] = v[j];\n                }\n"
          << "            } else {\n                _Pragma(\"unroll\") for (int u = 0; u < U; ++u)\n"
          << "                    _Pragma(\"unroll\") for (int j = 0; j < VL; ++j) {\n"
          << "                        const int64_t c = c0 + u * (64 * VL) + j;\n"
          << "                        r" << k << "[u * VL + j] = (c < cols && c >= p.leaf_lo[" << k << "] && c < p.leaf_hi[" << k
          << "]) ? base[c] : T(1);\n                    }\n            }\n        }\n";
    }
    for (int k = 0; k < p.n_imm; ++k)
        o << "        _Pragma(\"unroll\") for (int j = 0; j < V; ++j) r" << (nreg - 1 - k) << "[j] = imm" << k << ";\n";
    for (int i = 0; i < p.n_instr; ++i) {
        const uint32_t w = p.code[i];
        const int op = w & 0xff, dst = (w >> 8) & 15;
        const int src[4] = {int(w >> 12) & 15, int(w >> 16) & 15, int(w >> 20) & 15, int(w >> 24) & 15};
        o << "        {  // instruction " << i << "\n";
        if (op == AGMI_PROGRAM_STORE) {
            o << "            T *base = static_cast<T *>(p.out[" << src[1] << "]) + static_cast<int64_t>(cur_row) * p.out_rs[" << src[1]
              << "];\n            _Pragma(\"unroll\") for (int u = 0; u < U; ++u) {\n                vec_t v;\n"
              << "                _Pragma(\"unroll\") for (int j = 0; j < VL; ++j) v[j] = r" << src[0] << "[u * VL + j];\n"
              << "                if (interior) __builtin_nontemporal_store(v, reinterpret_cast<vec_t *>(base + c0 + u * (64 * VL)));\n"
              << "                else store_partial<T, VL>(base, c0 + u * (64 * VL), cols, v);\n            }\n        }\n";
            continue;
        }
        o << "            T o_[V];\n";
        if (op == AGMI_PROGRAM_MASK) {
            o << "            const int64_t lo = p.mask_lo[" << src[1] << "], hi = p.mask_hi[" << src[1] << "];\n"
              << "            _Pragma(\"unroll\") for (int u = 0; u < U; ++u)\n                _Pragma(\"unroll\") for (int j = 0; j < VL; ++j) {\n"
              << "                    const int64_t cc = c0 + u * (64 * VL) + j;\n"
              << "                    o_[u * VL + j] = (cc >= lo && cc < hi) ? r" << src[0] << "[u * VL + j] : r" << src[2]
              << "[u * VL + j];\n                }\n";
        } else if (op == AGMI_PROGRAM_ROWSUM || op == AGMI_PROGRAM_ROWLSE) {
            o << "            const T total = program_row_reduce<" << (op == AGMI_PROGRAM_ROWSUM ? "AccSum" : "AccLse")
              << "<T>, T, VL, U>(row_values[threadIdx.x >> 6], lane, cols, p.row_group, r" << src[0] << ");\n"
              << "            _Pragma(\"unroll\") for (int j = 0; j < V; ++j) o_[j] = total;\n";
        } else {
            const char *fn = functor_name(op);
            const int arity = functor_arity(op);
            o << "            _Pragma(\"unroll\") for (int j = 0; j < V; ++j) {\n                const T in_[4] = {";
            for (int k = 0; k < 4; ++k) {
                if (k < arity) o << "r" << src[k] << "[j]";
                else o << "T(0)";
                o << (k < 3 ? ", " : "};\n");
            }
            o << "                T out_[1];\n                " << fn << "<T>::apply(in_, out_);\n                o_[j] = out_[0];\n            }\n";
        }
        o << "            _Pragma(\"unroll\") for (int j = 0; j < V; ++j) r" << dst << "[j] = o_[j];\n        }\n";
    }
    o << R"SRC(        t += p.step_rows * tpr + p.step_chunks;
        row += p.step_rows;
        chunk += p.step_chunks;
        if (chunk >= tpr) {
            chunk -= tpr;
            ++row;
        }
        if (t >= p.n_tiles) break;
    }
}
)SRC";
    return o.str();
}

static bool spec_compile(const std::string &source, const std::string &name, SpecKernel *k, std::string *log) {
    hiprtcProgram prog = nullptr;
    if (hiprtcCreateProgram(&prog, source.c_str(), "agmi_specialized.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
        *log = "hiprtcCreateProgram failed";
        return false;
    }
    // the flags the library itself is built with: no fused multiply-adds the rules do not have, no packed float32 forms
    const char *options[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
                             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    const hiprtcResult rc = hiprtcCompileProgram(prog, sizeof(options) / sizeof(options[0]), options);
    if (rc != HIPRTC_SUCCESS) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        log->assign(n, '\0');
        if (n) hiprtcGetProgramLog(prog, &(*log)[0]);
        hiprtcDestroyProgram(&prog);
        return false;
    }
    size_t size = 0;
    hiprtcGetCodeSize(prog, &size);
    std::vector<char> code(size);
    hiprtcGetCode(prog, code.data());
    hiprtcDestroyProgram(&prog);
    if (hipModuleLoadData(&k->module, code.data()) != hipSuccess) {
        (void)hipGetLastError();
        *log = "hipModuleLoadData failed";
        return false;
    }
    if (hipModuleGetFunction(&k->function, k->module, name.c_str()) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipModuleUnload(k->module);
        k->module = nullptr;
        *log = "hipModuleGetFunction failed";
        return false;
    }
    return true;
}

// 0: launched; 1: no specialised kernel for this program (the caller runs the interpreter); < 0: error
int launch_specialized(bool f32, int nreg, const ProgParams &p0, int64_t rows, hipStream_t s) {
    std::lock_guard<std::mutex> lock(g_spec_mutex);
    if (g_spec_after < 0) {
        const char *e = std::getenv("AUTOGRAD_AMD_SPECIALIZE");
        g_spec_after = e ? std::max(0, std::atoi(e)) : 3;
    }
    if (g_spec_after == 0) return 1;
    int device = 0;
    (void)hipGetDevice(&device);
    std::string key;
    key.reserve(32 + 4 * static_cast<size_t>(p0.n_instr));
    const int32_t head[6] = {f32 ? 1 : 0, nreg, p0.n_leaf, p0.n_imm, p0.row_group > 0 ? 1 : 0, device};
    key.append(reinterpret_cast<const char *>(head), sizeof(head));
    key.append(reinterpret_cast<const char *>(p0.code), sizeof(uint32_t) * static_cast<size_t>(p0.n_instr));
    auto it = g_spec.find(key);
    if (it == g_spec.end()) {
        if (g_spec.size() >= kSpecMaxSeen) {  // programs that came by once or twice and never again: forget them
            for (auto e = g_spec.begin(); e != g_spec.end();) e = e->second.state == 0 ? g_spec.erase(e) : std::next(e);
        }
        it = g_spec.emplace(key, SpecKernel()).first;
    }
    SpecKernel &k = it->second;
    if (k.state < 0) return 1;
    if (k.state == 0) {
        if (++k.seen < g_spec_after || g_spec_compiled >= kSpecMaxKernels) return 1;
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &capturing) != hipSuccess) (void)hipGetLastError();
        if (capturing != hipStreamCaptureStatusNone) return 1;  // a module cannot be loaded while a graph is recorded
        std::string log;
        const std::string name = spec_name(f32, p0);
        if (!spec_compile(spec_source(f32, nreg, p0, name), name, &k, &log)) {
            k.state = -1;
            set_error("program: specialising a recurring program failed, the interpreter keeps running it: %.400s", log.c_str());
            return 1;
        }
        k.state = 1;
        k.name = name;
        ++g_spec_compiled;
    }
    ProgParams p = p0;
    constexpr int64_t kWavesPerBlock = 4;
    const int64_t TW = 64 * 2 * (f32 ? 4 : 2);
    const int64_t tpr = ceil_div(p.cols, TW), n_tiles = tpr * rows;
    if (tpr >= 0x7fffffffLL || n_tiles >= 0x7fffffffLL) return 1;
    // a tile per wave up to a grid that fills the part many times over, then a few tiles per wave
    const int64_t blocks = std::min<int64_t>(ceil_div(n_tiles, kWavesPerBlock), 256 * 64);
    const int64_t n_waves = blocks * kWavesPerBlock;
    p.tiles_per_row = static_cast<uint32_t>(tpr);
    p.n_tiles = static_cast<uint32_t>(n_tiles);
    p.step_rows = static_cast<uint32_t>(n_waves / tpr);
    p.step_chunks = static_cast<uint32_t>(n_waves % tpr);
    size_t size = sizeof(p);
    void *extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &p, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
    set_kernel_name("%s[%lldx%lld]", k.name.c_str(), (long long)rows, (long long)p.cols);
    const hipError_t rc = hipModuleLaunchKernel(k.function, static_cast<unsigned>(blocks), 1, 1, 256, 1, 1, 0, s, nullptr, extra);
    if (rc != hipSuccess) return hip_check(rc, "specialised program launch");
    ++g_spec_launches;
    return 0;
}

}  // namespace agmi

using namespace agmi;

extern "C" int agmi_program_specialize(int after) {
    std::lock_guard<std::mutex> lock(g_spec_mutex);
    if (g_spec_after < 0) {
        const char *e = std::getenv("AUTOGRAD_AMD_SPECIALIZE");
        g_spec_after = e ? std::max(0, std::atoi(e)) : 3;
    }
    const int before = g_spec_after;
    if (after >= 0) g_spec_after = after;
    return before;
}

extern "C" void agmi_program_specialized(long long *compiled, long long *launches) {
    std::lock_guard<std::mutex> lock(g_spec_mutex);
    if (compiled) *compiled = g_spec_compiled;
    if (launches) *launches = g_spec_launches;
}

extern "C" long long agmi_program_source(int dtype, int n_leaf, int n_imm, int n_instr, const uint32_t *code, int n_regs,
                                         int row_sums, char *text, size_t capacity) {
    if ((dtype != AGMI_F32 && dtype != AGMI_F64) || n_leaf < 0 || n_leaf > kProgMaxLeaf || n_imm < 0 || n_imm > kProgMaxImm ||
        n_instr < 1 || n_instr > kProgMaxInstr || !code) {
        set_error("program_source: bad counts or null code");
        return AGMI_ERR_ARG;
    }
    ProgParams p = {};
    p.n_leaf = n_leaf;
    p.n_imm = n_imm;
    p.n_instr = n_instr;
    p.row_group = row_sums ? 1 : 0;
    for (int i = 0; i < n_instr; ++i) {
        const int op = code[i] & 0xff;
        if (op != AGMI_PROGRAM_STORE && op != AGMI_PROGRAM_MASK && op != AGMI_PROGRAM_ROWSUM && op != AGMI_PROGRAM_ROWLSE &&
            !functor_name(op)) {
            set_error("program_source: instruction %d has unknown op %d", i, op);
            return AGMI_ERR_ARG;
        }
        p.code[i] = code[i];
    }
    const int nreg = (n_regs <= 8 && dtype == AGMI_F64) ? 8 : 16;
    const std::string source = spec_source(dtype == AGMI_F32, nreg, p, spec_name(dtype == AGMI_F32, p));
    if (text && capacity > 0) {
        const size_t n = std::min(capacity - 1, source.size());
        std::memcpy(text, source.data(), n);
        text[n] = '\0';
    }
    return static_cast<long long>(source.size());
}
