// Host-level Tiled broadcast and mapreduce: stand-ins for `_tiled_broadcast!` + `broadcast_kernel`
// (reference: src/broadcast.jl:75-129) and `_mapreducedim!` + `mapreduce_kernel`
// (reference: src/mapreduce.jl:13-129).
//
// The reference compiles one Tile IR kernel per (function tree, argument types) the first time it
// is used and caches it.  The same happens here with hiprtc: the expression tree arrives as text
// (tiled_expr.h), Julia's element-type rules give every node its type, and one fused HIP kernel is
// generated, compiled for gfx950, loaded and cached per device; later calls are a hash lookup and a
// launch.  What is baked into a kernel: the tree, the element types, the number of dimensions left
// after merging, which leaves vary along dimension 0, whether 16-byte accesses are legal, and the
// cache policy.  Sizes, strides, pointers and scalar values are run-time arguments.
//
// Mapping to the chip (instead of the reference's power-of-two tiles of 4096 elements,
// src/utils.jl:50-72): dimensions are merged wherever the memory layout allows, every lane moves
// 16 bytes per access along dimension 0, and a reduction runs in one of two shapes --
//   "run":    dimension 0 is reduced: a workgroup (64 or 256 lanes) per output element, lanes
//             stride over the contiguous run, wave64 shuffles + LDS finish;
//   "column": dimension 0 is kept: a lane owns 16 bytes of consecutive outputs and walks the
//             reduced dimensions, the rows of a workgroup share the walk and combine through LDS.
// Too few outputs to fill 256 CUs: the reduced range is split over P workgroups that write
// partials to the caller's workspace and the same kernel shape reduces the P partials (two passes,
// fixed order, no atomics -- results are reproducible, unlike src/mapreduce.jl:91-108).
#include <dlfcn.h>
#include <hip/hiprtc.h>
#include <mutex>
#include <string>
#include <unordered_map>
#include "common.h"
#include "tiled_device.h"
#include "tiled_expr.h"

namespace {

using namespace mi;
using namespace mi::tiled;

// ---- run-time compilation ------------------------------------------------------------------------
std::mutex g_mu;
std::unordered_map<std::string, hipFunction_t> g_cache;   // key: device id + generated source
bool g_dry_run = false;                                   // compile only: no module load, no launch
int g_compiles = 0;

// hiprtc is loaded on first use, so that the ahead-of-time entry points of the library do not depend on
// libhiprtc.so being present; only the Tiled entry points need it.
struct Rtc {
    decltype(&hiprtcCreateProgram) create = nullptr;
    decltype(&hiprtcCompileProgram) compile = nullptr;
    decltype(&hiprtcGetProgramLogSize) log_size = nullptr;
    decltype(&hiprtcGetProgramLog) log = nullptr;
    decltype(&hiprtcGetCodeSize) code_size = nullptr;
    decltype(&hiprtcGetCode) code = nullptr;
    decltype(&hiprtcDestroyProgram) destroy = nullptr;
    decltype(&hiprtcGetErrorString) error_string = nullptr;
    bool ok = false;
};
const Rtc& rtc() {
    static const Rtc r = [] {
        Rtc t;
        void* h = nullptr;
        for (const char* name : {"libhiprtc.so", "libhiprtc.so.7", "/opt/rocm/lib/libhiprtc.so"}) {
            h = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
            if (h) break;
        }
        if (!h) return t;
#define SYM(field, name) t.field = reinterpret_cast<decltype(t.field)>(dlsym(h, #name))
        SYM(create, hiprtcCreateProgram);
        SYM(compile, hiprtcCompileProgram);
        SYM(log_size, hiprtcGetProgramLogSize);
        SYM(log, hiprtcGetProgramLog);
        SYM(code_size, hiprtcGetCodeSize);
        SYM(code, hiprtcGetCode);
        SYM(destroy, hiprtcDestroyProgram);
        SYM(error_string, hiprtcGetErrorString);
#undef SYM
        t.ok = t.create && t.compile && t.log_size && t.log && t.code_size && t.code && t.destroy && t.error_string;
        return t;
    }();
    return r;
}

int compile(const std::string& gen, const char* kernel, hipFunction_t* fn) {
    int dev = 0;
    if (!g_dry_run && hipGetDevice(&dev) != hipSuccess) return (int)hipGetLastError();
    const std::string key = std::to_string(dev) + "#" + gen;
    bool dry;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        auto it = g_cache.find(key);
        if (it != g_cache.end()) { *fn = it->second; return MI_OK; }
        dry = g_dry_run;
    }
    // The compilation itself (a few tenths of a second) runs outside the lock: other threads keep launching
    // the kernels they already have.  Two threads that meet the same new expression both compile it; the
    // first to finish enters the cache.
    const Rtc& R = rtc();
    if (!R.ok) {
        fprintf(stderr, "libmi355tile: libhiprtc.so could not be loaded; the Tiled entry points need it\n");
        return MI_E_UNSUPPORTED;
    }
    const std::string src = std::string(kDevicePreamble) + gen;
    if (getenv("MI_TILED_DUMP")) fprintf(stderr, "%s\n", gen.c_str());
    hiprtcProgram prog;
    if (R.create(&prog, src.c_str(), "mi_tiled.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS) return MI_E_UNSUPPORTED;
    const char* opts[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    const hiprtcResult rc = R.compile(prog, (int)(sizeof(opts) / sizeof(opts[0])), opts);
    if (rc != HIPRTC_SUCCESS) {
        size_t n = 0;
        R.log_size(prog, &n);
        std::string log(n, '\0');
        if (n) R.log(prog, &log[0]);
        fprintf(stderr, "libmi355tile: run-time compilation failed (%s)\n%s\n---- generated source ----\n%s\n",
                R.error_string(rc), log.c_str(), gen.c_str());
        R.destroy(&prog);
        return MI_E_UNSUPPORTED;
    }
    hipFunction_t f = nullptr;
    if (!dry) {
        size_t n = 0;
        R.code_size(prog, &n);
        std::string code(n, '\0');
        R.code(prog, &code[0]);
        hipModule_t mod;
        hipError_t e = hipModuleLoadData(&mod, code.data());   // stays loaded until the process ends
        if (e == hipSuccess) e = hipModuleGetFunction(&f, mod, kernel);
        if (e != hipSuccess) { R.destroy(&prog); return (int)e; }
    }
    R.destroy(&prog);
    std::lock_guard<std::mutex> lock(g_mu);
    ++g_compiles;
    auto ins = g_cache.emplace(key, f);
    *fn = ins.first->second;
    return MI_OK;
}

// Kernels already built, by a short key (expression text + the constants baked into the kernel), so
// that a repeated call does not have to regenerate the source text just to find its kernel.
std::unordered_map<std::string, hipFunction_t> g_by_key;

template <typename MakeSource>
int kernel_for(const std::string& key, const char* kernel, MakeSource make_source, hipFunction_t* fn) {
    int dev = 0;
    if (!g_dry_run && hipGetDevice(&dev) != hipSuccess) return (int)hipGetLastError();
    const std::string k = std::to_string(dev) + "#" + key;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        auto it = g_by_key.find(k);
        if (it != g_by_key.end()) { *fn = it->second; return MI_OK; }
    }
    MI_CHECK(compile(make_source(), kernel, fn));
    std::lock_guard<std::mutex> lock(g_mu);
    g_by_key.emplace(k, *fn);
    return MI_OK;
}

int launch(hipFunction_t f, int64_t blocks, int threads, void* args, size_t bytes, hipStream_t s) {
    if (g_dry_run) return MI_OK;
    if (blocks <= 0) return MI_OK;
    if (blocks > 0x7fffffffLL) return MI_E_GRID;
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &bytes, HIP_LAUNCH_PARAM_END};
    const hipError_t e = hipModuleLaunchKernel(f, (unsigned)blocks, 1, 1, (unsigned)threads, 1, 1, 0, s, nullptr, extra);
    return e == hipSuccess ? MI_OK : (int)e;
}

// set_variant keeps the pointer it is given: names built at run time live in this per-thread string.
void set_variant_text(const char* text) {
    static thread_local std::string keep;
    keep = text;
    set_variant(keep.c_str());
}

int tiled_dtype_size(int dt) { return dt == MI_BOOL ? 1 : (dt == MI_F8E4M3FN || dt == MI_F8E5M2 ? 0 : dtype_size(dt)); }

// Arrays of this API: 0 to 4 dimensions, any element strides, pointer aligned to the element.
int check_tiled(const mi_tile_array* a) {
    if (!a) return MI_E_NULL;
    if (a->ndim < 0 || a->ndim > 4) return MI_E_RANK;
    const int es = tiled_dtype_size(a->dtype);
    if (es == 0) return MI_E_DTYPE;
    int64_t n = 1;
    for (int i = 0; i < a->ndim; ++i) {
        if (a->sizes[i] < 0) return MI_E_SHAPE;
        n *= a->sizes[i];
    }
    if (n > 0 && !a->ptr) return MI_E_NULL;
    if (((uintptr_t)a->ptr) % (uintptr_t)es) return MI_E_ALIGN;
    return MI_OK;
}
int64_t size_of(const mi_tile_array* a, int d) { return d < a->ndim ? a->sizes[d] : 1; }
int64_t stride_of(const mi_tile_array* a, int d) { return d < a->ndim ? a->strides[d] : 0; }

struct ScalarArgs { double sf[kMaxScalars]; long long si[kMaxScalars]; };

int pack_scalars(const mi_tile_scalar* sc, int ns, int32_t* dts, ScalarArgs* out) {
    if (ns < 0 || ns > kMaxScalars) return MI_E_UNSUPPORTED;
    if (ns && !sc) return MI_E_NULL;
    for (int i = 0; i < kMaxScalars; ++i) { out->sf[i] = 0; out->si[i] = 0; }
    for (int i = 0; i < ns; ++i) {
        dts[i] = sc[i].dtype;
        if (!dt_ok(sc[i].dtype)) return MI_E_DTYPE;
        if (dt_is_float(sc[i].dtype)) out->sf[i] = sc[i].value.f;
        else out->si[i] = sc[i].dtype == MI_BOOL ? (sc[i].value.i != 0) : sc[i].value.i;
    }
    return MI_OK;
}

// `const float s0 = (float)A.sf[0];` ... for the scalars the tree uses.
std::string scalar_decls(const Expr& e, const int32_t* dts) {
    std::string o;
    char buf[128];
    for (int i = 0; i < e.scalars_used; ++i) {
        const bool fl = dt_is_float(dts[i]);
        snprintf(buf, sizeof buf, "    const %s s%d = cvt<%s>(A.%s[%d]);\n", carrier(dts[i]), i, tag(dts[i]), fl ? "sf" : "si", i);
        o += buf;
    }
    return o;
}
std::string eval_params(const Expr& e, const int32_t* leaf_dt, const int32_t* scal_dt) {
    std::string o;
    char buf[64];
    bool first = true;
    for (int i = 0; i < e.leaves_used; ++i) { snprintf(buf, sizeof buf, "%s%s a%d", first ? "" : ", ", carrier(leaf_dt[i]), i); o += buf; first = false; }
    for (int i = 0; i < e.scalars_used; ++i) { snprintf(buf, sizeof buf, "%s%s s%d", first ? "" : ", ", carrier(scal_dt[i]), i); o += buf; first = false; }
    return o;
}

int pow2ceil(int64_t v) { int p = 1; while (p < v && p < (1 << 30)) p <<= 1; return p; }

// ================================================================================================
// Broadcast
// ================================================================================================
struct BcLeafArg { const void* p; long long st[4]; };
struct BcArgs {
    void* d;
    long long dst[4];
    long long size[4];
    BcLeafArg leaf[kMaxLeaves];
    double sf[kMaxScalars];
    long long si[kMaxScalars];
    long long nbx;
};

int broadcast_impl(const mi_tile_array* dest, const char* text, const mi_tile_array* const* leaves, int nl,
                   const mi_tile_scalar* scalars, int ns, hipStream_t stream) {
    MI_CHECK(check_tiled(dest));
    if (nl < 0 || nl > kMaxLeaves) return MI_E_UNSUPPORTED;
    if (nl && !leaves) return MI_E_NULL;
    int32_t leaf_dt[kMaxLeaves] = {0}, scal_dt[kMaxScalars] = {0};
    for (int i = 0; i < nl; ++i) { MI_CHECK(check_tiled(leaves[i])); leaf_dt[i] = leaves[i]->dtype; }
    ScalarArgs sa;
    MI_CHECK(pack_scalars(scalars, ns, scal_dt, &sa));
    Expr e;
    MI_CHECK(parse_expr(text, e));
    MI_CHECK(infer_types(e, leaf_dt, nl, scal_dt, ns));

    // Base.Broadcast.check_broadcast_axes: a leaf dimension equals the destination's or is 1.
    const int nd = dest->ndim;
    for (int i = 0; i < nl; ++i)
        for (int d = 0; d < 4; ++d) {
            const int64_t s = size_of(leaves[i], d);
            if (s != 1 && s != size_of(dest, d)) return MI_E_SHAPE;
        }
    int64_t total = 1;
    for (int d = 0; d < nd; ++d) total *= dest->sizes[d];
    if (total == 0) return MI_OK;

    // Merge dimensions: drop extent-1 dimensions, fuse neighbours that are one run in every array.
    int64_t size[4], dst[4], lst[kMaxLeaves][4];
    int n = 0;
    for (int d = 0; d < 4; ++d) {
        const int64_t s = size_of(dest, d);
        if (s == 1) continue;
        bool fuse = n > 0 && stride_of(dest, d) == dst[n - 1] * size[n - 1];
        for (int i = 0; i < nl && fuse; ++i) {
            const int64_t st = size_of(leaves[i], d) == 1 ? 0 : stride_of(leaves[i], d);
            fuse = st == lst[i][n - 1] * size[n - 1];
        }
        if (fuse) { size[n - 1] *= s; continue; }
        size[n] = s;
        dst[n] = stride_of(dest, d);
        for (int i = 0; i < nl; ++i) lst[i][n] = size_of(leaves[i], d) == 1 ? 0 : stride_of(leaves[i], d);
        ++n;
    }
    if (n == 0) { size[0] = 1; dst[0] = 1; for (int i = 0; i < nl; ++i) lst[i][0] = 0; n = 1; }
    for (int d = n; d < 4; ++d) { size[d] = 1; dst[d] = 0; for (int i = 0; i < nl; ++i) lst[i][d] = 0; }

    // Elements per lane: 16 bytes of the widest type that runs along dimension 0.
    int widest = tiled_dtype_size(dest->dtype);
    int64_t bytes = total * widest;
    for (int i = 0; i < e.leaves_used; ++i) {
        const int es = tiled_dtype_size(leaf_dt[i]);
        if (lst[i][0] != 0 && es > widest) widest = es;
        int64_t ln = 1;
        for (int d = 0; d < n; ++d) if (lst[i][d] != 0) ln *= size[d];
        bytes += ln * es;
    }
    int V = 16 / widest;
    if (V > 8) V = 8;
    auto vec_ok = [&](const void* p, int es, const int64_t* st) {
        if (st[0] != 1) return false;
        if (((uintptr_t)p) % (uintptr_t)(V * es < 16 ? V * es : 16)) return false;
        for (int d = 1; d < n; ++d) if ((st[d] * es) % (V * es < 16 ? V * es : 16)) return false;
        return true;
    };
    const bool vec_d = vec_ok(dest->ptr, tiled_dtype_size(dest->dtype), dst);
    bool keep0[kMaxLeaves], vec_l[kMaxLeaves];
    for (int i = 0; i < nl; ++i) {
        keep0[i] = lst[i][0] != 0;
        vec_l[i] = keep0[i] && vec_ok(leaves[i]->ptr, tiled_dtype_size(leaf_dt[i]), lst[i]);
    }
    const int64_t nvec0 = cld(size[0], (int64_t)V);
    const int TX = nvec0 >= 256 ? 256 : pow2ceil(nvec0);
    const int TY = 256 / TX;
    const int U = nvec0 >= 4 * (int64_t)TX ? 4 : 1;
    const bool NT = stream_hint(bytes);
    const int64_t rows = size[1] * size[2] * size[3];
    if (rows > 0x7fffffffLL || nvec0 > 0x7fffffffLL * 64) return MI_E_GRID;
    const int64_t nbx = cld(nvec0, (int64_t)TX * U), nby = cld(rows, (int64_t)TY);
    if (nbx > 0x7fffffffLL || nbx * nby > 0x7fffffffLL) return MI_E_GRID;

    // ---- kernel: looked up by what is baked into it, generated and compiled on a miss ----
    char buf[512];
    std::string key = "bc|";
    key += text;
    snprintf(buf, sizeof buf, "|%d|%d,%d,%d,%d,%d,%d,%d|", dest->dtype, V, U, TX, TY, n, NT ? 1 : 0, vec_d ? 1 : 0);
    key += buf;
    for (int i = 0; i < e.leaves_used; ++i) { snprintf(buf, sizeof buf, "%d%c%c,", leaf_dt[i], keep0[i] ? 'k' : 'b', vec_l[i] ? 'v' : 's'); key += buf; }
    key += "|";
    for (int i = 0; i < e.scalars_used; ++i) { snprintf(buf, sizeof buf, "%d,", scal_dt[i]); key += buf; }
    auto make_source = [&]() {
    std::string g;
    snprintf(buf, sizeof buf, "constexpr int V = %d, U = %d, TX = %d, TY = %d, NDIM = %d;\nconstexpr bool NT = %s, VECD = %s;\n", V, U, TX, TY,
             n, NT ? "true" : "false", vec_d ? "true" : "false");
    g += buf;
    snprintf(buf, sizeof buf, "typedef %s DST;\nconstexpr int DEST = %s;\n", storage(dest->dtype), tag(dest->dtype));
    g += buf;
    g += "struct Leaf { const void* p; long long st[4]; };\n"
         "struct Args { void* d; long long dst[4]; long long size[4]; Leaf leaf[8]; double sf[8]; long long si[8]; long long nbx; };\n";
    g += "__device__ __forceinline__ car<DEST> eval(" + eval_params(e, leaf_dt, scal_dt) + ") {\n" + emit_body(e);
    snprintf(buf, sizeof buf, "    return cvt<DEST>(t%d);\n}\n", e.root);
    g += buf;
    g += "extern \"C\" __global__ __launch_bounds__(256) void tiled_bc(Args A) {\n"
         "    const unsigned nbx = (unsigned)A.nbx;\n"
         "    const unsigned bx = blockIdx.x % nbx, by = blockIdx.x / nbx;\n"
         "    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;\n"
         "    const long long n0 = A.size[0];\n"
         "    const unsigned rows = (unsigned)(A.size[1] * A.size[2] * A.size[3]);\n"
         "    const unsigned row = by * TY + ty;\n"
         "    if (row >= rows) return;\n"
         "    unsigned i1 = row, i2 = 0, i3 = 0;\n"
         "    if constexpr (NDIM >= 3) { i2 = row / (unsigned)A.size[1]; i1 = row - i2 * (unsigned)A.size[1]; }\n"
         "    if constexpr (NDIM == 4) { i3 = i2 / (unsigned)A.size[2]; i2 = i2 - i3 * (unsigned)A.size[2]; }\n"
         "    DST* dp = (DST*)A.d + i1 * A.dst[1] + i2 * A.dst[2] + i3 * A.dst[3];\n";
    g += scalar_decls(e, scal_dt);
    for (int i = 0; i < e.leaves_used; ++i) {
        snprintf(buf, sizeof buf,
                 "    typedef %s L%d;\n    const L%d* p%d = (const L%d*)A.leaf[%d].p + i1 * A.leaf[%d].st[1] + i2 * A.leaf[%d].st[2] + i3 * A.leaf[%d].st[3];\n",
                 storage(leaf_dt[i]), i, i, i, i, i, i, i, i);
        g += buf;
        if (keep0[i]) { snprintf(buf, sizeof buf, "    L%d r%d[U][V] = {};\n", i, i); g += buf; }
        else { snprintf(buf, sizeof buf, "    const car<%s> c%d = to_car(ldg<false>(p%d));\n", tag(leaf_dt[i]), i, i); g += buf; }
    }
    // The block body is emitted twice: without predicates for blocks that lie wholly inside
    // dimension 0 (all loads of a lane are issued before the first use), with them for the last one.
    auto emit_block = [&](bool guard) {
        const char* left = guard ? "n0 - i0" : "(long long)V";
        g += "#pragma unroll\n        for (int u = 0; u < U; ++u) {\n"
             "            const long long i0 = (((long long)bx * U + u) * TX + tx) * V;\n";
        if (guard) g += "            if (i0 < n0) {\n";
        for (int i = 0; i < e.leaves_used; ++i)
            if (keep0[i]) {
                snprintf(buf, sizeof buf, "            load_run<L%d, V, %s, NT>(p%d + i0 * A.leaf[%d].st[0], %s, A.leaf[%d].st[0], r%d[u]);\n", i,
                         vec_l[i] ? "true" : "false", i, i, left, i, i);
                g += buf;
            }
        if (guard) g += "            }\n";
        g += "        }\n"
             "#pragma unroll\n        for (int u = 0; u < U; ++u) {\n"
             "            const long long i0 = (((long long)bx * U + u) * TX + tx) * V;\n";
        if (guard) g += "            if (i0 < n0) {\n";
        g += "            DST o[V];\n"
             "#pragma unroll\n            for (int q = 0; q < V; ++q) o[q] = to_sto<DST>(eval(";
        bool first = true;
        for (int i = 0; i < e.leaves_used; ++i) {
            if (keep0[i]) snprintf(buf, sizeof buf, "%sto_car(r%d[u][q])", first ? "" : ", ", i);
            else snprintf(buf, sizeof buf, "%sc%d", first ? "" : ", ", i);
            g += buf;
            first = false;
        }
        for (int i = 0; i < e.scalars_used; ++i) { snprintf(buf, sizeof buf, "%ss%d", first ? "" : ", ", i); g += buf; first = false; }
        g += "));\n";
        snprintf(buf, sizeof buf, "            store_run<DST, V, VECD, NT>(dp + i0 * A.dst[0], %s, A.dst[0], o);\n", left);
        g += buf;
        if (guard) g += "            }\n";
        g += "        }\n";
    };
    g += "    if (((long long)bx + 1) * U * TX * V <= n0) {\n";
    emit_block(false);
    g += "    } else {\n";
    emit_block(true);
    g += "    }\n}\n";

    return g;
    };
    hipFunction_t fn = nullptr;
    MI_CHECK(kernel_for(key, "tiled_bc", make_source, &fn));
    BcArgs a;
    memset(&a, 0, sizeof a);
    a.d = dest->ptr;
    for (int d = 0; d < 4; ++d) { a.dst[d] = dst[d]; a.size[d] = size[d]; }
    for (int i = 0; i < nl; ++i) {
        a.leaf[i].p = leaves[i]->ptr;
        for (int d = 0; d < 4; ++d) a.leaf[i].st[d] = lst[i][d];
    }
    memcpy(a.sf, sa.sf, sizeof a.sf);
    memcpy(a.si, sa.si, sizeof a.si);
    a.nbx = nbx;
    snprintf(buf, sizeof buf, "tiled_bc_v%d_u%d_tx%d_nd%d%s", V, U, TX, n, NT ? "_stream" : "");
    set_variant_text(buf);
    return launch(fn, nbx * nby, 256, &a, sizeof a, stream);
}

// ================================================================================================
// Mapreduce
// ================================================================================================
struct MrArgs {
    const void* src;
    void* dst;
    long long size[4];
    long long sst[4];
    long long dstr[4];
    long long P;
    long long nbx;
    long long nk;        // number of outputs (partials of split p start at nk * p in the column shape)
    long long chunk;     // reduced indices per split: split p owns [p * chunk, (p + 1) * chunk)
    double sf[kMaxScalars];
    long long si[kMaxScalars];
};

// The two kernel shapes; constants and the functions mapf / redop / neutral precede this text.
// RMASK: bit d set = dimension d is reduced.  Outputs are numbered over the kept dimensions in
// order, the reduced index space over the reduced ones; both are unpacked with 32-bit divisions
// that the compiler drops for dimensions of the other role.
const char* const kRunKernel = R"SRC(
// LANES lanes (a power of two up to the workgroup) share one output; a workgroup holds T / LANES outputs.
extern "C" __global__ __launch_bounds__(T) void tiled_mr(Args A) {
    constexpr int G = T / LANES;
    const unsigned P = (unsigned)A.P;
    const unsigned p = blockIdx.x % P;
    const unsigned o = (blockIdx.x / P) * G + threadIdx.x / LANES;
    const unsigned lane = threadIdx.x % LANES;
    const bool live = o < (unsigned long long)A.nk;
    long long soff = 0, doff = 0;
    {
        unsigned rest = o;
#pragma unroll
        for (int d = 1; d < 4; ++d)
            if (!((RMASK >> d) & 1)) {
                const unsigned n = (unsigned)A.size[d], k = rest % n;
                rest /= n;
                soff += k * A.sst[d];
                doff += k * A.dstr[d];
            }
    }
    const SST* base = (const SST*)A.src + soff;
    const long long n0 = A.size[0];
    const unsigned nvec0 = (unsigned)((n0 + V - 1) / V);
    unsigned long long nq = nvec0;
#pragma unroll
    for (int d = 1; d < 4; ++d) if ((RMASK >> d) & 1) nq *= (unsigned long long)A.size[d];
    unsigned long long qend = (unsigned long long)(p + 1) * (unsigned long long)A.chunk;
    if (qend > nq) qend = nq;
    if (!live) qend = 0;
    SCALARS
    AC acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = neutral();
#pragma unroll UNR
    for (unsigned long long q = (unsigned long long)p * (unsigned long long)A.chunk + lane; q < qend; q += LANES) {
        unsigned v0 = (unsigned)q;
        long long off = 0;
        if constexpr ((RMASK & 14) != 0) {
            unsigned rest = (unsigned)q / nvec0;
            v0 = (unsigned)q - rest * nvec0;
#pragma unroll
            for (int d = 1; d < 4; ++d)
                if ((RMASK >> d) & 1) {
                    // the highest reduced dimension takes what is left: no division for it
                    if ((RMASK >> (d + 1)) == 0) { off += rest * A.sst[d]; }
                    else {
                        const unsigned n = (unsigned)A.size[d], r = rest % n;
                        rest /= n;
                        off += r * A.sst[d];
                    }
                }
        }
        const long long i0 = (long long)v0 * V, left = n0 - i0;
        SST r[V] = {};
        load_run<SST, V, VEC, NT>(base + i0 * A.sst[0] + off, left, A.sst[0], r);
#pragma unroll
        for (int e = 0; e < V; ++e) if (e < left) acc[e] = redop(acc[e], MAPF(to_car(r[e])));
    }
    AC a = acc[0];
#pragma unroll
    for (int e = 1; e < V; ++e) a = redop(a, acc[e]);
#pragma unroll
    for (int m = (LANES < 64 ? LANES : 64) / 2; m >= 1; m >>= 1) a = redop(a, xor_lane(a, m));
    if constexpr (LANES > 64) {
        __shared__ AC sh[T / 64];
        if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = a;
        __syncthreads();
        if (lane == 0) for (int w = 1; w < LANES / 64; ++w) a = redop(a, sh[(threadIdx.x >> 6) + w]);
    }
    if (lane == 0 && live) {
        if constexpr (OUT_WS) ((AC*)A.dst)[p + (unsigned long long)P * o] = a;
        else ((DST*)A.dst)[doff] = to_sto<DST>(a);
    }
}
)SRC";

const char* const kColumnKernel = R"SRC(
extern "C" __global__ __launch_bounds__(TX * TY) void tiled_mr(Args A) {
    const unsigned P = (unsigned)A.P, nbx = (unsigned)A.nbx;
    unsigned b = blockIdx.x;
    const unsigned bx = b % nbx; b /= nbx;
    const unsigned p = b % P, kb = b / P;
    long long soff = 0, doff = 0;
    {
        unsigned rest = kb;
#pragma unroll
        for (int d = 1; d < 4; ++d)
            if (!((RMASK >> d) & 1)) {
                const unsigned n = (unsigned)A.size[d], k = rest % n;
                rest /= n;
                soff += k * A.sst[d];
                doff += k * A.dstr[d];
            }
    }
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const long long n0 = A.size[0];
    const long long i0 = ((long long)bx * TX + tx) * V, left = n0 - i0;
    const bool live = i0 < n0;
    unsigned long long nq = 1;
#pragma unroll
    for (int d = 1; d < 4; ++d) if ((RMASK >> d) & 1) nq *= (unsigned long long)A.size[d];
    const SST* base = (const SST*)A.src + i0 * A.sst[0] + soff;
    SCALARS
    AC acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = neutral();
    unsigned long long qend = (unsigned long long)(p + 1) * (unsigned long long)A.chunk;
    if (qend > nq) qend = nq;
    if (live) {
#pragma unroll UNR
        for (unsigned long long q = (unsigned long long)p * (unsigned long long)A.chunk + ty; q < qend; q += TY) {
            unsigned rest = (unsigned)q;
            long long off = 0;
#pragma unroll
            for (int d = 1; d < 4; ++d)
                if ((RMASK >> d) & 1) {
                    // the highest reduced dimension takes what is left: no division for it
                    if ((RMASK >> (d + 1)) == 0) { off += rest * A.sst[d]; }
                    else {
                        const unsigned n = (unsigned)A.size[d], r = rest % n;
                        rest /= n;
                        off += r * A.sst[d];
                    }
                }
            SST r[V] = {};
            load_run<SST, V, VEC, NT>(base + off, left, A.sst[0], r);
#pragma unroll
            for (int e = 0; e < V; ++e) if (e < left) acc[e] = redop(acc[e], MAPF(to_car(r[e])));
        }
    }
    if constexpr (TY > 1) {
        __shared__ AC sh[(TY / 2) * TX * V];
        for (int s = TY / 2; s >= 1; s >>= 1) {
            if (ty >= s && ty < 2 * s) {
#pragma unroll
                for (int e = 0; e < V; ++e) sh[((ty - s) * TX + tx) * V + e] = acc[e];
            }
            __syncthreads();
            if (ty < s) {
#pragma unroll
                for (int e = 0; e < V; ++e) acc[e] = redop(acc[e], sh[(ty * TX + tx) * V + e]);
            }
            __syncthreads();
        }
    }
    if (ty == 0 && live) {
        if constexpr (OUT_WS) {
            AC* w = (AC*)A.dst + (i0 + n0 * kb) + (unsigned long long)A.nk * p;
#pragma unroll
            for (int e = 0; e < V; ++e) if (e < left) w[e] = acc[e];
        } else {
            DST o[V];
#pragma unroll
            for (int e = 0; e < V; ++e) o[e] = to_sto<DST>(acc[e]);
            store_run<DST, V, VECD, false>((DST*)A.dst + i0 * A.dstr[0] + doff, left, A.dstr[0], o);
        }
    }
}
)SRC";

const char* neutral_text(int op, int dt) {
    const bool f64 = dt == MI_F64, fl = dt_is_float(dt);
    switch (op) {
        case MI_OP_ADD: case MI_OP_OR: return "(AC)0";
        case MI_OP_MUL: return "(AC)1";
        case MI_OP_AND: return dt == MI_BOOL ? "true" : "(AC)-1";
        case MI_OP_MAX:
            if (fl) return f64 ? "-__builtin_huge_val()" : "-__builtin_huge_valf()";
            return dt == MI_I32 ? "(-2147483647 - 1)" : dt == MI_I64 ? "(-9223372036854775807LL - 1)" : "false";
        default:
            if (fl) return f64 ? "__builtin_huge_val()" : "__builtin_huge_valf()";
            return dt == MI_I32 ? "2147483647" : dt == MI_I64 ? "9223372036854775807LL" : "true";
    }
}
const char* op_fn(int op) {
    switch (op) {
        case MI_OP_ADD: return "f_add";
        case MI_OP_MUL: return "f_mul";
        case MI_OP_MAX: return "f_max";
        case MI_OP_MIN: return "f_min";
        case MI_OP_AND: return "f_and";
        default: return "f_or";
    }
}
// The type partial results are stored in between the two passes: the carrier of the accumulator.
int carrier_dtype(int dt) { return (dt == MI_F16 || dt == MI_BF16) ? MI_F32 : dt; }

struct MrShape {
    int rmask;           // bit d: dimension d is reduced; bit 0 decides the kernel shape
    int64_t size[4], sst[4], dstr[4];
    bool run() const { return rmask & 1; }
    bool red(int d) const { return (rmask >> d) & 1; }
};
struct MrPlan {
    int V, T, TX, TY, UNR, LANES;
    bool vec, vecd, nt;
    int64_t P, nbx, blocks, nk, chunk;
};

// Tuning overrides (environment): workgroups a split reduction aims for, iterations a lane should
// at least have, unroll factor of the accumulation loop.
int knob(const char* name, int dflt) {
    const char* e = getenv(name);
    const int v = e ? atoi(e) : 0;
    return v > 0 ? v : dflt;
}
int knob_blocks() { static const int v = knob("MI_TILED_BLOCKS", 2048); return v; }
int knob_column_blocks() { static const int v = knob("MI_TILED_COLUMN_BLOCKS", 2048); return v; }
int knob_min_tx() { static const int v = knob("MI_TILED_MIN_TX", 32); return v; }   // 32 lanes x 16 B = 512-byte runs: the shortest that read at full rate
int knob_iters() { static const int v = knob("MI_TILED_ITERS", 8); return v; }
int knob_unroll() { static const int v = knob("MI_TILED_UNROLL", 4); return v; }

// Launch geometry of one pass; `allow_split` false for the pass over the partials.
int plan_pass(const MrShape& sh, int src_dt, int acc_dt, const void* src, const void* dst, bool allow_split, MrPlan* pl) {
    const int es = tiled_dtype_size(src_dt), ds = tiled_dtype_size(acc_dt);
    int V = 16 / es;
    if (V > 8) V = 8;
    const int vb = V * es < 16 ? V * es : 16;
    pl->V = V;
    pl->vec = sh.sst[0] == 1 && ((uintptr_t)src) % (uintptr_t)vb == 0;
    for (int d = 1; d < 4; ++d) if ((sh.sst[d] * es) % vb) pl->vec = false;
    const int64_t nvec0 = cld(sh.size[0], (int64_t)V);
    int64_t srcn = 1, nred = 1, nkept = 1;            // products over dimensions 1..3 by role
    for (int d = 0; d < 4; ++d) srcn *= sh.size[d];
    for (int d = 1; d < 4; ++d) (sh.red(d) ? nred : nkept) *= sh.size[d];
    // Dimensions 1..3 are unpacked with 32-bit divisions in the kernels.  Dimension 0 is walked in 64 bits; what
    // limits it is the number of vectors (below 2^32 where it is reduced, checked below) or of workgroups.
    for (int d = 1; d < 4; ++d) if (sh.size[d] > 0x7fffffffLL) return MI_E_GRID;
    if (nvec0 >= (1ll << 32)) return MI_E_GRID;
    pl->nt = stream_hint(srcn * es);
    pl->UNR = knob_unroll();
    pl->vecd = false;
    if (sh.run()) {
        const int64_t nq = nvec0 * nred, nk = nkept;
        if (nq >= (1ll << 32) || nk > 0x7fffffffLL) return MI_E_GRID;
        // lanes per output: at least four vectors each, more when there are too few outputs to
        // fill the chip otherwise
        int lanes = 1;
        while (lanes < 256 && (int64_t)lanes * 8 <= nq) lanes <<= 1;
        while (lanes < 256 && lanes < nq && nk * lanes < (int64_t)256 * 1024) lanes <<= 1;
        pl->LANES = lanes;
        pl->T = 256;
        pl->TX = pl->T; pl->TY = 1;
        int64_t P = 1;
        if (allow_split && lanes == 256) {
            P = cld(nq, (int64_t)lanes * knob_iters());
            const int64_t want = nk >= knob_blocks() ? 1 : knob_blocks() / (nk ? nk : 1);
            if (P > want) P = want;
            if (P < 1) P = 1;
        }
        pl->chunk = cld(cld(nq, P), (int64_t)lanes) * lanes;
        P = pl->chunk ? cld(nq, pl->chunk) : 1;
        if (P < 1) P = 1;
        pl->P = P; pl->nbx = 1; pl->nk = nk; pl->blocks = cld(nk, (int64_t)(pl->T / lanes)) * P;
    } else {
        const int64_t nq = nred, nk = sh.size[0] * nkept;
        if (nq >= (1ll << 32) || nkept > 0x7fffffffLL) return MI_E_GRID;
        // Lanes along dimension 0: as wide as the extent allows, narrowed (down to knob_min_tx) while
        // that leaves the chip short of workgroups and the reduced range can use the freed rows.
        int tx = nvec0 >= 256 ? 256 : pow2ceil(nvec0);
        while (tx > knob_min_tx() && cld(nvec0, (int64_t)tx) * nkept < 512 && (int64_t)(256 / tx) * 2 <= nq) tx >>= 1;
        pl->TX = tx;
        int ty = 256 / pl->TX;
        while (ty > 1 && ty > nq) ty >>= 1;
        pl->TY = ty;
        pl->T = pl->TX * pl->TY;
        pl->nbx = cld(nvec0, (int64_t)pl->TX);
        if (pl->nbx < 1) pl->nbx = 1;
        const int64_t b0 = pl->nbx * nkept;
        int64_t P = 1;
        if (allow_split) {
            P = cld(nq, (int64_t)pl->TY * knob_iters());
            const int64_t want = b0 >= knob_column_blocks() ? 1 : knob_column_blocks() / (b0 ? b0 : 1);
            if (P > want) P = want;
            if (P < 1) P = 1;
        }
        pl->chunk = cld(cld(nq, P), (int64_t)pl->TY) * pl->TY;
        P = pl->chunk ? cld(nq, pl->chunk) : 1;
        if (P < 1) P = 1;
        pl->P = P; pl->nk = nk; pl->blocks = b0 * P; pl->LANES = 1;
        const int dvb = V * ds < 16 ? V * ds : 16;
        pl->vecd = sh.dstr[0] == 1 && ((uintptr_t)dst) % (uintptr_t)dvb == 0;
        for (int d = 1; d < 4; ++d) if (!sh.red(d) && (sh.dstr[d] * ds) % dvb) pl->vecd = false;
    }
    if (pl->blocks > 0x7fffffffLL) return MI_E_GRID;
    return MI_OK;
}

// Shape of a reduction after merging: extent-1 dimensions dropped, neighbours of one role that form a
// single run in src (and dest, for kept ones) fused, padded to four with kept extent-1 dimensions.
int canonical_shape(const mi_tile_array* dest, const mi_tile_array* src, MrShape* out) {
    int n = 0;
    bool red[4];
    out->rmask = 0;
    for (int d = 0; d < 4; ++d) {
        const int64_t s = size_of(src, d), ds = size_of(dest, d);
        if (ds != s && ds != 1) return MI_E_SHAPE;
        if (s == 1) continue;
        const bool r = ds == 1;
        const int64_t st = stride_of(src, d), dt = r ? 0 : stride_of(dest, d);
        // (a fused dimension other than 0 has to stay within 31 bits: the kernels unpack it with 32-bit divisions)
        if (n > 0 && red[n - 1] == r && st == out->sst[n - 1] * out->size[n - 1] && (r || dt == out->dstr[n - 1] * out->size[n - 1]) &&
            (n == 1 || out->size[n - 1] * s <= 0x7fffffffLL)) {
            out->size[n - 1] *= s;
            continue;
        }
        out->size[n] = s; out->sst[n] = st; out->dstr[n] = dt; red[n] = r;
        if (r) out->rmask |= 1 << n;
        ++n;
    }
    for (; n < 4; ++n) { out->size[n] = 1; out->sst[n] = n == 0 ? 1 : 0; out->dstr[n] = n == 0 ? 1 : 0; }
    return MI_OK;
}

std::string mr_source(const Expr& e, const int32_t* scal_dt, int src_dt, int acc_dt, int op, const MrShape& sh, const MrPlan& pl, bool out_ws) {
    std::string g;
    char buf[512];
    snprintf(buf, sizeof buf,
             "constexpr int SRC = %s, ACC = %s, V = %d, T = %d, TX = %d, TY = %d, RMASK = %d, LANES = %d;\n"
             "constexpr bool NT = %s, VEC = %s, VECD = %s, OUT_WS = %s;\n#define UNR %d\n",
             tag(src_dt), tag(acc_dt), pl.V, pl.T, pl.TX, pl.TY, sh.rmask, pl.LANES, pl.nt ? "true" : "false", pl.vec ? "true" : "false",
             pl.vecd ? "true" : "false", out_ws ? "true" : "false", pl.UNR);
    g += buf;
    snprintf(buf, sizeof buf, "typedef %s SST;\ntypedef %s DST;\ntypedef car<ACC> AC;\n", storage(src_dt), storage(acc_dt));
    g += buf;
    g += "struct Args { const void* src; void* dst; long long size[4]; long long sst[4]; long long dstr[4]; long long P; long long nbx; long long nk; long long chunk; "
         "double sf[8]; long long si[8]; };\n";
    int32_t leaf_dt[1] = {src_dt};
    g += "__device__ __forceinline__ AC mapf(" + eval_params(e, leaf_dt, scal_dt) + ") {\n" + emit_body(e);
    snprintf(buf, sizeof buf, "    return cvt<ACC>(t%d);\n}\n", e.root);
    g += buf;
    snprintf(buf, sizeof buf, "__device__ __forceinline__ AC redop(AC a, AC b) { return %s<ACC>(a, b); }\n__device__ __forceinline__ AC neutral() { return %s; }\n",
             op_fn(op), neutral_text(op, acc_dt));
    g += buf;
    std::string call = "#define MAPF(x) mapf(x";
    for (int i = 0; i < e.scalars_used; ++i) { snprintf(buf, sizeof buf, ", s%d", i); call += buf; }
    g += call + ")\n";
    std::string sc = scalar_decls(e, scal_dt);
    for (char& c : sc) if (c == '\n') c = ' ';
    g += "#define SCALARS " + sc + "\n";
    g += sh.run() ? kRunKernel : kColumnKernel;
    return g;
}

int run_pass(const Expr& e, const char* text, const int32_t* scal_dt, const ScalarArgs& sa, int src_dt, int acc_dt, int op, const MrShape& sh,
             const MrPlan& pl, const void* src, void* dst, bool out_ws, hipStream_t stream) {
    char kb[256];
    snprintf(kb, sizeof kb, "|%d,%d,%d|%d,%d,%d,%d,%d,%d,%d|%d,%d,%d,%d|", src_dt, acc_dt, op, pl.V, pl.T, pl.TX, pl.TY, sh.rmask, pl.LANES, pl.UNR,
             pl.nt ? 1 : 0, pl.vec ? 1 : 0, pl.vecd ? 1 : 0, out_ws ? 1 : 0);
    std::string key = "mr|";
    key += text;
    key += kb;
    for (int i = 0; i < e.scalars_used; ++i) { snprintf(kb, sizeof kb, "%d,", scal_dt[i]); key += kb; }
    hipFunction_t fn = nullptr;
    MI_CHECK(kernel_for(key, "tiled_mr", [&]() { return mr_source(e, scal_dt, src_dt, acc_dt, op, sh, pl, out_ws); }, &fn));
    MrArgs a;
    memset(&a, 0, sizeof a);
    a.src = src;
    a.dst = dst;
    for (int d = 0; d < 4; ++d) { a.size[d] = sh.size[d]; a.sst[d] = sh.sst[d]; a.dstr[d] = sh.dstr[d]; }
    a.P = pl.P;
    a.nbx = pl.nbx;
    a.nk = pl.nk;
    a.chunk = pl.chunk;
    memcpy(a.sf, sa.sf, sizeof a.sf);
    memcpy(a.si, sa.si, sizeof a.si);
    return launch(fn, pl.blocks, pl.T, &a, sizeof a, stream);
}

int mapreduce_impl(const mi_tile_array* dest, const mi_tile_array* src, const char* f_text, const mi_tile_scalar* scalars, int ns, int op,
                   void* workspace, int64_t workspace_bytes, int64_t* need_only, hipStream_t stream) {
    MI_CHECK(check_tiled(dest));
    MI_CHECK(check_tiled(src));
    if (op < MI_OP_ADD || op > MI_OP_OR) return MI_E_ARG;
    if ((op == MI_OP_AND || op == MI_OP_OR) && dt_is_float(dest->dtype)) return MI_E_DTYPE;
    MrShape sh;
    MI_CHECK(canonical_shape(dest, src, &sh));
    int64_t dn = 1;
    for (int d = 0; d < dest->ndim; ++d) dn *= dest->sizes[d];
    if (dn == 0) { if (need_only) *need_only = 0; return MI_OK; }
    MrPlan p1;
    MI_CHECK(plan_pass(sh, src->dtype, dest->dtype, src->ptr, dest->ptr, true, &p1));
    const int cdt = carrier_dtype(dest->dtype);
    const int64_t need = p1.P > 1 ? p1.P * p1.nk * (int64_t)tiled_dtype_size(cdt) : 0;
    if (need_only) { *need_only = need; return MI_OK; }

    int32_t scal_dt[kMaxScalars] = {0};
    ScalarArgs sa;
    MI_CHECK(pack_scalars(scalars, ns, scal_dt, &sa));
    Expr e;
    MI_CHECK(parse_expr(f_text ? f_text : "a0", e));
    if (e.leaves_used > 1) return MI_E_ARG;
    e.leaves_used = 1;
    int32_t leaf_dt[1] = {src->dtype};
    MI_CHECK(infer_types(e, leaf_dt, 1, scal_dt, ns));

    char buf[96];
    if (p1.P == 1) {
        snprintf(buf, sizeof buf, "tiled_mr_%s_l%d_ty%d", sh.run() ? "run" : "column", p1.LANES, p1.TY);
        set_variant_text(buf);
        return run_pass(e, f_text ? f_text : "a0", scal_dt, sa, src->dtype, dest->dtype, op, sh, p1, src->ptr, dest->ptr, false, stream);
    }
    if (!workspace || workspace_bytes < need) return MI_E_ARG;
    if (((uintptr_t)workspace) % 16) return MI_E_ALIGN;
    MI_CHECK(run_pass(e, f_text ? f_text : "a0", scal_dt, sa, src->dtype, dest->dtype, op, sh, p1, src->ptr, workspace, true, stream));
    // Second pass: the P partials of every output, identity map.  The partials form a dense array
    // whose kept dimensions keep their place; P takes the place of dimension 0 (run shape: partials
    // of one output are adjacent) or of the first reduced dimension (column shape: P planes of nk).
    MrShape s2;
    int slot = 0;
    if (!sh.run()) { slot = 1; while (slot < 4 && !sh.red(slot)) ++slot; }
    s2.rmask = 1 << slot;
    int64_t st = sh.run() ? p1.P : 1;
    for (int d = 0; d < 4; ++d) {
        if (d == slot) { s2.size[d] = p1.P; s2.sst[d] = sh.run() ? 1 : p1.nk; s2.dstr[d] = 0; continue; }
        if (sh.red(d)) { s2.size[d] = 1; s2.sst[d] = 0; s2.dstr[d] = 0; continue; }
        s2.size[d] = sh.size[d]; s2.sst[d] = st; s2.dstr[d] = sh.dstr[d];
        st *= sh.size[d];
    }
    MrPlan p2;
    MI_CHECK(plan_pass(s2, cdt, dest->dtype, workspace, dest->ptr, false, &p2));
    Expr id;
    MI_CHECK(parse_expr("a0", id));
    int32_t l2[1] = {cdt};
    MI_CHECK(infer_types(id, l2, 1, scal_dt, 0));
    snprintf(buf, sizeof buf, "tiled_mr_%s_l%d_ty%d_split%lld", sh.run() ? "run" : "column", p1.LANES, p1.TY, (long long)p1.P);
    set_variant_text(buf);
    ScalarArgs none;
    memset(&none, 0, sizeof none);
    return run_pass(id, "a0", scal_dt, none, cdt, dest->dtype, op, s2, p2, workspace, dest->ptr, false, stream);
}

}  // namespace

extern "C" {

int mi_tiled_broadcast(const mi_tile_array* dest, const char* expr, const mi_tile_array* const* leaves, int n_leaves,
                       const mi_tile_scalar* scalars, int n_scalars, void* stream) {
    return broadcast_impl(dest, expr, leaves, n_leaves, scalars, n_scalars, (hipStream_t)stream);
}

int mi_tiled_broadcast_eltype(const char* expr, const int32_t* leaf_dtypes, int n_leaves, const int32_t* scalar_dtypes, int n_scalars,
                              int32_t* out_dtype) {
    if (!out_dtype) return MI_E_NULL;
    if (n_leaves < 0 || n_leaves > kMaxLeaves || n_scalars < 0 || n_scalars > kMaxScalars) return MI_E_UNSUPPORTED;
    if ((n_leaves && !leaf_dtypes) || (n_scalars && !scalar_dtypes)) return MI_E_NULL;
    Expr e;
    MI_CHECK(parse_expr(expr, e));
    MI_CHECK(infer_types(e, leaf_dtypes, n_leaves, scalar_dtypes, n_scalars));
    *out_dtype = e.nodes[e.root].dtype;
    return MI_OK;
}

int mi_tiled_mapreduce(const mi_tile_array* dest, const mi_tile_array* src, const char* f_expr, const mi_tile_scalar* scalars, int n_scalars,
                       int op, void* workspace, int64_t workspace_bytes, void* stream) {
    return mapreduce_impl(dest, src, f_expr, scalars, n_scalars, op, workspace, workspace_bytes, nullptr, (hipStream_t)stream);
}

int mi_tiled_mapreduce_workspace(const mi_tile_array* dest, const mi_tile_array* src, int op, int64_t* bytes) {
    if (!bytes) return MI_E_NULL;
    return mapreduce_impl(dest, src, nullptr, nullptr, 0, op, nullptr, 0, bytes, nullptr);
}

int mi_tiled_mapreduce_eltype(const char* f_expr, int32_t src_dtype, const int32_t* scalar_dtypes, int n_scalars, int op, int widen,
                              int32_t* out_dtype) {
    if (!out_dtype) return MI_E_NULL;
    if (n_scalars < 0 || n_scalars > kMaxScalars) return MI_E_UNSUPPORTED;
    if (op < MI_OP_ADD || op > MI_OP_OR) return MI_E_ARG;
    Expr e;
    MI_CHECK(parse_expr(f_expr ? f_expr : "a0", e));
    if (e.leaves_used > 1) return MI_E_ARG;
    MI_CHECK(infer_types(e, &src_dtype, 1, scalar_dtypes, n_scalars));
    int t = e.nodes[e.root].dtype;
    // promote_op(op, T, T): + on Bool counts; add_sum / mul_prod also widen Int32 (Base reduce.jl).
    if (op == MI_OP_ADD && t == MI_BOOL) t = MI_I64;
    if (widen && (op == MI_OP_ADD || op == MI_OP_MUL) && (t == MI_I32 || t == MI_BOOL)) t = MI_I64;
    if ((op == MI_OP_AND || op == MI_OP_OR) && dt_is_float(t)) return MI_E_DTYPE;
    *out_dtype = t;
    return MI_OK;
}

int mi_tiled_set_dry_run(int on) {
    std::lock_guard<std::mutex> lock(g_mu);
    const int old = g_dry_run ? 1 : 0;
    if ((on != 0) != g_dry_run) { g_cache.clear(); g_by_key.clear(); }   // entries of a dry run hold no loaded function
    g_dry_run = on != 0;
    return old;
}

int mi_tiled_compile_count(void) {
    std::lock_guard<std::mutex> lock(g_mu);
    return g_compiles;
}

}  // extern "C"
