// Expression trees of the host-level Tiled broadcast / mapreduce entry points: the text form a
// caller hands over, Julia's element-type rules for every node, and the device source of one
// fused evaluation function.  Host-only code.
//
// The reference walks a Base.Broadcast.Broadcasted tree inside its kernel (src/broadcast.jl:101-113,
// `_eval_bc`): array leaves are loaded as tiles, numbers pass through, every inner node applies its
// function element-wise.  Here the tree crosses the C ABI as text in prefix form,
//     expr  := name '(' expr { ',' expr } ')'  |  'a' index  |  's' index
// where a<i> is the i-th array leaf, s<i> the i-th scalar, and `name` one of the functions of the
// table below (Julia's `+` is `add`, `.^` is `pow`, `Float32(x)` is `f32`, ...).  Only names from
// the table are accepted, so the text can never inject source.
#pragma once
#include <stdint.h>
#include <string.h>
#include <string>
#include <vector>
#include "../../include/mi355tile.h"

namespace mi {
namespace tiled {

constexpr int kMaxLeaves = 8;
constexpr int kMaxScalars = 8;
constexpr int kMaxNodes = 128;

enum Kind { kLeaf = 0, kScalar = 1, kCall = 2 };

// How a function's result type follows from its arguments (Julia semantics).
enum Rule {
    R_ARITH,     // promote_type; Bool op Bool widens to Int64 (true + true == 2)
    R_MUL,       // promote_type (Bool * Bool stays Bool)
    R_SAME,      // type of the (promoted) arguments
    R_NEG,       // like R_SAME, Bool -> Int64
    R_DIV,       // `/`: integers give Float64, floats promote
    R_POW,       // `^`: the base keeps its type for integer / Bool exponents (Julia's ^(x::T, p::Integer)), otherwise promote
    R_FLOAT,     // math functions: integers are converted with float() (Float64), floats keep their type
    R_BOOL,      // predicates and comparisons
    R_LOGIC,     // & | xor !: Bool or integers (bitwise), promote
    R_IFELSE,    // ifelse(cond::Bool, a, b): promote_type(a, b)
    R_FIRST,     // type of the first argument (copysign)
    R_CONVERT,   // constructors: fixed result type
    R_INTDIV,    // div / rem / mod / fld / cld: promote (integers stay integers)
    R_SHIFT      // << >> >>>: type of the shifted integer (Bool widens to Int64), any integer count
};

struct FnInfo {
    const char* name;   // name in the text form
    int arity;
    Rule rule;
    int fixed;          // R_CONVERT: result dtype
    const char* dev;    // device function (template on the result dtype tag)
};

// name, arity, rule, fixed dtype, device function
static const FnInfo kFns[] = {
    {"identity", 1, R_SAME, 0, "f_identity"},
    {"add", 2, R_ARITH, 0, "f_add"},
    {"sub", 2, R_ARITH, 0, "f_sub"},
    {"mul", 2, R_MUL, 0, "f_mul"},
    {"div", 2, R_DIV, 0, "f_div"},
    {"pow", 2, R_POW, 0, "f_pow"},
    {"neg", 1, R_NEG, 0, "f_neg"},
    {"abs", 1, R_SAME, 0, "f_abs"},
    {"abs2", 1, R_SAME, 0, "f_abs2"},
    {"sign", 1, R_SAME, 0, "f_sign"},
    {"max", 2, R_SAME, 0, "f_max"},
    {"min", 2, R_SAME, 0, "f_min"},
    {"fma", 3, R_SAME, 0, "f_fma"},
    {"muladd", 3, R_SAME, 0, "f_fma"},
    {"clamp", 3, R_SAME, 0, "f_clamp"},
    {"copysign", 2, R_FIRST, 0, "f_copysign"},
    {"floor", 1, R_SAME, 0, "f_floor"},
    {"ceil", 1, R_SAME, 0, "f_ceil"},
    {"round", 1, R_SAME, 0, "f_round"},
    {"trunc", 1, R_SAME, 0, "f_trunc"},
    {"sqrt", 1, R_FLOAT, 0, "f_sqrt"},
    {"cbrt", 1, R_FLOAT, 0, "f_cbrt"},
    {"inv", 1, R_FLOAT, 0, "f_inv"},
    {"exp", 1, R_FLOAT, 0, "f_exp"},
    {"exp2", 1, R_FLOAT, 0, "f_exp2"},
    {"exp10", 1, R_FLOAT, 0, "f_exp10"},
    {"expm1", 1, R_FLOAT, 0, "f_expm1"},
    {"log", 1, R_FLOAT, 0, "f_log"},
    {"log2", 1, R_FLOAT, 0, "f_log2"},
    {"log10", 1, R_FLOAT, 0, "f_log10"},
    {"log1p", 1, R_FLOAT, 0, "f_log1p"},
    {"sin", 1, R_FLOAT, 0, "f_sin"},
    {"cos", 1, R_FLOAT, 0, "f_cos"},
    {"tan", 1, R_FLOAT, 0, "f_tan"},
    {"asin", 1, R_FLOAT, 0, "f_asin"},
    {"acos", 1, R_FLOAT, 0, "f_acos"},
    {"atan", 1, R_FLOAT, 0, "f_atan"},
    {"sinh", 1, R_FLOAT, 0, "f_sinh"},
    {"cosh", 1, R_FLOAT, 0, "f_cosh"},
    {"tanh", 1, R_FLOAT, 0, "f_tanh"},
    {"atan2", 2, R_FLOAT, 0, "f_atan2"},
    {"hypot", 2, R_FLOAT, 0, "f_hypot"},
    {"lt", 2, R_BOOL, 0, "f_lt"},
    {"le", 2, R_BOOL, 0, "f_le"},
    {"gt", 2, R_BOOL, 0, "f_gt"},
    {"ge", 2, R_BOOL, 0, "f_ge"},
    {"eq", 2, R_BOOL, 0, "f_eq"},
    {"ne", 2, R_BOOL, 0, "f_ne"},
    {"isnan", 1, R_BOOL, 0, "f_isnan"},
    {"isinf", 1, R_BOOL, 0, "f_isinf"},
    {"isfinite", 1, R_BOOL, 0, "f_isfinite"},
    {"signbit", 1, R_BOOL, 0, "f_signbit"},
    {"iszero", 1, R_BOOL, 0, "f_iszero"},
    {"not", 1, R_LOGIC, 0, "f_not"},
    {"and", 2, R_LOGIC, 0, "f_and"},
    {"or", 2, R_LOGIC, 0, "f_or"},
    {"xor", 2, R_LOGIC, 0, "f_xor"},
    {"ifelse", 3, R_IFELSE, 0, "f_ifelse"},
    {"div_int", 2, R_INTDIV, 0, "f_divi"},
    {"rem", 2, R_INTDIV, 0, "f_rem"},
    {"mod", 2, R_INTDIV, 0, "f_mod"},
    {"fld", 2, R_INTDIV, 0, "f_fld"},
    {"cld", 2, R_INTDIV, 0, "f_cld"},
    {"rsqrt", 1, R_FLOAT, 0, "f_rsqrt"},
    {"shl", 2, R_SHIFT, 0, "f_shl"},
    {"shr", 2, R_SHIFT, 0, "f_shr"},
    {"lshr", 2, R_SHIFT, 0, "f_lshr"},
    {"mul_hi", 2, R_LOGIC, 0, "f_mul_hi"},
    {"f16", 1, R_CONVERT, MI_F16, "f_convert"},
    {"bf16", 1, R_CONVERT, MI_BF16, "f_convert"},
    {"f32", 1, R_CONVERT, MI_F32, "f_convert"},
    {"f64", 1, R_CONVERT, MI_F64, "f_convert"},
    {"i32", 1, R_CONVERT, MI_I32, "f_convert"},
    {"i64", 1, R_CONVERT, MI_I64, "f_convert"},
    {"bool", 1, R_CONVERT, MI_BOOL, "f_convert"},
};
constexpr int kNumFns = (int)(sizeof(kFns) / sizeof(kFns[0]));

struct Node {
    int kind = kLeaf;
    int index = 0;      // leaf / scalar number, or function number
    int nargs = 0;
    int args[3] = {0, 0, 0};
    int dtype = -1;
};

struct Expr {
    std::vector<Node> nodes;   // children precede parents
    int root = -1;
    int leaves_used = 0;       // 1 + highest leaf index
    int scalars_used = 0;
};

static inline bool dt_is_float(int dt) { return dt == MI_F32 || dt == MI_F64 || dt == MI_F16 || dt == MI_BF16; }
static inline bool dt_is_int(int dt) { return dt == MI_I32 || dt == MI_I64; }
static inline bool dt_ok(int dt) { return dt_is_float(dt) || dt_is_int(dt) || dt == MI_BOOL; }

// Julia's promote_type restricted to the element types of this library.
static inline int promote(int a, int b) {
    if (a == b) return a;
    if (a == MI_BOOL) return b;
    if (b == MI_BOOL) return a;
    if (dt_is_int(a) && dt_is_int(b)) return MI_I64;
    if (dt_is_int(a)) return b;          // Int + AbstractFloat -> the float type
    if (dt_is_int(b)) return a;
    if (a == MI_F64 || b == MI_F64) return MI_F64;
    if (a == MI_F32 || b == MI_F32) return MI_F32;
    return MI_F32;                        // Float16 with BFloat16
}

// ---- parser ------------------------------------------------------------------------------------
struct Parser {
    const char* s;
    Expr* e;
    int err = MI_OK;
    void skip() { while (*s == ' ' || *s == '\t' || *s == '\n') ++s; }
    int number() {
        if (*s < '0' || *s > '9') { err = MI_E_ARG; return 0; }
        int v = 0;
        while (*s >= '0' && *s <= '9') { v = v * 10 + (*s - '0'); if (v > 1000) { err = MI_E_ARG; return 0; } ++s; }
        return v;
    }
    int parse() {
        skip();
        if (err) return -1;
        if ((int)e->nodes.size() >= kMaxNodes) { err = MI_E_UNSUPPORTED; return -1; }
        const char* b = s;
        while ((*s >= 'a' && *s <= 'z') || (*s >= '0' && *s <= '9') || *s == '_') ++s;
        const size_t len = (size_t)(s - b);
        if (len == 0) { err = MI_E_ARG; return -1; }
        skip();
        if (*s != '(') {   // leaf or scalar: one letter then digits
            if ((b[0] != 'a' && b[0] != 's') || len < 2) { err = MI_E_ARG; return -1; }
            const char* save = s;
            s = b + 1;
            const int idx = number();
            if (err || s != b + len) { err = MI_E_ARG; return -1; }
            s = save;
            Node n;
            n.kind = b[0] == 'a' ? kLeaf : kScalar;
            n.index = idx;
            if (n.kind == kLeaf) { if (idx >= kMaxLeaves) { err = MI_E_UNSUPPORTED; return -1; } if (idx + 1 > e->leaves_used) e->leaves_used = idx + 1; }
            else { if (idx >= kMaxScalars) { err = MI_E_UNSUPPORTED; return -1; } if (idx + 1 > e->scalars_used) e->scalars_used = idx + 1; }
            e->nodes.push_back(n);
            return (int)e->nodes.size() - 1;
        }
        int fn = -1;
        for (int i = 0; i < kNumFns; ++i)
            if (strlen(kFns[i].name) == len && memcmp(kFns[i].name, b, len) == 0) { fn = i; break; }
        if (fn < 0) { err = MI_E_UNSUPPORTED; return -1; }
        ++s;  // '('
        Node n;
        n.kind = kCall;
        n.index = fn;
        for (;;) {
            if (n.nargs >= 3) { err = MI_E_ARG; return -1; }
            const int c = parse();
            if (err) return -1;
            n.args[n.nargs++] = c;
            skip();
            if (*s == ',') { ++s; continue; }
            if (*s == ')') { ++s; break; }
            err = MI_E_ARG;
            return -1;
        }
        if (n.nargs != kFns[fn].arity) { err = MI_E_ARG; return -1; }
        e->nodes.push_back(n);
        return (int)e->nodes.size() - 1;
    }
};

static inline int parse_expr(const char* text, Expr& e) {
    if (!text) return MI_E_NULL;
    if (strlen(text) > 4096) return MI_E_UNSUPPORTED;
    Parser p{text, &e};
    e.root = p.parse();
    if (p.err) return p.err;
    p.skip();
    if (*p.s != '\0') return MI_E_ARG;
    return MI_OK;
}

// ---- element types -----------------------------------------------------------------------------
static inline int infer_types(Expr& e, const int32_t* leaf_dt, int nl, const int32_t* scal_dt, int ns) {
    if (e.leaves_used > nl || e.scalars_used > ns) return MI_E_ARG;
    for (Node& n : e.nodes) {
        if (n.kind == kLeaf) { n.dtype = leaf_dt[n.index]; if (!dt_ok(n.dtype)) return MI_E_DTYPE; continue; }
        if (n.kind == kScalar) { n.dtype = scal_dt[n.index]; if (!dt_ok(n.dtype)) return MI_E_DTYPE; continue; }
        const FnInfo& f = kFns[n.index];
        int t = e.nodes[n.args[0]].dtype;
        for (int i = 1; i < n.nargs; ++i) t = promote(t, e.nodes[n.args[i]].dtype);
        switch (f.rule) {
            case R_ARITH: n.dtype = t == MI_BOOL ? MI_I64 : t; break;
            case R_MUL: case R_SAME: n.dtype = t; break;
            case R_NEG: n.dtype = t == MI_BOOL ? MI_I64 : t; break;
            case R_DIV: n.dtype = dt_is_float(t) ? t : MI_F64; break;
            case R_POW: {
                const int b = e.nodes[n.args[0]].dtype, x = e.nodes[n.args[1]].dtype;
                n.dtype = !dt_is_float(x) ? b : t;   // Int32 ^ Int64 is Int32, Bool ^ Int is Bool, Float32 ^ Int is Float32
                break;
            }
            case R_FLOAT: n.dtype = dt_is_float(t) ? t : MI_F64; break;
            case R_BOOL: n.dtype = MI_BOOL; break;
            case R_LOGIC: if (dt_is_float(t)) return MI_E_DTYPE; n.dtype = t; break;
            case R_IFELSE:
                if (e.nodes[n.args[0]].dtype != MI_BOOL) return MI_E_DTYPE;
                n.dtype = promote(e.nodes[n.args[1]].dtype, e.nodes[n.args[2]].dtype);
                break;
            case R_FIRST: n.dtype = e.nodes[n.args[0]].dtype; break;
            case R_CONVERT: n.dtype = f.fixed; break;
            case R_INTDIV: n.dtype = t == MI_BOOL ? MI_I64 : t; break;
            case R_SHIFT: {
                const int x = e.nodes[n.args[0]].dtype, c = e.nodes[n.args[1]].dtype;
                if (dt_is_float(x) || dt_is_float(c)) return MI_E_DTYPE;
                n.dtype = x == MI_BOOL ? MI_I64 : x;
                break;
            }
        }
    }
    return MI_OK;
}

// ---- device source -----------------------------------------------------------------------------
// A value of element type T travels in registers as its carrier: float for Float16 / BFloat16 /
// Float32 (re-rounded to T after every operation, which is how Julia defines Float16 arithmetic),
// double, int, long long, bool.
static inline const char* carrier(int dt) {
    switch (dt) {
        case MI_F64: return "double";
        case MI_I32: return "int";
        case MI_I64: return "long long";
        case MI_BOOL: return "bool";
        default: return "float";
    }
}
static inline const char* tag(int dt) {
    switch (dt) {
        case MI_F32: return "DT_F32";
        case MI_F64: return "DT_F64";
        case MI_F16: return "DT_F16";
        case MI_BF16: return "DT_BF16";
        case MI_I32: return "DT_I32";
        case MI_I64: return "DT_I64";
        default: return "DT_BOOL";
    }
}
static inline const char* storage(int dt) {
    switch (dt) {
        case MI_F32: return "float";
        case MI_F64: return "double";
        case MI_F16: return "_Float16";
        case MI_BF16: return "bf16_t";
        case MI_I32: return "int";
        case MI_I64: return "long long";
        default: return "unsigned char";
    }
}

// Body of `eval`: one statement per node, the value of node i in t<i>.  Leaves read the
// parameters a<i> (already carriers), scalars the parameters s<i>.
static inline std::string emit_body(const Expr& e) {
    std::string o;
    char buf[64];
    for (size_t i = 0; i < e.nodes.size(); ++i) {
        const Node& n = e.nodes[i];
        snprintf(buf, sizeof buf, "    const %s t%zu = ", carrier(n.dtype), i);
        o += buf;
        if (n.kind == kLeaf) { snprintf(buf, sizeof buf, "a%d;\n", n.index); o += buf; continue; }
        if (n.kind == kScalar) { snprintf(buf, sizeof buf, "s%d;\n", n.index); o += buf; continue; }
        const FnInfo& f = kFns[n.index];
        // Arguments are first converted to the type the operation works in.
        int work = n.dtype;
        if (f.rule == R_BOOL || f.rule == R_CONVERT) {
            work = e.nodes[n.args[0]].dtype;
            for (int k = 1; k < n.nargs; ++k) work = promote(work, e.nodes[n.args[k]].dtype);
        }
        o += f.dev;
        o += "<";
        o += tag(f.rule == R_CONVERT ? n.dtype : work);
        o += ">(";
        for (int k = 0; k < n.nargs; ++k) {
            const Node& a = e.nodes[n.args[k]];
            int want = work;
            if (f.rule == R_IFELSE && k == 0) want = MI_BOOL;
            if (f.rule == R_POW && k == 1 && !dt_is_float(a.dtype)) want = MI_I64;
            if (f.rule == R_CONVERT) want = a.dtype;
            if (f.rule == R_SHIFT && k == 1) want = MI_I64;
            if (k) o += ", ";
            if (want == a.dtype) snprintf(buf, sizeof buf, "t%d", n.args[k]);
            else snprintf(buf, sizeof buf, "cvt<%s>(t%d)", tag(want), n.args[k]);
            o += buf;
        }
        o += ");\n";
    }
    return o;
}

}  // namespace tiled
}  // namespace mi
