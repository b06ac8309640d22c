// StableHLO text -> Function.  Statement-oriented: one op is the text up to the
// first newline at bracket depth zero; operands, attributes and the type
// signature are then picked out of that text.
#include <ctype.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "hlo.h"

namespace mhlo {

// ---------------------------------------------------------------- small helpers
uint16_t f32_to_bf16_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    if (f != f) return 0x7FC0;
    return (uint16_t)((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}

uint16_t f32_to_f16_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    int32_t exp = (int32_t)((x >> 23) & 0xFF) - 127 + 15;
    uint32_t man = x & 0x7FFFFFu;
    if (((x >> 23) & 0xFF) == 0xFF) return (uint16_t)(sign | 0x7C00u | (man ? 0x200u : 0));
    if (exp >= 31) return (uint16_t)(sign | 0x7C00u);
    if (exp <= 0) {
        if (exp < -10) return (uint16_t)sign;
        man |= 0x800000u;
        const int shift = 14 - exp;
        uint32_t half = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1), mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) half++;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)exp << 10) | (man >> 13);
    const uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++;
    return (uint16_t)(sign | half);
}

static std::string trim(const std::string& s) {
    size_t a = 0, b = s.size();
    while (a < b && isspace((unsigned char)s[a])) a++;
    while (b > a && isspace((unsigned char)s[b - 1])) b--;
    return s.substr(a, b - a);
}

static bool starts_with(const std::string& s, const char* p) { return s.compare(0, strlen(p), p) == 0; }

static int parse_dtype(const std::string& t, int line) {
    static const std::pair<const char*, int> tab[] = {
        {"f16", F16}, {"f32", F32}, {"f64", F64}, {"bf16", BF16}, {"i1", I1}, {"i8", I8},
        {"i16", I16}, {"i32", I32}, {"i64", I64}, {"ui8", UI8}, {"ui16", UI16}, {"ui32", UI32},
        {"ui64", UI64}, {"si8", I8}, {"si16", I16}, {"si32", I32}, {"si64", I64}};
    for (auto& e : tab)
        if (t == e.first) return e.second;
    throw UnsupportedOp("line " + std::to_string(line) + ": element type '" + t + "' is not supported");
}

// "tensor<2x3xf32>" starting at s[p]; advances p past '>'.
static TensorType parse_type(const std::string& s, size_t& p, int line) {
    while (p < s.size() && isspace((unsigned char)s[p])) p++;
    if (s.compare(p, 7, "tensor<") != 0)
        throw ParseError("line " + std::to_string(line) + ": expected tensor<...> near '" + s.substr(p, 24) + "'");
    p += 7;
    const size_t e = s.find('>', p);
    if (e == std::string::npos) throw ParseError("line " + std::to_string(line) + ": unterminated tensor type");
    const std::string body = s.substr(p, e - p);
    p = e + 1;
    TensorType t;
    size_t i = 0;
    while (i < body.size()) {
        size_t j = i;
        while (j < body.size() && isdigit((unsigned char)body[j])) j++;
        if (j > i && j < body.size() && body[j] == 'x') {
            t.shape.push_back(strtoll(body.substr(i, j - i).c_str(), nullptr, 10));
            i = j + 1;
        } else {
            break;
        }
    }
    const std::string et = trim(body.substr(i));
    if (!et.empty() && et[0] == '?') throw UnsupportedOp("line " + std::to_string(line) + ": dynamic shapes are not supported");
    t.dtype = parse_dtype(et, line);
    return t;
}

// Index of the first ':' at bracket depth 0 outside strings, or npos.
static size_t top_level_colon(const std::string& s) {
    int depth = 0;
    bool in_str = false;
    for (size_t i = 0; i < s.size(); i++) {
        const char c = s[i];
        if (in_str) {
            if (c == '\\') i++;
            else if (c == '"') in_str = false;
            continue;
        }
        if (c == '"') in_str = true;
        else if (c == '-' && i + 1 < s.size() && s[i + 1] == '>') i++;
        else if (c == '(' || c == '[' || c == '{' || c == '<') depth++;
        else if (c == ')' || c == ']' || c == '}' || c == '>') depth--;
        else if (c == ':' && depth == 0) return i;
    }
    return std::string::npos;
}

// Integers of the first "[...]" or "array<i64: ...>" that follows `key` (whole word).
static bool ints_after_key(const std::string& s, const std::string& key, std::vector<int64_t>& out,
                           size_t from = 0, size_t* end = nullptr) {
    size_t k = from;
    for (;;) {
        k = s.find(key, k);
        if (k == std::string::npos) return false;
        const bool left_ok = k == 0 || !(isalnum((unsigned char)s[k - 1]) || s[k - 1] == '_');
        const size_t r = k + key.size();
        const bool right_ok = r >= s.size() || !(isalnum((unsigned char)s[r]) || s[r] == '_');
        if (left_ok && right_ok) break;
        k += key.size();
    }
    size_t i = k + key.size();
    while (i < s.size() && s[i] != '[' && s.compare(i, 6, "array<") != 0 && s[i] != ',' && s[i] != '}') i++;
    if (i >= s.size() || s[i] == ',' || s[i] == '}') return false;
    char close = ']';
    if (s[i] == '[') {
        i++;
    } else {
        close = '>';
        i = s.find(':', i);
        if (i == std::string::npos) return false;
        i++;
    }
    out.clear();
    while (i < s.size() && s[i] != close) {
        if (isdigit((unsigned char)s[i]) || s[i] == '-') {
            char* e;
            out.push_back(strtoll(s.c_str() + i, &e, 10));
            i = e - s.c_str();
        } else {
            i++;
        }
    }
    if (end) *end = i;
    return true;
}

static bool int_after_key(const std::string& s, const std::string& key, int64_t& out) {
    size_t k = s.find(key);
    while (k != std::string::npos) {
        const bool left_ok = k == 0 || !(isalnum((unsigned char)s[k - 1]) || s[k - 1] == '_');
        size_t i = k + key.size();
        while (i < s.size() && isspace((unsigned char)s[i])) i++;
        if (left_ok && i < s.size() && s[i] == '=') {
            i++;
            while (i < s.size() && isspace((unsigned char)s[i])) i++;
            if (i < s.size() && (isdigit((unsigned char)s[i]) || s[i] == '-')) {
                out = strtoll(s.c_str() + i, nullptr, 10);
                return true;
            }
        }
        k = s.find(key, k + 1);
    }
    return false;
}

// ---------------------------------------------------------------- constants
static void store_scalar(std::vector<uint8_t>& buf, size_t idx, int dtype, double fv, int64_t iv, bool is_int_lit,
                         uint64_t raw_bits, bool is_hex) {
    const int es = dtype_bytes(dtype);
    uint8_t* p = buf.data() + idx * es;
    if (dtype_is_float(dtype)) {
        if (is_hex) {            // hex literal = bit pattern of the element type
            memcpy(p, &raw_bits, es);
            return;
        }
        const double v = is_int_lit ? (double)iv : fv;
        if (dtype == F64) { memcpy(p, &v, 8); }
        else if (dtype == F32) { const float f = (float)v; memcpy(p, &f, 4); }
        else if (dtype == BF16) { const uint16_t h = f32_to_bf16_bits((float)v); memcpy(p, &h, 2); }
        else { const uint16_t h = f32_to_f16_bits((float)v); memcpy(p, &h, 2); }
    } else {
        // integer literals keep all 64 bits (no trip through double)
        const int64_t v = is_hex ? (int64_t)raw_bits : (is_int_lit ? iv : (int64_t)fv);
        if (dtype == I1) { p[0] = v != 0; return; }
        memcpy(p, &v, es);   // little endian truncation
    }
}

static void parse_dense(const std::string& body, Op& op) {
    const TensorType& t = op.out;
    const int es = dtype_bytes(t.dtype);
    const int64_t n = t.numel();
    std::string b = trim(body);
    if (!b.empty() && b[0] == '"') {   // dense<"0x...."> raw little-endian bytes
        std::string hex = b.substr(1, b.size() - 2);
        if (starts_with(hex, "0x") || starts_with(hex, "0X")) hex = hex.substr(2);
        std::vector<uint8_t> raw;
        for (size_t i = 0; i + 1 < hex.size(); i += 2) raw.push_back((uint8_t)strtoul(hex.substr(i, 2).c_str(), nullptr, 16));
        if ((int64_t)raw.size() == n * es) { op.constant = raw; return; }
        if ((int64_t)raw.size() == es) {
            op.splat = true; op.splat_bits = 0; memcpy(&op.splat_bits, raw.data(), es);
            return;
        }
        throw ParseError("line " + std::to_string(op.line) + ": dense hex string has the wrong length");
    }
    struct Lit { double f; int64_t i; bool is_int, is_hex; uint64_t bits; };
    std::vector<Lit> lits;
    size_t i = 0;
    while (i < b.size()) {
        const char c = b[i];
        if (c == '[' || c == ']' || c == ',' || isspace((unsigned char)c)) { i++; continue; }
        Lit l{0, 0, false, false, 0};
        if (b.compare(i, 4, "true") == 0) { l.i = 1; l.is_int = true; i += 4; }
        else if (b.compare(i, 5, "false") == 0) { l.i = 0; l.is_int = true; i += 5; }
        else if (b.compare(i, 2, "0x") == 0 || b.compare(i, 2, "0X") == 0) {
            char* e; l.bits = strtoull(b.c_str() + i, &e, 16); l.is_hex = true; i = e - b.c_str();
        } else {
            size_t j = i;
            bool is_int = true;
            while (j < b.size() && (isalnum((unsigned char)b[j]) || b[j] == '.' || b[j] == '-' || b[j] == '+')) {
                if (b[j] == '.' || b[j] == 'e' || b[j] == 'E' || b[j] == 'n' || b[j] == 'i') is_int = false;
                j++;
            }
            if (j == i) throw ParseError("line " + std::to_string(op.line) + ": bad dense literal near '" + b.substr(i, 16) + "'");
            const std::string tok = b.substr(i, j - i);
            l.is_int = is_int;
            if (is_int) l.i = tok[0] == '-' ? strtoll(tok.c_str(), nullptr, 10) : (int64_t)strtoull(tok.c_str(), nullptr, 10);   // ui64 keeps all 64 bits
            else l.f = strtod(tok.c_str(), nullptr);
            i = j;
        }
        lits.push_back(l);
    }
    if (lits.empty() && n == 0) return;
    if (lits.size() == 1) {
        std::vector<uint8_t> one(8, 0);
        one.resize(8);
        store_scalar(one, 0, t.dtype, lits[0].f, lits[0].i, lits[0].is_int, lits[0].bits, lits[0].is_hex);
        op.splat = true;
        op.splat_bits = 0;
        memcpy(&op.splat_bits, one.data(), es);
        return;
    }
    if ((int64_t)lits.size() != n)
        throw ParseError("line " + std::to_string(op.line) + ": dense literal has " + std::to_string(lits.size()) +
                         " elements, type wants " + std::to_string(n));
    op.constant.assign((size_t)n * es, 0);
    for (int64_t k = 0; k < n; k++)
        store_scalar(op.constant, k, t.dtype, lits[k].f, lits[k].i, lits[k].is_int, lits[k].bits, lits[k].is_hex);
}

// ---------------------------------------------------------------- module
namespace {

struct Parser {
    const std::string& s;
    size_t p = 0;
    int line = 1;
    Function fn;
    std::map<std::string, int> names;

    explicit Parser(const std::string& text) : s(text) {}

    [[noreturn]] void fail(const std::string& m) { throw ParseError("line " + std::to_string(line) + ": " + m); }

    void skip_ws() {
        for (;;) {
            while (p < s.size() && isspace((unsigned char)s[p])) { if (s[p] == '\n') line++; p++; }
            if (p + 1 < s.size() && s[p] == '/' && s[p + 1] == '/') { while (p < s.size() && s[p] != '\n') p++; continue; }
            break;
        }
    }

    int value_id(const std::string& name, bool define) {
        auto it = names.find(name);
        if (it != names.end()) {
            if (define) fail("value " + name + " defined twice");
            return it->second;
        }
        if (!define) fail("use of undefined value " + name);
        const int id = fn.num_values++;
        names[name] = id;
        return id;
    }

    // One statement: text up to a newline at depth 0 (strings and brackets respected).
    std::string read_statement() {
        std::string out;
        int depth = 0;
        bool in_str = false;
        while (p < s.size()) {
            const char c = s[p];
            if (in_str) {
                out += c;
                if (c == '\\' && p + 1 < s.size()) { out += s[p + 1]; p += 2; continue; }
                if (c == '"') in_str = false;
                p++;
                continue;
            }
            if (c == '/' && p + 1 < s.size() && s[p + 1] == '/') { while (p < s.size() && s[p] != '\n') p++; continue; }
            if (c == '"') in_str = true;
            else if (c == '-' && p + 1 < s.size() && s[p + 1] == '>') { out += "->"; p += 2; continue; }
            else if (c == '(' || c == '[' || c == '{' || c == '<') depth++;
            else if (c == ')' || c == ']' || c == '>') depth--;
            else if (c == '}') { if (depth == 0) break; depth--; }
            else if (c == '\n') { line++; if (depth <= 0) { p++; break; } }
            out += c;
            p++;
        }
        return out;
    }

    std::vector<std::string> value_refs(const std::string& t) {
        std::vector<std::string> r;
        bool in_str = false;
        for (size_t i = 0; i < t.size(); i++) {
            if (in_str) { if (t[i] == '\\') i++; else if (t[i] == '"') in_str = false; continue; }
            if (t[i] == '"') { in_str = true; continue; }
            if (t[i] == '%') {
                size_t j = i + 1;
                while (j < t.size() && (isalnum((unsigned char)t[j]) || t[j] == '_' || t[j] == '.' || t[j] == '$' || t[j] == '-')) j++;
                if (j < t.size() && t[j] == '#') {        // %r#1: result 1 of a multi-result op
                    j++;
                    while (j < t.size() && isdigit((unsigned char)t[j])) j++;
                }
                r.push_back(t.substr(i, j - i));
                i = j - 1;
            }
        }
        return r;
    }

    void parse_signature(const std::string& sig, Op& op) {
        size_t q = 0;
        auto ws = [&] { while (q < sig.size() && isspace((unsigned char)sig[q])) q++; };
        ws();
        std::vector<TensorType> ins, outs;
        if (q < sig.size() && sig[q] == '(') {
            q++;
            ws();
            while (q < sig.size() && sig[q] != ')') {
                ins.push_back(parse_type(sig, q, line));
                ws();
                if (q < sig.size() && sig[q] == ',') q++;
                ws();
            }
            q++;
            ws();
            if (sig.compare(q, 2, "->") != 0) fail("expected '->' in the type signature");
            q += 2;
            ws();
            if (q < sig.size() && sig[q] == '(') {
                q++;
                ws();
                while (q < sig.size() && sig[q] != ')') {
                    outs.push_back(parse_type(sig, q, line));
                    ws();
                    if (q < sig.size() && sig[q] == ',') q++;
                    ws();
                }
            } else {
                outs.push_back(parse_type(sig, q, line));
            }
            if (outs.size() != 1 && op.name != "call")
                throw UnsupportedOp("line " + std::to_string(line) + ": ops with " + std::to_string(outs.size()) + " results are not supported");
            op.in_types = ins;
            if (!outs.empty()) op.out = outs[0];
            op.out_types = outs;
        } else {
            while (q < sig.size()) {
                ws();
                if (q >= sig.size() || sig.compare(q, 7, "tensor<") != 0) break;
                ins.push_back(parse_type(sig, q, line));
                ws();
                if (q < sig.size() && sig[q] == ',') q++;
            }
            if (ins.empty()) fail("missing type after ':'");
            op.out = ins.back();
            op.in_types = ins;
            ws();
            if (sig.compare(q, 2, "->") == 0) {   // "t1, t2 -> t3"
                q += 2;
                op.out = parse_type(sig, q, line);
            }
        }
    }

    void decode_attrs(Op& op) {
        const std::string& h = op.attrs;
        const std::string& n = op.name;
        if (n == "transpose") {
            if (!ints_after_key(h, "dims", op.dims) && !ints_after_key(h, "permutation", op.dims)) fail("transpose without a permutation");
        } else if (n == "broadcast_in_dim") {
            if (!ints_after_key(h, "dims", op.dims) && !ints_after_key(h, "broadcast_dimensions", op.dims)) fail("broadcast_in_dim without dims");
        } else if (n == "reduce") {
            if (!ints_after_key(h, "dimensions", op.dims)) fail("reduce without dimensions");
            static const char* ops[] = {"maximum", "minimum", "multiply", "add"};
            for (auto o : ops)
                if (h.find(std::string("stablehlo.") + o) != std::string::npos) { op.reducer = o; break; }
            if (op.reducer.empty()) {
                if (h.find("compare") != std::string::npos && (h.find("GT") != std::string::npos || h.find("GE") != std::string::npos)) op.reducer = "maximum";
                else if (h.find("compare") != std::string::npos) op.reducer = "minimum";
            }
        } else if (n == "iota") {
            if (!int_after_key(h, "dim", op.iota_dim) && !int_after_key(h, "iota_dimension", op.iota_dim)) fail("iota without dim");
        } else if (n == "compare") {
            static const char* dirs[] = {"EQ", "NE", "LT", "LE", "GT", "GE"};
            size_t best = std::string::npos;
            for (auto d : dirs) {
                size_t k = 0;
                while ((k = h.find(d, k)) != std::string::npos) {
                    const bool l_ok = k == 0 || !isalnum((unsigned char)h[k - 1]);
                    const bool r_ok = k + 2 >= h.size() || !isalnum((unsigned char)h[k + 2]);
                    if (l_ok && r_ok && k < best) { best = k; op.direction = d; }
                    k += 2;
                }
            }
            if (op.direction.empty()) fail("compare without a direction");
        } else if (n == "dot_general") {
            size_t e = 0;
            std::vector<int64_t> a, b;
            if (ints_after_key(h, "batching_dims", a, 0, &e)) {
                op.lhs_batch = a;
                ints_after_key(h, "x", b, e);      // "[..] x [..]"
                op.rhs_batch = b;
                if (!ints_after_key(h, "contracting_dims", a, 0, &e)) fail("dot_general without contracting_dims");
                op.lhs_contract = a;
                ints_after_key(h, "x", b, e);
                op.rhs_contract = b;
            } else if (ints_after_key(h, "contracting_dims", a, 0, &e)) {
                op.lhs_contract = a;
                ints_after_key(h, "x", b, e);
                op.rhs_contract = b;
            } else {
                ints_after_key(h, "lhs_batching_dimensions", op.lhs_batch);
                ints_after_key(h, "rhs_batching_dimensions", op.rhs_batch);
                if (!ints_after_key(h, "lhs_contracting_dimensions", op.lhs_contract) ||
                    !ints_after_key(h, "rhs_contracting_dimensions", op.rhs_contract))
                    fail("dot_general without dimension numbers");
            }
        } else if (n == "slice") {
            // pretty: [0:2, 1:3:1]   generic: start_indices / limit_indices / strides
            if (!ints_after_key(h, "start_indices", op.starts)) {
                const size_t b0 = h.find('[');
                const size_t b1 = h.find(']', b0);
                if (b0 == std::string::npos || b1 == std::string::npos) fail("slice without indices");
                const std::string body = h.substr(b0 + 1, b1 - b0 - 1);
                size_t i = 0;
                while (i < body.size()) {
                    size_t j = body.find(',', i);
                    if (j == std::string::npos) j = body.size();
                    const std::string part = body.substr(i, j - i);
                    long long a = 0, b = 0, c = 1;
                    const int got = sscanf(part.c_str(), " %lld : %lld : %lld", &a, &b, &c);
                    if (got < 2) fail("bad slice range '" + part + "'");
                    op.starts.push_back(a); op.limits.push_back(b); op.strides.push_back(got == 3 ? c : 1);
                    i = j + 1;
                }
            } else {
                ints_after_key(h, "limit_indices", op.limits);
                if (!ints_after_key(h, "strides", op.strides)) op.strides.assign(op.starts.size(), 1);
            }
        } else if (n == "custom_call") {
            size_t a = h.find('@');
            if (a != std::string::npos) {
                size_t b = a + 1;
                while (b < h.size() && (isalnum((unsigned char)h[b]) || h[b] == '_' || h[b] == '.')) b++;
                op.target = h.substr(a + 1, b - a - 1);
            } else {
                const size_t k = h.find("call_target_name");
                if (k == std::string::npos) fail("custom_call without a target");
                const size_t q0 = h.find('"', k), q1 = h.find('"', q0 + 1);
                op.target = h.substr(q0 + 1, q1 - q0 - 1);
            }
            const size_t k = h.find("backend_config");
            if (k != std::string::npos) {
                size_t q0 = h.find('"', k);
                if (q0 != std::string::npos) {
                    std::string v;
                    size_t i = q0 + 1;
                    while (i < h.size() && h[i] != '"') {
                        if (h[i] == '\\' && i + 1 < h.size()) { v += h[i + 1]; i += 2; }
                        else v += h[i++];
                    }
                    op.backend_config = v;
                }
            }
        } else if (n == "gather") {
            ints_after_key(h, "slice_sizes", op.limits);
            ints_after_key(h, "collapsed_slice_dims", op.dims);
            ints_after_key(h, "start_index_map", op.starts);
            ints_after_key(h, "offset_dims", op.strides);
            if (!int_after_key(h, "index_vector_dim", op.iota_dim)) op.iota_dim = -1;
            ints_after_key(h, "operand_batching_dims", op.lhs_batch);
            ints_after_key(h, "start_indices_batching_dims", op.rhs_batch);
        } else if (n == "constant") {
            const size_t d = h.find("dense<");
            if (d == std::string::npos) fail("constant without dense<...>");
            int depth = 0;
            size_t i = d + 5, start = d + 6;
            bool in_str = false;
            for (; i < h.size(); i++) {
                if (in_str) { if (h[i] == '"') in_str = false; continue; }
                if (h[i] == '"') in_str = true;
                else if (h[i] == '<') depth++;
                else if (h[i] == '>') { depth--; if (depth == 0) break; }
            }
            parse_dense(h.substr(start, i - start), op);
        }
    }

    void parse_statement(const std::string& raw) {
        std::string t = trim(raw);
        if (t.empty()) return;
        if (starts_with(t, "reducer")) {           // region of the preceding reduce
            if (!fn.ops.empty() && fn.ops.back().name == "reduce" && fn.ops.back().reducer.empty()) {
                Op& r = fn.ops.back();
                r.attrs += " " + t;
                static const char* ops[] = {"maximum", "minimum", "multiply", "add"};
                for (auto o : ops)
                    if (t.find(std::string("stablehlo.") + o) != std::string::npos) { r.reducer = o; break; }
            }
            return;
        }
        for (const char* r : {"func.return", "stablehlo.return", "return"}) {
            if (starts_with(t, r)) {
                const size_t c = top_level_colon(t);
                for (auto& v : value_refs(t.substr(strlen(r), c == std::string::npos ? std::string::npos : c - strlen(r))))
                    fn.returns.push_back(value_id(v, false));
                return;
            }
        }
        Op op;
        op.line = line;
        std::string result;
        if (t[0] == '%') {
            const size_t eq = t.find('=');
            if (eq == std::string::npos) fail("expected '=' after the result name");
            result = trim(t.substr(0, eq));
            t = trim(t.substr(eq + 1));
        }
        std::string name;
        size_t q = 0;
        if (t[0] == '"') {
            const size_t e = t.find('"', 1);
            name = t.substr(1, e - 1);
            q = e + 1;
        } else {
            while (q < t.size() && !isspace((unsigned char)t[q]) && t[q] != '(') q++;
            name = t.substr(0, q);
        }
        for (const char* pre : {"stablehlo.", "mhlo.", "chlo.", "func."})
            if (starts_with(name, pre)) { name = name.substr(strlen(pre)); break; }
        op.name = name;
        // `%r:2 = call ...` defines %r#0 and %r#1; `%a, %b = call ...` names them one by one
        std::vector<std::string> result_names;
        if (!result.empty()) {
            const size_t colon = result.find(':');
            if (colon != std::string::npos || result.find(',') != std::string::npos) {
                if (name != "call") throw UnsupportedOp("line " + std::to_string(line) + ": multi-result op " + result);
                if (colon != std::string::npos) {
                    const int n = atoi(result.c_str() + colon + 1);
                    const std::string base = trim(result.substr(0, colon));
                    if (n < 1 || n > 64) fail("bad result count in " + result);
                    for (int i = 0; i < n; i++) result_names.push_back(base + "#" + std::to_string(i));
                } else {
                    result_names = value_refs(result);
                }
            } else {
                result_names.push_back(result);
            }
        }
        const std::string rest = t.substr(q);
        const size_t c = top_level_colon(rest);
        if (c == std::string::npos) fail("op '" + name + "' has no type signature");
        op.attrs = rest.substr(0, c);
        parse_signature(rest.substr(c + 1), op);
        // generic form with a region, `"stablehlo.reduce"(%x, %init) ({ ^bb0(...): ... }) {attrs}`:
        // the values named inside the region are the body's own, not operands
        std::string outer = op.attrs;
        const size_t r0 = outer.find("({");
        if (r0 != std::string::npos) {
            int depth = 0;
            size_t r1 = r0 + 1;
            for (; r1 < outer.size(); r1++) {
                if (outer[r1] == '{') depth++;
                else if (outer[r1] == '}' && --depth == 0) break;
            }
            const size_t close = outer.find(')', r1);
            if (depth != 0 || close == std::string::npos) fail("unterminated region of '" + name + "'");
            outer = outer.substr(0, r0) + outer.substr(close + 1);
        }
        for (auto& v : value_refs(outer)) op.operands.push_back(value_id(v, false));
        if (name == "call") {
            const size_t at = op.attrs.find('@');
            if (at == std::string::npos) fail("call without a callee");
            size_t e = at + 1;
            while (e < op.attrs.size() && (isalnum((unsigned char)op.attrs[e]) || op.attrs[e] == '_' || op.attrs[e] == '.' || op.attrs[e] == '$')) e++;
            op.target = op.attrs.substr(at + 1, e - at - 1);
            if (op.out_types.size() != result_names.size())
                fail("call @" + op.target + " names " + std::to_string(result_names.size()) + " results, its signature has " +
                     std::to_string(op.out_types.size()));
            if (result_names.empty()) return;              // a call without results computes nothing here
            op.result = value_id(result_names[0], true);
            for (size_t i = 1; i < result_names.size(); i++) op.more_results.push_back(value_id(result_names[i], true));
            fn.ops.push_back(std::move(op));
            return;
        }
        decode_attrs(op);
        if (result_names.empty()) fail("op '" + name + "' has no result");
        op.result = value_id(result_names[0], true);
        fn.ops.push_back(std::move(op));
    }

    bool parse_function() {
        // "func.func [public|private] @name(args) -> results [attributes {...}] {"
        const size_t f = s.find("func.func", p);
        if (f == std::string::npos) return false;
        for (size_t i = p; i < f; i++) if (s[i] == '\n') line++;
        p = f + 9;
        skip_ws();
        fn = Function();
        names.clear();
        const size_t at = s.find('@', p);
        size_t e = at + 1;
        while (e < s.size() && (isalnum((unsigned char)s[e]) || s[e] == '_' || s[e] == '.')) e++;
        fn.name = s.substr(at + 1, e - at - 1);
        p = e;
        skip_ws();
        if (p >= s.size() || s[p] != '(') fail("expected '(' after the function name");
        p++;
        for (;;) {
            skip_ws();
            if (p < s.size() && s[p] == ')') { p++; break; }
            if (p >= s.size() || s[p] != '%') fail("expected an argument name");
            size_t j = p + 1;
            while (j < s.size() && (isalnum((unsigned char)s[j]) || s[j] == '_' || s[j] == '.')) j++;
            const std::string an = s.substr(p, j - p);
            p = j;
            skip_ws();
            if (s[p] != ':') fail("expected ':' after " + an);
            p++;
            fn.arg_types.push_back(parse_type(s, p, line));
            fn.arg_ids.push_back(value_id(an, true));
            skip_ws();
            if (p < s.size() && s[p] == '{') {       // argument attributes
                int d = 0;
                do { if (s[p] == '{') d++; else if (s[p] == '}') d--; p++; } while (p < s.size() && d > 0);
                skip_ws();
            }
            if (s.compare(p, 4, "loc(") == 0) { int d = 0; do { if (s[p] == '(') d++; else if (s[p] == ')') d--; p++; } while (p < s.size() && d > 0); skip_ws(); }
            if (p < s.size() && s[p] == ',') p++;
        }
        skip_ws();
        if (s.compare(p, 2, "->") == 0) {
            p += 2;
            skip_ws();
            const bool paren = s[p] == '(';
            if (paren) p++;
            for (;;) {
                skip_ws();
                if (paren && s[p] == ')') { p++; break; }
                fn.result_types.push_back(parse_type(s, p, line));
                skip_ws();
                if (!paren) break;       // a '{' here opens the body
                if (p < s.size() && s[p] == '{') { int d = 0; do { if (s[p] == '{') d++; else if (s[p] == '}') d--; p++; } while (p < s.size() && d > 0); skip_ws(); }
                if (s[p] == ',') p++;
            }
        }
        skip_ws();
        if (s.compare(p, 10, "attributes") == 0) {
            p += 10;
            skip_ws();
            int d = 0;
            do { if (s[p] == '{') d++; else if (s[p] == '}') d--; p++; } while (p < s.size() && d > 0);
            skip_ws();
        }
        if (p >= s.size() || s[p] != '{') fail("expected '{' to open the body of @" + fn.name);
        p++;
        for (;;) {
            skip_ws();
            if (p >= s.size()) fail("unterminated function body");
            if (s[p] == '}') { p++; break; }
            parse_statement(read_statement());
        }
        if (fn.returns.size() != fn.result_types.size() && !fn.result_types.empty())
            fail("@" + fn.name + " returns " + std::to_string(fn.returns.size()) + " values, signature declares " +
                 std::to_string(fn.result_types.size()));
        return true;
    }
};

}  // namespace

// Replaces every call in `f` by the callee's operations (callees inlined first; recursion is an
// error): the callee's arguments become the call's operands, its other values get fresh ids in the
// caller, and uses of the call's results become uses of the values the callee returns.
static void inline_calls(Function& f, const std::map<std::string, Function>& all, std::vector<std::string>& stack) {
    bool any = false;
    for (auto& op : f.ops) any |= op.name == "call";
    if (!any) return;
    if (stack.size() > 64) throw ParseError("calls nested deeper than 64 functions");
    stack.push_back(f.name);
    std::vector<Op> out;
    std::map<int, int> subst;          // caller value -> the value that replaces it
    auto mapped = [&](int v) { auto it = subst.find(v); return it == subst.end() ? v : it->second; };
    for (auto& op : f.ops) {
        for (int& v : op.operands) v = mapped(v);
        if (op.name != "call") { out.push_back(std::move(op)); continue; }
        auto it = all.find(op.target);
        if (it == all.end()) throw ParseError("line " + std::to_string(op.line) + ": call of unknown function @" + op.target);
        for (auto& s : stack)
            if (s == op.target) throw ParseError("line " + std::to_string(op.line) + ": recursive call of @" + op.target);
        Function callee = it->second;
        inline_calls(callee, all, stack);
        if (callee.arg_ids.size() != op.operands.size())
            throw ParseError("line " + std::to_string(op.line) + ": @" + op.target + " takes " + std::to_string(callee.arg_ids.size()) +
                             " arguments, the call passes " + std::to_string(op.operands.size()));
        if (callee.returns.size() != op.out_types.size())
            throw ParseError("line " + std::to_string(op.line) + ": @" + op.target + " returns " + std::to_string(callee.returns.size()) +
                             " values, the call expects " + std::to_string(op.out_types.size()));
        for (size_t i = 0; i < callee.arg_types.size(); i++)
            if (!op.in_types.empty() && i < op.in_types.size() && !(op.in_types[i] == callee.arg_types[i]))
                throw ParseError("line " + std::to_string(op.line) + ": argument " + std::to_string(i) + " of @" + op.target + " has another type");
        std::map<int, int> local;      // callee value -> caller value
        for (size_t i = 0; i < callee.arg_ids.size(); i++) local[callee.arg_ids[i]] = op.operands[i];
        for (auto& c : callee.ops) {
            Op n = c;
            for (int& v : n.operands) v = local.at(v);
            n.result = f.num_values++;
            local[c.result] = n.result;
            out.push_back(std::move(n));
        }
        std::vector<int> results = {op.result};
        results.insert(results.end(), op.more_results.begin(), op.more_results.end());
        for (size_t i = 0; i < results.size(); i++) {
            if (!(callee.result_types.empty() || callee.result_types[i] == op.out_types[i]))
                throw ParseError("line " + std::to_string(op.line) + ": result " + std::to_string(i) + " of @" + op.target + " has another type");
            subst[results[i]] = local.at(callee.returns[i]);
        }
    }
    for (int& r : f.returns) r = mapped(r);
    f.ops = std::move(out);
    stack.pop_back();
}

Function parse_module(const std::string& text) {
    Parser ps(text);
    std::vector<Function> fns;
    while (ps.parse_function()) fns.push_back(ps.fn);
    if (fns.empty()) throw ParseError("no func.func found in the module");
    std::map<std::string, Function> all;
    for (auto& f : fns) all.emplace(f.name, f);
    Function* entry = &fns[0];
    for (auto& f : fns)
        if (f.name == "main") { entry = &f; break; }
    std::vector<std::string> stack;
    inline_calls(*entry, all, stack);
    return *entry;
}

// ---------------------------------------------------------------- backend_config
double Config::get_float(const std::string& k, double d) const {
    auto it = num.find(k);
    return it == num.end() ? d : it->second;
}
int64_t Config::get_int(const std::string& k, int64_t d) const {
    auto it = num.find(k);
    return it == num.end() ? d : (int64_t)it->second;
}
bool Config::get_bool(const std::string& k, bool d) const {
    auto it = boolean.find(k);
    if (it != boolean.end()) return it->second;
    auto n = num.find(k);
    if (n != num.end() && n->second == floor(n->second)) return n->second != 0;
    return d;
}
std::string Config::get_string(const std::string& k, const std::string& d) const {
    auto it = str.find(k);
    return it == str.end() ? d : it->second;
}
std::vector<int64_t> Config::get_int_array(const std::string& k, const std::vector<int64_t>& d) const {
    auto it = arr.find(k);
    if (it == arr.end()) return d;
    std::vector<int64_t> r;
    for (double v : it->second) r.push_back((int64_t)v);
    return r;
}

Config parse_config(const std::string& j) {
    Config c, empty;
    size_t i = 0;
    auto ws = [&] { while (i < j.size() && isspace((unsigned char)j[i])) i++; };
    ws();
    if (i >= j.size() || j[i] != '{') return empty;
    i++;
    for (;;) {
        ws();
        if (i < j.size() && j[i] == '}') return c;
        if (i >= j.size() || j[i] != '"') return empty;
        const size_t e = j.find('"', i + 1);
        if (e == std::string::npos) return empty;
        const std::string key = j.substr(i + 1, e - i - 1);
        i = e + 1;
        ws();
        if (i >= j.size() || j[i] != ':') return empty;
        i++;
        ws();
        if (i >= j.size()) return empty;
        if (j[i] == '"') {
            const size_t e2 = j.find('"', i + 1);
            if (e2 == std::string::npos) return empty;
            c.str[key] = j.substr(i + 1, e2 - i - 1);
            i = e2 + 1;
        } else if (j.compare(i, 4, "true") == 0) { c.boolean[key] = true; i += 4; }
        else if (j.compare(i, 5, "false") == 0) { c.boolean[key] = false; i += 5; }
        else if (j[i] == '[') {
            i++;
            std::vector<double> v;
            std::vector<std::string> sv;
            for (;;) {
                ws();
                if (i < j.size() && j[i] == ']') { i++; break; }
                if (i < j.size() && j[i] == '"') {          // an array of strings (the operation list of fused_elementwise)
                    const size_t e3 = j.find('"', i + 1);
                    if (e3 == std::string::npos) return empty;
                    sv.push_back(j.substr(i + 1, e3 - i - 1));
                    i = e3 + 1;
                    ws();
                    if (i < j.size() && j[i] == ',') i++;
                    continue;
                }
                char* e2;
                const double d = strtod(j.c_str() + i, &e2);
                if (e2 == j.c_str() + i) return empty;
                v.push_back(d);
                i = e2 - j.c_str();
                ws();
                if (i < j.size() && j[i] == ',') i++;
            }
            if (!sv.empty()) {
                if (!v.empty()) return empty;
                c.sarr[key] = sv;
            } else {
                c.arr[key] = v;
            }
        } else {
            char* e2;
            const double d = strtod(j.c_str() + i, &e2);
            if (e2 == j.c_str() + i) return empty;
            c.num[key] = d;
            i = e2 - j.c_str();
        }
        ws();
        if (i < j.size() && j[i] == ',') i++;
    }
}

}  // namespace mhlo
