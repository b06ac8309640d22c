// Minimal StableHLO IR + text front-end for the host executor.
//
// Covers the operator subset the fused transformer path needs (the reference's
// full 92-op parser is Sources/MetalHLOCore/Parser/Parser.swift; the grammar
// forms accepted here are the ones listed for it: pretty and generic op forms,
// both dot_general attribute spellings, both reduce spellings, dense constants).
#pragma once
#include <stdint.h>

#include <map>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

namespace mhlo {

// Element type codes are MHLOElementType / mhip_dtype.
enum DType { F16 = 0, F32 = 1, F64 = 2, BF16 = 3, I1 = 4, I8 = 5, I16 = 6, I32 = 7, I64 = 8,
             UI8 = 9, UI16 = 10, UI32 = 11, UI64 = 12 };

// Storage bytes per element (i1 is one byte per element on the device).
inline int dtype_bytes(int dt) {
    switch (dt) {
        case F16: case BF16: case I16: case UI16: return 2;
        case F32: case I32: case UI32: return 4;
        case F64: case I64: case UI64: return 8;
        default: return 1;
    }
}
inline const char* dtype_name(int dt) {
    static const char* const names[13] = {"f16", "f32", "f64", "bf16", "i1", "i8", "i16", "i32", "i64", "ui8", "ui16", "ui32", "ui64"};
    return dt >= 0 && dt < 13 ? names[dt] : "?";
}
inline bool dtype_is_float(int dt) { return dt == F16 || dt == F32 || dt == F64 || dt == BF16; }

struct TensorType {
    std::vector<int64_t> shape;
    int dtype = F32;
    int64_t numel() const { int64_t n = 1; for (auto d : shape) n *= d; return n; }
    size_t bytes() const { return (size_t)numel() * dtype_bytes(dtype); }
    bool operator==(const TensorType& o) const { return dtype == o.dtype && shape == o.shape; }
};

struct ParseError : std::runtime_error { using std::runtime_error::runtime_error; };
struct UnsupportedOp : std::runtime_error { using std::runtime_error::runtime_error; };

struct Op {
    std::string name;                 // "add", "dot_general", "custom_call", ...
    std::vector<int> operands;        // value ids
    std::vector<TensorType> in_types; // as written in the signature (may be empty)
    TensorType out;
    int result = -1;                  // value id
    std::string attrs;                // raw text between the operands and the signature
    // decoded attributes
    std::vector<int64_t> dims;        // broadcast dims / permutation / reduce dims
    std::vector<int64_t> lhs_batch, rhs_batch, lhs_contract, rhs_contract;
    std::vector<int64_t> starts, limits, strides;   // slice
    int64_t iota_dim = 0;
    std::string target, backend_config, direction, reducer;
    // `call` only, and only until parse_module has inlined it: the other results of a
    // multi-result call (`%r:2 = call ...`, used as %r#0, %r#1) and all result types
    std::vector<int> more_results;
    std::vector<TensorType> out_types;
    std::vector<uint8_t> constant;    // dense bytes in `out` layout (splat already expanded)
    bool splat = false;
    uint64_t splat_bits = 0;
    int line = 0;
};

struct Function {
    std::string name;
    std::vector<TensorType> arg_types;
    std::vector<int> arg_ids;
    std::vector<Op> ops;
    std::vector<int> returns;
    std::vector<TensorType> result_types;
    int num_values = 0;
};

// Parses a module (or a bare func.func) and returns its entry function (`main` when present,
// else the first) with every `call` / `func.call` of another function of the module inlined
// (the reference resolves callees the same way, Parser/Parser.swift:31-226; tracing front ends
// emit private helper functions such as @_where routinely).  Throws ParseError / UnsupportedOp.
Function parse_module(const std::string& text);

// Rewrites decomposed softmax / GELU(tanh) / LayerNorm / RMSNorm / attention /
// matmul+bias+activation subgraphs into the fused custom_calls (fusion.cpp); returns the
// number of rewrites.  Values used outside a pattern are never absorbed.
int fuse_patterns(Function& fn, const std::set<std::string>* disabled = nullptr);

// parse_module + fuse_patterns (unless `opt_level` is 0) with the environment's switches:
// METALHLO_DISABLED_PASSES (comma-separated names of the reference's fusion passes),
// METALHLO_DEBUG_PASSES=1 (one line per pass on stderr), METALHLO_DUMP_OPTIMIZED=<file>.
Function build_function(const std::string& text, int opt_level);

// Flat JSON object {"k": number | bool | "string" | [numbers]} as used by
// backend_config (Compiler/CustomCallHandlers.swift:102-168).  Anything that
// does not parse yields an empty config.
struct Config {
    std::map<std::string, double> num;
    std::map<std::string, bool> boolean;
    std::map<std::string, std::string> str;
    std::map<std::string, std::vector<double>> arr;
    std::map<std::string, std::vector<std::string>> sarr;
    double get_float(const std::string& k, double d) const;
    int64_t get_int(const std::string& k, int64_t d) const;
    bool get_bool(const std::string& k, bool d) const;
    std::string get_string(const std::string& k, const std::string& d) const;
    std::vector<int64_t> get_int_array(const std::string& k, const std::vector<int64_t>& d) const;
    std::vector<std::string> get_string_array(const std::string& k) const { auto it = sarr.find(k); return it == sarr.end() ? std::vector<std::string>() : it->second; }
};
Config parse_config(const std::string& json);

// float <-> 16-bit helpers used for constants (round to nearest even).
uint16_t f32_to_bf16_bits(float f);
uint16_t f32_to_f16_bits(float f);

}  // namespace mhlo
