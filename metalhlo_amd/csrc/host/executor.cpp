#include "executor.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <chrono>
#include <map>

#include "../../../include/mhip.h"

namespace mhlo {

// ---------------------------------------------------------------- memory
DevicePool::~DevicePool() {
    for (auto& kv : free_) (void)hipFree(kv.second);
}

static size_t bucket(size_t bytes) {
    size_t b = 256;
    while (b < bytes) b <<= 1;
    return bytes > (64u << 20) ? ((bytes + (2u << 20) - 1) & ~((size_t)(2u << 20) - 1)) : b;
}

void* DevicePool::alloc(size_t bytes) {
    const size_t b = bucket(bytes ? bytes : 1);
    {
        std::lock_guard<std::mutex> g(mu_);
        auto it = free_.find(b);
        if (it != free_.end()) {
            void* p = it->second;
            free_.erase(it);
            return p;
        }
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, b);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        {   // give cached blocks back and retry once
            std::lock_guard<std::mutex> g(mu_);
            for (auto& kv : free_) (void)hipFree(kv.second);
            free_.clear();
        }
        e = hipMalloc(&p, b);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            throw BufferError(std::string("hipMalloc of ") + std::to_string(b) + " bytes failed: " + hipGetErrorString(e));
        }
    }
    return p;
}

void DevicePool::release(void* p, size_t bytes) {
    std::lock_guard<std::mutex> g(mu_);
    free_.emplace(bucket(bytes ? bytes : 1), p);
}

DeviceTensor Client::allocate(const TensorType& t) {
    if (device < 0) throw NoDevice("no HIP device: buffers cannot be created");
    DeviceTensor d;
    d.type = t;
    d.mem = std::make_shared<DeviceMem>();
    d.mem->pool = &pool;
    d.mem->bytes = t.bytes();
    d.mem->ptr = pool.alloc(d.mem->bytes);
    return d;
}

Executable::~Executable() {
    for (auto& g : graphs) if (g.exec) (void)hipGraphExecDestroy(g.exec);
    if (arena) (void)hipFree(arena);
}

// Where the allocations of one walk over the program come from.
struct Allocator {
    enum Mode { POOL, RECORD, ARENA } mode = POOL;
    Client* client = nullptr;
    ArenaPlan* plan = nullptr;
    char* base = nullptr;
    bool escaping_in_arena = false;
    std::vector<std::shared_ptr<DeviceMem>>* presets = nullptr;   // by slot: storage allocated ahead for the escaping slots
    size_t next = 0;

    DeviceTensor allocate(const TensorType& t) {
        if (mode == POOL) return client->allocate(t);
        DeviceTensor d;
        d.type = t;
        d.mem = std::make_shared<DeviceMem>();
        d.mem->bytes = t.bytes();
        const size_t rounded = (t.bytes() + 255) & ~(size_t)255;
        if (mode == RECORD) {
            ArenaPlan::Slot sl;
            sl.bytes = rounded;
            sl.begin = plan->clock++;
            plan->slots.push_back(sl);
            d.mem->recorder = plan;
            d.mem->slot = (int)plan->slots.size() - 1;
            return d;
        }
        if (next >= plan->slots.size() || plan->slots[next].bytes != rounded)
            throw ExecError("the execution does not follow the memory plan made at compile time");
        const size_t slot_no = next;
        const ArenaPlan::Slot& sl = plan->slots[next++];
        if (sl.escapes && presets) {
            d.mem = (*presets)[slot_no];
            if (!d.mem) throw ExecError("the execution does not follow the memory plan made at compile time");
        } else if (sl.escapes && !escaping_in_arena) {
            d.mem->pool = &client->pool;
            d.mem->ptr = client->pool.alloc(d.mem->bytes);
        } else {
            d.mem->ptr = base + sl.offset;     // not owned: the arena outlives the execution
        }
        return d;
    }
};

// Offsets for the recorded slots: largest first, each at the lowest 256-byte boundary where it
// meets no already placed slot that is alive at the same time.
static size_t place_slots(ArenaPlan& plan, bool escaping, size_t floor) {
    std::vector<int> order;
    for (int i = 0; i < (int)plan.slots.size(); i++) if (plan.slots[i].escapes == escaping) order.push_back(i);
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return plan.slots[a].bytes > plan.slots[b].bytes; });
    std::vector<int> placed;
    size_t top = floor;
    for (int i : order) {
        ArenaPlan::Slot& s = plan.slots[i];
        std::vector<std::pair<size_t, size_t>> busy;     // [offset, end) of the slots alive together with s
        for (int j : placed) {
            const ArenaPlan::Slot& o = plan.slots[j];
            if (o.begin <= s.end && s.begin <= o.end) busy.emplace_back(o.offset, o.offset + o.bytes);
        }
        std::sort(busy.begin(), busy.end());
        size_t at = floor;
        for (auto& b : busy) {
            if (at + s.bytes <= b.first) break;
            at = std::max(at, b.second);
        }
        s.offset = at;
        top = std::max(top, at + s.bytes);
        placed.push_back(i);
    }
    return top;
}

// The same slots placed in the order the execution allocates them, each in the block of its own
// size that was released last (else the smallest larger block, split; else new bytes at the top,
// after merging free neighbours).  A value then tends to land where its predecessor in the
// program was read a moment ago, bytes that are still in the caches, instead of at the lowest
// address that happens to be free.  May need more bytes than place_slots; the caller compares.
static size_t place_slots_recent(ArenaPlan& plan, bool escaping, size_t floor) {
    struct Event { int time; int slot; bool release; };
    std::vector<Event> ev;
    for (int i = 0; i < (int)plan.slots.size(); i++) {
        if (plan.slots[i].escapes != escaping) continue;
        ev.push_back({plan.slots[i].begin, i, false});
        ev.push_back({plan.slots[i].end, i, true});
    }
    // a release at the time of an allocation (cannot happen with the recording clock) comes second
    std::stable_sort(ev.begin(), ev.end(), [](const Event& a, const Event& b) { return a.time != b.time ? a.time < b.time : a.release < b.release; });
    struct Block { size_t offset, bytes; int released; };
    std::vector<Block> free_blocks;
    size_t top = floor;
    auto merge = [&]() {
        std::sort(free_blocks.begin(), free_blocks.end(), [](const Block& a, const Block& b) { return a.offset < b.offset; });
        std::vector<Block> out;
        for (const Block& b : free_blocks) {
            if (!out.empty() && out.back().offset + out.back().bytes == b.offset) {
                out.back().bytes += b.bytes;
                out.back().released = std::max(out.back().released, b.released);
            } else out.push_back(b);
        }
        if (!out.empty() && out.back().offset + out.back().bytes == top) { top = out.back().offset; out.pop_back(); }
        free_blocks.swap(out);
    };
    auto take = [&](size_t bytes, size_t& offset) {
        int best = -1;
        for (int i = 0; i < (int)free_blocks.size(); i++)
            if (free_blocks[i].bytes == bytes && (best < 0 || free_blocks[i].released > free_blocks[best].released)) best = i;
        if (best < 0)
            for (int i = 0; i < (int)free_blocks.size(); i++)
                if (free_blocks[i].bytes > bytes && (best < 0 || free_blocks[i].bytes < free_blocks[best].bytes)) best = i;
        if (best < 0) return false;
        offset = free_blocks[best].offset;
        if (free_blocks[best].bytes == bytes) free_blocks.erase(free_blocks.begin() + best);
        else { free_blocks[best].offset += bytes; free_blocks[best].bytes -= bytes; }
        return true;
    };
    size_t high = floor;
    for (const Event& e : ev) {
        ArenaPlan::Slot& s = plan.slots[e.slot];
        if (e.release) { free_blocks.push_back({s.offset, s.bytes, e.time}); continue; }
        if (!take(s.bytes, s.offset)) {
            merge();
            if (!take(s.bytes, s.offset)) { s.offset = top; top += s.bytes; }
        }
        high = std::max(high, std::max(top, s.offset + s.bytes));
    }
    return high;
}

// ---------------------------------------------------------------- op tables
static const std::map<std::string, int> kUnary = {
    {"exponential", MHIP_UN_EXP}, {"tanh", MHIP_UN_TANH}, {"rsqrt", MHIP_UN_RSQRT}, {"sqrt", MHIP_UN_SQRT},
    {"negate", MHIP_UN_NEG}, {"logistic", MHIP_UN_LOGISTIC}, {"abs", MHIP_UN_ABS}, {"log", MHIP_UN_LOG},
    {"erf", MHIP_UN_ERF}, {"sine", MHIP_UN_SIN}, {"cosine", MHIP_UN_COS}, {"floor", MHIP_UN_FLOOR}, {"ceil", MHIP_UN_CEIL}};
static const std::map<std::string, int> kBinary = {
    {"add", MHIP_BIN_ADD}, {"subtract", MHIP_BIN_SUB}, {"multiply", MHIP_BIN_MUL}, {"divide", MHIP_BIN_DIV},
    {"maximum", MHIP_BIN_MAX}, {"minimum", MHIP_BIN_MIN}, {"power", MHIP_BIN_POW}};
static const std::map<std::string, int> kCompare = {{"EQ", MHIP_CMP_EQ}, {"NE", MHIP_CMP_NE}, {"LT", MHIP_CMP_LT},
                                                    {"LE", MHIP_CMP_LE}, {"GT", MHIP_CMP_GT}, {"GE", MHIP_CMP_GE}};
static const std::map<std::string, int> kReduce = {{"add", MHIP_RED_SUM}, {"maximum", MHIP_RED_MAX},
                                                   {"minimum", MHIP_RED_MIN}, {"multiply", MHIP_RED_PROD}};
static const std::map<std::string, int> kActivation = {{"none", MHIP_ACT_NONE}, {"relu", MHIP_ACT_RELU},
                                                       {"gelu", MHIP_ACT_GELU}, {"silu", MHIP_ACT_SILU},
                                                       {"tanh", MHIP_ACT_TANH}, {"sigmoid", MHIP_ACT_SIGMOID},
                                                       {"gelu_approximate", MHIP_ACT_GELU}, {"geluApproximate", MHIP_ACT_GELU},
                                                       {"swish", MHIP_ACT_SILU}, {"gelu_exact", MHIP_ACT_GELU_ERF}};
// custom_call targets served by a kernel (Compiler/CustomCallHandlers.swift:75-89)
static const char* kTargets[] = {"fused_scaled_dot_product_attention", "fused_layer_norm", "fused_rms_norm",
                                 "fused_softmax", "fused_gelu", "fused_matmul_bias_activation", "fused_ffn",
                                 "fused_rope", "fused_elementwise", "fused_batch_norm", "fused_depth_attention",
                                 "fused_token_embedding"};

// The operation list of a fused_elementwise call ("ops", or "operations": CustomCallHandlers.swift:941-943)
// as codes for mhip_elementwise_chain, and the number of inputs the chain consumes.  The names are
// the reference's (:969-1065): six binary operations and twelve unary ones.
static std::vector<int> chain_ops(const Op& op, const Config& cfg, size_t* inputs_needed) {
    static const std::map<std::string, int> binary = {{"add", MHIP_BIN_ADD}, {"subtract", MHIP_BIN_SUB}, {"multiply", MHIP_BIN_MUL},
                                                      {"divide", MHIP_BIN_DIV}, {"maximum", MHIP_BIN_MAX}, {"minimum", MHIP_BIN_MIN}};
    static const std::map<std::string, int> unary = {{"negate", MHIP_UN_NEG}, {"abs", MHIP_UN_ABS}, {"exponential", MHIP_UN_EXP},
                                                     {"log", MHIP_UN_LOG}, {"sqrt", MHIP_UN_SQRT}, {"rsqrt", MHIP_UN_RSQRT},
                                                     {"tanh", MHIP_UN_TANH}, {"logistic", MHIP_UN_LOGISTIC}, {"sine", MHIP_UN_SIN},
                                                     {"cosine", MHIP_UN_COS}, {"floor", MHIP_UN_FLOOR}, {"ceil", MHIP_UN_CEIL}};
    std::vector<std::string> names = cfg.get_string_array("ops");
    if (names.empty()) names = cfg.get_string_array("operations");
    if (names.empty()) throw ParseError("line " + std::to_string(op.line) + " (fused_elementwise): Missing 'ops' or 'operations' in the config");
    if (names.size() > MHIP_CHAIN_MAX_OPS) throw UnsupportedOp("line " + std::to_string(op.line) + " (fused_elementwise): more than 16 operations in one chain");
    std::vector<int> codes;
    size_t need = 1;
    for (auto& n : names) {
        if (binary.count(n)) { codes.push_back(MHIP_CHAIN_BINARY + binary.at(n)); need++; }
        else if (unary.count(n)) codes.push_back(unary.at(n));
        else throw ParseError("line " + std::to_string(op.line) + " (fused_elementwise): Unsupported operation in fused chain: " + n);
    }
    if (inputs_needed) *inputs_needed = need;
    return codes;
}

static std::string where(const Op& op) { return "line " + std::to_string(op.line) + " (stablehlo." + op.name + "): "; }

static bool is_kernel_float(int dt) { return dt == F32 || dt == F16 || dt == BF16; }

// Shapes/dtypes of every value, filled while validating.
static std::vector<TensorType> value_types(const Function& fn) {
    std::vector<TensorType> t(fn.num_values);
    for (size_t i = 0; i < fn.arg_ids.size(); i++) t[fn.arg_ids[i]] = fn.arg_types[i];
    for (auto& op : fn.ops) t[op.result] = op.out;
    return t;
}

struct DotPlan {
    int64_t B = 1, M = 1, N = 1, K = 1;
    bool lhs_copy = false, rhs_copy = false;   // need a transposing copy into canonical order
    bool trans_a = false, trans_b = false;
    std::vector<int64_t> lhs_perm, rhs_perm;   // canonical orders [batch, free, contract] / [batch, contract, free]
};

static bool is_identity_after(const std::vector<int64_t>& perm) {
    for (size_t i = 0; i < perm.size(); i++) if (perm[i] != (int64_t)i) return false;
    return true;
}

static DotPlan plan_dot(const Op& op, const TensorType& lt, const TensorType& rt) {
    DotPlan p;
    std::vector<int64_t> lb = op.lhs_batch, rb = op.rhs_batch, lc = op.lhs_contract, rc = op.rhs_contract;
    if (op.name == "dot") {
        lc = {(int64_t)lt.shape.size() - 1};
        rc = {0};
    }
    auto in = [](const std::vector<int64_t>& v, int64_t d) { return std::find(v.begin(), v.end(), d) != v.end(); };
    std::vector<int64_t> lf, rf;
    for (int64_t d = 0; d < (int64_t)lt.shape.size(); d++) if (!in(lb, d) && !in(lc, d)) lf.push_back(d);
    for (int64_t d = 0; d < (int64_t)rt.shape.size(); d++) if (!in(rb, d) && !in(rc, d)) rf.push_back(d);
    if (lb.size() != rb.size() || lc.size() != rc.size()) throw ParseError(where(op) + "mismatched dimension numbers");
    for (size_t i = 0; i < lb.size(); i++) {
        if (lt.shape.at(lb[i]) != rt.shape.at(rb[i])) throw ParseError(where(op) + "batch sizes differ");
        p.B *= lt.shape[lb[i]];
    }
    for (size_t i = 0; i < lc.size(); i++) {
        if (lt.shape.at(lc[i]) != rt.shape.at(rc[i])) throw ParseError(where(op) + "contracting sizes differ");
        p.K *= lt.shape[lc[i]];
    }
    for (auto d : lf) p.M *= lt.shape[d];
    for (auto d : rf) p.N *= rt.shape[d];
    auto cat = [](std::vector<int64_t> a, const std::vector<int64_t>& b, const std::vector<int64_t>& c) {
        a.insert(a.end(), b.begin(), b.end());
        a.insert(a.end(), c.begin(), c.end());
        return a;
    };
    // lhs: [batch, free, contract] is A[M,K]; [batch, contract, free] is A stored [K,M]
    if (is_identity_after(cat(lb, lf, lc))) p.trans_a = false;
    else if (is_identity_after(cat(lb, lc, lf))) p.trans_a = true;
    else { p.lhs_copy = true; p.lhs_perm = cat(lb, lf, lc); }
    // rhs: [batch, contract, free] is B[K,N]; [batch, free, contract] is B stored [N,K]
    if (is_identity_after(cat(rb, rc, rf))) p.trans_b = false;
    else if (is_identity_after(cat(rb, rf, rc))) p.trans_b = true;
    else { p.rhs_copy = true; p.rhs_perm = cat(rb, rc, rf); }
    return p;
}

static std::vector<int64_t> dense_strides(const std::vector<int64_t>& shape) {
    std::vector<int64_t> s(shape.size(), 1);
    for (int i = (int)shape.size() - 2; i >= 0; i--) s[i] = s[i + 1] * shape[i + 1];
    return s;
}

// stablehlo.gather as the descriptor mhip_gather takes.  Attribute slots of Op: limits =
// slice_sizes, dims = collapsed_slice_dims, starts = start_index_map, strides = offset_dims,
// iota_dim = index_vector_dim, lhs_batch / rhs_batch = operand / start_indices batching dims.
struct GatherPlan {
    bool whole_rows = false;          // operand [rows, d], indices pick rows: the embedding-lookup kernel
    std::vector<int64_t> out_op_stride, out_idx_stride, comp_op_stride, comp_max;
    int64_t comp_stride = 0;
};

static GatherPlan plan_gather(const Op& op, const TensorType& xt, const TensorType& it) {
    GatherPlan p;
    const int64_t xr = (int64_t)xt.shape.size(), ir = (int64_t)it.shape.size(), rr = (int64_t)op.out.shape.size();
    if (it.dtype != I32 && it.dtype != I64) throw UnsupportedOp(where(op) + "gather indices must be i32 or i64");
    if (op.out.dtype != xt.dtype) throw ParseError(where(op) + "gather changes the element type");
    const int64_t ivd = op.iota_dim < 0 ? ir : op.iota_dim;
    auto has = [](const std::vector<int64_t>& v, int64_t d) { return std::find(v.begin(), v.end(), d) != v.end(); };
    if ((int64_t)op.limits.size() != xr || ivd > ir || rr > 8 || op.starts.size() > 8 || op.lhs_batch.size() != op.rhs_batch.size())
        throw ParseError(where(op) + "bad gather dimension numbers");
    const int64_t n_comp = ivd < ir ? it.shape[ivd] : 1;
    if ((int64_t)op.starts.size() != n_comp) throw ParseError(where(op) + "start_index_map does not match the index vector");
    const auto xs = dense_strides(xt.shape), is = dense_strides(it.shape);
    for (int64_t d = 0; d < xr; d++) {
        if (op.limits[d] < 0 || op.limits[d] > xt.shape[d]) throw ParseError(where(op) + "slice size outside the operand");
        if ((has(op.dims, d) || has(op.lhs_batch, d)) && op.limits[d] > 1) throw ParseError(where(op) + "collapsed / batching dims need slice size 1");
    }
    // operand dims that stay in the result, in order: one per offset dim
    std::vector<int64_t> kept;
    for (int64_t d = 0; d < xr; d++) if (!has(op.dims, d) && !has(op.lhs_batch, d)) kept.push_back(d);
    if (kept.size() != op.strides.size() || (int64_t)(op.strides.size() + (size_t)(ir - (ivd < ir ? 1 : 0))) != rr)
        throw ParseError(where(op) + "offset_dims do not match the result rank");
    // batch dims of the result walk the dims of start_indices other than index_vector_dim
    std::vector<int64_t> idx_dims;
    for (int64_t d = 0; d < ir; d++) if (d != ivd) idx_dims.push_back(d);
    p.out_op_stride.assign(rr, 0);
    p.out_idx_stride.assign(rr, 0);
    size_t nb = 0, no = 0;
    for (int64_t r = 0; r < rr; r++) {
        if (has(op.strides, r)) {
            const int64_t d = kept.at(no++);
            if (op.out.shape[r] != op.limits[d]) throw ParseError(where(op) + "result shape does not match slice_sizes");
            p.out_op_stride[r] = xs[d];
        } else {
            const int64_t d = idx_dims.at(nb++);
            if (op.out.shape[r] != it.shape[d]) throw ParseError(where(op) + "result shape does not match start_indices");
            p.out_idx_stride[r] = is[d];
            for (size_t b = 0; b < op.rhs_batch.size(); b++)
                if (op.rhs_batch[b] == d) {
                    const int64_t od = op.lhs_batch[b];
                    if (od < 0 || od >= xr || xt.shape[od] != it.shape[d]) throw ParseError(where(op) + "batching dims differ in size");
                    p.out_op_stride[r] = xs[od];
                }
        }
    }
    p.comp_stride = ivd < ir ? is[ivd] : 0;
    for (int64_t c = 0; c < n_comp; c++) {
        const int64_t d = op.starts[c];
        if (d < 0 || d >= xr) throw ParseError(where(op) + "start_index_map out of range");
        p.comp_op_stride.push_back(xs[d]);
        p.comp_max.push_back(xt.shape[d] - op.limits[d]);
    }
    p.whole_rows = xr == 2 && op.dims == std::vector<int64_t>{0} && op.starts == std::vector<int64_t>{0} &&
                   op.limits == std::vector<int64_t>{1, xt.shape[1]} && op.lhs_batch.empty() &&
                   (ivd == ir || (ivd == ir - 1 && it.shape[ivd] == 1)) && op.strides == std::vector<int64_t>{rr - 1};
    return p;
}

// Reduced dims must form one contiguous block [a, b]; gives outer/len/inner.
static bool reduce_block(const std::vector<int64_t>& shape, std::vector<int64_t> dims, int64_t& outer, int64_t& len,
                         int64_t& inner) {
    std::sort(dims.begin(), dims.end());
    for (size_t i = 1; i < dims.size(); i++) if (dims[i] != dims[i - 1] + 1) return false;
    outer = len = inner = 1;
    for (int64_t d = 0; d < (int64_t)shape.size(); d++) {
        if (dims.empty() || d < dims.front()) outer *= shape[d];
        else if (d > dims.back()) inner *= shape[d];
        else len *= shape[d];
    }
    return true;
}

static double scalar_constant(const Op& c) {
    if (!c.splat && c.constant.empty()) throw UnsupportedOp(where(c) + "reduce init must be a scalar constant");
    uint64_t bits = c.splat_bits;
    if (!c.splat) memcpy(&bits, c.constant.data(), std::min<size_t>(8, c.constant.size()));
    switch (c.out.dtype) {
        case F32: { float f; memcpy(&f, &bits, 4); return f; }
        case F64: { double d; memcpy(&d, &bits, 8); return d; }
        case BF16: { uint32_t w = (uint32_t)(bits & 0xFFFF) << 16; float f; memcpy(&f, &w, 4); return f; }
        case F16: {
            const uint32_t h = bits & 0xFFFF, s = (h >> 15) & 1, e = (h >> 10) & 31, m = h & 1023;
            double v = e == 0 ? ldexp((double)m, -24) : e == 31 ? (m ? NAN : INFINITY) : ldexp((double)(m | 1024), (int)e - 25);
            return s ? -v : v;
        }
        case I32: { int32_t v; memcpy(&v, &bits, 4); return v; }
        case I64: { int64_t v; memcpy(&v, &bits, 8); return (double)v; }
        default: return (double)(int64_t)bits;
    }
}

static void plan_memory(Executable& exe);

// ---------------------------------------------------------------- validation
// Many programs convert every fp32 parameter to the 16-bit compute type where it is used: a
// launch per tensor, most of them tiny.  Converts that depend on nothing but an argument are
// moved to the front and run as one batched launch (mhip_convert_batch); the converted tensors
// then live for the whole execution.  Only from eight such converts on, and not at level 0.
static void hoist_parameter_converts(Executable& exe) {
    Function& fn = exe.fn;
    exe.batched_converts = 0;
    if (exe.opt_level < 1) return;
    std::vector<bool> is_arg(fn.num_values, false);
    for (int a : fn.arg_ids) is_arg[a] = true;
    std::vector<TensorType> arg_type(fn.num_values);
    for (size_t i = 0; i < fn.arg_ids.size(); i++) arg_type[fn.arg_ids[i]] = fn.arg_types[i];
    int dst = -1;
    std::vector<size_t> picked;
    for (size_t i = 0; i < fn.ops.size(); i++) {
        const Op& op = fn.ops[i];
        if (op.name != "convert" || op.operands.size() != 1 || !is_arg[op.operands[0]]) continue;
        if (arg_type[op.operands[0]].dtype != F32 || (op.out.dtype != BF16 && op.out.dtype != F16)) continue;
        if (arg_type[op.operands[0]].shape != op.out.shape) continue;
        if (dst < 0) dst = op.out.dtype;
        if (op.out.dtype != dst) continue;
        picked.push_back(i);
    }
    if (picked.size() < 8) return;
    std::vector<Op> front, rest;
    size_t k = 0;
    for (size_t i = 0; i < fn.ops.size(); i++) {
        if (k < picked.size() && picked[k] == i) { front.push_back(std::move(fn.ops[i])); k++; }
        else rest.push_back(std::move(fn.ops[i]));
    }
    exe.batched_converts = front.size();
    front.insert(front.end(), std::make_move_iterator(rest.begin()), std::make_move_iterator(rest.end()));
    fn.ops = std::move(front);
}

// [batch dims, lhs free dims, rhs free dims]: the shape dot / dot_general writes
static std::vector<int64_t> dot_result_shape(const Op& op, const TensorType& lt, const TensorType& rt) {
    std::vector<int64_t> lb = op.lhs_batch, rb = op.rhs_batch, lc = op.lhs_contract, rc = op.rhs_contract;
    if (op.name == "dot") { lc = {(int64_t)lt.shape.size() - 1}; rc = {0}; }
    auto in = [](const std::vector<int64_t>& v, int64_t d) { return std::find(v.begin(), v.end(), d) != v.end(); };
    std::vector<int64_t> shape;
    for (auto d : lb) shape.push_back(lt.shape.at(d));
    for (int64_t d = 0; d < (int64_t)lt.shape.size(); d++) if (!in(lb, d) && !in(lc, d)) shape.push_back(lt.shape[d]);
    for (int64_t d = 0; d < (int64_t)rt.shape.size(); d++) if (!in(rb, d) && !in(rc, d)) shape.push_back(rt.shape[d]);
    return shape;
}

// The fused kernels derive every extent from their operands and write a result of the operands'
// element type: a custom_call whose declared result (or an operand) says otherwise would be an
// out-of-bounds write or a misread buffer, so it is refused here, before anything runs.
static void check_custom_call_types(const Op& op, const std::vector<TensorType>& vt) {
    auto in = [&](size_t i) -> const TensorType& { return vt[op.operands.at(i)]; };
    const int dt = op.out.dtype;
    if (op.target == "fused_token_embedding") {
        // ids [B, S] i32, table [vocab, d] f32, positions [P, d] f32 -> [B, S, d]; token (b, s)
        // gets table[ids[b, s]] + positions[first_position + s]
        const TensorType &ids = in(0), &table = in(1), &pos = in(2);
        const int64_t p0 = parse_config(op.backend_config).get_int("first_position", 0);
        if (ids.dtype != I32 || ids.shape.size() != 2 || table.dtype != F32 || table.shape.size() != 2 || table.shape[0] < 1 ||
            pos.dtype != F32 || pos.shape.size() != 2 || pos.shape[1] != table.shape[1])
            throw ParseError(where(op) + "expected ids [B, S] i32, table [vocab, d] f32 and positions [P, d] f32");
        if (p0 < 0 || p0 + ids.shape[1] > pos.shape[0]) throw ParseError(where(op) + "positions outside their table");
        if (op.out.shape != std::vector<int64_t>{ids.shape[0], ids.shape[1], table.shape[1]})
            throw ParseError(where(op) + "the result shape is not [B, S, d]");
        return;
    }
    for (size_t i = 0; i < op.operands.size(); i++)
        if (in(i).dtype != dt) throw ParseError(where(op) + "every operand must have the result's element type");
    const Config cfg = parse_config(op.backend_config);
    const TensorType& xt = in(0);
    const int64_t cols = xt.shape.empty() ? 1 : xt.shape.back();
    if (op.target == "fused_rope") {
        // x [.., S, D], freqs [S, D] (cos | sin) or [S, D / 2] (angles), leading axes of extent 1 allowed
        // (CustomCallHandlers.swift:733-812); the third form there, separate cos and sin operands of
        // another width, is not served
        const TensorType& ft = in(1);
        if (xt.shape.size() < 2 || cols % 2 != 0 || !(xt == op.out)) throw ParseError(where(op) + "expected x [.., S, D] with even D and a result of x's type");
        const int64_t S = xt.shape[xt.shape.size() - 2], fd = ft.shape.empty() ? 0 : ft.shape.back();
        if ((fd != cols && fd != cols / 2) || ft.numel() != S * fd)
            throw UnsupportedOp(where(op) + "frequencies must be [S, D] (cos | sin) or [S, D / 2] (angles)");
        return;
    }
    if (op.target == "fused_batch_norm") {
        // x [.., C], gamma / beta / mean / variance with C elements each (CustomCallHandlers.swift:430-434)
        if (xt.shape.empty() || !(xt == op.out)) throw ParseError(where(op) + "expected x [.., C] and a result of x's type");
        for (size_t i = 1; i < 5; i++)
            if (in(i).numel() != cols) throw ParseError(where(op) + "gamma, beta, mean and variance must have one element per channel");
        return;
    }
    if (op.target == "fused_depth_attention") {
        // query [.., 1, H] or [.., H], keys and values [.., depth, H] (CustomCallHandlers.swift:1101-1103)
        const TensorType &kt = in(1), &vt2 = in(2);
        if (kt.shape.size() < 2 || !(kt == vt2) || !(xt == op.out)) throw ParseError(where(op) + "expected keys and values [.., depth, H] and a result of the query's type");
        std::vector<int64_t> lead(kt.shape.begin(), kt.shape.end() - 2), with_row = lead, without = lead;
        with_row.push_back(1); with_row.push_back(kt.shape.back());
        without.push_back(kt.shape.back());
        if (xt.shape != with_row && xt.shape != without) throw ParseError(where(op) + "the query must be [.., 1, H] or [.., H] over the keys' leading axes");
        const int64_t depth = kt.shape[kt.shape.size() - 2];
        if (depth < 1 || depth > 64) throw UnsupportedOp(where(op) + "1 to 64 key / value rows are served");
        return;
    }
    if (op.target == "fused_elementwise") {
        size_t need = 0;
        (void)chain_ops(op, cfg, &need);
        if (need > MHIP_CHAIN_MAX_INPUTS) throw UnsupportedOp(where(op) + "more than 8 inputs in one chain");
        if (op.operands.size() < need) throw ParseError(where(op) + "Not enough inputs for the operations of the chain");
        for (size_t i = 0; i < need; i++)
            if (in(i).numel() != op.out.numel() && in(i).numel() != 1)
                throw UnsupportedOp(where(op) + "every input must have the result's shape or one element");
        return;
    }
    if (op.target == "fused_softmax" || op.target == "fused_gelu" || op.target == "fused_layer_norm" || op.target == "fused_rms_norm") {
        if (!(xt == op.out)) throw ParseError(where(op) + "the result type must be the input's");
        if (op.target == "fused_layer_norm" || op.target == "fused_rms_norm") {
            if (in(1).numel() != cols) throw ParseError(where(op) + "gamma must be [cols] of the input type");
            if (op.target == "fused_layer_norm" && in(2).numel() != cols) throw ParseError(where(op) + "beta must be [cols] of the input type");
        }
    } else if (op.target == "fused_matmul_bias_activation") {
        const bool ta = cfg.get_bool("trans_a", false), tb = cfg.get_bool("trans_b", false);
        const TensorType& wt = in(1);
        if (wt.shape.size() != 2 || xt.shape.size() < 2 || (ta && xt.shape.size() != 2))
            throw ParseError(where(op) + "expected x [.., M, K] and w [K, N]");
        const int64_t K = ta ? xt.shape[0] : cols;
        const int64_t Kb = tb ? wt.shape[1] : wt.shape[0], N = tb ? wt.shape[0] : wt.shape[1];
        std::vector<int64_t> want = ta ? std::vector<int64_t>{xt.shape[1]} : std::vector<int64_t>(xt.shape.begin(), xt.shape.end() - 1);
        want.push_back(N);
        if (K != Kb) throw ParseError(where(op) + "operand shapes do not contract");
        if (op.out.shape != want) throw ParseError(where(op) + "the result shape is not [.., M, N]");
        const bool has_res = cfg.get_bool("has_residual", false);
        const size_t n_plain = op.operands.size() - (has_res ? 1 : 0);
        if (has_res && op.operands.size() < 3) throw ParseError(where(op) + "has_residual without a residual operand");
        if (n_plain > 2 && in(2).numel() != N) throw ParseError(where(op) + "bias must be [N] of the input type");
        if (has_res && !(in(op.operands.size() - 1) == op.out)) throw ParseError(where(op) + "the residual must have the result's type");
    } else if (op.target == "fused_ffn") {
        // x [.., M, d], up [d, F], down [F, d2] -> [.., M, d2]  (CustomCallHandlers.swift:861-882)
        const TensorType &up = in(1), &down = in(2);
        if (xt.shape.size() < 2 || up.shape.size() != 2 || down.shape.size() != 2 || up.shape[0] != cols || down.shape[0] != up.shape[1])
            throw ParseError(where(op) + "expected x [.., M, d], up [d, F] and down [F, d2]");
        std::vector<int64_t> want(xt.shape.begin(), xt.shape.end() - 1);
        want.push_back(down.shape[1]);
        if (op.out.shape != want) throw ParseError(where(op) + "the result shape is not [.., M, d2]");
        // "is_gated" is read and ignored, as the reference's handler does (CustomCallHandlers.swift:871)
    } else if (op.target == "fused_scaled_dot_product_attention" && cfg.get_int_array("views", {}).empty()) {
        const TensorType& kt = in(1);
        const size_t r = xt.shape.size();
        if (r < 2 || kt.shape.size() != r || !(in(2) == kt) || kt.shape[r - 1] != xt.shape[r - 1])
            throw ParseError(where(op) + "expected q [.., Sq, D] and k, v [.., Skv, D]");
        for (size_t d = 0; d + 2 < r; d++)
            if (kt.shape[d] != xt.shape[d]) throw ParseError(where(op) + "q and k differ in a batch / head dimension");
        if (!(xt == op.out)) throw ParseError(where(op) + "the result type must be q's");
    }
}

void compile(Executable& exe) {
    hoist_parameter_converts(exe);
    Function& fn = exe.fn;
    std::vector<TensorType> vt = value_types(fn);
    std::map<int, const Op*> producer;
    for (auto& op : fn.ops) producer[op.result] = &op;
    exe.constants.assign(fn.ops.size(), DeviceTensor());
    for (size_t oi = 0; oi < fn.ops.size(); oi++) {
        Op& op = fn.ops[oi];
        auto in = [&](size_t i) -> const TensorType& {
            if (i >= op.operands.size()) throw ParseError(where(op) + "expected at least " + std::to_string(i + 1) + " operands");
            return vt[op.operands[i]];
        };
        const std::string& n = op.name;
        if (n == "constant") {
            if (exe.client && exe.client->device >= 0) {
                DeviceTensor d = exe.client->allocate(op.out);
                // (the fill goes to the client's stream and the copy waits for it: neither while another
                // thread captures that stream)
                std::lock_guard<std::mutex> stream_lock(exe.client->stream_mu);
                if (op.splat) {
                    if (mhip_fill(exe.client->stream, d.data(), op.out.numel(), op.splat_bits, dtype_bytes(op.out.dtype)) != MHIP_OK)
                        throw ExecError(std::string("constant fill failed: ") + mhip_last_error());
                } else if (!op.constant.empty()) {
                    if (hipMemcpy(d.data(), op.constant.data(), op.constant.size(), hipMemcpyHostToDevice) != hipSuccess)
                        throw BufferError("constant upload failed");
                }
                exe.constants[oi] = d;
            }
        } else if (kUnary.count(n)) {
            if (!(in(0) == op.out)) throw ParseError(where(op) + "operand and result types differ");
            const bool is_int = op.out.dtype >= I8 && op.out.dtype <= UI64;
            const bool int_ok = (n == "negate" || n == "abs") && is_int;
            if (!is_kernel_float(op.out.dtype) && op.out.dtype != F64 && !int_ok) throw UnsupportedOp(where(op) + "element type not supported");
        } else if (kBinary.count(n)) {
            if (!(in(0) == op.out) || !(in(1) == op.out)) throw ParseError(where(op) + "operand and result types differ");
            if (op.out.dtype == I1 && (n == "divide" || n == "power")) throw UnsupportedOp(where(op) + "not defined on booleans");
        } else if (n == "convert") {
            if (in(0).shape != op.out.shape) throw ParseError(where(op) + "convert changes the shape");
            auto cv = [](int d) { return d >= F16 && d <= UI64; };   // every element type the parser knows
            if (!cv(in(0).dtype) || !cv(op.out.dtype)) throw UnsupportedOp(where(op) + "element type not supported");
        } else if (n == "reshape") {
            if (in(0).numel() != op.out.numel() || in(0).dtype != op.out.dtype) throw ParseError(where(op) + "reshape changes the element count or type");
        } else if (n == "transpose") {
            if (op.dims.size() != in(0).shape.size() || op.dims.size() > 8) throw ParseError(where(op) + "bad permutation");
            for (size_t d = 0; d < op.dims.size(); d++)
                if (op.dims[d] < 0 || op.dims[d] >= (int64_t)op.dims.size() || op.out.shape.at(d) != in(0).shape[op.dims[d]])
                    throw ParseError(where(op) + "permutation does not match the result shape");
        } else if (n == "broadcast_in_dim") {
            if (op.dims.size() != in(0).shape.size() || op.out.shape.size() > 8) throw ParseError(where(op) + "bad broadcast dims");
            for (size_t d = 0; d < op.dims.size(); d++) {
                if (op.dims[d] < 0 || op.dims[d] >= (int64_t)op.out.shape.size()) throw ParseError(where(op) + "broadcast dim out of range");
                const int64_t a = in(0).shape[d], b = op.out.shape[op.dims[d]];
                if (a != b && a != 1) throw ParseError(where(op) + "operand dim is neither 1 nor the result dim");
            }
        } else if (n == "slice") {
            const size_t r = in(0).shape.size();
            if (op.starts.size() != r || op.limits.size() != r || op.strides.size() != r || r > 8) throw ParseError(where(op) + "bad slice indices");
            for (size_t d = 0; d < r; d++) {
                if (op.strides[d] <= 0 || op.starts[d] < 0 || op.limits[d] > in(0).shape[d] || op.starts[d] > op.limits[d])
                    throw ParseError(where(op) + "slice range outside the operand");
                if ((op.limits[d] - op.starts[d] + op.strides[d] - 1) / op.strides[d] != op.out.shape.at(d))
                    throw ParseError(where(op) + "slice range does not match the result shape");
            }
        } else if (n == "reduce") {
            if (!kReduce.count(op.reducer)) throw UnsupportedOp(where(op) + "reducer body is not add / maximum / minimum / multiply");
            auto it = producer.find(op.operands.at(1));
            if (it == producer.end() || it->second->name != "constant") throw UnsupportedOp(where(op) + "init value must be a constant");
            if (!is_kernel_float(in(0).dtype) && in(0).dtype != I32 && in(0).dtype != I64) throw UnsupportedOp(where(op) + "element type not supported");
            for (auto d : op.dims) if (d < 0 || d >= (int64_t)in(0).shape.size()) throw ParseError(where(op) + "dimension out of range");
            // the kernel writes one element per kept position: the declared result must be exactly that
            std::vector<int64_t> kept;
            for (int64_t d = 0; d < (int64_t)in(0).shape.size(); d++)
                if (std::find(op.dims.begin(), op.dims.end(), d) == op.dims.end()) kept.push_back(in(0).shape[d]);
            if (op.out.shape != kept || op.out.dtype != in(0).dtype)
                throw ParseError(where(op) + "the result type is not the operand's without the reduced dimensions");
        } else if (n == "dot" || n == "dot_general") {
            // operands of one type; the result has that type, or a wider floating one (the
            // operands are then converted first and the product is taken in the result type)
            auto dot_type = [](int d) { return is_kernel_float(d) || d == F64 || d == I32 || d == I64; };
            const bool widen = is_kernel_float(in(0).dtype) && (op.out.dtype == F32 || op.out.dtype == F64) &&
                               dtype_bytes(op.out.dtype) > dtype_bytes(in(0).dtype);
            if (!dot_type(in(0).dtype) || in(0).dtype != in(1).dtype || (op.out.dtype != in(0).dtype && !widen))
                throw UnsupportedOp(where(op) + "dot needs f32 / f16 / bf16 / f64 / i32 / i64 operands of one type");
            (void)plan_dot(op, in(0), in(1));
            if (op.out.shape != dot_result_shape(op, in(0), in(1)))
                throw ParseError(where(op) + "the result shape is not [batch, lhs free, rhs free]");
        } else if (n == "iota") {
            if (op.iota_dim < 0 || op.iota_dim >= (int64_t)op.out.shape.size()) throw ParseError(where(op) + "iota dim out of range");
        } else if (n == "compare") {
            if (!(in(0) == in(1)) || op.out.dtype != I1 || op.out.shape != in(0).shape) throw ParseError(where(op) + "bad compare types");

        } else if (n == "select") {
            if (!(in(1) == op.out) || !(in(2) == op.out) || in(0).dtype != I1) throw ParseError(where(op) + "bad select types");
            if (in(0).numel() != 1 && in(0).shape != op.out.shape) throw ParseError(where(op) + "predicate shape mismatch");
        } else if (n == "gather") {
            (void)plan_gather(op, in(0), in(1));
        } else if (n == "custom_call") {
            bool ok = false;
            for (auto t : kTargets) ok |= op.target == t;
            if (!ok) throw UnsupportedOp(where(op) + "Unsupported custom call target: " + op.target);
            const size_t need = op.target == "fused_scaled_dot_product_attention" || op.target == "fused_layer_norm" || op.target == "fused_ffn" ||
                                        op.target == "fused_token_embedding" ? 3
                              : op.target == "fused_batch_norm" ? 5 : op.target == "fused_depth_attention" ? 3
                              : op.target == "fused_rms_norm" || op.target == "fused_matmul_bias_activation" || op.target == "fused_rope" ? 2 : 1;
            if (op.operands.size() < need)
                throw ParseError(where(op) + "Invalid input count: expected " + std::to_string(need) + ", got " + std::to_string(op.operands.size()));
            if (!is_kernel_float(op.target == "fused_token_embedding" ? op.out.dtype : in(0).dtype))
                throw UnsupportedOp(where(op) + "element type not supported");
            if (op.target == "fused_matmul_bias_activation" &&
                !kActivation.count(parse_config(op.backend_config).get_string("activation", "none")))
                throw UnsupportedOp(where(op) + "unknown activation");
            check_custom_call_types(op, vt);
        } else {
            throw UnsupportedOp(where(op) + "operation is outside the supported subset");
        }
    }
    if (exe.client && exe.client->device >= 0) {
        std::lock_guard<std::mutex> stream_lock(exe.client->stream_mu);     // another thread may be capturing the stream
        (void)hipStreamSynchronize(exe.client->stream);
    }
    plan_memory(exe);
}

// ---------------------------------------------------------------- execution
static void check(int st, const Op& op) {
    if (st != MHIP_OK) throw ExecError(where(op) + mhip_last_error());
}

static DeviceTensor permuted_copy(Allocator& al, bool dry, void* stream, const DeviceTensor& x,
                                  const std::vector<int64_t>& perm, const Op& op) {
    TensorType t;
    t.dtype = x.type.dtype;
    const auto st = dense_strides(x.type.shape);
    std::vector<int64_t> in_str;
    for (auto d : perm) { t.shape.push_back(x.type.shape[d]); in_str.push_back(st[d]); }
    DeviceTensor y = al.allocate(t);
    if (!dry)
        check(mhip_strided_copy(stream, x.data(), y.data(), (int)perm.size(), t.shape.data(), in_str.data(), 0,
                                dtype_bytes(t.dtype)), op);
    return y;
}

// One walk over the program in order: every allocation comes from `al`, every launch goes to
// the client's stream; with `dry` nothing is launched (the walk only shows `al` which
// allocations an execution makes and when each is released).  Returns the value of each result.
#define RUN(call) do { if (!dry) check((call), op); } while (0)
// `marks` (optional): one HIP event is recorded on the stream in front of the first launch and one
// behind every operation; marks[i].first = index of the operation the event closes (-1: the start).
static std::vector<DeviceTensor> run_ops(Executable& exe, const std::vector<DeviceTensor>& inputs, Allocator& al, bool dry,
                                         std::vector<std::pair<int, hipEvent_t>>* marks = nullptr, hipStream_t on_stream = nullptr) {
    const Function& fn = exe.fn;
    void* s = on_stream ? on_stream : (exe.client ? exe.client->stream : nullptr);
    auto mark = [&](int op_index) {
        if (!marks || dry) return;
        hipEvent_t e = nullptr;
        if (hipEventCreate(&e) != hipSuccess || hipEventRecord(e, static_cast<hipStream_t>(s)) != hipSuccess) {
            (void)hipGetLastError();
            if (e) (void)hipEventDestroy(e);
            return;
        }
        marks->emplace_back(op_index, e);
    };
    mark(-1);
    std::vector<DeviceTensor> val(fn.num_values);
    for (size_t i = 0; i < inputs.size(); i++) val[fn.arg_ids[i]] = inputs[i];
    // last use of every value, so that intermediates return to the pool early
    std::vector<int> last(fn.num_values, -1);
    for (size_t oi = 0; oi < fn.ops.size(); oi++) for (int v : fn.ops[oi].operands) last[v] = (int)oi;
    for (int r : fn.returns) last[r] = (int)fn.ops.size();
    std::map<int, const Op*> producer;
    for (auto& op : fn.ops) producer[op.result] = &op;

    if (exe.batched_converts) {            // the parameter converts at the head of the program, one launch
        std::vector<const void*> xs;
        std::vector<void*> ys;
        std::vector<int64_t> ns;
        for (size_t oi = 0; oi < exe.batched_converts; oi++) {
            const Op& op = fn.ops[oi];
            DeviceTensor out = al.allocate(op.out);
            xs.push_back(val[op.operands[0]].data());
            ys.push_back(out.data());
            ns.push_back(op.out.numel());
            val[op.result] = out;
        }
        const Op& op = fn.ops[0];
        RUN(mhip_convert_batch(s, (int)xs.size(), xs.data(), ys.data(), ns.data(), F32, op.out.dtype));
        mark((int)exe.batched_converts - 1);
    }
    for (size_t oi = exe.batched_converts; oi < fn.ops.size(); oi++) {
        const Op& op = fn.ops[oi];
        const std::string& n = op.name;
        auto in = [&](size_t i) -> const DeviceTensor& { return val[op.operands.at(i)]; };
        DeviceTensor out;
        if (n == "constant") {
            out = exe.constants[oi];
            out.type = op.out;
        } else if (n == "reshape") {
            out = in(0);
            out.type = op.out;
        } else {
            out = al.allocate(op.out);
            const int dt = op.out.dtype;
            const int64_t cnt = op.out.numel();
            if (kUnary.count(n)) {
                RUN(mhip_unary(s, kUnary.at(n), in(0).data(), out.data(), cnt, dt));
            } else if (kBinary.count(n)) {
                RUN(mhip_binary(s, kBinary.at(n), in(0).data(), in(1).data(), out.data(), cnt, dt));
            } else if (n == "convert") {
                if (in(0).type.dtype == dt) RUN(mhip_copy(s, in(0).data(), out.data(), (int64_t)op.out.bytes()));
                else RUN(mhip_convert(s, in(0).data(), out.data(), cnt, in(0).type.dtype, dt));
            } else if (n == "transpose") {
                const auto st = dense_strides(in(0).type.shape);
                std::vector<int64_t> is;
                for (auto d : op.dims) is.push_back(st[d]);
                RUN(mhip_strided_copy(s, in(0).data(), out.data(), (int)op.dims.size(), op.out.shape.data(), is.data(), 0,
                                        dtype_bytes(dt)));
            } else if (n == "broadcast_in_dim") {
                const auto st = dense_strides(in(0).type.shape);
                std::vector<int64_t> is(op.out.shape.size(), 0);
                for (size_t d = 0; d < op.dims.size(); d++)
                    is[op.dims[d]] = in(0).type.shape[d] == 1 ? 0 : st[d];
                RUN(mhip_strided_copy(s, in(0).data(), out.data(), (int)op.out.shape.size(), op.out.shape.data(), is.data(),
                                        0, dtype_bytes(dt)));
            } else if (n == "slice") {
                const auto st = dense_strides(in(0).type.shape);
                std::vector<int64_t> is;
                int64_t off = 0;
                for (size_t d = 0; d < st.size(); d++) { is.push_back(st[d] * op.strides[d]); off += st[d] * op.starts[d]; }
                RUN(mhip_strided_copy(s, in(0).data(), out.data(), (int)st.size(), op.out.shape.data(), is.data(), off,
                                        dtype_bytes(dt)));
            } else if (n == "reduce") {
                const double init = scalar_constant(*producer.at(op.operands.at(1)));
                int64_t outer, len, inner;
                DeviceTensor x = in(0);
                if (!reduce_block(x.type.shape, op.dims, outer, len, inner)) {
                    // move the reduced dims to the end, then reduce the trailing block
                    std::vector<int64_t> perm, red = op.dims;
                    std::sort(red.begin(), red.end());
                    for (int64_t d = 0; d < (int64_t)x.type.shape.size(); d++)
                        if (std::find(red.begin(), red.end(), d) == red.end()) perm.push_back(d);
                    const size_t kept = perm.size();
                    perm.insert(perm.end(), red.begin(), red.end());
                    x = permuted_copy(al, dry, s, x, perm, op);
                    outer = len = 1;
                    inner = 1;
                    for (size_t d = 0; d < perm.size(); d++) (d < kept ? outer : len) *= x.type.shape[d];
                }
                RUN(mhip_reduce(s, kReduce.at(op.reducer), x.data(), out.data(), outer, len, inner, init, dt));
            } else if (n == "dot" || n == "dot_general") {
                DotPlan p = plan_dot(op, in(0).type, in(1).type);
                DeviceTensor a = in(0), b = in(1);
                if (a.type.dtype != dt) {    // result wider than the operands: convert, then multiply in the result type
                    DeviceTensor a2 = al.allocate(TensorType{a.type.shape, dt}), b2 = al.allocate(TensorType{b.type.shape, dt});
                    RUN(mhip_convert(s, a.data(), a2.data(), a.type.numel(), a.type.dtype, dt));
                    RUN(mhip_convert(s, b.data(), b2.data(), b.type.numel(), b.type.dtype, dt));
                    a = a2; b = b2;
                }
                if (p.lhs_copy) a = permuted_copy(al, dry, s, a, p.lhs_perm, op);
                if (p.rhs_copy) b = permuted_copy(al, dry, s, b, p.rhs_perm, op);
                RUN(mhip_gemm(s, a.data(), b.data(), nullptr, out.data(), p.M, p.N, p.K, p.B, p.M * p.K, p.K * p.N,
                                p.M * p.N, p.trans_a, p.trans_b, MHIP_ACT_NONE, dt));
            } else if (n == "iota") {
                int64_t outer = 1, inner = 1;
                for (int64_t d = 0; d < (int64_t)op.out.shape.size(); d++) {
                    if (d < op.iota_dim) outer *= op.out.shape[d];
                    else if (d > op.iota_dim) inner *= op.out.shape[d];
                }
                RUN(mhip_iota(s, out.data(), outer, op.out.shape[op.iota_dim], inner, dt));
            } else if (n == "compare") {
                RUN(mhip_compare(s, kCompare.at(op.direction), in(0).data(), in(1).data(), out.data(), cnt, in(0).type.dtype));
            } else if (n == "select") {
                RUN(mhip_select(s, in(0).data(), in(1).data(), in(2).data(), out.data(), cnt, dtype_bytes(dt),
                                  in(0).type.numel() == 1 && cnt != 1));
            } else if (n == "gather") {
                const GatherPlan p = plan_gather(op, in(0).type, in(1).type);
                if (p.whole_rows)
                    RUN(mhip_gather_rows(s, in(0).data(), in(1).data(), out.data(), in(1).type.numel(), in(0).type.shape[0],
                                           in(0).type.shape[1], in(0).type.dtype, in(1).type.dtype));
                else
                    RUN(mhip_gather(s, in(0).data(), in(1).data(), out.data(), (int)op.out.shape.size(), op.out.shape.data(),
                                      p.out_op_stride.data(), p.out_idx_stride.data(), (int)p.comp_max.size(), p.comp_stride,
                                      p.comp_op_stride.data(), p.comp_max.data(), dtype_bytes(dt), in(1).type.dtype));
            } else if (n == "custom_call") {
                const Config cfg = parse_config(op.backend_config);
                const TensorType& xt = in(0).type;
                const int64_t cols = xt.shape.empty() ? 1 : xt.shape.back();
                const int64_t rows = cols ? xt.numel() / cols : 0;
                if (op.target == "fused_token_embedding") {
                    const TensorType &ids = in(0).type, &table = in(1).type;
                    const int64_t d = table.shape[1], p0 = cfg.get_int("first_position", 0);
                    RUN(mhip_embed_tokens(s, in(0).data(), in(1).data(), static_cast<const float*>(in(2).data()) + p0 * d, out.data(),
                                          ids.shape[0], ids.shape[1], d, table.shape[0], MHIP_F32, dt));
                } else if (op.target == "fused_rope") {
                    const int64_t S = xt.shape[xt.shape.size() - 2], fd = in(1).type.shape.back();
                    RUN(mhip_rope(s, in(0).data(), in(1).data(), out.data(), rows, S, cols, fd == cols / 2 ? 1 : 0, dt));
                } else if (op.target == "fused_batch_norm") {
                    RUN(mhip_batch_norm(s, in(0).data(), in(1).data(), in(2).data(), in(3).data(), in(4).data(), out.data(), rows, cols,
                                        (float)cfg.get_float("eps", 1e-5), dt));
                } else if (op.target == "fused_depth_attention") {
                    const TensorType& kt = in(1).type;
                    RUN(mhip_depth_attention(s, in(0).data(), in(1).data(), in(2).data(), out.data(), rows, kt.shape[kt.shape.size() - 2],
                                             cols, (float)cfg.get_float("scale", 1.0), dt));
                } else if (op.target == "fused_elementwise") {
                    size_t need = 0;
                    const std::vector<int> codes = chain_ops(op, cfg, &need);
                    std::vector<const void*> ptrs;
                    std::vector<int64_t> counts;
                    for (size_t i = 0; i < need; i++) { ptrs.push_back(in(i).data()); counts.push_back(in(i).type.numel()); }
                    RUN(mhip_elementwise_chain(s, (int)need, ptrs.data(), counts.data(), (int)codes.size(), codes.data(), out.data(), cnt, dt));
                } else if (op.target == "fused_softmax") {
                    int64_t axis = cfg.get_int("axis", -1);
                    if (axis < 0) axis += (int64_t)xt.shape.size();
                    if (axis < 0 || axis >= (int64_t)xt.shape.size()) throw ExecError(where(op) + "softmax axis out of range");
                    int64_t outer = 1, inner = 1;
                    outer = inner = 1;
                    for (int64_t d = 0; d < axis; d++) outer *= xt.shape[d];
                    for (int64_t d = axis + 1; d < (int64_t)xt.shape.size(); d++) inner *= xt.shape[d];
                    RUN(mhip_softmax_strided(s, in(0).data(), out.data(), outer, xt.shape[axis], inner, dt));
                } else if (op.target == "fused_gelu") {
                    // "approximate": false alone means the tanh form too, as in the reference
                    // (CustomCallHandlers.swift:694-707); the recogniser marks a decomposed erf GELU
                    // with "erf": true, which runs the exact form
                    if (cfg.get_bool("erf", false)) RUN(mhip_bias_gelu_erf(s, in(0).data(), nullptr, out.data(), rows, cols, dt));
                    else RUN(mhip_bias_gelu(s, in(0).data(), nullptr, out.data(), rows, cols, dt));
                } else if (op.target == "fused_ffn") {
                    // act(x . up) . down: two GEMMs, the hidden activations in a temporary
                    const TensorType &up = in(1).type, &down = in(2).type;
                    const int64_t F = up.shape[1], d2 = down.shape[1];
                    DeviceTensor hidden = al.allocate(TensorType{{rows, F}, dt});
                    // an activation name the handler does not know means no activation (CustomCallHandlers.swift:905)
                    const std::string act_name = cfg.get_string("activation", "gelu");
                    RUN(mhip_gemm(s, in(0).data(), in(1).data(), nullptr, hidden.data(), rows, F, cols, 1, 0, 0, 0, 0, 0,
                                  kActivation.count(act_name) ? kActivation.at(act_name) : MHIP_ACT_NONE, dt));
                    RUN(mhip_gemm(s, hidden.data(), in(2).data(), nullptr, out.data(), rows, d2, F, 1, 0, 0, 0, 0, 0, MHIP_ACT_NONE, dt));
                } else if (op.target == "fused_layer_norm" || op.target == "fused_rms_norm") {
                    const auto axes = cfg.get_int_array("axes", {-1});
                    if (axes.size() != 1 || (axes[0] != -1 && axes[0] != (int64_t)xt.shape.size() - 1))
                        throw ExecError(where(op) + "only normalisation over the last axis is supported");
                    const float eps = (float)cfg.get_float("eps", 1e-5);
                    if (in(1).type.numel() != cols || in(1).type.dtype != dt) throw ExecError(where(op) + "gamma must be [cols] of the input type");
                    if (op.target == "fused_layer_norm") {
                        if (in(2).type.numel() != cols || in(2).type.dtype != dt) throw ExecError(where(op) + "beta must be [cols] of the input type");
                        RUN(mhip_layer_norm(s, in(0).data(), in(1).data(), in(2).data(), out.data(), rows, cols, eps, dt));
                    } else {
                        RUN(mhip_rms_norm(s, in(0).data(), in(1).data(), out.data(), rows, cols, eps, dt));
                    }
                } else if (op.target == "fused_matmul_bias_activation") {
                    const bool ta = cfg.get_bool("trans_a", false), tb = cfg.get_bool("trans_b", false);
                    const TensorType& wt = in(1).type;
                    if (wt.shape.size() != 2 || xt.shape.size() < 2 || (ta && xt.shape.size() != 2))
                        throw ExecError(where(op) + "expected x [.., M, K] and w [K, N]");
                    const int64_t K = ta ? xt.shape[0] : cols, M = ta ? xt.shape[1] : rows;
                    const int64_t Kb = tb ? wt.shape[1] : wt.shape[0], N = tb ? wt.shape[0] : wt.shape[1];
                    if (K != Kb || op.out.numel() != M * N) throw ExecError(where(op) + "operand shapes do not contract");
                    // operands: x, w, [bias], [residual, when the config says "has_residual"]
                    const bool has_res = cfg.get_bool("has_residual", false);
                    const size_t n_plain = op.operands.size() - (has_res ? 1 : 0);
                    if (has_res && op.operands.size() < 3) throw ExecError(where(op) + "has_residual without a residual operand");
                    const void* bias = n_plain > 2 ? in(2).data() : nullptr;
                    if (bias && (in(2).type.numel() != N || in(2).type.dtype != dt)) throw ExecError(where(op) + "bias must be [N] of the input type");
                    const DeviceTensor* res = has_res ? &in(op.operands.size() - 1) : nullptr;
                    if (res && !(res->type == op.out)) throw ExecError(where(op) + "the residual must have the result's type");
                    RUN(mhip_gemm_residual(s, in(0).data(), in(1).data(), bias, res ? res->data() : nullptr, out.data(), M, N, K, 1, 0, 0, 0,
                                           ta, tb, kActivation.at(cfg.get_string("activation", "none")), dt));
                } else if (!cfg.get_int_array("views", {}).empty()) {   // attention reading / writing views in place
                    const auto dims = cfg.get_int_array("dims", {});
                    const auto vw = cfg.get_int_array("views", {});
                    if (dims.size() != 5 || vw.size() != 16) throw ExecError(where(op) + "views need dims [B,H,Sq,Skv,D] and 16 view entries");
                    const int64_t B = dims[0], H = dims[1], Sq = dims[2], Skv = dims[3], D = dims[4];
                    const int64_t es = dtype_bytes(dt);
                    // every view must stay inside the tensor it is a window of
                    const int64_t rows[4] = {Sq, Skv, Skv, Sq};
                    const int64_t have[4] = {in(0).type.numel(), in(1).type.numel(), in(2).type.numel(), op.out.numel()};
                    int64_t strides[12];
                    for (int t = 0; t < 4; t++) {
                        const int64_t off = vw[4 * t], sb = vw[4 * t + 1], sh = vw[4 * t + 2], sr = vw[4 * t + 3];
                        if (off < 0 || sb < 0 || sh < 0 || sr < D ||
                            off + (B - 1) * sb + (H - 1) * sh + (rows[t] - 1) * sr + D > have[t])
                            throw ExecError(where(op) + "a view reaches outside its tensor");
                        strides[3 * t] = sb; strides[3 * t + 1] = sh; strides[3 * t + 2] = sr;
                    }
                    if (in(0).type.dtype != dt || in(1).type.dtype != dt || in(2).type.dtype != dt)
                        throw ExecError(where(op) + "q, k, v and the result must have one element type");
                    const bool has_mask = cfg.get_bool("has_mask", false) && op.operands.size() > 3;
                    const void* mask = nullptr;
                    int64_t msb = 0, msh = 0;
                    if (has_mask) {
                        const TensorType& mt = in(3).type;
                        const size_t mr = mt.shape.size();
                        if (mr < 2 || mt.shape[mr - 1] != Skv || mt.shape[mr - 2] != Sq || mt.dtype != dt)
                            throw ExecError(where(op) + "mask must end in [Sq, Skv] and have the input type");
                        const int64_t mh = mr >= 3 ? mt.shape[mr - 3] : 1;
                        int64_t mb = 1;
                        for (size_t d = 0; d + 3 < mr; d++) mb *= mt.shape[d];
                        if ((mh != 1 && mh != H) || (mb != 1 && mb != B)) throw ExecError(where(op) + "mask does not broadcast to [B, H, Sq, Skv]");
                        msh = mh == H && H != 1 ? Sq * Skv : 0;
                        msb = mb == B && B != 1 ? mh * Sq * Skv : 0;
                        mask = in(3).data();
                    }
                    auto at = [&](const void* p, int64_t off) { return static_cast<const char*>(p) + off * es; };
                    RUN(mhip_flash_attention_strided(s, at(in(0).data(), vw[0]), at(in(1).data(), vw[4]), at(in(2).data(), vw[8]), mask,
                                                     const_cast<char*>(at(out.data(), vw[12])), B, H, Sq, Skv, D,
                                                     (float)cfg.get_float("scale", 1.0), cfg.get_bool("is_causal", false), msb, msh, dt,
                                                     strides));
                } else {   // fused_scaled_dot_product_attention
                    const TensorType& kt = in(1).type;
                    if (xt.shape.size() < 2 || kt.shape.size() != xt.shape.size() || !(in(2).type == kt) || kt.dtype != dt)
                        throw ExecError(where(op) + "expected q [.., Sq, D] and k, v [.., Skv, D]");
                    const size_t r = xt.shape.size();
                    const int64_t D = xt.shape[r - 1], Sq = xt.shape[r - 2], Skv = kt.shape[r - 2];
                    const int64_t H = r >= 3 ? xt.shape[r - 3] : 1;
                    int64_t B = 1;
                    for (size_t d = 0; d + 3 < r; d++) B *= xt.shape[d];
                    const float scale = (float)cfg.get_float("scale", 1.0);
                    const bool has_mask = cfg.get_bool("has_mask", false) && op.operands.size() > 3;
                    const void* mask = nullptr;
                    int64_t msb = 0, msh = 0;
                    if (has_mask) {
                        const TensorType& mt = in(3).type;
                        const size_t mr = mt.shape.size();
                        if (mr < 2 || mt.shape[mr - 1] != Skv || mt.shape[mr - 2] != Sq || mt.dtype != dt)
                            throw ExecError(where(op) + "mask must end in [Sq, Skv] and have the input type");
                        const int64_t mh = mr >= 3 ? mt.shape[mr - 3] : 1;
                        int64_t mb = 1;
                        for (size_t d = 0; d + 3 < mr; d++) mb *= mt.shape[d];
                        if ((mh != 1 && mh != H) || (mb != 1 && mb != B)) throw ExecError(where(op) + "mask does not broadcast to [B, H, Sq, Skv]");
                        msh = mh == H && H != 1 ? Sq * Skv : 0;
                        msb = mb == B && B != 1 ? mh * Sq * Skv : 0;
                        mask = in(3).data();
                    }
                    RUN(mhip_flash_attention(s, in(0).data(), in(1).data(), in(2).data(), mask, out.data(), B, H, Sq, Skv, D,
                                               scale, cfg.get_bool("is_causal", false), msb, msh, dt));
                }
            }
        }
        val[op.result] = out;
        if (n != "constant" && n != "reshape") mark((int)oi);
        for (int v : op.operands)
            if (last[v] == (int)oi) val[v] = DeviceTensor();
    }
    std::vector<DeviceTensor> rets;
    for (int r : fn.returns) rets.push_back(val[r]);
    return rets;
}
#undef RUN

static bool env_flag(const char* name, bool dflt) {
    const char* v = getenv(name);
    return v && *v ? atoi(v) != 0 : dflt;
}

static void plan_memory(Executable& exe) {
    exe.plan = ArenaPlan();
    try {
        Allocator al;
        al.mode = Allocator::RECORD;
        al.plan = &exe.plan;
        std::vector<DeviceTensor> ins;
        for (auto& t : exe.fn.arg_types) { DeviceTensor d; d.type = t; ins.push_back(d); }
        {
            const std::vector<DeviceTensor> rets = run_ops(exe, ins, al, true);
            for (auto& r : rets) if (r.mem && r.mem->recorder) exe.plan.slots[r.mem->slot].escapes = true;
        }
        for (auto& sl : exe.plan.slots) {
            if (sl.escapes) sl.end = 0x7FFFFFFF;
            else exe.plan.sum_bytes += sl.bytes;
        }
        // Both placements are made; the one by recency is kept unless it needs over a quarter more
        // bytes than the packed one (METALHLO_ARENA_PLACEMENT=packed keeps the packed one regardless).
        // GPT-2-small forward, B8 S1024: 361 MB against 319 MB, and 0.02-0.03 ms of 3.5 ms faster.
        const char* how = getenv("METALHLO_ARENA_PLACEMENT");
        const size_t packed = place_slots(exe.plan, false, 0);
        exe.plan.core_bytes = packed;
        if (!how || strcmp(how, "packed")) {
            const std::vector<ArenaPlan::Slot> keep = exe.plan.slots;
            const size_t recent = place_slots_recent(exe.plan, false, 0);
            if (recent <= packed + packed / 4) exe.plan.core_bytes = recent;
            else exe.plan.slots = keep;
        }
        exe.plan.full_bytes = place_slots(exe.plan, true, exe.plan.core_bytes);
        exe.plan.valid = true;
    } catch (const std::exception&) {
        exe.plan = ArenaPlan();     // the execution reports the problem; it allocates per value
    }
}

static void ensure_arena(Executable& exe, size_t bytes) {
    bytes = std::max<size_t>(bytes, 256);
    if (exe.arena && exe.arena_size >= bytes) return;
    Client& c = *exe.client;
    (void)hipStreamSynchronize(c.stream);
    for (auto& g : exe.graphs) if (g.exec) (void)hipGraphExecDestroy(g.exec);     // they hold addresses of the old arena
    exe.graphs.clear();
    if (exe.arena) (void)hipFree(exe.arena);
    exe.arena = nullptr;
    exe.arena_size = 0;
    if (hipMalloc(&exe.arena, bytes) != hipSuccess) {
        (void)hipGetLastError();
        exe.arena = nullptr;
        throw BufferError("hipMalloc of the " + std::to_string(bytes) + "-byte arena failed");
    }
    exe.arena_size = bytes;
}

// Captures one walk over the program (every value, results included, at its arena address) into
// a graph.  False when the capture or the instantiation fails; the stream is usable again then.
// True when every returned value is an allocation of its own (no input, constant or alias among the
// results, none returned twice): the results of a captured graph can then live in buffers of their own.
static bool direct_results(const Executable& exe) {
    size_t escaping = 0;
    for (auto& sl : exe.plan.slots) escaping += sl.escapes;
    return escaping == exe.fn.returns.size();
}

static bool capture_graph(Executable& exe, const std::vector<DeviceTensor>& inputs, Executable::CapturedGraph& out) {
    Client& c = *exe.client;
    // storage of the results, allocated before the capture begins (nothing may allocate inside it)
    std::vector<std::shared_ptr<DeviceMem>> presets;
    const bool direct = direct_results(exe);
    if (direct) {
        presets.resize(exe.plan.slots.size());
        for (size_t i = 0; i < exe.plan.slots.size(); i++) {
            if (!exe.plan.slots[i].escapes) continue;
            auto m = std::make_shared<DeviceMem>();
            m->bytes = exe.plan.slots[i].bytes;             // the slot's size (the value's, rounded up to 256)
            m->pool = &c.pool;
            m->ptr = c.pool.alloc(m->bytes);
            m->replay_result = true;
            presets[i] = m;
        }
    }
    // The capture runs on the client's capture stream (see Client), in relaxed mode: nothing inside the
    // capture allocates or synchronises (the replay tests hold every kernel wrapper to that), and
    // what other threads call meanwhile -- the pool's hipMalloc, the transfer engine's pinned blocks
    // and event waits -- cannot invalidate it.  The caller (execute) holds c.stream_mu.
    if (c.capture_broken) return false;
    if (!c.capture_stream && hipStreamCreateWithFlags(&c.capture_stream, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        c.capture_stream = nullptr;
        return false;
    }
    if (hipStreamBeginCapture(c.capture_stream, hipStreamCaptureModeRelaxed) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    Allocator al;
    al.mode = Allocator::ARENA;
    al.client = &c;
    al.plan = &exe.plan;
    al.base = static_cast<char*>(exe.arena);
    al.escaping_in_arena = !direct;
    if (direct) al.presets = &presets;
    std::vector<DeviceTensor> rets;
    bool ok = true;
    std::string why;
    try { rets = run_ops(exe, inputs, al, false, nullptr, c.capture_stream); } catch (const std::exception& x) { ok = false; why = x.what(); }
    hipGraph_t g = nullptr;
    const hipError_t e = hipStreamEndCapture(c.capture_stream, &g);
    if (e != hipSuccess || !ok) {
        (void)hipGetLastError();
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        const hipError_t q = hipStreamIsCapturing(c.capture_stream, &st);
        (void)hipGetLastError();
        // a failed capture can leave its stream in the capturing state for good (seen with an
        // invalidated capture); nothing more is captured on this client then
        if (q != hipSuccess || st != hipStreamCaptureStatusNone) c.capture_broken = true;
        if (getenv("METALHLO_DEBUG_GRAPH"))
            fprintf(stderr, "[metalhlo] graph capture failed: launches: %s; end of capture: %s; stream capture status afterwards: %d (%s)\n",
                    ok ? "ok" : why.c_str(), hipGetErrorString(e), (int)st, hipGetErrorString(q));
    }
    hipGraphExec_t ex = nullptr;
    if (ok && e == hipSuccess && g && hipGraphInstantiate(&ex, g, nullptr, nullptr, 0) != hipSuccess) ex = nullptr;
    if (g) (void)hipGraphDestroy(g);
    if (!ex) {
        (void)hipGetLastError();
        return false;
    }
    out.exec = ex;
    out.inputs.clear();
    for (auto& t : inputs) out.inputs.push_back(t.data());
    out.returns.clear();
    out.results.clear();
    if (direct) {
        for (auto& r : rets) {
            if (!r.mem || !r.mem->replay_result) {          // not what the plan promised: keep this program eager
                (void)hipGraphExecDestroy(ex);
                return false;
            }
            out.results.push_back(r);
        }
    } else {
        for (auto& r : rets) out.returns.emplace_back(r.data(), r.type);
    }
    return true;
}

std::vector<DeviceTensor> execute(Executable& exe, const std::vector<DeviceTensor>& inputs, double* encode_s,
                                  double* gpu_s) {
    Client& c = *exe.client;
    if (c.device < 0) throw NoDevice("no HIP device: cannot execute");
    const Function& fn = exe.fn;
    if (inputs.size() != fn.arg_types.size())
        throw InputMismatch("Expected " + std::to_string(fn.arg_types.size()) + " inputs, got " + std::to_string(inputs.size()));
    for (size_t i = 0; i < inputs.size(); i++)
        if (!(inputs[i].type == fn.arg_types[i]))
            throw InputMismatch("Input " + std::to_string(i) + " has the wrong shape or element type");
    const bool use_arena = exe.plan.valid && env_flag("METALHLO_ARENA", true);
    // a replay costs one graph launch plus the copies of the results out of the arena: it pays
    // from roughly twenty launches per execution on, so short programs stay eager by default
    size_t launches = 0;
    for (auto& op : fn.ops) launches += op.name != "constant" && op.name != "reshape";
    const bool profile_env = env_flag("METALHLO_PROFILE_GPU", false);
    const bool profile = profile_env || exe.profile_next;          // a profiled execution is eager: events between the launches
    exe.profile_next = false;
    const bool want_graph = !profile && use_arena && env_flag("METALHLO_HIP_GRAPH", exe.opt_level >= 3 && launches >= 16);
    std::vector<std::pair<int, hipEvent_t>> marks;
    std::unique_lock<std::mutex> run_lock(exe.run_mu, std::defer_lock);
    if (use_arena) run_lock.lock();          // the arena belongs to one execution at a time
    const auto t0 = std::chrono::steady_clock::now();
    std::vector<DeviceTensor> rets;
    bool replayed = false;
    // Every call that touches the client's stream happens under its lock, from here to the end of the
    // copy-out: the synchronisation in front of a new arena, eager launches, the capture, graph
    // launches and the synchronisations.  Another thread that executes another program on this
    // client (or a PJRT transfer) can then never launch into, or wait for, a stream that is being
    // captured, where its work would be recorded into the graph instead of run.
    std::unique_lock<std::mutex> stream_lock(c.stream_mu);
    if (use_arena) ensure_arena(exe, want_graph && !direct_results(exe) ? exe.plan.full_bytes : exe.plan.core_bytes);
    // the first execution runs eagerly (kernels set their attributes, tuning tables load); from the
    // second on the op list is one graph per set of input addresses
    if (want_graph && !exe.graph_failed && exe.eager_runs > 0) {
        // A graph with result buffers of its own can run again only when the caller has released
        // what its previous replay handed out.  A caller that still holds the results of step n when
        // it starts step n + 1 (the usual pattern of a training or serving loop) gets a second and a
        // third graph for the same inputs, each with its own result buffers, and the replays rotate
        // over whichever is free; with all of them held this execution is eager.
        constexpr size_t kResultSets = 3;
        Executable::CapturedGraph* hit = nullptr;
        size_t same_inputs = 0;
        for (auto& g : exe.graphs) {
            bool same = g.inputs.size() == inputs.size();
            for (size_t i = 0; same && i < inputs.size(); i++) same = g.inputs[i] == inputs[i].data();
            if (!same) continue;
            same_inputs++;
            bool busy = false;
            for (auto& r : g.results) busy = busy || r.mem.use_count() > 1;
            if (!busy) { hit = &g; break; }
        }
        if (!hit && same_inputs < kResultSets) {
            Executable::CapturedGraph g;
            if (capture_graph(exe, inputs, g)) {
                if (exe.graphs.size() >= 8) {
                    // the oldest graph whose results the caller does not hold makes room
                    size_t victim = exe.graphs.size();
                    for (size_t i = 0; i < exe.graphs.size() && victim == exe.graphs.size(); i++) {
                        bool busy = false;
                        for (auto& r : exe.graphs[i].results) busy = busy || r.mem.use_count() > 1;
                        if (!busy) victim = i;
                    }
                    if (victim == exe.graphs.size()) victim = 0;
                    (void)hipStreamSynchronize(c.stream);
                    (void)hipGraphExecDestroy(exe.graphs[victim].exec);
                    exe.graphs.erase(exe.graphs.begin() + victim);
                }
                exe.graphs.push_back(std::move(g));
                hit = &exe.graphs.back();
                exe.graph_captures++;
            } else if (same_inputs == 0) {
                exe.graph_failed = true;     // this program stays on eager launches
            }
        }
        if (hit) {
            if (hipGraphLaunch(hit->exec, c.stream) != hipSuccess) {
                const hipError_t e = hipGetLastError();
                throw ExecError(std::string("graph launch failed: ") + hipGetErrorString(e));
            }
            exe.graph_replays++;
            for (auto& r : hit->results) rets.push_back(r);
            for (auto& r : hit->returns) {
                DeviceTensor t;
                t.type = r.second;
                t.mem = std::make_shared<DeviceMem>();
                t.mem->ptr = const_cast<void*>(r.first);      // not owned: copied out below
                t.mem->bytes = r.second.bytes();
                rets.push_back(t);
            }
            replayed = true;
        }
    }
    if (!replayed) {
        Allocator al;
        al.client = &c;
        if (use_arena) {
            al.mode = Allocator::ARENA;
            al.plan = &exe.plan;
            al.base = static_cast<char*>(exe.arena);
            al.escaping_in_arena = false;
        }
        rets = run_ops(exe, inputs, al, false, profile ? &marks : nullptr);
        exe.eager_runs++;
    }
    const auto t1 = std::chrono::steady_clock::now();
    if (hipStreamSynchronize(c.stream) != hipSuccess) {
        const hipError_t e = hipGetLastError();
        throw ExecError(std::string("execution failed: ") + hipGetErrorString(e));
    }
    const auto t2 = std::chrono::steady_clock::now();
    if (profile) {
        exe.last_profile.clear();
        for (size_t i = 1; i < marks.size(); i++) {
            float ms = 0.f;
            if (hipEventElapsedTime(&ms, marks[i - 1].second, marks[i].second) != hipSuccess) { (void)hipGetLastError(); continue; }
            const Op& op = fn.ops[marks[i].first];
            Executable::OpTime t;
            const bool batch = exe.batched_converts && marks[i].first == (int)exe.batched_converts - 1;
            t.name = batch ? "convert x" + std::to_string(exe.batched_converts) : (op.name == "custom_call" ? op.target : op.name);
            for (size_t d = 0; d < op.out.shape.size(); d++) t.shape += (d ? "x" : "") + std::to_string(op.out.shape[d]);
            t.shape += (t.shape.empty() ? "" : "x") + std::string(dtype_name(op.out.dtype));
            t.us = ms * 1e3;
            if (profile_env) fprintf(stderr, "[metalhlo gpu] %3zu %-36s %-24s %9.1f us\n", i - 1, t.name.c_str(), t.shape.c_str(), t.us);
            exe.last_profile.push_back(std::move(t));
        }
        for (auto& m : marks) (void)hipEventDestroy(m.second);
    }
    if (encode_s) *encode_s = std::chrono::duration<double>(t1 - t0).count();
    if (gpu_s) *gpu_s = std::chrono::duration<double>(t2 - t0).count();
    std::vector<DeviceTensor> outs;
    for (size_t i = 0; i < rets.size(); i++) {
        DeviceTensor o = std::move(rets[i]);
        rets[i] = DeviceTensor();
        if (!o.mem) throw ExecError("a returned value was never produced");
        // an output must own its storage: inputs, constants, aliases, repeated results and
        // values that lie in the arena are copied out
        const bool shared = !o.mem->replay_result && (o.mem.use_count() > 1 || !o.mem->pool);
        if (shared) {
            DeviceTensor cpy = c.allocate(o.type);
            if (mhip_copy(c.stream, o.data(), cpy.data(), (int64_t)o.type.bytes()) != MHIP_OK) throw ExecError(mhip_last_error());
            (void)hipStreamSynchronize(c.stream);
            o = cpy;
        }
        outs.push_back(o);
    }
    return outs;
}

}  // namespace mhlo
