// Pattern recogniser: rewrites decomposed StableHLO subgraphs into the fused
// custom_calls the kernels serve -- the job of the reference's SoftmaxPattern /
// GELUPattern / LayerNormPattern / RMSNormPattern / AttentionPattern
// (Sources/MetalHLOCore/Optimizer/FusionPatterns.swift:18-1142) and of its
// MatMulBiasActFusionPass (Compiler/PassManager.swift:1436-1570).
//
// A match is only rewritten when every interior value is used inside the pattern
// alone (the reference's rule, Analyzer.swift:1715-1721): that is what makes the
// rewrite semantics-preserving.  Matching is structural and strict: constants
// must have the right values, reductions the right axis and neutral element, and
// commutative operands are accepted in either order.  Forms the kernels would
// answer differently (erf GELU, attention with dropout, ...) are left unfused.
#include <math.h>
#include <stdio.h>
#include <string.h>

#include <stdlib.h>

#include <algorithm>
#include <set>

#include "hlo.h"

namespace mhlo {
namespace {

struct Rewriter {
    Function& fn;
    std::map<int, size_t> def;          // value id -> index of the op that defines it
    std::map<int, TensorType> type;     // value id -> type
    std::vector<bool> dead;
    int fused = 0;

    explicit Rewriter(Function& f) : fn(f) { reindex(); }

    void reindex() {
        def.clear();
        type.clear();
        for (size_t i = 0; i < fn.arg_ids.size(); i++) type[fn.arg_ids[i]] = fn.arg_types[i];
        for (size_t i = 0; i < fn.ops.size(); i++) {
            def[fn.ops[i].result] = i;
            type[fn.ops[i].result] = fn.ops[i].out;
        }
        dead.assign(fn.ops.size(), false);
    }

    const Op* op_of(int v) const {
        auto it = def.find(v);
        return (it == def.end() || dead[it->second]) ? nullptr : &fn.ops[it->second];
    }
    const Op* op_named(int v, const char* name) const {
        const Op* o = op_of(v);
        return (o && o->name == name) ? o : nullptr;
    }
    size_t index_of(const Op* o) const { return (size_t)(o - fn.ops.data()); }

    // every use of the values defined by `interior` ops (root excluded) lies inside the pattern
    bool closed(const std::set<size_t>& interior, size_t root) const {
        std::set<int> vals;
        for (size_t i : interior)
            if (i != root) vals.insert(fn.ops[i].result);
        for (int r : fn.returns)
            if (vals.count(r)) return false;
        for (size_t i = 0; i < fn.ops.size(); i++) {
            if (dead[i] || interior.count(i)) continue;
            for (int v : fn.ops[i].operands)
                if (vals.count(v)) return false;
        }
        return true;
    }

    static bool decode(const Op& c, double& out) {
        if (c.name != "constant" || (!c.splat && c.out.numel() != 1)) return false;
        uint64_t bits = c.splat_bits;
        if (!c.splat) {
            if (c.constant.empty()) return false;
            bits = 0;
            memcpy(&bits, c.constant.data(), std::min<size_t>(8, c.constant.size()));
        }
        switch (c.out.dtype) {
            case F32: { float f; memcpy(&f, &bits, 4); out = f; return true; }
            case F64: { memcpy(&out, &bits, 8); return true; }
            case BF16: { uint32_t w = (uint32_t)(bits & 0xFFFF) << 16; float f; memcpy(&f, &w, 4); out = f; return true; }
            case F16: {
                const uint32_t h = bits & 0xFFFF, s = (h >> 15) & 1, e = (h >> 10) & 31, m = h & 1023;
                double v = e == 0 ? ldexp((double)m, -24) : e == 31 ? (m ? NAN : INFINITY) : ldexp((double)(m | 1024), (int)e - 25);
                out = s ? -v : v;
                return true;
            }
            case I32: { int32_t v; memcpy(&v, &bits, 4); out = v; return true; }
            case I64: { int64_t v; memcpy(&v, &bits, 8); out = (double)v; return true; }
            default: return false;
        }
    }

    // the single value a tensor is filled with: a splat constant, possibly behind
    // broadcast_in_dim / reshape / convert
    bool splat_value(int v, double& out, std::set<size_t>* via = nullptr) const {
        for (int hop = 0; hop < 4; hop++) {
            const Op* o = op_of(v);
            if (!o) return false;
            if (o->name == "constant") return decode(*o, out);
            if (o->name != "broadcast_in_dim" && o->name != "reshape" && o->name != "convert") return false;
            if (via) via->insert(index_of(o));
            v = o->operands.at(0);
        }
        return false;
    }

    static bool near(double a, double b, double tol) { return fabs(a - b) <= tol; }
    // the element types the fused kernels compute in
    static bool fused_float(int dt) { return dt == F32 || dt == F16 || dt == BF16; }
    // `c` is the constant `want` as a program of element type `dt` can spell it: `want` rounded to
    // that type, give or take one unit in the last place (another value is another function)
    static bool is_const(double c, double want, int dt) {
        double r = (double)(float)want, rel = 2.4e-7;
        if (dt == BF16) {
            const uint32_t w = (uint32_t)f32_to_bf16_bits((float)want) << 16;
            float f; memcpy(&f, &w, 4); r = f; rel = 1.0 / 128;
        } else if (dt == F16) {
            r = (double)(float)(_Float16)(float)want; rel = 1.0 / 1024;
        }
        return fabs(c - r) <= fabs(r) * rel;
    }

    // Statistics (one value per row) are often carried in keepdims style: reshaped or broadcast
    // to a shape with extra unit dims, computed on there, and spread over the row at the end.
    // relabel_src skips the ops that only rename the dims of `v` (reshape; broadcast_in_dim that
    // keeps the element count and the order); both keep the linear order of the elements.
    int relabel_src(int v, std::set<size_t>& nodes) const {
        for (int hop = 0; hop < 4; hop++) {
            const Op* o = op_of(v);
            if (!o || o->operands.empty()) return v;
            const bool same_count = type.at(o->operands[0]).numel() == o->out.numel();
            bool rename = o->name == "reshape" && same_count;
            if (o->name == "broadcast_in_dim" && same_count) {
                rename = true;
                for (size_t i = 1; i < o->dims.size(); i++) rename &= o->dims[i] > o->dims[i - 1];
            }
            if (!rename) return v;
            nodes.insert(index_of(o));
            v = o->operands[0];
        }
        return v;
    }
    // v = a per-row statistic spread over exactly one axis of the result shape: broadcast_in_dim
    // with increasing dims whose operand has, for every result dim but `axis`, either that dim
    // in full or nothing where the dim is 1.  Returns the statistic (renames skipped), -1 if not.
    int spread_src(int v, int64_t& axis, std::set<size_t>& nodes) const {
        const Op* b = op_named(v, "broadcast_in_dim");
        if (!b) return -1;
        const auto& S = b->out.shape;
        const auto& T = type.at(b->operands[0]).shape;
        if (b->dims.size() != T.size()) return -1;
        std::vector<int64_t> got(S.size(), 1);
        for (size_t i = 0; i < T.size(); i++) {
            const int64_t d = b->dims[i];
            if (d < 0 || d >= (int64_t)S.size() || (i > 0 && d <= b->dims[i - 1])) return -1;
            if (T[i] != S[d] && T[i] != 1) return -1;
            got[d] = T[i];
        }
        int64_t a = -1;
        for (size_t d = 0; d < S.size(); d++)
            if (got[d] != S[d]) {
                if (a >= 0) return -1;
                a = (int64_t)d;
            }
        if (a < 0) return -1;
        axis = a;
        nodes.insert(index_of(b));
        return relabel_src(b->operands[0], nodes);
    }

    // reduce of `x` over the single axis `axis` with `reducer`; the neutral element is checked
    const Op* reduce_over(int v, const char* reducer, int64_t& axis, int& x) const {
        const Op* r = op_named(v, "reduce");
        if (!r || r->reducer != reducer || r->dims.size() != 1 || r->operands.size() != 2) return nullptr;
        double init;
        if (!splat_value(r->operands[1], init)) return nullptr;
        if (!strcmp(reducer, "add") ? init != 0.0 : !(init <= -1e30)) return nullptr;
        axis = r->dims[0];
        x = r->operands[0];
        return r;
    }

    void replace(size_t root, const std::set<size_t>& interior, const std::string& target,
                 const std::vector<int>& operands, const std::string& config) {
        Op& o = fn.ops[root];
        o.name = "custom_call";
        o.target = target;
        o.backend_config = config;
        o.operands = operands;
        o.in_types.clear();
        for (int v : operands) o.in_types.push_back(type.at(v));
        o.attrs.clear();
        o.dims.clear();
        for (size_t i : interior)
            if (i != root) dead[i] = true;
        fused++;
    }

    // ------------------------------------------------------------------ token + position embedding
    // convert(add(gather(table, ids), broadcast_in_dim(positions, dims = [1, 2]))) -- or the add
    // alone where the program computes in f32: whole rows of an f32 table [vocab, d] picked by
    // ids [B, S] (i32), plus f32 positions [S, d] repeated over the batch, the positions possibly
    // rows p0 .. p0+S of a longer table (slice with unit strides over whole rows).  One kernel
    // reads both rows, adds them in f32 and rounds once, as the three operations in a row do.
    bool embedding(size_t ri) {
        const Op& root = fn.ops[ri];
        std::set<size_t> nodes{ri};
        const Op* sum = root.name == "add" ? &root : root.name == "convert" ? op_named(root.operands[0], "add") : nullptr;
        if (!sum || sum->out.dtype != F32 || sum->out.shape.size() != 3 || !fused_float(root.out.dtype) || root.out.shape != sum->out.shape)
            return false;
        nodes.insert(index_of(sum));
        const int64_t B = sum->out.shape[0], S = sum->out.shape[1], d = sum->out.shape[2];
        if (B < 1 || S < 1 || d < 1) return false;
        for (int k = 0; k < 2; k++) {
            const Op* g = op_named(sum->operands[k], "gather");
            const Op* b = op_named(sum->operands[1 - k], "broadcast_in_dim");
            if (!g || !b || g->operands.size() != 2) continue;
            const TensorType &tt = type.at(g->operands[0]), &it = type.at(g->operands[1]);
            // the whole-row form of gather, indices without a trailing unit dim
            if (tt.dtype != F32 || tt.shape.size() != 2 || tt.shape[1] != d || tt.shape[0] < 1 || it.dtype != I32 ||
                it.shape != std::vector<int64_t>{B, S} || g->dims != std::vector<int64_t>{0} ||
                g->starts != std::vector<int64_t>{0} || g->limits != std::vector<int64_t>{1, d} || !g->lhs_batch.empty() ||
                !g->rhs_batch.empty() || g->iota_dim != 2 || g->strides != std::vector<int64_t>{2})
                continue;
            int pos = b->operands[0];
            const TensorType& pt = type.at(pos);
            if (b->dims != std::vector<int64_t>{1, 2} || pt.dtype != F32 || pt.shape != std::vector<int64_t>{S, d}) continue;
            std::set<size_t> all = nodes;
            all.insert(index_of(g));
            all.insert(index_of(b));
            int64_t p0 = 0;
            if (const Op* sl = op_named(pos, "slice")) {
                const TensorType& st = type.at(sl->operands[0]);
                if (st.dtype == F32 && st.shape.size() == 2 && st.shape[1] == d && sl->strides == std::vector<int64_t>{1, 1} &&
                    sl->starts.size() == 2 && sl->limits.size() == 2 && sl->starts[1] == 0 && sl->limits[1] == d &&
                    sl->starts[0] >= 0 && sl->limits[0] == sl->starts[0] + S && sl->limits[0] <= st.shape[0]) {
                    p0 = sl->starts[0];
                    pos = sl->operands[0];
                    all.insert(index_of(sl));
                }
            }
            if (!closed(all, ri)) continue;
            replace(ri, all, "fused_token_embedding", {g->operands[1], g->operands[0], pos},
                    "{\"first_position\": " + std::to_string(p0) + "}");
            return true;
        }
        return false;
    }

    // ------------------------------------------------------------------ softmax
    // divide(e, bcast(reduce_add(e))), e = exp(subtract(x, bcast(reduce_max(x))))
    bool softmax(size_t ri) {
        const Op& root = fn.ops[ri];
        if (root.name != "divide" || !fused_float(root.out.dtype)) return false;
        const Op* e = op_named(root.operands[0], "exponential");
        if (!e) return false;
        std::set<size_t> in = {ri, index_of(e)};
        int64_t ax_s, ax_m, ax_b;
        int e_in, x;
        const int sum = spread_src(root.operands[1], ax_b, in);
        if (sum < 0) return false;
        const Op* s = reduce_over(sum, "add", ax_s, e_in);
        if (!s || e_in != e->result || ax_s != ax_b) return false;
        const Op* sh = op_named(e->operands[0], "subtract");
        if (!sh) {
            // exp(x) / sum(exp(x)) without the shift by the row maximum: the same function wherever the
            // spelled form does not overflow (the fused kernel always shifts, so it stays finite there too)
            x = e->operands[0];
            if (!(type.at(x) == root.out)) return false;
            in.insert(index_of(s));
            if (!closed(in, ri)) return false;
            char cfg0[64];
            snprintf(cfg0, sizeof cfg0, "{\"axis\": %lld}", (long long)ax_s);
            replace(ri, in, "fused_softmax", {x}, cfg0);
            return true;
        }
        const int mx = spread_src(sh->operands[1], ax_b, in);
        if (mx < 0) return false;
        const Op* m = reduce_over(mx, "maximum", ax_m, x);
        if (!m || ax_m != ax_s || ax_b != ax_s || x != sh->operands[0]) return false;
        if (!(type.at(x) == root.out)) return false;
        in.insert(index_of(s));
        in.insert(index_of(sh));
        in.insert(index_of(m));
        if (!closed(in, ri)) return false;
        char cfg[64];
        snprintf(cfg, sizeof cfg, "{\"axis\": %lld}", (long long)ax_s);
        replace(ri, in, "fused_softmax", {x}, cfg);
        return true;
    }

    // ------------------------------------------------------------------ GELU (tanh form)
    // leaves of a product: nested multiplies are opened while their value has no other use
    void product_leaves(int v, bool is_root, std::vector<int>& leaves, std::set<size_t>& nodes) const {
        const Op* o = op_named(v, "multiply");
        if (o && (is_root || uses(v) == 1)) {
            nodes.insert(index_of(o));
            product_leaves(o->operands[0], false, leaves, nodes);
            product_leaves(o->operands[1], false, leaves, nodes);
        } else {
            leaves.push_back(v);
        }
    }
    int uses(int v) const {
        int n = 0;
        for (int r : fn.returns) n += r == v;
        for (size_t i = 0; i < fn.ops.size(); i++)
            if (!dead[i])
                for (int u : fn.ops[i].operands) n += u == v;
        return n;
    }
    // add(const c, other) in either order
    const Op* add_const(int v, double c, double tol, int& other, std::set<size_t>& nodes) const {
        const Op* a = op_named(v, "add");
        if (!a) return nullptr;
        for (int k = 0; k < 2; k++) {
            double got;
            if (splat_value(a->operands[k], got) && near(got, c, tol)) {
                other = a->operands[1 - k];
                nodes.insert(index_of(a));
                return a;
            }
        }
        return nullptr;
    }

    bool gelu(size_t ri) {
        const Op& root = fn.ops[ri];
        if (root.name != "multiply" || !fused_float(root.out.dtype)) return false;
        const int dt = root.out.dtype;
        std::vector<int> leaves;
        std::set<size_t> in;
        product_leaves(root.result, true, leaves, in);
        if (leaves.size() != 3) return false;
        int x = -1, opt = -1, halves = 0, t = -1;
        for (int v : leaves) {
            double c;
            int inner;
            std::set<size_t> tmp;
            if (splat_value(v, c) && near(c, 0.5, 1e-6)) halves++;
            else if (add_const(v, 1.0, 1e-6, inner, tmp) && op_named(inner, "tanh")) { opt = v; t = inner; in.insert(tmp.begin(), tmp.end()); }
            else x = v;
        }
        if (halves != 1 || x < 0 || opt < 0) return false;
        const Op* th = op_named(t, "tanh");
        in.insert(index_of(th));
        // tanh argument: sqrt(2/pi) * (x + 0.044715 x^3)
        std::vector<int> l2;
        product_leaves(th->operands[0], true, l2, in);
        if (l2.size() != 2) return false;
        int inner = -1, ks = 0;
        for (int v : l2) {
            double c;
            if (splat_value(v, c) && is_const(c, 0.7978845608028654, dt)) ks++;
            else inner = v;
        }
        if (ks != 1 || inner < 0) return false;
        const Op* ia = op_named(inner, "add");
        if (!ia) return false;
        in.insert(index_of(ia));
        int cubic = ia->operands[0] == x ? ia->operands[1] : ia->operands[1] == x ? ia->operands[0] : -1;
        if (cubic < 0) return false;
        std::vector<int> l3;
        product_leaves(cubic, true, l3, in);
        int xs = 0, cs = 0;
        for (int v : l3) {
            double c;
            if (v == x) xs++;
            else if (splat_value(v, c) && is_const(c, 0.044715, dt)) cs++;
            else return false;
        }
        if (xs != 3 || cs != 1 || !(type.at(x) == root.out)) return false;
        if (!closed(in, ri)) return false;
        replace(ri, in, "fused_gelu", {x}, "{\"approximate\": true}");
        return true;
    }

    // ------------------------------------------------------------------ GELU (erf form)
    // x * (1 + erf(x / sqrt 2)) * 0.5 in any association and operand order, the last factor also as
    // a division by 2, the erf argument as x * (1 / sqrt 2) or x / sqrt 2: what
    // jax.nn.gelu(approximate=False) lowers to.  It becomes a fused_gelu marked "erf": true, which
    // runs the exact function (not the tanh approximation the reference substitutes).
    bool gelu_erf(size_t ri) {
        const Op& root = fn.ops[ri];
        if (!fused_float(root.out.dtype)) return false;
        const int dt = root.out.dtype;
        std::set<size_t> in = {ri};
        std::vector<int> leaves;
        int halves = 0;
        if (root.name == "divide") {                     // (...) / 2
            double c;
            if (!splat_value(root.operands[1], c) || c != 2.0) return false;
            halves = 1;
            product_leaves(root.operands[0], uses(root.operands[0]) == 1, leaves, in);
        } else if (root.name == "multiply") {
            product_leaves(root.result, true, leaves, in);
        } else {
            return false;
        }
        int x = -1, er = -1;
        for (int v : leaves) {
            double c;
            int inner;
            std::set<size_t> tmp;
            if (splat_value(v, c) && c == 0.5) halves++;
            else if (add_const(v, 1.0, 0.0, inner, tmp) && op_named(inner, "erf")) { er = inner; in.insert(tmp.begin(), tmp.end()); }
            else if (x < 0) x = v;
            else return false;
        }
        if (halves != 1 || x < 0 || er < 0 || leaves.size() != (root.name == "divide" ? 2u : 3u)) return false;
        const Op* e = op_named(er, "erf");
        in.insert(index_of(e));
        const Op* arg = op_of(e->operands[0]);
        if (!arg || (arg->name != "multiply" && arg->name != "divide")) return false;
        in.insert(index_of(arg));
        bool ok = false;
        for (int k = 0; k < 2 && !ok; k++) {
            if (arg->name == "divide" && k == 0) continue;          // x / sqrt 2: the constant is the divisor
            double c;
            if (arg->operands[1 - k] != x || !splat_value(arg->operands[k], c)) continue;
            ok = arg->name == "divide" ? is_const(c, 1.4142135623730951, dt) : is_const(c, 0.7071067811865476, dt);
        }
        if (!ok || !(type.at(x) == root.out) || !closed(in, ri)) return false;
        replace(ri, in, "fused_gelu", {x}, "{\"approximate\": false, \"erf\": true}");
        return true;
    }

    // ------------------------------------------------------------------ LayerNorm / RMSNorm
    // mean over the last axis: reduce_add(u) / N  or  reduce_add(u) * (1/N)
    bool mean_last(int v, int& u, std::set<size_t>& nodes) const {
        v = relabel_src(v, nodes);
        const Op* o = op_of(v);
        if (!o || (o->name != "divide" && o->name != "multiply")) return false;
        for (int k = 0; k < 2; k++) {
            if (o->name == "divide" && k == 1) break;
            double c;
            int64_t axis;
            int src;
            std::set<size_t> via;
            const Op* r = reduce_over(relabel_src(o->operands[k], nodes), "add", axis, src);
            if (!r || !splat_value(o->operands[1 - k], c, &via)) continue;
            const auto& shp = type.at(src).shape;
            if (shp.empty() || axis != (int64_t)shp.size() - 1) continue;
            const double n = (double)shp.back();
            if (o->name == "divide" ? !near(c, n, 1e-6 * n) : !near(c * n, 1.0, 1e-5)) continue;
            u = src;
            nodes.insert(index_of(o));
            nodes.insert(index_of(r));
            return true;
        }
        return false;
    }
    // v = a statistic spread over the last axis; returns the statistic, -1 if not
    int spread_last(int v, size_t rank, std::set<size_t>& nodes) const {
        int64_t axis;
        std::set<size_t> t = nodes;
        const int src = spread_src(v, axis, t);
        if (src < 0 || axis != (int64_t)rank - 1) return -1;
        nodes = t;
        return src;
    }
    // The variance spelled mean(x * x) - mean(x) * mean(x) (the one-pass form jax.numpy.var and
    // flax's LayerNorm with use_fast_variance emit), with `c` = x - bcast(mean(x)) of the same
    // mean.  The fused kernel computes the two-pass variance: the same quantity without the
    // cancellation of the spelled form.
    bool one_pass_variance(int var, int c, size_t rank, const std::set<size_t>& base, int& x, std::set<size_t>& nodes) const {
        std::set<size_t> t = base;
        const Op* vs = op_named(relabel_src(var, t), "subtract");
        if (!vs) return false;
        int sq;
        if (!mean_last(vs->operands[0], sq, t)) return false;
        const Op* sqo = op_named(sq, "multiply");
        if (!sqo || sqo->operands[0] != sqo->operands[1]) return false;
        const int xx = sqo->operands[0];
        const Op* m2 = op_named(relabel_src(vs->operands[1], t), "multiply");
        if (!m2 || m2->operands[0] != m2->operands[1]) return false;
        int mx;
        if (!mean_last(m2->operands[0], mx, t) || mx != xx) return false;
        const Op* sub = op_named(c, "subtract");
        if (!sub || sub->operands[0] != xx) return false;
        const int spread = spread_last(sub->operands[1], rank, t);
        std::set<size_t> scratch;
        if (spread < 0 || relabel_src(spread, scratch) != relabel_src(m2->operands[0], scratch)) return false;
        t.insert(index_of(vs));
        t.insert(index_of(sqo));
        t.insert(index_of(m2));
        t.insert(index_of(sub));
        x = xx;
        nodes.insert(t.begin(), t.end());
        return true;
    }
    // v = c * bcast(rsqrt(mean(c*c) + eps)); centred: c = x - bcast(mean(x))
    bool norm_core(int v, int& x, double& eps, bool& centred, std::set<size_t>& nodes) const {
        const Op* m = op_named(v, "multiply");
        if (!m) return false;
        const size_t rank = m->out.shape.size();
        if (rank < 1) return false;
        for (int k = 0; k < 2; k++) {
            std::set<size_t> tmp = {index_of(m)};
            const int stat = spread_last(m->operands[k], rank, tmp);
            if (stat < 0) continue;
            const int c = m->operands[1 - k];
            const Op* rs = op_named(stat, "rsqrt");
            if (!rs) continue;
            const Op* ve = op_named(relabel_src(rs->operands[0], tmp), "add");
            if (!ve) continue;
            tmp.insert(index_of(rs));
            tmp.insert(index_of(ve));
            for (int j = 0; j < 2; j++) {
                double e;
                int sq;
                std::set<size_t> t2 = tmp;
                if (!splat_value(ve->operands[j], e) || !(e > 0 && e < 1e-1)) continue;
                if (one_pass_variance(ve->operands[1 - j], c, rank, tmp, x, nodes)) {   // mean(x^2) - mean(x)^2
                    centred = true;
                    eps = e;
                    return true;
                }
                if (!mean_last(ve->operands[1 - j], sq, t2)) continue;
                const Op* sqo = op_named(sq, "multiply");
                if (!sqo || sqo->operands[0] != c || sqo->operands[1] != c) continue;
                t2.insert(index_of(sqo));
                const Op* sub = op_named(c, "subtract");
                int mx;
                std::set<size_t> t3 = t2;
                const int mean = sub ? spread_last(sub->operands[1], rank, t3) : -1;
                if (sub && mean >= 0 && mean_last(mean, mx, t3) && mx == sub->operands[0]) {
                    t3.insert(index_of(sub));
                    x = mx;
                    centred = true;
                    nodes.insert(t3.begin(), t3.end());
                } else {
                    x = c;
                    centred = false;
                    nodes.insert(t2.begin(), t2.end());
                }
                eps = e;
                return true;
            }
        }
        return false;
    }
    // v = bcast of a [cols] vector along the last axis
    bool param_vector(int v, size_t rank, int64_t cols, int dtype, int& vec, std::set<size_t>& nodes) const {
        const Op* b = op_named(v, "broadcast_in_dim");
        if (!b || b->dims != std::vector<int64_t>{(int64_t)rank - 1}) return false;
        const TensorType& t = type.at(b->operands[0]);
        if (t.shape != std::vector<int64_t>{cols} || t.dtype != dtype) return false;
        vec = b->operands[0];
        nodes.insert(index_of(b));
        return true;
    }

    bool norm(size_t ri) {
        const Op& root = fn.ops[ri];
        if (!dtype_is_float(root.out.dtype) || root.out.dtype == F64 || root.out.shape.empty()) return false;
        const size_t rank = root.out.shape.size();
        const int64_t cols = root.out.shape.back();
        int x;
        double eps;
        bool centred;
        if (root.name == "add") {            // (core * gamma) + beta
            for (int k = 0; k < 2; k++) {
                std::set<size_t> t = {ri};
                int b;
                if (!param_vector(root.operands[k], rank, cols, root.out.dtype, b, t)) continue;
                const Op* y = op_named(root.operands[1 - k], "multiply");
                if (!y) continue;
                for (int j = 0; j < 2; j++) {
                    std::set<size_t> t2 = t;
                    int g;
                    t2.insert(index_of(y));
                    if (!param_vector(y->operands[j], rank, cols, root.out.dtype, g, t2)) continue;
                    if (!norm_core(y->operands[1 - j], x, eps, centred, t2) || !centred) continue;
                    if (!closed(t2, ri)) continue;
                    char cfg[96];
                    snprintf(cfg, sizeof cfg, "{\"eps\": %.9g, \"axes\": [-1]}", eps);
                    replace(ri, t2, "fused_layer_norm", {x, g, b}, cfg);
                    return true;
                }
            }
            return false;
        }
        if (root.name != "multiply") return false;
        // core * gamma (RMSNorm)
        for (int j = 0; j < 2; j++) {
            std::set<size_t> t2 = {ri};
            int g;
            if (!param_vector(root.operands[j], rank, cols, root.out.dtype, g, t2)) continue;
            if (!norm_core(root.operands[1 - j], x, eps, centred, t2) || centred) continue;
            if (!closed(t2, ri)) continue;
            char cfg[96];
            snprintf(cfg, sizeof cfg, "{\"eps\": %.9g, \"axes\": [-1]}", eps);
            replace(ri, t2, "fused_rms_norm", {x, g}, cfg);
            return true;
        }
        return false;
    }

    // ------------------------------------------------------------------ attention
    static bool iota_prefix(const std::vector<int64_t>& v, size_t n) {
        if (v.size() != n) return false;
        for (size_t i = 0; i < n; i++)
            if (v[i] != (int64_t)i) return false;
        return true;
    }
    // mask [S, S] = select(compare(key index, query index), ...) over two iotas that keeps (adds 0)
    // where key <= query and adds -inf (or anything <= -1e30) elsewhere: the kernel's causal flag
    bool causal_mask(int mask) const {
        const Op* sel = op_named(mask, "select");
        if (!sel || sel->operands.size() != 3 || sel->out.shape.size() != 2 || sel->out.shape[0] != sel->out.shape[1]) return false;
        const Op* cmp = op_named(sel->operands[0], "compare");
        if (!cmp || cmp->operands.size() != 2 || cmp->out.shape != sel->out.shape) return false;
        const Op* l = op_named(cmp->operands[0], "iota");
        const Op* r = op_named(cmp->operands[1], "iota");
        if (!l || !r || l->out.shape != sel->out.shape || r->out.shape != sel->out.shape || dtype_is_float(l->out.dtype) ||
            l->out.dtype != r->out.dtype || l->iota_dim + r->iota_dim != 1)
            return false;
        // written as <key> DIR <query>: swap the direction when the query index (dim 0) is on the left
        std::string dir = cmp->direction;
        if (l->iota_dim == 0) dir = dir == "LE" ? "GE" : dir == "GE" ? "LE" : dir == "LT" ? "GT" : dir == "GT" ? "LT" : dir;
        const bool pred_keeps = dir == "LE", pred_masks = dir == "GT";
        if (!pred_keeps && !pred_masks) return false;
        double keep, drop;
        if (!splat_value(sel->operands[pred_keeps ? 1 : 2], keep) || !splat_value(sel->operands[pred_keeps ? 2 : 1], drop)) return false;
        return keep == 0.0 && drop <= -1e30;
    }

    bool attention(size_t ri) {
        const Op& pv = fn.ops[ri];
        if (pv.name != "dot_general" || !dtype_is_float(pv.out.dtype) || pv.out.dtype == F64) return false;
        const size_t r = pv.out.shape.size();
        if (r < 2 || r > 4) return false;
        const std::vector<int64_t> last = {(int64_t)r - 1}, prev = {(int64_t)r - 2};
        if (!iota_prefix(pv.lhs_batch, r - 2) || !iota_prefix(pv.rhs_batch, r - 2) || pv.lhs_contract != last ||
            pv.rhs_contract != prev)
            return false;
        const Op* p = op_named(pv.operands[0], "custom_call");
        if (!p || p->target != "fused_softmax") return false;
        const long long axis = parse_config(p->backend_config).get_int("axis", -1);
        if (axis != -1 && axis != (long long)r - 1) return false;
        std::set<size_t> in = {ri, index_of(p)};
        int cur = p->operands[0], mask = -1;
        double scale = 1.0;
        if (const Op* a = op_named(cur, "add")) {          // scores + mask
            const bool lhs_scores = op_named(a->operands[0], "multiply") || op_named(a->operands[0], "divide") ||
                                    op_named(a->operands[0], "dot_general");
            mask = a->operands[lhs_scores ? 1 : 0];
            cur = a->operands[lhs_scores ? 0 : 1];
            in.insert(index_of(a));
        }
        if (const Op* m = op_named(cur, "multiply")) {      // scores * scale
            double c;
            int k = splat_value(m->operands[1], c) ? 1 : splat_value(m->operands[0], c) ? 0 : -1;
            if (k < 0) return false;
            scale = c;
            cur = m->operands[1 - k];
            in.insert(index_of(m));
        } else if (const Op* d = op_named(cur, "divide")) { // scores / sqrt(D)
            double c;
            if (!splat_value(d->operands[1], c) || c == 0.0) return false;
            scale = 1.0 / c;
            cur = d->operands[0];
            in.insert(index_of(d));
        }
        const Op* qk = op_named(cur, "dot_general");
        if (!qk || !iota_prefix(qk->lhs_batch, r - 2) || !iota_prefix(qk->rhs_batch, r - 2) || qk->lhs_contract != last)
            return false;
        in.insert(index_of(qk));
        const int q = qk->operands[0], v = pv.operands[1];
        int k = qk->operands[1];
        if (qk->rhs_contract == prev) {                     // explicit transpose of K
            const Op* t = op_named(k, "transpose");
            if (!t || t->dims.size() != r) return false;
            for (size_t i = 0; i + 2 < r; i++)
                if (t->dims[i] != (int64_t)i) return false;
            if (t->dims[r - 2] != (int64_t)r - 1 || t->dims[r - 1] != (int64_t)r - 2) return false;
            in.insert(index_of(t));
            k = t->operands[0];
        } else if (qk->rhs_contract != last) {
            return false;
        }
        const TensorType &qt = type.at(q), &kt = type.at(k), &vt = type.at(v);
        if (qt.dtype != pv.out.dtype || !(kt == vt) || kt.dtype != qt.dtype || qt.shape.size() != r || kt.shape.size() != r)
            return false;
        if (qt.shape[r - 1] != kt.shape[r - 1]) return false;
        for (size_t i = 0; i + 2 < r; i++)
            if (qt.shape[i] != kt.shape[i]) return false;
        if (mask >= 0) {
            // a mask broadcast along leading axes only need not be materialised
            if (const Op* mbc = op_named(mask, "broadcast_in_dim")) {
                const size_t mr0 = type.at(mbc->operands[0]).shape.size();
                bool trailing = mbc->dims.size() == mr0 && mr0 >= 2 && mr0 <= r;
                for (size_t i = 0; trailing && i < mr0; i++) trailing = mbc->dims[i] == (int64_t)(r - mr0 + i);
                if (trailing && uses(mask) == 1) {
                    in.insert(index_of(mbc));
                    mask = mbc->operands[0];
                }
            }
        }
        bool causal = false;
        if (mask >= 0 && qt.shape[r - 2] == kt.shape[r - 2] && type.at(mask).shape == std::vector<int64_t>{qt.shape[r - 2], kt.shape[r - 2]} &&
            causal_mask(mask)) {
            causal = true;      // the mask's producers stay behind for other users and are swept when there are none
            mask = -1;
        }
        if (mask >= 0) {                                    // must end in [Sq, Skv] and broadcast over batch / heads
            const TensorType& mt = type.at(mask);
            const size_t mr = mt.shape.size();
            const int64_t Sq = qt.shape[r - 2], Skv = kt.shape[r - 2];
            if (mt.dtype != qt.dtype || mr < 2 || mr > r || mt.shape[mr - 1] != Skv || mt.shape[mr - 2] != Sq) return false;
            const int64_t H = r >= 3 ? qt.shape[r - 3] : 1;
            int64_t B = 1, mb = 1;
            for (size_t i = 0; i + 3 < r; i++) B *= qt.shape[i];
            const int64_t mh = mr >= 3 ? mt.shape[mr - 3] : 1;
            for (size_t i = 0; i + 3 < mr; i++) mb *= mt.shape[i];
            if ((mh != 1 && mh != H) || (mb != 1 && mb != B)) return false;
        }
        if (!closed(in, ri)) return false;
        char cfg[128];
        snprintf(cfg, sizeof cfg, "{\"scale\": %.9g, \"has_mask\": %s, \"is_causal\": %s}", scale, mask >= 0 ? "true" : "false",
                 causal ? "true" : "false");
        std::vector<int> ops = {q, k, v};
        if (mask >= 0) ops.push_back(mask);
        replace(ri, in, "fused_scaled_dot_product_attention", ops, cfg);
        return true;
    }

    // ------------------------------------------------------------------ attention on views
    // A [B,H,S,D] operand that is only a re-arranged window of a [B,S,W] tensor --
    // transpose{0,2,1,3}(reshape [B,S,H*D] -> [B,S,H,D] (slice [:, :, off : off + H*D] (t))), the
    // slice optional -- is read in place: element (b,h,s,d) lies at off + b*S*W + s*W + h*D + d.
    struct View { int src; int64_t off, sb, sh, sr; };
    bool head_view(int v, View& out) const {
        const Op* t = op_named(v, "transpose");
        if (!t || t->dims != std::vector<int64_t>{0, 2, 1, 3}) return false;
        const Op* r = op_named(t->operands[0], "reshape");
        if (!r || r->out.shape.size() != 4) return false;
        const int64_t B = r->out.shape[0], S = r->out.shape[1], H = r->out.shape[2], D = r->out.shape[3];
        const TensorType& rt = type.at(r->operands[0]);
        if (rt.shape != std::vector<int64_t>{B, S, H * D}) return false;
        out = View{r->operands[0], 0, S * H * D, D, H * D};
        if (const Op* sl = op_named(r->operands[0], "slice")) {
            const TensorType& bt = type.at(sl->operands[0]);
            if (bt.shape.size() == 3 && sl->strides == std::vector<int64_t>{1, 1, 1} && sl->starts[0] == 0 && sl->starts[1] == 0 &&
                sl->limits[0] == B && sl->limits[1] == S && bt.shape[0] == B && bt.shape[1] == S) {
                const int64_t W = bt.shape[2];
                out = View{sl->operands[0], sl->starts[2], S * W, D, W};
            }
        }
        return out.off % 8 == 0 && out.sr % 8 == 0 && out.sb % 8 == 0;
    }
    // Rewrites a fused attention whose operands (or whose only consumer) are such views to read
    // (write) them in place: the config gains "dims" [B,H,Sq,Skv,D] and "views" = {offset, batch,
    // head, row strides} x {q, k, v, o}; the glue operations lose their users and are swept.
    bool attention_views(size_t ri) {
        Op& at = fn.ops[ri];
        if (at.name != "custom_call" || at.target != "fused_scaled_dot_product_attention" || at.out.shape.size() != 4) return false;
        if (at.out.dtype != BF16 && at.out.dtype != F16) return false;
        const Config cfg = parse_config(at.backend_config);
        if (!cfg.get_int_array("views", {}).empty()) return false;
        const TensorType qt = type.at(at.operands[0]), kt = type.at(at.operands[1]);
        const int64_t B = qt.shape[0], H = qt.shape[1], Sq = qt.shape[2], D = qt.shape[3], Skv = kt.shape[2];
        if (D != 64 && D != 128) return false;
        View views[4];
        bool any = false;
        for (int i = 0; i < 3; i++) {
            const int64_t S = i == 0 ? Sq : Skv;
            views[i] = View{at.operands[i], 0, H * S * D, S * D, D};          // packed [B,H,S,D]
            View w;
            if (head_view(at.operands[i], w)) { views[i] = w; any = true; }
        }
        // the result: written as [B,S,H,D] when its only use is the head merge
        views[3] = View{-1, 0, H * Sq * D, Sq * D, D};
        size_t root = ri;
        const Op* tr = nullptr;
        const Op* rs = nullptr;
        if (uses(at.result) == 1) {
            for (size_t i = 0; i < fn.ops.size() && !tr; i++)
                if (!dead[i] && fn.ops[i].name == "transpose" && fn.ops[i].operands[0] == at.result &&
                    fn.ops[i].dims == std::vector<int64_t>{0, 2, 1, 3})
                    tr = &fn.ops[i];
            if (tr && uses(tr->result) == 1)
                for (size_t i = 0; i < fn.ops.size() && !rs; i++)
                    if (!dead[i] && fn.ops[i].name == "reshape" && fn.ops[i].operands[0] == tr->result &&
                        fn.ops[i].out.shape == std::vector<int64_t>{B, Sq, H * D})
                        rs = &fn.ops[i];
        }
        if (rs) {
            views[3] = View{-1, 0, Sq * H * D, D, H * D};
            root = index_of(rs);
            any = true;
        }
        if (!any) return false;
        std::string c;
        char num[64];
        snprintf(num, sizeof num, "%.9g", cfg.get_float("scale", 1.0));
        c = std::string("{\"scale\": ") + num + ", \"has_mask\": " + (cfg.get_bool("has_mask", false) ? "true" : "false") +
            ", \"is_causal\": " + (cfg.get_bool("is_causal", false) ? "true" : "false") + ", \"dims\": [" + std::to_string(B) + ", " +
            std::to_string(H) + ", " + std::to_string(Sq) + ", " + std::to_string(Skv) + ", " + std::to_string(D) + "], \"views\": [";
        for (int i = 0; i < 4; i++)
            c += std::to_string(views[i].off) + ", " + std::to_string(views[i].sb) + ", " + std::to_string(views[i].sh) + ", " +
                 std::to_string(views[i].sr) + (i < 3 ? ", " : "]}");
        std::vector<int> operands = {views[0].src, views[1].src, views[2].src};
        for (size_t i = 3; i < at.operands.size(); i++) operands.push_back(at.operands[i]);
        std::set<size_t> interior = {root};
        if (root != ri) { interior.insert(ri); interior.insert(index_of(tr)); }
        replace(root, interior, "fused_scaled_dot_product_attention", operands, c);
        return true;
    }

    // ------------------------------------------------------------------ matmul + bias (+ activation)
    bool plain_matmul(const Op* d) const {
        if (!d || (d->name != "dot" && d->name != "dot_general") || d->operands.size() != 2) return false;
        const TensorType &xt = type.at(d->operands[0]), &wt = type.at(d->operands[1]);
        if (wt.shape.size() != 2 || xt.shape.size() < 2 || !fused_float(xt.dtype) || wt.dtype != xt.dtype)
            return false;
        // a widening product (16-bit operands, f32 result) is not what the fused kernel computes
        if (d->out.dtype != xt.dtype) return false;
        if (d->name == "dot") return xt.shape.size() == 2;
        if (d->name != "dot_general") return false;
        return d->lhs_batch.empty() && d->rhs_batch.empty() &&
               d->lhs_contract == std::vector<int64_t>{(int64_t)xt.shape.size() - 1} &&
               d->rhs_contract == std::vector<int64_t>{0};
    }
    bool matmul_bias_act(size_t ri) {
        const Op& root = fn.ops[ri];
        std::string act = "none";
        std::set<size_t> in = {ri};
        const Op* add = nullptr;
        if (root.name == "add") {
            add = &root;
        } else {
            int src = -1;
            if (root.name == "tanh") { act = "tanh"; src = root.operands[0]; }
            else if (root.name == "logistic") { act = "sigmoid"; src = root.operands[0]; }
            else if (root.name == "custom_call" && root.target == "fused_gelu") {
                act = parse_config(root.backend_config).get_bool("erf", false) ? "gelu_exact" : "gelu";
                src = root.operands[0];
            }
            else if (root.name == "maximum") {
                double c;
                for (int k = 0; k < 2; k++)
                    if (splat_value(root.operands[k], c) && c == 0.0) { act = "relu"; src = root.operands[1 - k]; }
            } else if (root.name == "multiply") {          // h * logistic(h): SiLU
                for (int k = 0; k < 2; k++) {
                    const Op* lg = op_named(root.operands[k], "logistic");
                    if (lg && lg->operands[0] == root.operands[1 - k] && uses(lg->result) == 1) {
                        act = "silu";
                        src = root.operands[1 - k];
                        in.insert(index_of(lg));
                    }
                }
            }
            if (src < 0) return false;
            add = op_named(src, "add");
            if (!add) return false;
            in.insert(index_of(add));
        }
        const size_t rank = add->out.shape.size();
        if (rank < 2) return false;
        for (int k = 0; k < 2; k++) {
            std::set<size_t> t = in;
            int bias;
            if (!param_vector(add->operands[k], rank, add->out.shape.back(), add->out.dtype, bias, t)) continue;
            const Op* d = op_of(add->operands[1 - k]);
            if (!plain_matmul(d)) continue;
            t.insert(index_of(d));
            if (!closed(t, ri)) continue;
            const std::vector<int> ops = {d->operands[0], d->operands[1], bias};
            replace(ri, t, "fused_matmul_bias_activation", ops, "{\"activation\": \"" + act + "\"}");
            return true;
        }
        return false;
    }

    // add(r, fused_matmul_bias_activation(x, w, bias)) with the product used nowhere else: the
    // residual goes into the GEMM epilogue (last operand, "has_residual"); the kernel adds it after
    // rounding the product, so the bits are those of the separate add
    bool matmul_residual(size_t ri) {
        const Op& root = fn.ops[ri];
        if (root.name != "add" || !dtype_is_float(root.out.dtype) || root.out.dtype == F64) return false;
        for (int k = 0; k < 2; k++) {
            const Op* mm = op_named(root.operands[k], "custom_call");
            if (!mm || mm->target != "fused_matmul_bias_activation" || mm->operands.size() != 3 || uses(mm->result) != 1) continue;
            if (parse_config(mm->backend_config).get_bool("has_residual", false)) continue;
            const int r = root.operands[1 - k];
            if (!(type.at(r) == root.out) || !(mm->out == root.out)) continue;
            std::string cfg = mm->backend_config;
            const size_t close = cfg.rfind('}');
            if (close == std::string::npos) continue;
            cfg = cfg.substr(0, close) + ", \"has_residual\": true}";
            const std::vector<int> ops = {mm->operands[0], mm->operands[1], mm->operands[2], r};
            replace(ri, {ri, index_of(mm)}, "fused_matmul_bias_activation", ops, cfg);
            return true;
        }
        return false;
    }

    // drop rewritten ops and everything that has become unused
    void sweep() {
        bool changed = true;
        while (changed) {
            changed = false;
            for (size_t i = fn.ops.size(); i-- > 0;) {
                if (dead[i]) continue;
                if (uses(fn.ops[i].result) == 0) { dead[i] = true; changed = true; }
            }
        }
        std::vector<Op> keep;
        for (size_t i = 0; i < fn.ops.size(); i++)
            if (!dead[i]) keep.push_back(std::move(fn.ops[i]));
        fn.ops = std::move(keep);
        reindex();
    }

    template <typename F>
    void pass(F&& try_at) {
        for (size_t i = fn.ops.size(); i-- > 0;)
            if (!dead[i]) try_at(i);
        sweep();
    }
};

}  // namespace

int fuse_patterns(Function& fn, const std::set<std::string>* disabled) {
    // malformed operations are reported by the validation that follows; do not look inside them
    static const std::map<std::string, size_t> kArity = {
        {"add", 2}, {"subtract", 2}, {"multiply", 2}, {"divide", 2}, {"maximum", 2}, {"minimum", 2}, {"dot", 2},
        {"dot_general", 2}, {"reduce", 2}, {"exponential", 1}, {"tanh", 1}, {"rsqrt", 1}, {"logistic", 1}, {"erf", 1},
        {"broadcast_in_dim", 1}, {"reshape", 1}, {"convert", 1}, {"transpose", 1}};
    for (const Op& op : fn.ops) {
        auto it = kArity.find(op.name);
        if (it != kArity.end() && op.operands.size() != it->second) return 0;
        for (int v : op.operands)
            if (v < 0 || v >= fn.num_values) return 0;
    }
    Rewriter rw(fn);
    // The passes under the names the reference gives its pattern-fusion passes
    // (Compiler/PassManager.swift:154-201), so that METALHLO_DISABLED_PASSES means the same thing.
    // Later passes build on earlier ones: attention needs the fused softmax, the GELU epilogue the
    // fused GELU, the residual epilogue the fused matmul.  METALHLO_DEBUG_PASSES=1 prints one line
    // per pass, `[*] name ops: N -> M` (asterisk = the pass changed the program; PassManager.swift:255-278).
    const char* dbg = getenv("METALHLO_DEBUG_PASSES");
    const bool debug = dbg && !strcmp(dbg, "1");
    auto run = [&](const char* name, auto&& try_at) {
        if (disabled && disabled->count(name)) return;
        const size_t before = fn.ops.size();
        const int fused_before = rw.fused;
        rw.pass(try_at);
        if (debug) fprintf(stderr, "[%c] %s ops: %zu -> %zu\n", rw.fused != fused_before ? '*' : ' ', name, before, fn.ops.size());
    };
    run("softmax-fusion", [&](size_t i) { rw.softmax(i); });
    run("gelu-fusion", [&](size_t i) { rw.gelu(i) || rw.gelu_erf(i); });
    run("norm-fusion", [&](size_t i) { rw.norm(i); });
    run("attention-fusion", [&](size_t i) { rw.attention(i); });
    run("matmul-bias-act-fusion", [&](size_t i) { rw.matmul_bias_act(i); });
    run("transpose-folding", [&](size_t i) { rw.attention_views(i); });
    run("residual-chain-fusion", [&](size_t i) { rw.matmul_residual(i); });
    // no counterpart among the reference's passes: the lookup at the head of a language model
    run("embedding-fusion", [&](size_t i) { rw.embedding(i); });
    return rw.fused;
}

// The text front end with the environment's diagnostics: parse (calls inlined), recognise the
// fused patterns unless the level is O0, write the result to the file METALHLO_DUMP_OPTIMIZED
// names (one line per operation: result = name inputs=[...]; Compiler/MetalHLOCompiler.swift:205-218).
// METALHLO_DISABLED_PASSES (comma-separated pass names) is honoured on every surface.
Function build_function(const std::string& text, int opt_level) {
    Function fn = parse_module(text);
    std::set<std::string> disabled;
    if (const char* d = getenv("METALHLO_DISABLED_PASSES")) {
        std::string cur;
        for (const char* c = d;; c++) {
            if (*c == ',' || *c == 0) {
                if (!cur.empty()) disabled.insert(cur);
                cur.clear();
                if (!*c) break;
            } else if (*c != ' ') {
                cur += *c;
            }
        }
    }
    if (opt_level >= 1) fuse_patterns(fn, &disabled);
    if (const char* path = getenv("METALHLO_DUMP_OPTIMIZED")) {
        if (FILE* f = fopen(path, "w")) {
            fprintf(f, "// optimized IR -- %zu ops\n", fn.ops.size());
            for (const Op& op : fn.ops) {
                fprintf(f, "%%%d = %s inputs=[", op.result, op.name == "custom_call" ? op.target.c_str() : op.name.c_str());
                for (size_t i = 0; i < op.operands.size(); i++) fprintf(f, "%s%%%d", i ? "," : "", op.operands[i]);
                fprintf(f, "]%s%s\n", op.backend_config.empty() ? "" : " config=", op.backend_config.c_str());
            }
            fclose(f);
        }
    }
    return fn;
}

}  // namespace mhlo
