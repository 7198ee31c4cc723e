#include "codegen.hpp"

#include <algorithm>
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <map>
#include <set>
#include <sstream>

namespace dsc {

namespace {

using std::string;
using std::to_string;

string S(int64_t v) { return to_string((long long)v); }

string hex32(uint32_t bits) {
    char buf[16];
    std::snprintf(buf, sizeof buf, "0x%08xu", bits);
    return buf;
}

const int64_t kMaxIndex = (int64_t)1 << 31;

// Largest linear index (+1) a view may produce into its input, i.e. the input's element count.
int64_t input_extent(const dsc_view& v) { return element_count(v.in_shape); }

// How a linear element id was formed from named integer coordinates: id = base + sum coef_i * name_i with
// name_i in [0, extent_i).  Lets a consumer's coordinates be turned into a producer's coordinates digit by
// digit (no division of the combined id) whenever the terms occupy disjoint digit ranges.
struct IndexForm {
    bool valid = false;
    int64_t base = 0;
    std::vector<string> names;
    std::vector<int64_t> coefs, extents;
};

bool is_identifier(const string& s) {
    if (s.empty() || !(std::isalpha((unsigned char)s[0]) || s[0] == '_')) return false;
    for (char c : s)
        if (!(std::isalnum((unsigned char)c) || c == '_')) return false;
    return true;
}

// A leaky ReLU as the reference writes it, select(x > 0, x, x * c) with a literal 0 < c < 1: the larger of x and x * c
// (for x > 0 that is x, for x < 0 it is x * c, and where the two are equal -- zeros, infinities -- either is the
// value; a NaN x gives NaN both ways).  One v_max_f32 where the select is a compare, a wait for its mask and a
// conditional move.
bool leaky_relu_select(const dsc_kernel_desc& pe, const dsc_pe_op& op) {
    if (op.kind != DSC_PE_SELECT || op.op != DSC_CMP_GT || op.args[2] != op.args[0]) return false;
    const dsc_pe_op& zero = pe.ops[op.args[1]];
    const dsc_pe_op& scaled = pe.ops[op.args[3]];
    if (zero.kind != DSC_PE_LITERAL_F32 || zero.bits != 0u || scaled.kind != DSC_PE_BINARY || scaled.op != DSC_BIN_MUL) return false;
    int lit = -1;
    if (scaled.args[0] == op.args[0]) lit = scaled.args[1];
    else if (scaled.args[1] == op.args[0]) lit = scaled.args[0];
    if (lit < 0 || pe.ops[lit].kind != DSC_PE_LITERAL_F32) return false;
    float c;
    std::memcpy(&c, &pe.ops[lit].bits, 4);
    return c > 0.f && c < 1.f;
}

struct Emitter {
    const FusedKernel& fk;
    std::ostringstream funcs;  // device functions, emitted before the kernel
    std::map<string, string> instances;  // (virtual, index form signature) -> function name

    explicit Emitter(const FusedKernel& k) : fk(k) {}

    // ---- parameters ---------------------------------------------------------------------------------
    string params_decl() const {
        string s;
        for (int i = 0; i < fk.n_buffers; ++i) {
            if (i) s += ", ";
            s += (fk.buffer_is_output[i] ? "float* __restrict__ b" : "const float* __restrict__ b") + to_string(i);
        }
        s += (fk.n_buffers ? ", " : "");
        s += "uint rand_seed";
        return s;
    }
    // The __global__ signature: the seed arrives by value, or -- when seed_cell is not null -- through a one-word
    // device cell, so that a captured launch sequence can be replayed with a new seed without touching its
    // kernel arguments.
    string kernel_params_decl() const {
        string s;
        for (int i = 0; i < fk.n_buffers; ++i)
            s += (fk.buffer_is_output[i] ? "float* __restrict__ b" : "const float* __restrict__ b") + to_string(i) + ", ";
        return s + "const uint* __restrict__ seed_cell, const uint seed_value";
    }
    string params_pass() const {
        string s;
        for (int i = 0; i < fk.n_buffers; ++i) s += "b" + to_string(i) + ", ";
        return s + "rand_seed";
    }

    // ---- coordinates --------------------------------------------------------------------------------
    // Emits the row-major decomposition of `gid` over `shape` as ints named <pfx>0.. and returns the names.
    std::vector<string> emit_coords(std::ostream& o, const dsc_shape& shape, const string& gid, const string& pfx) {
        std::vector<string> names(shape.rank);
        if (shape.rank == 1) {
            names[0] = pfx + "0";
            o << "    const int " << names[0] << " = (int)(" << gid << ");\n";
            return names;
        }
        const string rem = pfx + "r";
        o << "    uint " << rem << " = (uint)(" << gid << ");\n";
        for (int i = shape.rank - 1; i >= 1; --i) {
            names[i] = pfx + to_string(i);
            if (shape.dims[i] == 1) {
                o << "    const int " << names[i] << " = 0;\n";
            } else {
                o << "    const int " << names[i] << " = (int)(" << rem << " % " << S(shape.dims[i]) << "u); " << rem
                  << " /= " << S(shape.dims[i]) << "u;\n";
            }
        }
        names[0] = pfx + "0";
        o << "    const int " << names[0] << " = (int)" << rem << ";\n";
        return names;
    }

    // Decomposition of an id given as an IndexForm: every term must start exactly on a digit boundary of
    // `shape` and the terms' digit ranges must not overlap (then no carries cross between them).  Returns an
    // empty vector when the form does not separate.
    std::vector<string> emit_coords_separable(std::ostream& o, const dsc_shape& shape, const IndexForm& form, const string& pfx) {
        if (!form.valid || form.base != 0) return {};
        int64_t st[DSC_MAX_DIM];
        strides_of(shape, st);
        std::vector<int> owner(shape.rank, -1);
        struct Span { int hi, lo; };
        std::vector<Span> spans(form.names.size(), Span{-1, -1});
        for (size_t t = 0; t < form.names.size(); ++t) {
            if (form.coefs[t] == 0 || form.extents[t] <= 1) continue;
            if (form.coefs[t] < 0) return {};
            int lo = -1;
            for (int i = shape.rank - 1; i >= 0; --i)
                if (st[i] == form.coefs[t] && shape.dims[i] > 1) { lo = i; break; }
            if (lo < 0) return {};
            int hi = lo;
            int64_t cover = st[lo] * shape.dims[lo];
            const int64_t need = form.coefs[t] * form.extents[t];
            while (cover < need) {
                if (--hi < 0) return {};
                cover *= shape.dims[hi];
            }
            for (int i = hi; i <= lo; ++i) {
                if (owner[i] >= 0) return {};
                owner[i] = (int)t;
            }
            spans[t] = Span{hi, lo};
        }
        std::vector<string> names(shape.rank);
        for (int i = 0; i < shape.rank; ++i) names[i] = "0";
        for (size_t t = 0; t < form.names.size(); ++t) {
            if (spans[t].lo < 0) continue;
            const int hi = spans[t].hi, lo = spans[t].lo;
            if (hi == lo) { names[lo] = form.names[t]; continue; }
            const string rem = pfx + "q" + to_string(t);
            o << "    uint " << rem << " = (uint)" << form.names[t] << ";\n";
            for (int i = lo; i > hi; --i) {
                names[i] = pfx + to_string(i);
                if (shape.dims[i] == 1) { o << "    const int " << names[i] << " = 0;\n"; continue; }
                o << "    const int " << names[i] << " = (int)(" << rem << " % " << S(shape.dims[i]) << "u); " << rem << " /= "
                  << S(shape.dims[i]) << "u;\n";
            }
            names[hi] = pfx + to_string(hi);
            o << "    const int " << names[hi] << " = (int)" << rem << ";\n";
        }
        return names;
    }

    // Linear index into the view's input for output coordinates `coord` (kernel.rs:89-133).
    string index_expr(const dsc_view& v, const std::vector<string>& coord) const {
        int64_t st[DSC_MAX_DIM];
        strides_of(v.in_shape, st);
        int64_t constant = 0;
        std::map<string, int64_t> affine;  // coordinate name -> coefficient (un-clamped axes folded together)
        string clamped;
        for (int i = 0; i < v.in_shape.rank; ++i) {
            if (!needs_clamp(v, i)) {
                constant += v.in_offset[i] * st[i];
                for (int j = 0; j < v.out_shape.rank; ++j)
                    if (v.map_axis[j] == i && v.out_shape.dims[j] > 1) affine[coord[j]] += v.map_step[j] * st[i];
            } else {
                string e = S(v.in_offset[i]);
                for (int j = 0; j < v.out_shape.rank; ++j)
                    if (v.map_axis[j] == i && v.out_shape.dims[j] > 1) e += " + (" + S(v.map_step[j]) + ")*" + coord[j];
                clamped += " + clampi(" + e + ", 0, " + S(v.in_shape.dims[i] - 1) + ")*" + S(st[i]);
            }
        }
        string e = "(" + S(constant);
        for (auto& kv : affine)
            if (kv.second != 0) e += " + (" + S(kv.second) + ")*" + kv.first;
        return e + clamped + ")";
    }

    // The same index as an IndexForm, when the view needs no clamp and the coordinates are plain names.
    IndexForm index_form(const dsc_view& v, const std::vector<string>& coord) const {
        IndexForm f;
        int64_t coef[DSC_MAX_DIM];
        if (!affine_form(v, &f.base, coef)) return f;
        for (int j = 0; j < v.out_shape.rank; ++j) {
            if (coef[j] == 0 || v.out_shape.dims[j] <= 1) continue;
            if (!is_identifier(coord[j])) return f;
            // the same name on two axes would need a combined extent: give up
            for (auto& n : f.names)
                if (n == coord[j]) return f;
            f.names.push_back(coord[j]);
            f.coefs.push_back(coef[j]);
            f.extents.push_back(v.out_shape.dims[j]);
        }
        f.valid = true;
        return f;
    }

    // The index as one term per axis of the view's input (clamped where the view pads), for views index_form gives up on.
    bool axis_form(const dsc_view& v, const std::vector<string>& coord, IndexForm* f, std::vector<string>* args) const {
        int64_t st[DSC_MAX_DIM];
        strides_of(v.in_shape, st);
        for (int i = 0; i < v.in_shape.rank; ++i) {
            if (v.in_shape.dims[i] <= 1) continue;
            string e = S(v.in_offset[i]);
            bool driven = false;
            for (int j = 0; j < v.out_shape.rank; ++j)
                if (v.map_axis[j] == i && v.out_shape.dims[j] > 1) {
                    e += " + (" + S(v.map_step[j]) + ")*" + coord[j];
                    driven = true;
                }
            if (!driven) {
                if (v.in_offset[i] != 0) return false;  // a fixed slice of the producer: the linear form handles it
                continue;
            }
            if (needs_clamp(v, i)) e = "clampi(" + e + ", 0, " + S(v.in_shape.dims[i] - 1) + ")";
            args->push_back("(" + e + ")");
            f->names.push_back("axis" + to_string(i));
            f->coefs.push_back(st[i]);
            f->extents.push_back(v.in_shape.dims[i]);
        }
        if (args->empty()) return false;
        f->valid = true;
        return true;
    }

    // Expression for the element of source `s` that view `v` selects at coordinates `coord`.
    string load_view(const Source& s, const dsc_view& v, const std::vector<string>& coord) {
        if (s.buffer >= 0) return "b" + to_string(s.buffer) + "[" + index_expr(v, coord) + "]";
        IndexForm form = index_form(v, coord);
        if (!form.valid) {
            // a padded (clamped) view: one argument per axis of the producer, the clamp applied here, so that a
            // coordinate that is a constant at the call stays one inside the producer
            IndexForm per_axis;
            std::vector<string> args;
            if (axis_form(v, coord, &per_axis, &args)) {
                const string fn = instantiate(s.virt, per_axis);
                string list;
                for (auto& a : args) list += a + ", ";
                return fn + "(" + list + params_pass() + ")";
            }
            const string fn = instantiate(s.virt, IndexForm{});
            return fn + "(" + index_expr(v, coord) + ", " + params_pass() + ")";
        }
        const string fn = instantiate(s.virt, form);
        string args;
        for (auto& n : form.names) args += n + ", ";
        return fn + "(" + args + params_pass() + ")";
    }
    // Element `idx` (a linear id expression) of source `s`.
    string load_linear(const Source& s, const string& idx) {
        if (s.buffer >= 0) return "b" + to_string(s.buffer) + "[" + idx + "]";
        return instantiate(s.virt, IndexForm{}) + "(" + idx + ", " + params_pass() + ")";
    }

    // A device function evaluating virtual producer `virt` for ids of the given form: parameters are the
    // form's coordinates (or the linear id when the form is invalid), then the kernel's parameters.
    string instantiate(int virt, const IndexForm& form) {
        string sig = to_string(virt) + "|";
        if (form.valid) {
            sig += S(form.base);
            for (size_t t = 0; t < form.names.size(); ++t) sig += "," + S(form.coefs[t]) + "x" + S(form.extents[t]);
        } else {
            sig += "lin";
        }
        auto it = instances.find(sig);
        if (it != instances.end()) return it->second;
        const string name = "virt" + to_string(virt) + "_" + to_string(instances.size());
        instances[sig] = name;
        const Virtual& vi = fk.virtuals[virt];
        std::ostringstream body;
        IndexForm local;  // the form re-expressed over this function's own parameter names
        string decl;
        if (form.valid) {
            local = form;
            string gid = S(form.base);
            for (size_t t = 0; t < form.names.size(); ++t) {
                local.names[t] = "a" + to_string(t);
                decl += "int a" + to_string(t) + ", ";
                gid += " + (" + S(form.coefs[t]) + ")*a" + to_string(t);
            }
            body << "    const int gid = " << gid << ";\n";
        } else {
            decl = "int gid, ";
        }
        const dsc_kernel_desc& pd = vi.pe.raw();
        if (pd.kind == DSC_KERNEL_PER_ELEMENT) {
            emit_pe(body, pd, vi.inputs, "gid", "v", {}, form.valid ? &local : nullptr);
            body << "    return vt" << vi.out_op << ";\n";
        } else if (pd.kind == DSC_KERNEL_UNPAD) {
            // one element of an Unpad on demand: the padded elements that the replicate padding took from it, in the
            // standalone kernel's order (src/kernel.rs:645-710); one of them away from the border
            const dsc_view& v = pd.inputs[0];
            std::vector<string> oc;
            if (form.valid) oc = emit_coords_separable(body, pd.shape, local, "vo");
            if (oc.empty()) oc = emit_coords(body, pd.shape, "gid", "vo");
            body << "    const int in_c = " << oc[pd.axis] << " + " << pd.pad << ";\n";
            body << "    const int k_min = in_c - ((" << oc[pd.axis] << " == 0) ? " << pd.pad << " : 0);\n";
            body << "    const int k_max = in_c + ((" << oc[pd.axis] << " == " << S(pd.shape.dims[pd.axis] - 1) << ") ? " << pd.pad << " : 0);\n";
            body << "    float acc = 0.f;\n    for (int kk = k_min; kk <= k_max; ++kk) {\n";
            auto ic = oc;
            ic[pd.axis] = "kk";
            body << "        acc += " << load_view(vi.inputs[0], v, ic) << ";\n    }\n    return acc;\n";
        } else if (pd.kind == DSC_KERNEL_WINDOWS_TO_IMAGE) {
            // one pixel of a WindowsToImage on demand: the windows that cover it, in the standalone kernel's order
            // (src/kernel.rs:713-810, with the test that the window exists)
            const dsc_view& v = pd.inputs[0];
            const int r = v.out_shape.rank, bd = pd.shape.rank - 3;
            const int64_t out_h = v.out_shape.dims[r - 6], out_w = v.out_shape.dims[r - 5];
            const int64_t fh = v.out_shape.dims[r - 3], fw = v.out_shape.dims[r - 2], group_nc = v.out_shape.dims[r - 1];
            const int64_t sw = pd.stride_w, sh = pd.stride_h;
            std::vector<string> oc;
            if (form.valid) oc = emit_coords_separable(body, pd.shape, local, "vo");
            if (oc.empty()) oc = emit_coords(body, pd.shape, "gid", "vo");
            body << "    const int in_y = " << oc[bd] << ", in_x = " << oc[bd + 1] << ", in_c = " << oc[bd + 2] << ";\n";
            body << "    const int group_index = in_c / " << S(group_nc) << ", group_c = in_c % " << S(group_nc) << ";\n";
            body << "    const int fbx = in_x % " << S(sw) << ", fby = in_y % " << S(sh) << ";\n";
            body << "    const int oxb = in_x / " << S(sw) << ", oyb = in_y / " << S(sh) << ";\n";
            body << "    float acc = 0.f;\n";
            body << "#pragma unroll\n    for (int iy = 0; iy < " << S((fh + sh - 1) / sh) << "; ++iy)\n";
            body << "#pragma unroll\n    for (int ix = 0; ix < " << S((fw + sw - 1) / sw) << "; ++ix) {\n";
            body << "        const int fx = fbx + " << S(sw) << " * ix, fy = fby + " << S(sh) << " * iy;\n";
            body << "        const int ox = oxb - ix, oy = oyb - iy;\n";
            // (as in the standalone kernel, a tap without a window reads a valid element and adds zero: the taps' loads
            // are then independent of the tests and in flight together -- behind a branch each, they were four round
            // trips one after another)
            body << "        const bool ok = fx < " << S(fw) << " && fy < " << S(fh) << " && ox >= 0 && ox < " << S(out_w) << " && oy >= 0 && oy < " << S(out_h) << ";\n";
            body << "        const int fxc = min(fx, " << S(fw - 1) << "), fyc = min(fy, " << S(fh - 1) << "), oxc = clampi(ox, 0, " << S(out_w - 1)
                 << "), oyc = clampi(oy, 0, " << S(out_h - 1) << ");\n";
            std::vector<string> ic(r);
            for (int i = 0; i < bd; ++i) ic[i] = oc[i];
            ic[bd] = "oyc"; ic[bd + 1] = "oxc"; ic[bd + 2] = "group_index"; ic[bd + 3] = "fyc"; ic[bd + 4] = "fxc"; ic[bd + 5] = "group_c";
            body << "        const float w = " << load_view(vi.inputs[0], v, ic) << ";\n        acc += ok ? w : 0.f;\n    }\n    return acc;\n";
        } else if (pd.kind == DSC_KERNEL_MATMUL) {
            // one element of a product over a very short k on demand (an outer product: the gradient of a depthwise
            // filter's windows), summed in k order with fused multiply-adds like the row-per-thread kernel
            const MatMulDims g = matmul_dims(pd);
            dsc_shape os{};  // the product as the kernel stores it
            os.rank = 3;
            const bool by_rows = pd.output_mode == DSC_MATMUL_ROWS;
            os.dims[0] = by_rows ? g.m : g.batch; os.dims[1] = by_rows ? g.batch : g.m; os.dims[2] = g.n;
            std::vector<string> oc;
            if (form.valid) oc = emit_coords_separable(body, os, local, "vo");
            if (oc.empty()) oc = emit_coords(body, os, "gid", "vo");
            body << "    const int cn = " << oc[2] << ", cm = " << oc[by_rows ? 0 : 1] << ", cb = " << oc[by_rows ? 1 : 0] << ";\n";
            body << "    float acc = 0.f;\n#pragma unroll\n    for (int ck = 0; ck < " << S(g.k) << "; ++ck)\n";
            body << "        acc = fmaf(" << load_view(vi.inputs[0], pd.inputs[0], {"cb", "cm", "ck"}) << ", " << load_view(vi.inputs[1], pd.inputs[1], {"cb", "ck", "cn"}) << ", acc);\n";
            body << "    return acc;\n";
        } else {  // DSC_KERNEL_REDUCE evaluated on demand: one output element = a loop over the reduced axis
            const dsc_view& v = pd.inputs[0];
            std::vector<string> oc;
            if (form.valid) oc = emit_coords_separable(body, pd.shape, local, "vo");
            if (oc.empty()) oc = emit_coords(body, pd.shape, "gid", "vo");
            const bool is_max = pd.reduce_op == DSC_REDUCE_MAX;
            body << "    float acc = " << (is_max ? "U2F(0xff800000u)" : "0.f") << ";\n";
            body << "    for (int kk = 0; kk < " << S(v.out_shape.dims[pd.axis]) << "; ++kk) {\n";
            auto ic = oc;
            ic[pd.axis] = "kk";
            body << "        const float x = " << load_view(vi.inputs[0], v, ic) << ";\n";
            body << "        acc = " << (is_max ? "glsl_max(acc, x)" : "acc + x") << ";\n    }\n";
            body << "    return acc;\n";
        }
        funcs << "DSC_INLINE float " << name << "(" << decl << params_decl() << ") {\n" << body.str() << "}\n\n";
        return name;
    }

    // Decomposition of an id given as an IndexForm whose terms each lie inside one axis of `shape`, several of them
    // possibly inside the same axis (an id over [img, y, x, g, fy, fx] read as [img * y * x, g, fy * fx]): a coordinate
    // is then the sum of its terms, none of which can carry into the next axis.  An axis that one term with the
    // axis' own stride fills keeps the term's name.  Empty when a term straddles axes or an axis could overflow.
    std::vector<string> emit_coords_grouped(std::ostream& o, const dsc_shape& shape, const IndexForm& form, const string& pfx) {
        if (!form.valid || form.base != 0) return {};
        int64_t st[DSC_MAX_DIM];
        strides_of(shape, st);
        std::vector<std::vector<std::pair<int64_t, string>>> parts(shape.rank);
        std::vector<int64_t> reach(shape.rank, 0);
        for (size_t t = 0; t < form.names.size(); ++t) {
            if (form.coefs[t] == 0 || form.extents[t] <= 1) continue;
            if (form.coefs[t] < 0) return {};
            int axis = -1;
            for (int i = 0; i < shape.rank; ++i)
                if (shape.dims[i] > 1 && st[i] <= form.coefs[t]) { axis = i; break; }  // the outermost axis whose stride the term reaches
            if (axis < 0 || form.coefs[t] % st[axis] != 0) return {};
            const int64_t mult = form.coefs[t] / st[axis];
            parts[axis].push_back({mult, form.names[t]});
            reach[axis] += mult * (form.extents[t] - 1);
        }
        std::vector<string> names(shape.rank);
        for (int i = 0; i < shape.rank; ++i) {
            if (reach[i] >= shape.dims[i]) return {};
            if (parts[i].empty()) { names[i] = "0"; continue; }
            if (parts[i].size() == 1 && parts[i][0].first == 1) { names[i] = parts[i][0].second; continue; }
            names[i] = pfx + "g" + to_string(i);
            o << "    const int " << names[i] << " = ";
            for (size_t j = 0; j < parts[i].size(); ++j) o << (j ? " + " : "") << "(" << S(parts[i][j].first) << ")*" << parts[i][j].second;
            o << ";\n";
        }
        return names;
    }

    // ---- four elements along any coordinate -----------------------------------------------------------
    // The elements of source `s` that view `v` selects at coord, with coordinate `q` taking coord[q] .. coord[q] + 3
    // (a multiple of four inside an extent that is one), as a float4.  Where the quad's elements are not neighbours
    // in the source -- four groups of a depthwise convolution, far apart in a product's own layout -- the index
    // arithmetic of every level is still done once per quad, and the buffers at the end are read with one 16-byte load
    // where the quad does walk memory there (the four channels of a pixel), with four words otherwise.  "" when a
    // level cannot be evaluated that way (the caller then evaluates single elements).
    string load_view_q(const Source& s, const dsc_view& v, const std::vector<string>& coord, int q) {
        if (q < 0 || q >= v.out_shape.rank || v.out_shape.dims[q] % 4 != 0 || !is_identifier(coord[q])) return "";
        int64_t base = 0, coef[DSC_MAX_DIM];
        if (!affine_form(v, &base, coef)) return "";
        if (s.buffer >= 0) {
            const string b = "b" + to_string(s.buffer), idx = index_expr(v, coord);
            if (coef[q] == 0) return "dsc_splat4(" + b + "[" + idx + "])";
            bool aligned = coef[q] == 1 && base % 4 == 0;
            for (int j = 0; j < v.out_shape.rank; ++j)
                if (j != q && v.out_shape.dims[j] > 1 && coef[j] % 4 != 0) aligned = false;
            if (aligned) return "*(const float4*)(" + b + " + " + idx + ")";
            return "dsc_load4_strided(" + b + " + " + idx + ", " + S(coef[q]) + ")";
        }
        if (coef[q] == 0) {
            const string one = load_view(s, v, coord);
            return "dsc_splat4(" + one + ")";
        }
        IndexForm form = index_form(v, coord);
        if (!form.valid) return "";
        int qt = -1;
        for (size_t t = 0; t < form.names.size(); ++t)
            if (form.names[t] == coord[q]) qt = (int)t;
        if (qt < 0) return "";
        string fn;
        {
            // four consecutive ids of a per-element or Reduce producer: the form for consecutive quads knows every op
            const int vk = fk.virtuals[s.virt].pe.raw().kind;
            if ((vk == DSC_KERNEL_PER_ELEMENT || vk == DSC_KERNEL_REDUCE) && form.coefs[qt] == 1) {
                IndexForm last = form;  // the quad's term last, as that form wants it
                std::swap(last.names[qt], last.names.back());
                std::swap(last.coefs[qt], last.coefs.back());
                std::swap(last.extents[qt], last.extents.back());
                const string f4 = instantiate4(s.virt, last);
                if (!f4.empty()) {
                    string args4;
                    for (auto& n : last.names) args4 += n + ", ";
                    return f4 + "(" + args4 + params_pass() + ")";
                }
            }
        }
        fn = instantiate_q(s.virt, form, qt);
        if (fn.empty()) return "";
        string args;
        for (auto& n : form.names) args += n + ", ";
        return fn + "(" + args + params_pass() + ")";
    }

    // The float4 of virtual producer `virt` for ids of the given form whose term `qt` takes its coordinate .. + 3.
    string instantiate_q(int virt, const IndexForm& form, int qt) {
        if (!form.valid || form.extents[qt] % 4 != 0) return "";
        string sig = "Q" + to_string(virt) + "|" + to_string(qt) + "|" + S(form.base);
        for (size_t t = 0; t < form.names.size(); ++t) sig += "," + S(form.coefs[t]) + "x" + S(form.extents[t]);
        auto it = instances.find(sig);
        if (it != instances.end()) return it->second;
        const Virtual& vi = fk.virtuals[virt];
        const dsc_kernel_desc& pd = vi.pe.raw();
        const string name = "virt" + to_string(virt) + "_" + to_string(instances.size()) + "_q";
        instances[sig] = name;  // (the graph of virtuals is acyclic)
        IndexForm local = form;
        string decl;
        for (size_t t = 0; t < form.names.size(); ++t) {
            local.names[t] = "a" + to_string(t);
            decl += "int a" + to_string(t) + ", ";
        }
        const string qname = local.names[qt];
        std::ostringstream body;
        auto fail = [&]() { return instances[sig] = ""; };
        // the axis of `shape` that the quad's term is the coordinate of
        auto axis_of_quad = [&](const std::vector<string>& oc) {
            for (size_t i = 0; i < oc.size(); ++i)
                if (oc[i] == qname) return (int)i;
            return -1;
        };
        const char* add4 = "    acc = make_float4(acc.x + w.x, acc.y + w.y, acc.z + w.z, acc.w + w.w);\n";
        if (pd.kind == DSC_KERNEL_PER_ELEMENT) {
            // a pure copy hands the quad on through its view; anything else is not evaluated this way
            if (!(pd.n_inputs == 1 && pd.n_outputs == 1 && pd.n_ops >= 1 && pd.n_ops <= 2 && pd.ops[0].kind == DSC_PE_LOAD &&
                  (pd.n_ops == 1 || (pd.ops[1].kind == DSC_PE_UNARY && pd.ops[1].op == DSC_UN_MOV && pd.ops[1].args[0] == 0)) &&
                  vi.out_op == pd.n_ops - 1))
                return fail();
            const dsc_view& v = pd.inputs[0];
            std::vector<string> oc = emit_coords_separable(body, v.out_shape, local, "vo");
            if (oc.empty()) oc = emit_coords_grouped(body, v.out_shape, local, "vo");
            const int qa = oc.empty() ? -1 : axis_of_quad(oc);
            if (qa < 0) return fail();
            const string x = load_view_q(vi.inputs[0], v, oc, qa);
            if (x.empty()) return fail();
            body << "    return " << x << ";\n";
        } else if (pd.kind == DSC_KERNEL_UNPAD) {
            const dsc_view& v = pd.inputs[0];
            std::vector<string> oc = emit_coords_separable(body, pd.shape, local, "vo");
            if (oc.empty()) oc = emit_coords_grouped(body, pd.shape, local, "vo");
            const int qa = oc.empty() ? -1 : axis_of_quad(oc);
            if (qa < 0 || qa == pd.axis) return fail();
            auto ic = oc;
            ic[pd.axis] = "kk";
            const string x = load_view_q(vi.inputs[0], v, ic, qa);
            if (x.empty()) return fail();
            body << "    const int in_c = " << oc[pd.axis] << " + " << pd.pad << ";\n";
            body << "    const int k_min = in_c - ((" << oc[pd.axis] << " == 0) ? " << pd.pad << " : 0);\n";
            body << "    const int k_max = in_c + ((" << oc[pd.axis] << " == " << S(pd.shape.dims[pd.axis] - 1) << ") ? " << pd.pad << " : 0);\n";
            body << "    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);\n    for (int kk = k_min; kk <= k_max; ++kk) {\n";
            body << "        const float4 w = " << x << ";\n    " << add4 << "    }\n    return acc;\n";
        } else if (pd.kind == DSC_KERNEL_WINDOWS_TO_IMAGE) {
            const dsc_view& v = pd.inputs[0];
            const int r = v.out_shape.rank, bd = pd.shape.rank - 3;
            const int64_t out_h = v.out_shape.dims[r - 6], out_w = v.out_shape.dims[r - 5];
            const int64_t fh = v.out_shape.dims[r - 3], fw = v.out_shape.dims[r - 2], group_nc = v.out_shape.dims[r - 1];
            const int64_t sw = pd.stride_w, sh = pd.stride_h;
            std::vector<string> oc = emit_coords_separable(body, pd.shape, local, "vo");
            if (oc.empty()) oc = emit_coords_grouped(body, pd.shape, local, "vo");
            const int qa = oc.empty() ? -1 : axis_of_quad(oc);
            // the quad runs over channels: four of one group, or four groups of one channel each
            if (qa != bd + 2 || !(group_nc % 4 == 0 || group_nc == 1)) return fail();
            std::vector<string> ic(r);
            for (int i = 0; i < bd; ++i) ic[i] = oc[i];
            ic[bd] = "oyc"; ic[bd + 1] = "oxc"; ic[bd + 2] = "group_index"; ic[bd + 3] = "fyc"; ic[bd + 4] = "fxc"; ic[bd + 5] = "group_c";
            const string x = load_view_q(vi.inputs[0], v, ic, group_nc == 1 ? bd + 2 : bd + 5);
            if (x.empty()) return fail();
            body << "    const int in_y = " << oc[bd] << ", in_x = " << oc[bd + 1] << ", in_c = " << oc[bd + 2] << ";\n";
            body << "    const int group_index = in_c / " << S(group_nc) << ", group_c = in_c % " << S(group_nc) << ";\n";
            body << "    const int fbx = in_x % " << S(sw) << ", fby = in_y % " << S(sh) << ";\n";
            body << "    const int oxb = in_x / " << S(sw) << ", oyb = in_y / " << S(sh) << ";\n";
            body << "    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);\n";
            body << "#pragma unroll\n    for (int iy = 0; iy < " << S((fh + sh - 1) / sh) << "; ++iy)\n";
            body << "#pragma unroll\n    for (int ix = 0; ix < " << S((fw + sw - 1) / sw) << "; ++ix) {\n";
            body << "        const int fx = fbx + " << S(sw) << " * ix, fy = fby + " << S(sh) << " * iy;\n";
            body << "        const int ox = oxb - ix, oy = oyb - iy;\n";
            body << "        const bool ok = fx < " << S(fw) << " && fy < " << S(fh) << " && ox >= 0 && ox < " << S(out_w) << " && oy >= 0 && oy < " << S(out_h) << ";\n";
            body << "        const int fxc = min(fx, " << S(fw - 1) << "), fyc = min(fy, " << S(fh - 1) << "), oxc = clampi(ox, 0, " << S(out_w - 1)
                 << "), oyc = clampi(oy, 0, " << S(out_h - 1) << ");\n";
            body << "        const float4 w = " << x << ";\n";
            body << "        acc = make_float4(acc.x + (ok ? w.x : 0.f), acc.y + (ok ? w.y : 0.f), acc.z + (ok ? w.z : 0.f), acc.w + (ok ? w.w : 0.f));\n    }\n";
            body << "    return acc;\n";
        } else if (pd.kind == DSC_KERNEL_MATMUL) {
            const MatMulDims g = matmul_dims(pd);
            dsc_shape os{};
            os.rank = 3;
            const bool by_rows = pd.output_mode == DSC_MATMUL_ROWS;
            os.dims[0] = by_rows ? g.m : g.batch; os.dims[1] = by_rows ? g.batch : g.m; os.dims[2] = g.n;
            std::vector<string> oc = emit_coords_separable(body, os, local, "vo");
            if (oc.empty()) oc = emit_coords_grouped(body, os, local, "vo");
            const int qa = oc.empty() ? -1 : axis_of_quad(oc);
            if (qa < 0) return fail();
            const string cb = oc[by_rows ? 1 : 0], cm = oc[by_rows ? 0 : 1], cn = oc[2];
            const int q_is = qa == 2 ? 2 : (qa == (by_rows ? 1 : 0) ? 0 : 1);  // 0: batch, 1: row, 2: column
            // (coordinates that are literal zeros -- an extent of one -- are passed as they are: their axes carry no term)
            const string xa = q_is == 2 ? "dsc_splat4(" + load_view(vi.inputs[0], pd.inputs[0], {cb, cm, "ck"}) + ")" : load_view_q(vi.inputs[0], pd.inputs[0], {cb, cm, "ck"}, q_is == 0 ? 0 : 1);
            const string xb = q_is == 1 ? "dsc_splat4(" + load_view(vi.inputs[1], pd.inputs[1], {cb, "ck", cn}) + ")" : load_view_q(vi.inputs[1], pd.inputs[1], {cb, "ck", cn}, q_is == 0 ? 0 : 2);
            if (xa.empty() || xb.empty()) return fail();
            body << "    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);\n#pragma unroll\n    for (int ck = 0; ck < " << S(g.k) << "; ++ck) {\n";
            body << "        const float4 x = " << xa << ";\n        const float4 y = " << xb << ";\n";
            body << "        acc = make_float4(fmaf(x.x, y.x, acc.x), fmaf(x.y, y.y, acc.y), fmaf(x.z, y.z, acc.z), fmaf(x.w, y.w, acc.w));\n    }\n";
            body << "    return acc;\n";
        } else {
            return fail();
        }
        funcs << "DSC_INLINE float4 " << name << "(" << decl << params_decl() << ") {\n" << body.str() << "}\n\n";
        return name;
    }

    // ---- four consecutive elements at once ------------------------------------------------------------
    // A consumer that wants elements id .. id + 3 of a source, id a multiple of four and the four of them inside one
    // run of the innermost axis of every view on the way, gets them from ONE evaluation: the index arithmetic of each
    // view (the divisions by its extents) is done once for the quad, a buffer is read with one 16-byte load where its
    // innermost axis walks memory (or one word, where the view repeats an element along that axis), and only the
    // arithmetic is done four times.  The reference has no counterpart: it evaluates one element per invocation
    // (src/kernel.rs:196-383).  Everything returns "" where a quad cannot be formed; callers then fall back on four
    // single evaluations.
    //
    // The view's element for the quad that starts at coordinates `coord` (the last one a multiple of four).
    string load_view4(const Source& s, const dsc_view& v, const std::vector<string>& coord) {
        const int L = v.out_shape.rank - 1;
        if (L < 0 || v.out_shape.dims[L] % 4 != 0) return "";
        int64_t base = 0, coef[DSC_MAX_DIM];
        if (!affine_form(v, &base, coef)) return "";
        if (v.out_shape.dims[L] > 1 && coef[L] == 0) {  // the same element four times
            const string one = load_view(s, v, coord);
            return "dsc_splat4(" + one + ")";
        }
        if (coef[L] != 1) return "";
        if (s.buffer >= 0) {
            bool aligned = base % 4 == 0;
            for (int j = 0; j < L; ++j)
                if (v.out_shape.dims[j] > 1 && coef[j] % 4 != 0) aligned = false;
            const string idx = index_expr(v, coord);
            const string b = "b" + to_string(s.buffer);
            if (aligned) return "*(const float4*)(" + b + " + " + idx + ")";
            return "dsc_load4_unaligned(" + b + " + " + idx + ")";
        }
        IndexForm form = index_form(v, coord);
        if (!form.valid || form.names.empty() || form.names.back() != coord[L] || form.coefs.back() != 1) return "";
        const string fn = instantiate4(s.virt, form);
        if (fn.empty()) return "";
        string args;
        for (auto& n : form.names) args += n + ", ";
        return fn + "(" + args + params_pass() + ")";
    }

    // The float4 counterpart of `instantiate`: elements id .. id + 3 of virtual producer `virt`, where the form's last
    // term is the quad's coordinate (coefficient one, a multiple of four at every call) and every other term moves the
    // id by a multiple of four.  "" when the producer cannot be evaluated that way.
    string instantiate4(int virt, const IndexForm& form) {
        if (!form.valid || form.names.empty() || form.coefs.back() != 1 || form.extents.back() % 4 != 0 || form.base % 4 != 0) return "";
        for (size_t t = 0; t + 1 < form.names.size(); ++t)
            if (form.coefs[t] % 4 != 0) return "";
        string sig = "q" + to_string(virt) + "|" + S(form.base);
        for (size_t t = 0; t < form.names.size(); ++t) sig += "," + S(form.coefs[t]) + "x" + S(form.extents[t]);
        auto it = instances.find(sig);
        if (it != instances.end()) return it->second;
        const Virtual& vi = fk.virtuals[virt];
        const dsc_kernel_desc& pd = vi.pe.raw();
        // (gathered sums evaluated on demand have one quad form, along any coordinate: here the last term's)
        if (pd.kind == DSC_KERNEL_UNPAD || pd.kind == DSC_KERNEL_WINDOWS_TO_IMAGE || pd.kind == DSC_KERNEL_MATMUL)
            return instances[sig] = instantiate_q(virt, form, (int)form.names.size() - 1);
        if (pd.kind != DSC_KERNEL_PER_ELEMENT && pd.kind != DSC_KERNEL_REDUCE) return instances[sig] = "";
        const string name = "virt" + to_string(virt) + "_" + to_string(instances.size()) + "_x4";
        instances[sig] = name;  // (a producer never reads itself: the graph of virtuals is acyclic)
        IndexForm local = form;
        string decl, gid = S(form.base);
        for (size_t t = 0; t < form.names.size(); ++t) {
            local.names[t] = "a" + to_string(t);
            decl += "int a" + to_string(t) + ", ";
            gid += " + (" + S(form.coefs[t]) + ")*a" + to_string(t);
        }
        std::ostringstream body;
        body << "    const int gid = " << gid << ";\n";
        if (pd.kind == DSC_KERNEL_REDUCE) {
            // four neighbouring results of a reduction along another axis than the innermost: one loop, quads added up
            const dsc_view& v = pd.inputs[0];
            const int L = pd.shape.rank - 1;
            if (L < 1 || pd.axis == L || pd.shape.dims[L] % 4 != 0) return instances[sig] = "";
            std::vector<string> oc = emit_coords_separable(body, pd.shape, local, "vo");
            if (oc.empty()) oc = emit_coords(body, pd.shape, "gid", "vo");
            auto ic = oc;
            ic[pd.axis] = "kk";
            const string x = load_view4(vi.inputs[0], v, ic);
            if (x.empty()) return instances[sig] = "";
            const bool is_max = pd.reduce_op == DSC_REDUCE_MAX;
            const string init = is_max ? "U2F(0xff800000u)" : "0.f";
            body << "    float4 acc = make_float4(" << init << ", " << init << ", " << init << ", " << init << ");\n";
            body << "    for (int kk = 0; kk < " << S(v.out_shape.dims[pd.axis]) << "; ++kk) {\n        const float4 x = " << x << ";\n";
            if (is_max) body << "        acc = make_float4(glsl_max(acc.x, x.x), glsl_max(acc.y, x.y), glsl_max(acc.z, x.z), glsl_max(acc.w, x.w));\n    }\n";
            else body << "        acc = make_float4(acc.x + x.x, acc.y + x.y, acc.z + x.z, acc.w + x.w);\n    }\n";
            body << "    return acc;\n";
            funcs << "DSC_INLINE float4 " << name << "(" << decl << params_decl() << ") {\n" << body.str() << "}\n\n";
            return name;
        }
        if (!emit_pe4(body, pd, vi.inputs, "gid", "v", &local)) return instances[sig] = "";
        body << "    return make_float4(vt" << vi.out_op << "[0], vt" << vi.out_op << "[1], vt" << vi.out_op << "[2], vt" << vi.out_op << "[3]);\n";
        funcs << "DSC_INLINE float4 " << name << "(" << decl << params_decl() << ") {\n" << body.str() << "}\n\n";
        return name;
    }

    // emit_pe for the quad gid .. gid + 3 (gid a multiple of four): op i is left in the array <pfx>t<i>[4].  False
    // when an op or a load cannot be done for a quad (nothing usable has been emitted then).
    bool emit_pe4(std::ostream& out, const dsc_kernel_desc& pe, const std::vector<Source>& srcs, const string& gid, const string& pfx,
                  const IndexForm* form) {
        std::ostringstream o;
        std::vector<std::pair<dsc_shape, std::vector<string>>> sets;
        auto coords_for = [&](const dsc_shape& shape) -> std::vector<string> {
            for (auto& s : sets)
                if (same_shape(s.first, shape)) return s.second;
            const string cp = pfx + "c" + to_string(sets.size()) + "_";
            std::vector<string> names;
            if (form) names = emit_coords_separable(o, shape, *form, cp);
            if (names.empty()) names = emit_coords(o, shape, gid, cp);
            sets.emplace_back(shape, names);
            return names;
        };
        auto T = [&](int i) { return pfx + "t" + to_string(i); };
        auto each = [&](int i, const std::function<string(int)>& rhs) {
            o << "    const float " << T(i) << "[4] = {" << rhs(0) << ", " << rhs(1) << ", " << rhs(2) << ", " << rhs(3) << "};\n";
        };
        auto E = [&](int i, int e) { return T(i) + "[" + to_string(e) + "]"; };
        for (int i = 0; i < pe.n_ops; ++i) {
            const dsc_pe_op& op = pe.ops[i];
            switch (op.kind) {
            case DSC_PE_LOAD: {
                const dsc_view& v = pe.inputs[op.input_index];
                const int L = v.out_shape.rank - 1;
                if (L < 0 || v.out_shape.dims[L] % 4 != 0) return false;
                const Source& src = srcs[op.input_index];
                string q;
                if (is_identity(v) && src.buffer >= 0) q = "*(const float4*)(b" + to_string(src.buffer) + " + " + gid + ")";
                else if (is_identity(v) && form && form->valid) {
                    // the producer's ids are this function's: hand the coordinates on as they came
                    const string fn = instantiate4(src.virt, *form);
                    if (!fn.empty()) {
                        string args;
                        for (auto& n : form->names) args += n + ", ";
                        q = fn + "(" + args + params_pass() + ")";
                    }
                }
                if (q.empty()) q = load_view4(src, v, coords_for(v.out_shape));
                if (q.empty()) return false;
                o << "    const float4 " << T(i) << "q = " << q << ";\n";
                o << "    const float " << T(i) << "[4] = {" << T(i) << "q.x, " << T(i) << "q.y, " << T(i) << "q.z, " << T(i) << "q.w};\n";
                break;
            }
            case DSC_PE_LITERAL_F32:
            case DSC_PE_LITERAL_U32: each(i, [&](int) { return "U2F(" + hex32(op.bits) + ")"; }); break;
            case DSC_PE_UNARY: {
                const int a = op.args[0];
                switch (op.op) {
                case DSC_UN_MOV: each(i, [&](int e) { return E(a, e); }); break;
                case DSC_UN_NEG: each(i, [&](int e) { return "-" + E(a, e); }); break;
                case DSC_UN_SQRT: each(i, [&](int e) { return "sqrtf(" + E(a, e) + ")"; }); break;
                case DSC_UN_FLOAT_TO_UINT: each(i, [&](int e) { return "U2F((uint)" + E(a, e) + ")"; }); break;
                case DSC_UN_UINT_TO_FLOAT: each(i, [&](int e) { return "(float)F2U(" + E(a, e) + ")"; }); break;
                default: return false;  // transcendental producers stay on the single-element path
                }
                break;
            }
            case DSC_PE_BINARY: {
                const int a = op.args[0], b = op.args[1];
                switch (op.op) {
                case DSC_BIN_ADD: each(i, [&](int e) { return E(a, e) + " + " + E(b, e); }); break;
                case DSC_BIN_SUB: each(i, [&](int e) { return E(a, e) + " - " + E(b, e); }); break;
                case DSC_BIN_MUL: each(i, [&](int e) { return E(a, e) + " * " + E(b, e); }); break;
                case DSC_BIN_DIV: each(i, [&](int e) { return E(a, e) + " / " + E(b, e); }); break;
                case DSC_BIN_UADD: each(i, [&](int e) { return "U2F(F2U(" + E(a, e) + ") + F2U(" + E(b, e) + "))"; }); break;
                case DSC_BIN_UMUL: each(i, [&](int e) { return "U2F(F2U(" + E(a, e) + ") * F2U(" + E(b, e) + "))"; }); break;
                case DSC_BIN_UBITXOR: each(i, [&](int e) { return "U2F(F2U(" + E(a, e) + ") ^ F2U(" + E(b, e) + "))"; }); break;
                default: return false;
                }
                break;
            }
            case DSC_PE_SELECT:
                if (leaky_relu_select(pe, op)) {
                    each(i, [&](int e) { return "fmaxf(" + E(op.args[0], e) + ", " + E(op.args[3], e) + ")"; });
                    break;
                }
                each(i, [&](int e) {
                    return "(" + E(op.args[0], e) + (op.op == DSC_CMP_EQ ? " == " : " > ") + E(op.args[1], e) + ") ? " + E(op.args[2], e) + " : " + E(op.args[3], e);
                });
                break;
            default: return false;  // coordinates, random numbers and gathers differ per element in more than a value
            }
        }
        out << o.str();
        return true;
    }

    // ---- per-element bodies ---------------------------------------------------------------------------
    // Emits the straight-line evaluation of `pe` at linear id `gid`; op i is left in variable <pfx>t<i>.
    // `override_load[input]` replaces the load of that input by an expression.  `form` (optional) says how
    // gid was composed, which lets coordinate sets be derived without dividing gid.
    void emit_pe(std::ostream& o, const dsc_kernel_desc& pe, const std::vector<Source>& srcs, const string& gid,
                 const string& pfx, const std::map<int, string>& override_load, const IndexForm* form = nullptr) {
        std::vector<std::pair<dsc_shape, std::vector<string>>> sets;
        auto coords_for = [&](const dsc_shape& shape) -> std::vector<string> {
            for (auto& s : sets)
                if (same_shape(s.first, shape)) return s.second;
            const string cp = pfx + "c" + to_string(sets.size()) + "_";
            std::vector<string> names;
            if (form) names = emit_coords_separable(o, shape, *form, cp);
            if (names.empty()) names = emit_coords(o, shape, gid, cp);
            sets.emplace_back(shape, names);
            return names;
        };
        auto T = [&](int i) { return pfx + "t" + to_string(i); };
        for (int i = 0; i < pe.n_ops; ++i) {
            const dsc_pe_op& op = pe.ops[i];
            string rhs;
            switch (op.kind) {
            case DSC_PE_LOAD: {
                auto ov = override_load.find(op.input_index);
                if (ov != override_load.end()) { rhs = ov->second; break; }
                const dsc_view& v = pe.inputs[op.input_index];
                // (a fused producer behind an identity view is handed the coordinates when the caller has them taken
                // apart already: it then divides nothing either)
                if (is_identity(v) && !(form && form->valid && srcs[op.input_index].virt >= 0 && v.out_shape.rank > 1))
                    rhs = load_linear(srcs[op.input_index], "(int)(" + gid + ")");
                else rhs = load_view(srcs[op.input_index], v, coords_for(v.out_shape));
                break;
            }
            case DSC_PE_LITERAL_F32:
            case DSC_PE_LITERAL_U32: rhs = "U2F(" + hex32(op.bits) + ")"; break;
            case DSC_PE_COORD: {
                const dsc_view& v = pe.builtin_views[op.view_index];
                rhs = "(float)" + index_expr(v, coords_for(v.out_shape));
                break;
            }
            case DSC_PE_RAND: {
                const dsc_view& v = pe.builtin_views[op.view_index];
                string idx = is_identity(v) ? "(int)(" + gid + ")" : index_expr(v, coords_for(v.out_shape));
                rhs = "rand_from_index(rand_seed, " + S(op.bits) + "u, " + idx + ")";
                break;
            }
            case DSC_PE_UNARY: {
                const string a = T(op.args[0]);
                switch (op.op) {
                case DSC_UN_MOV: rhs = a; break;
                case DSC_UN_NEG: rhs = "-" + a; break;
                case DSC_UN_SQRT: rhs = "sqrtf(" + a + ")"; break;
                case DSC_UN_EXP: rhs = "expf(" + a + ")"; break;
                case DSC_UN_LOG: rhs = "logf(" + a + ")"; break;
                case DSC_UN_SIN: rhs = "dsc_sin(" + a + ")"; break;
                case DSC_UN_COS: rhs = "dsc_cos(" + a + ")"; break;
                case DSC_UN_FLOAT_TO_UINT: rhs = "U2F((uint)" + a + ")"; break;
                case DSC_UN_UINT_TO_FLOAT: rhs = "(float)F2U(" + a + ")"; break;
                }
                break;
            }
            case DSC_PE_BINARY: {
                const string a = T(op.args[0]), b = T(op.args[1]);
                switch (op.op) {
                case DSC_BIN_ADD: rhs = a + " + " + b; break;
                case DSC_BIN_SUB: rhs = a + " - " + b; break;
                case DSC_BIN_MUL: rhs = a + " * " + b; break;
                case DSC_BIN_DIV: rhs = a + " / " + b; break;
                case DSC_BIN_POW: rhs = "powf(" + a + ", " + b + ")"; break;
                case DSC_BIN_UADD: rhs = "U2F(F2U(" + a + ") + F2U(" + b + "))"; break;
                case DSC_BIN_UMUL: rhs = "U2F(F2U(" + a + ") * F2U(" + b + "))"; break;
                case DSC_BIN_UREM: rhs = "U2F(F2U(" + a + ") % F2U(" + b + "))"; break;
                case DSC_BIN_UBITXOR: rhs = "U2F(F2U(" + a + ") ^ F2U(" + b + "))"; break;
                }
                break;
            }
            case DSC_PE_SELECT:
                if (leaky_relu_select(pe, op)) {
                    rhs = "fmaxf(" + T(op.args[0]) + ", " + T(op.args[3]) + ")";
                    break;
                }
                rhs = "(" + T(op.args[0]) + (op.op == DSC_CMP_EQ ? " == " : " > ") + T(op.args[1]) + ") ? " +
                      T(op.args[2]) + " : " + T(op.args[3]);
                break;
            case DSC_PE_GATHER: {
                const dsc_view& v = pe.inputs[op.input_index];
                auto names = coords_for(op.gather_shape);
                // The index comes from data, so its range is unknown when the kernel is generated.  The reference
                // (kernel.rs:336-351) loads with whatever it gets and leans on Vulkan's bounds-checked buffers; a HIP
                // load has no such net, so the index is clamped to the gathered axis (indices inside it are untouched).
                names[op.axis] = "clampi(F2I(" + T(op.args[0]) + "), 0, " + S(v.out_shape.dims[op.axis] - 1) + ")";
                rhs = load_view(srcs[op.input_index], v, names);
                break;
            }
            }
            o << "    const float " << T(i) << " = " << rhs << ";\n";
        }
    }
};

bool rows_kernel_applies(const FusedKernel& fk, const MatMulDims& g);
bool smallk_kernel_applies(const FusedKernel& fk, const MatMulDims& g);
bool tallk_kernel_applies(const FusedKernel& fk, const MatMulDims& g);
bool ksplit_kernel_applies(const FusedKernel& fk, const MatMulDims& g);
bool dot_kernel_applies(const FusedKernel& fk, const MatMulDims& g);
bool dot_kernel_for_many_rows(const FusedKernel& fk, const MatMulDims& g);

// Entry points carry the kernel kind and its size, so that a profiler's per-name statistics tell the kernels of
// a schedule apart: dsc_matmul_mfma_epilogue_b1_m8192_n8192_k8192, dsc_reduce_k4084_n144, dsc_per_element_n12544000.
string entry_name(const FusedKernel& fk) {
    const dsc_kernel_desc& d = fk.main.raw();
    auto count = [](int64_t v) { return to_string((long long)v); };
    if (fk.dgrad.on) {
        const MatMulDims g = matmul_dims(d);
        return string(fk.dgrad.wgrad_only ? "dsc_conv_wgrad_img" : fk.dgrad.wgrad ? "dsc_conv_bwd_img" : "dsc_conv_dgrad_img") + count(fk.dgrad.img) + "_" + count(fk.dgrad.oh) +
               "x" + count(fk.dgrad.ow) + "_g" + count(fk.dgrad.g) + "_k" + count(fk.dgrad.wgrad_only ? g.n : g.k) + "_c" + count(fk.dgrad.c);
    }
    if (fk.cfwd.on)
        return string(fk.has_epilogue ? "dsc_conv_fwd_epilogue_img" : "dsc_conv_fwd_img") + count(fk.cfwd.img) + "_" + count(fk.cfwd.h) + "x" +
               count(fk.cfwd.w) + "_g" + count(fk.cfwd.g) + "_c" + count(fk.cfwd.c) + "_f" + count(fk.cfwd.fh) + "x" + count(fk.cfwd.fw) + "_n" +
               count(matmul_dims(d).n);
    if (!fk.row_stages.empty()) return "dsc_row_fused_m" + count(fk.row_m) + "_n" + count(fk.row_n) + "_s" + count((int64_t)fk.row_stages.size());
    switch (d.kind) {
    case DSC_KERNEL_FILL: return "dsc_fill_n" + count(d.shape.dims[0]);
    case DSC_KERNEL_PER_ELEMENT: return "dsc_per_element_n" + count(d.shape.dims[0]) + (fk.row_width ? "_rows" + count(fk.row_width) : string());
    case DSC_KERNEL_REDUCE: {
        return string(fk.has_epilogue ? "dsc_reduce_epilogue_k" : "dsc_reduce_k") + count(d.inputs[0].out_shape.dims[d.axis]) + "_n" +
               count(element_count(d.shape));
    }
    case DSC_KERNEL_MATMUL: {
        const MatMulDims g = matmul_dims(d);
        string base = fk.pair.on                     ? "dsc_matmul_shortk"
                      : rows_kernel_applies(fk, g)   ? "dsc_matmul_rows"
                      : smallk_kernel_applies(fk, g) ? "dsc_matmul_shortk"
                      : tallk_kernel_applies(fk, g)  ? "dsc_matmul_tallk"
                      : ksplit_kernel_applies(fk, g) ? "dsc_matmul_ksplit"
                      : dot_kernel_applies(fk, g)    ? "dsc_matmul_dot"
                                                     : "dsc_matmul_mfma";
        if (fk.pair.on) base += "_wgrad";
        if (fk.has_epilogue) base += "_epilogue";
        if (fk.out_slice_width) base += "_slices" + count(fk.out_slice_width);
        return base + "_b" + count(g.batch) + "_m" + count(g.m) + "_n" + count(g.n) + "_k" + count(g.k);
    }
    case DSC_KERNEL_UNPAD: return string(fk.has_epilogue ? "dsc_unpad_epilogue_n" : "dsc_unpad_n") + count(element_count(d.shape));
    case DSC_KERNEL_WINDOWS_TO_IMAGE:
        return string(fk.has_epilogue ? "dsc_windows_to_image_epilogue_n" : "dsc_windows_to_image_n") + count(element_count(d.shape));
    case DSC_KERNEL_SCATTER_ADD: return "dsc_scatter_add_n" + count(element_count(d.inputs[0].out_shape));
    default: return "dsc_kernel";
    }
}

string check_sizes(const FusedKernel& fk) {
    auto chk = [](const dsc_kernel_desc& d) -> string {
        if (element_count(d.shape) >= kMaxIndex) return "kernel too large for 32-bit indexing";
        for (int i = 0; i < d.n_inputs; ++i)
            if (input_extent(d.inputs[i]) >= kMaxIndex || element_count(d.inputs[i].out_shape) >= kMaxIndex)
                return "input too large for 32-bit indexing";
        return "";
    };
    string e = chk(fk.main.raw());
    if (!e.empty()) return e;
    for (auto& v : fk.virtuals) {
        e = chk(v.pe.raw());
        if (!e.empty()) return e;
    }
    for (auto& st : fk.row_stages) {
        e = chk(st.k.raw());
        if (!e.empty()) return e;
    }
    if (fk.has_epilogue) return chk(fk.epilogue.raw());
    return "";
}

// The store of one result of a kernel that takes a fused per-element consumer (Reduce, WindowsToImage, Unpad):
// plain, or through the consumer cluster (emitted once as a device function).
struct ResultStore {
    Emitter& em;
    int n_res = 1;
    explicit ResultStore(Emitter& e) : em(e) {
        const FusedKernel& fk = em.fk;
        if (!fk.has_epilogue) return;
        const dsc_kernel_desc& pe = fk.epilogue.raw();
        n_res = pe.n_outputs;
        std::ostringstream body;
        std::map<int, string> ov;
        ov[fk.epilogue_product_input] = "product";
        em.emit_pe(body, pe, fk.epilogue_inputs, "gid", "e", ov);
        for (int o = 0; o < pe.n_outputs; ++o) body << "    result[" << o << "] = et" << pe.outputs[o] << ";\n";
        em.funcs << "DSC_INLINE void result_epilogue(float product, int gid, float* result, " << em.params_decl() << ") {\n"
                 << body.str() << "}\n";
        if (fk.epilogue_permuted) {
            // result r is element `r` of the product array; the epilogue element that reads it has, on every output
            // axis j of the view, the coordinate (c_i / step_j) % extent_j of the input axis i the axis walks
            const dsc_view& v = pe.inputs[fk.epilogue_product_input];
            int64_t ist[DSC_MAX_DIM], ost[DSC_MAX_DIM];
            strides_of(v.in_shape, ist);
            strides_of(v.out_shape, ost);
            std::ostringstream f;
            f << "DSC_INLINE int epilogue_element_of(int r) {\n    int e = 0;\n";
            for (int j = 0; j < v.out_shape.rank; ++j) {
                if (v.out_shape.dims[j] <= 1 || v.map_axis[j] < 0) continue;
                const int i = v.map_axis[j];
                f << "    e += (((r / " << S(ist[i]) << ") % " << S(v.in_shape.dims[i]) << ") / " << S(v.map_step[j]) << ") % " << S(v.out_shape.dims[j]) << " * "
                  << S(ost[j]) << ";\n";
            }
            f << "    return e;\n}\n";
            em.funcs << f.str();
        }
    }
    string one(const string& value, const string& oid) const {
        const FusedKernel& fk = em.fk;
        if (!fk.has_epilogue) return "b" + to_string(fk.outputs[0]) + "[" + oid + "] = " + value + ";";
        if (fk.epilogue_permuted) {
            string t = "{ float res[" + to_string(n_res) + "]; const int ee = epilogue_element_of((int)(" + oid + ")); result_epilogue(" + value + ", ee, res, " +
                       em.params_pass() + ");";
            for (int o = 0; o < n_res; ++o) t += " b" + to_string(fk.outputs[o]) + "[ee] = res[" + to_string(o) + "];";
            return t + " }";
        }
        string t = "{ float res[" + to_string(n_res) + "]; result_epilogue(" + value + ", (int)(" + oid + "), res, " + em.params_pass() + ");";
        for (int o = 0; o < n_res; ++o) t += " b" + to_string(fk.outputs[o]) + "[" + oid + "] = res[" + to_string(o) + "];";
        if (fk.epilogue_keeps_product) t += " b" + to_string(fk.outputs.back()) + "[" + oid + "] = " + value + ";";
        return t + " }";
    }
    string four(const string& value4, const string& oid) const {
        const FusedKernel& fk = em.fk;
        if (!fk.has_epilogue) return "*(float4*)(b" + to_string(fk.outputs[0]) + " + " + oid + ") = " + value4 + ";";
        if (fk.epilogue_permuted)
            return "{ " + one(value4 + ".x", oid) + " " + one(value4 + ".y", "(" + oid + ") + 1") + " " + one(value4 + ".z", "(" + oid + ") + 2") + " " +
                   one(value4 + ".w", "(" + oid + ") + 3") + " }";
        string t = "{ const float pv[4] = {" + value4 + ".x, " + value4 + ".y, " + value4 + ".z, " + value4 + ".w}; float res[4][" +
                   to_string(n_res) + "];\n#pragma unroll\n        for (int j = 0; j < 4; ++j) result_epilogue(pv[j], (int)(" + oid +
                   ") + j, res[j], " + em.params_pass() + ");";
        for (int o = 0; o < n_res; ++o)
            t += " *(float4*)(b" + to_string(fk.outputs[o]) + " + " + oid + ") = make_float4(res[0][" + to_string(o) + "], res[1][" +
                 to_string(o) + "], res[2][" + to_string(o) + "], res[3][" + to_string(o) + "]);";
        if (fk.epilogue_keeps_product) t += " *(float4*)(b" + to_string(fk.outputs.back()) + " + " + oid + ") = " + value4 + ";";
        return t + " }";
    }
};

unsigned blocks_for(int64_t threads, int block) { return (unsigned)((threads + block - 1) / block); }

// Read-only inputs of at most `max_floats` elements that a kernel and its fused producers read through plain views
// (a depthwise filter, a bias): (buffer, elements).  A kernel whose lanes read such a table at lane-dependent places
// pays a vector memory instruction per read -- a quarter wave per cycle through the address unit whatever the bytes --
// and can keep the table in LDS instead (`stage_small_tables`).
std::vector<std::pair<int, int64_t>> small_tables(const FusedKernel& fk, int64_t max_floats) {
    std::map<int, int64_t> extent;
    std::set<int> barred;
    auto visit = [&](const dsc_kernel_desc& d, const std::vector<Source>& srcs) {
        for (int i = 0; i < d.n_inputs && i < (int)srcs.size(); ++i) {
            if (srcs[i].buffer < 0) continue;
            const int b = srcs[i].buffer;
            extent[b] = std::max(extent[b], element_count(d.inputs[i].in_shape));
            if (d.kind == DSC_KERNEL_PER_ELEMENT)
                for (int o = 0; o < d.n_ops; ++o)
                    if (d.ops[o].kind == DSC_PE_GATHER && d.ops[o].input_index == i) barred.insert(b);
            if (d.kind == DSC_KERNEL_SCATTER_ADD) barred.insert(b);
        }
    };
    visit(fk.main.raw(), fk.inputs);
    for (auto& v : fk.virtuals) visit(v.pe.raw(), v.inputs);
    if (fk.has_epilogue) visit(fk.epilogue.raw(), fk.epilogue_inputs);
    std::vector<std::pair<int, int64_t>> out;
    for (auto& e : extent)
        if (e.second <= max_floats && !barred.count(e.first) && e.first < fk.n_buffers && !fk.buffer_is_output[e.first]) out.push_back(e);
    return out;
}

// Opens a block in which the names of the given buffers mean copies of them in LDS (every later read of b<i>, in the
// kernel and in the producers' functions it passes b<i> to, is then an LDS read); the caller closes the block with
// one more "}".  All 256 threads of the workgroup must reach this point.
void stage_small_tables(std::ostream& k, const std::vector<std::pair<int, int64_t>>& tables) {
    for (auto& t : tables) k << "    __shared__ float sb" << t.first << "[" << S(t.second) << "];\n";
    for (auto& t : tables)
        k << "    for (int i = threadIdx.x; i < " << S(t.second) << "; i += 256) sb" << t.first << "[i] = b" << t.first << "[i];\n";
    k << "    __syncthreads();\n    {\n";
    for (auto& t : tables) k << "    const float* const b" << t.first << " = sb" << t.first << ";\n";
}

// ---------------------------------------------------------------------------------------------------------

string gen_fill(Emitter& em, Generated* out) {
    const dsc_kernel_desc& d = em.fk.main.raw();
    const int64_t n = d.shape.dims[0];
    std::ostringstream k;
    const bool vec = n % 4 == 0;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(em.fk) << "(" << em.kernel_params_decl() << ") {\n    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    k << "    const uint i = blockIdx.x * 256u + threadIdx.x;\n";
    if (vec) {
        k << "    if (i >= " << S(n / 4) << "u) return;\n";
        k << "    const float v = U2F(" << hex32(d.fill_bits) << ");\n";
        k << "    ((float4*)b" << em.fk.outputs[0] << ")[i] = make_float4(v, v, v, v);\n";
    } else {
        k << "    if (i >= " << S(n) << "u) return;\n";
        k << "    b" << em.fk.outputs[0] << "[i] = U2F(" << hex32(d.fill_bits) << ");\n";
    }
    k << "}\n";
    out->grid = blocks_for(vec ? n / 4 : n, 256);
    out->block = 256;
    out->source = k.str();
    out->note = vec ? "fill x4" : "fill";
    return "";
}

}  // namespace

int64_t column_partition_width(const dsc_kernel_desc& d) {
    if (d.kind != DSC_KERNEL_PER_ELEMENT) return 0;
    for (int i = 0; i < d.n_ops; ++i) {
        const dsc_pe_op& op = d.ops[i];
        if (op.kind != DSC_PE_SELECT || op.op != DSC_CMP_GT) continue;
        const dsc_pe_op& lhs = d.ops[op.args[0]];
        const dsc_pe_op& rhs = d.ops[op.args[1]];
        if (lhs.kind != DSC_PE_COORD || (rhs.kind != DSC_PE_LITERAL_F32 && rhs.kind != DSC_PE_LITERAL_U32)) continue;
        const dsc_view& v = d.builtin_views[lhs.view_index];
        const int last = v.out_shape.rank - 1;
        if (last < 1 || element_count(v.out_shape) != d.shape.dims[0]) continue;
        int64_t base = 0, coef[DSC_MAX_DIM];
        if (!affine_form(v, &base, coef) || coef[last] == 0) continue;
        bool only_last = true;
        for (int a = 0; a < last; ++a)
            if (coef[a] != 0 && v.out_shape.dims[a] > 1) only_last = false;
        const int64_t w = v.out_shape.dims[last];
        if (only_last && w >= 2 && w <= 64) return w;
    }
    return 0;
}

namespace {
// One thread per row of a [rows, w] per-element kernel (see FusedKernel::row_width).
string gen_per_element_rows(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const int64_t n = d.shape.dims[0], W = fk.row_width;
    if (W < 2 || W > 64 || n % W != 0 || column_partition_width(d) != W) return "per-element rows: not a column partition of this width";
    const int64_t rows = n / W;
    if (rows >= kMaxIndex) return "per-element rows: too many rows";
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(em.fk) << "(" << em.kernel_params_decl() << ") {\n    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    // (the small tables a row gathers from -- the coarse levels of a hash grid -- stay in memory: copied into LDS per
    // workgroup, 2 / 8 / 15 / 28 thousand floats of them, the hash grid's encoding took 76 / 86 / 101 / 185 us against 74)
    k << "    const int dsc_row = (int)(blockIdx.x * 256u + threadIdx.x);\n";
    k << "    if (dsc_row >= " << S(rows) << ") return;\n";
    for (int o = 0; o < d.n_outputs; ++o) k << "    float o" << o << "[" << S(W) << "];\n";
    for (int64_t c = 0; c < W; ++c) {
        k << "    {\n    const int dsc_col = " << S(c) << ";\n";
        IndexForm form;
        form.valid = true;
        form.names = {"dsc_row", "dsc_col"};
        form.coefs = {W, 1};
        form.extents = {rows, W};
        em.emit_pe(k, d, fk.inputs, "(uint)(dsc_row * " + S(W) + " + dsc_col)", "", {}, &form);
        for (int o = 0; o < d.n_outputs; ++o) k << "    o" << o << "[" << S(c) << "] = t" << d.outputs[o] << ";\n";
        k << "    }\n";
    }
    for (int o = 0; o < d.n_outputs; ++o) {
        k << "    float* const row" << o << " = b" << fk.outputs[o] << " + (size_t)dsc_row * " << S(W) << ";\n";
        if (W % 4 == 0) {
            for (int64_t c = 0; c < W; c += 4)
                k << "    *(float4*)(row" << o << " + " << S(c) << ") = make_float4(o" << o << "[" << S(c) << "], o" << o << "[" << S(c + 1) << "], o" << o << "["
                  << S(c + 2) << "], o" << o << "[" << S(c + 3) << "]);\n";
        } else {
            for (int64_t c = 0; c < W; ++c) k << "    row" << o << "[" << S(c) << "] = o" << o << "[" << S(c) << "];\n";
        }
    }
    k << "}\n";
    out->grid = blocks_for(rows, 256);
    out->block = 256;
    out->source = k.str();
    out->note = "per-element: a thread per row of " + S(W) + " columns, the column a constant of each evaluation";
    return "";
}

string gen_per_element(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    if (fk.row_width) return gen_per_element_rows(em, out);
    const int64_t n = d.shape.dims[0];
    const int vec = (n % 4 == 0 && n >= 4096) ? 4 : 1;
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(em.fk) << "(" << em.kernel_params_decl() << ") {\n    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    k << "    const uint base = (blockIdx.x * 256u + threadIdx.x) * " << vec << "u;\n";
    k << "    if (base >= " << S(n) << "u) return;\n";
    std::map<int, string> override_load;
    dsc_shape quad_shape{};
    IndexForm quad_form;
    string quad_inner;
    if (vec == 4) {
        // identity-view loads of real buffers become one 16-byte load per thread; so do the loads through any view
        // whose innermost output axis walks the innermost input axis one to one in whole groups of four (a bias
        // broadcast over rows, the window of a pooling gradient over channels-last data): the thread's four elements
        // share every other coordinate, so the view's index is evaluated once, at the first of them
        auto quad_contiguous = [&](const dsc_view& v) {
            const int L = v.out_shape.rank - 1;
            if (L < 0 || element_count(v.out_shape) != n || v.out_shape.dims[L] % 4 != 0) return false;
            const int a = v.map_axis[L];
            if (a < 0 || v.map_step[L] != 1 || needs_clamp(v, a) || v.in_offset[a] % 4 != 0 || v.in_shape.dims[a] % 4 != 0) return false;
            for (int i = a + 1; i < v.in_shape.rank; ++i)
                if (v.in_shape.dims[i] != 1) return false;
            for (int j = 0; j < L; ++j)
                if (v.map_axis[j] == a && v.out_shape.dims[j] > 1) return false;
            return true;
        };
        for (int i = 0; i < d.n_inputs; ++i) {
            if (fk.inputs[i].buffer < 0) continue;
            bool loaded = false;
            for (int o = 0; o < d.n_ops; ++o) loaded = loaded || (d.ops[o].kind == DSC_PE_LOAD && d.ops[o].input_index == i);
            if (!loaded) continue;
            if (is_identity(d.inputs[i])) {
                k << "    const float4 q" << i << " = *(const float4*)(b" << fk.inputs[i].buffer << " + base);\n";
            } else if (quad_contiguous(d.inputs[i])) {
                auto c = em.emit_coords(k, d.inputs[i].out_shape, "base", "qb" + to_string(i) + "_");
                k << "    const float4 q" << i << " = *(const float4*)(b" << fk.inputs[i].buffer << " + " << em.index_expr(d.inputs[i], c) << ");\n";
            } else {
                continue;
            }
            k << "    const float l" << i << "[4] = {q" << i << ".x, q" << i << ".y, q" << i << ".z, q" << i << ".w};\n";
            override_load[i] = "l" + to_string(i) + "[e]";
        }
        for (int o = 0; o < d.n_outputs; ++o) k << "    float o" << o << "[4];\n";
        // The thread's four elements differ in the innermost coordinate only (when that axis is a multiple of four
        // long): the coordinates of the first are taken apart once, outside the loop, and handed to the views and
        // fused producers as names, so nothing divides the element id per element, and what the four evaluations
        // load from consecutive addresses can be merged by the compiler.
        for (int i = 0; i < d.n_inputs + d.n_builtin_views && quad_shape.rank == 0; ++i) {
            const dsc_view& v = i < d.n_inputs ? d.inputs[i] : d.builtin_views[i - d.n_inputs];
            if (i < d.n_inputs && override_load.count(i)) continue;
            const int L = v.out_shape.rank - 1;
            if (L >= 1 && element_count(v.out_shape) == n && v.out_shape.dims[L] % 4 == 0) quad_shape = v.out_shape;
        }
        if (quad_shape.rank) {
            auto c = em.emit_coords(k, quad_shape, "base", "qs_");
            int64_t st[DSC_MAX_DIM];
            strides_of(quad_shape, st);
            quad_form.valid = true;
            for (int j = 0; j < quad_shape.rank; ++j) {
                if (quad_shape.dims[j] <= 1) continue;
                quad_form.names.push_back(j == quad_shape.rank - 1 ? string("qs_inner") : c[j]);
                quad_form.coefs.push_back(st[j]);
                quad_form.extents.push_back(quad_shape.dims[j]);
            }
            quad_inner = c[quad_shape.rank - 1];
        }
        k << "#pragma unroll\n    for (int e = 0; e < 4; ++e) {\n    const uint gid = base + e;\n";
        if (quad_shape.rank) k << "    const int qs_inner = " << quad_inner << " + e;\n";
    } else {
        k << "    const uint gid = base;\n    {\n";
    }
    em.emit_pe(k, d, fk.inputs, "gid", "", override_load, quad_form.valid ? &quad_form : nullptr);
    for (int o = 0; o < d.n_outputs; ++o) {
        if (vec == 4) k << "    o" << o << "[e] = t" << d.outputs[o] << ";\n";
        else k << "    b" << fk.outputs[o] << "[gid] = t" << d.outputs[o] << ";\n";
    }
    k << "    }\n";
    if (vec == 4)
        for (int o = 0; o < d.n_outputs; ++o)
            k << "    *(float4*)(b" << fk.outputs[o] << " + base) = make_float4(o" << o << "[0], o" << o << "[1], o" << o
              << "[2], o" << o << "[3]);\n";
    k << "}\n";
    out->grid = blocks_for(n / vec, 256);
    out->block = 256;
    out->source = k.str();
    out->note = vec == 4 ? "per-element x4" : "per-element";
    return "";
}

int64_t pow2_ceil(int64_t v) {
    int64_t p = 1;
    while (p < v) p <<= 1;
    return p;
}

string gen_reduce(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const dsc_view& v = d.inputs[0];
    const int64_t n_out = element_count(d.shape);
    const int64_t K = v.out_shape.dims[d.axis];
    const bool is_max = d.reduce_op == DSC_REDUCE_MAX;
    const string init = is_max ? "U2F(0xff800000u)" : "0.f";
    auto combine = [&](const string& a, const string& b) { return is_max ? "glsl_max(" + a + ", " + b + ")" : a + " + " + b; };

    const ResultStore store(em);
    auto store_one = [&](const string& value, const string& oid) { return store.one(value, oid); };
    auto store_four = [&](const string& value4, const string& oid) { return store.four(value4, oid); };

    // is the reduced axis the one that walks memory fastest?
    bool k_fastest = false;
    if (fk.inputs[0].buffer >= 0) {
        int64_t base, coef[DSC_MAX_DIM];
        if (affine_form(v, &base, coef) && coef[d.axis] == 1 && K >= 4) k_fastest = true;
    }

    // can four adjacent outputs be fetched with one 16-byte load?  (input is a real buffer, the view is affine,
    // the innermost output axis that is not reduced walks memory with stride 1 and everything is 4-aligned)
    bool vec_outputs = false;
    if (!k_fastest && fk.inputs[0].buffer >= 0 && n_out % 4 == 0) {
        int64_t base, coef[DSC_MAX_DIM];
        int inner = d.shape.rank - 1;
        while (inner >= 0 && d.shape.dims[inner] == 1) --inner;
        if (inner >= 0 && inner != d.axis && affine_form(v, &base, coef) && coef[inner] == 1 && d.shape.dims[inner] % 4 == 0 && base % 4 == 0) {
            vec_outputs = true;
            for (int j = 0; j < d.shape.rank; ++j)
                if (j != inner && v.out_shape.dims[j] > 1 && coef[j] % 4 != 0) vec_outputs = false;
        }
    }

    // ... or, from a fused producer, with one evaluation of a quad (a pooling over a window copy of an image whose
    // channels walk memory: the copy's index arithmetic once per four channels, 16-byte loads)
    bool vec_virtual = false;
    if (!k_fastest && !vec_outputs && fk.inputs[0].virt >= 0 && n_out % 4 == 0 && v.out_shape.rank == d.shape.rank) {
        const int L = d.shape.rank - 1;
        if (L >= 1 && d.axis != L && d.shape.dims[L] % 4 == 0) {
            std::vector<string> pc;
            for (int i = 0; i < d.shape.rank; ++i) pc.push_back(d.shape.dims[i] == 1 && i != d.axis ? "0" : "oc" + to_string(i));
            pc[d.axis] = "kq0";
            vec_virtual = vec_outputs = !em.load_view4(fk.inputs[0], v, pc).empty();
        }
    }

    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(em.fk) << "(" << em.kernel_params_decl() << ") {\n    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    // The k loop runs over groups of U independent accumulators: the U loads of a group are issued before any of
    // them is used, with no bounds test in between (a test per load would be a branch per load, and the loads
    // would be issued one at a time).  What is left over is handled by groups of U/2, U/4, .. 1.
    // `first`/`step` give the thread's k sequence.
    auto pick_unroll = [&](int64_t step, int64_t max_u) {
        int64_t u = max_u;
        while (u > 1 && u * step > K) u /= 2;
        return (int)u;
    };
    auto emit_k_loop = [&](const std::vector<string>& oc, const string& first, int64_t step) {
        // a fused producer is code, not a load: fewer copies of it (groups of 4, then single steps)
        const bool heavy = fk.inputs[0].virt >= 0;
        const int U = pick_unroll(step, heavy ? 4 : 8);
        for (int u = 0; u < U; ++u) k << (u ? ", acc" : "    float acc") << u << " = " << init;
        k << ";\n    int kb = " << first << ";\n";
        for (int lvl = U; lvl >= 1; lvl = (heavy && lvl > 1) ? 1 : lvl / 2) {
            const string cond = "kb + " + S((lvl - 1) * step) + " < " + S(K);
            const bool loop = lvl == U || heavy;
            k << (loop ? "    for (; " + cond + "; kb += " + S(lvl * step) + ") {\n" : "    if (" + cond + ") {\n");
            for (int u = 0; u < lvl; ++u) {
                auto ic = oc;
                ic[d.axis] = "(kb + " + S(u * step) + ")";
                k << "        const float x" << u << " = " << em.load_view(fk.inputs[0], v, ic) << ";\n";
            }
            for (int u = 0; u < lvl; ++u) k << "        acc" << u << " = " << combine("acc" + to_string(u), "x" + to_string(u)) << ";\n";
            if (!loop) k << "        kb += " << S(lvl * step) << ";\n";
            k << "    }\n";
        }
        std::vector<string> terms;
        for (int u = 0; u < U; ++u) terms.push_back("acc" + to_string(u));
        while (terms.size() > 1) {
            std::vector<string> next;
            for (size_t i = 0; i + 1 < terms.size(); i += 2) next.push_back("(" + combine(terms[i], terms[i + 1]) + ")");
            terms = next;
        }
        k << "    float acc = " << terms[0] << ";\n";
    };
    if (k_fastest) {
        // lanes of a group walk k; groups of G lanes own one output; butterfly over the group
        const int64_t G = std::min<int64_t>(64, pow2_ceil(K));
        const int64_t per_block = 256 / G;
        k << "    const int grp = threadIdx.x / " << G << ", lk = threadIdx.x % " << G << ";\n";
        k << "    const uint oid = blockIdx.x * " << per_block << "u + grp;\n";
        k << "    if (oid >= " << S(n_out) << "u) return;\n";
        auto oc = em.emit_coords(k, d.shape, "oid", "oc");
        emit_k_loop(oc, "lk", G);
        for (int64_t off = G / 2; off >= 1; off /= 2)
            k << "    acc = " << combine("acc", "__shfl_xor(acc, " + S(off) + ", 64)") << ";\n";
        k << "    if (lk == 0) " << store_one("acc", "oid") << "\n}\n";
        out->grid = blocks_for(n_out, (int)per_block);
        out->note = "reduce: " + S(G) + " lanes along k, shuffle";
    } else if (vec_outputs) {
        // each thread owns 4 adjacent outputs that are adjacent in memory: 16-byte loads, lanes walk outputs;
        // k optionally split over TK thread rows combined through LDS
        const int64_t n_vec = n_out / 4;
        int64_t TK = 1;
        // (a workgroup per compute unit at least: the sum of 256 partial 256x256 products took 23.4 us with 128 workgroups)
        const int64_t want_threads = 65536;
        if (n_vec < want_threads && K >= 8) {
            while (TK < 64 && n_vec * TK < want_threads && TK * 4 <= K) TK *= 2;
        }
        const int64_t TO = 256 / TK;
        k << "    const int to = threadIdx.x % " << TO << ", tk = threadIdx.x / " << TO << ";\n";
        k << "    const uint vid = blockIdx.x * " << TO << "u + to;\n";
        if (TK > 1) k << "    __shared__ float4 red[256];\n";
        k << "    float4 result = make_float4(" << init << ", " << init << ", " << init << ", " << init << ");\n";
        k << "    if (vid < " << S(n_vec) << "u) {\n";
        k << "    const uint oid = vid * 4u;\n";
        auto oc = em.emit_coords(k, d.shape, "oid", "oc");
        const int U = pick_unroll(TK, vec_virtual ? 4 : 16);
        const char* comps[4] = {"x", "y", "z", "w"};
        for (int u = 0; u < U; ++u) k << (u ? ", a" : "    float4 a") << u << " = result";
        k << ";\n    int kb = " << (TK > 1 ? "tk" : "0") << ";\n";
        for (int lvl = U; lvl >= 1; lvl /= 2) {
            const string cond = "kb + " + S((lvl - 1) * TK) + " < " + S(K);
            k << (lvl == U ? "    for (; " + cond + "; kb += " + S(lvl * TK) + ") {\n" : "    if (" + cond + ") {\n");
            for (int u = 0; u < lvl; ++u) {
                auto ic = oc;
                ic[d.axis] = "(kb + " + S(u * TK) + ")";
                if (vec_virtual) {  // (a producer takes its coordinates by name)
                    ic[d.axis] = "kq" + to_string(u);
                    for (int i = 0; i < d.shape.rank; ++i)
                        if (d.shape.dims[i] == 1 && i != d.axis) ic[i] = "0";
                    k << "        const int kq" << u << " = kb + " << S(u * TK) << ";\n";
                    k << "        const float4 x" << u << " = " << em.load_view4(fk.inputs[0], v, ic) << ";\n";
                }
                else
                k << "        const float4 x" << u << " = *(const float4*)(b" << fk.inputs[0].buffer << " + " << em.index_expr(v, ic) << ");\n";
            }
            for (int u = 0; u < lvl; ++u) {
                const string a = "a" + to_string(u), x = "x" + to_string(u);
                k << "       ";
                for (const char* c : comps) k << " " << a << "." << c << " = " << combine(a + "." + c, x + "." + c) << ";";
                k << "\n";
            }
            if (lvl != U) k << "        kb += " << S(lvl * TK) << ";\n";
            k << "    }\n";
        }
        for (const char* c : comps) {
            std::vector<string> terms;
            for (int u = 0; u < U; ++u) terms.push_back("a" + to_string(u) + "." + c);
            while (terms.size() > 1) {
                std::vector<string> next;
                for (size_t i = 0; i + 1 < terms.size(); i += 2) next.push_back("(" + combine(terms[i], terms[i + 1]) + ")");
                terms = next;
            }
            k << "    result." << c << " = " << terms[0] << ";\n";
        }
        k << "    }\n";
        if (TK > 1) {
            k << "    red[threadIdx.x] = result;\n    __syncthreads();\n";
            k << "    if (tk == 0 && vid < " << S(n_vec) << "u) {\n";
            k << "        for (int j = 1; j < " << TK << "; ++j) { const float4 o = red[j * " << TO << " + to];";
            for (const char* c : {"x", "y", "z", "w"}) k << " result." << c << " = " << combine(string("result.") + c, string("o.") + c) << ";";
            k << " }\n";
            k << "        " << store_four("result", "vid * 4u") << "\n    }\n}\n";
        } else {
            k << "    if (vid < " << S(n_vec) << "u) " << store_four("result", "vid * 4u") << "\n}\n";
        }
        out->grid = blocks_for(n_vec, (int)TO);
        out->note = "reduce: lanes along outputs x4, k split " + S(TK);
    } else {
        // lanes walk outputs (coalesced); optional split of k over TK thread rows, combined through LDS
        int64_t TK = 1;
        if (n_out < 65536 && K >= 8) {
            while (TK < 64 && n_out * TK < 65536 && TK * 4 <= K) TK *= 2;
        }
        const int64_t TO = 256 / TK;
        k << "    const int to = threadIdx.x % " << TO << ", tk = threadIdx.x / " << TO << ";\n";
        k << "    const uint oid = blockIdx.x * " << TO << "u + to;\n";
        if (TK > 1) k << "    __shared__ float red[256];\n";
        k << "    float result = " << init << ";\n";
        k << "    if (oid < " << S(n_out) << "u) {\n";
        auto oc = em.emit_coords(k, d.shape, "oid", "oc");
        emit_k_loop(oc, TK > 1 ? "tk" : "0", TK);
        k << "    result = acc;\n    }\n";
        if (TK > 1) {
            k << "    red[threadIdx.x] = result;\n    __syncthreads();\n";
            k << "    if (tk == 0 && oid < " << S(n_out) << "u) {\n";
            k << "        for (int j = 1; j < " << TK << "; ++j) result = " << combine("result", "red[j * " + S(TO) + " + to]") << ";\n";
            k << "        " << store_one("result", "oid") << "\n    }\n}\n";
        } else {
            k << "    if (oid < " << S(n_out) << "u) " << store_one("result", "oid") << "\n}\n";
        }
        out->grid = blocks_for(n_out, (int)TO);
        out->note = "reduce: lanes along outputs, k split " + S(TK);
    }
    out->block = 256;
    out->source = k.str();
    return "";
}

string gen_unpad(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const dsc_view& v = d.inputs[0];
    const int64_t n = element_count(d.shape);
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(em.fk) << "(" << em.kernel_params_decl() << ") {\n    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    // (a chain of gathered sums evaluated on demand reads the small tables at its end -- a depthwise filter -- once per
    // evaluation and lane: from LDS)
    const auto tables = fk.inputs[0].virt >= 0 ? small_tables(fk, 1024) : std::vector<std::pair<int, int64_t>>();
    if (!tables.empty()) stage_small_tables(k, tables);
    // Four elements of the innermost axis per thread where the chain behind the input can be evaluated for a quad (the
    // four channels of a pixel share every index but the channel's, and the chain ends in 16-byte loads where the
    // channels walk memory): a kernel of this kind is bound by the load instructions it issues.
    {
        const int L = d.shape.rank - 1;
        string x4;
        if (fk.inputs[0].virt >= 0 && L >= 1 && d.axis != L && d.shape.dims[L] % 4 == 0 && n % 4 == 0) {
            std::vector<string> pc;
            for (int i = 0; i < d.shape.rank; ++i) pc.push_back("c" + to_string(i));
            pc[d.axis] = "kk";
            x4 = em.load_view_q(fk.inputs[0], v, pc, L);
        }
        if (!x4.empty()) {
            k << "    const uint gid = (blockIdx.x * 256u + threadIdx.x) * 4u;\n    if (gid >= " << S(n) << "u) return;\n";
            auto c = em.emit_coords(k, d.shape, "gid", "c");
            const string oc = c[d.axis];
            k << "    const int in_c = " << oc << " + " << d.pad << ";\n";
            k << "    const int k_min = in_c - ((" << oc << " == 0) ? " << d.pad << " : 0);\n";
            k << "    const int k_max = in_c + ((" << oc << " == " << S(d.shape.dims[d.axis] - 1) << ") ? " << d.pad << " : 0);\n";
            k << "    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);\n    for (int kk = k_min; kk <= k_max; ++kk) {\n";
            k << "        const float4 w = " << x4 << ";\n";
            k << "        sum = make_float4(sum.x + w.x, sum.y + w.y, sum.z + w.z, sum.w + w.w);\n    }\n";
            k << "    " << ResultStore(em).four("sum", "gid") << "\n" << (tables.empty() ? "" : "    }\n") << "}\n";
            out->grid = blocks_for(n / 4, 256);
            out->block = 256;
            out->source = k.str();
            out->note = string(fk.has_epilogue ? "unpad x4 +epilogue" : "unpad x4") + (tables.empty() ? "" : ", small tables in LDS");
            return "";
        }
    }
    k << "    const uint gid = blockIdx.x * 256u + threadIdx.x;\n    if (gid >= " << S(n) << "u) return;\n";
    auto c = em.emit_coords(k, d.shape, "gid", "c");
    const string oc = c[d.axis];
    k << "    const int in_c = " << oc << " + " << d.pad << ";\n";
    k << "    const int k_min = in_c - ((" << oc << " == 0) ? " << d.pad << " : 0);\n";
    k << "    const int k_max = in_c + ((" << oc << " == " << S(d.shape.dims[d.axis] - 1) << ") ? " << d.pad << " : 0);\n";
    // the candidates in_c - pad .. in_c + pad are all loaded (clamped into [k_min, k_max]) and the ones outside
    // that range add zero: no loop with a data-dependent trip count, every load in flight at once
    auto ic = c;
    if (fk.inputs[0].virt >= 0) {
        // (an input that is evaluated on demand -- sums of gathered elements themselves -- is evaluated only where it counts:
        // once away from the border, where the masked candidates would cost 2 pad + 1 evaluations)
        ic[d.axis] = "kk";
        k << "    float sum = 0.f;\n    for (int kk = k_min; kk <= k_max; ++kk) sum += " << em.load_view(fk.inputs[0], v, ic) << ";\n";
    } else {
    k << "    float sum = 0.f;\n#pragma unroll\n    for (int j = " << -d.pad << "; j <= " << d.pad << "; ++j) {\n";
    k << "        const int kk = in_c + j;\n        const int kc = clampi(kk, k_min, k_max);\n";
    ic[d.axis] = "kc";
    k << "        const float w = " << em.load_view(fk.inputs[0], v, ic) << ";\n";
    k << "        sum += (kk >= k_min && kk <= k_max) ? w : 0.f;\n    }\n";
    }
    k << "    " << ResultStore(em).one("sum", "gid") << "\n" << (tables.empty() ? "" : "    }\n") << "}\n";
    out->grid = blocks_for(n, 256);
    out->block = 256;
    out->source = k.str();
    out->note = string(fk.has_epilogue ? "unpad +epilogue" : "unpad") + (tables.empty() ? "" : ", small tables in LDS");
    return "";
}

string gen_windows_to_image(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const dsc_view& v = d.inputs[0];
    const int r = v.out_shape.rank;
    const int64_t out_h = v.out_shape.dims[r - 6], out_w = v.out_shape.dims[r - 5];
    const int64_t fh = v.out_shape.dims[r - 3], fw = v.out_shape.dims[r - 2], group_nc = v.out_shape.dims[r - 1];
    const int64_t sw = d.stride_w, sh = d.stride_h;
    const int bd = d.shape.rank - 3;
    const int64_t n = element_count(d.shape);
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(em.fk) << "(" << em.kernel_params_decl() << ") {\n    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    // Four channels of a pixel per thread where a group's channels come in fours: they share the pixel's windows, so the
    // index arithmetic is done once per quad and the loads are 16 bytes (a kernel of this kind is bound by the number
    // of load instructions it issues, not by their bytes).
    if (group_nc % 4 == 0 && n % 4 == 0) {
        std::vector<string> pc(r);
        for (int i = 0; i < bd; ++i) pc[i] = "c" + to_string(i);
        pc[bd] = "oyc"; pc[bd + 1] = "oxc"; pc[bd + 2] = "group_index"; pc[bd + 3] = "fyc"; pc[bd + 4] = "fxc"; pc[bd + 5] = "group_c";
        for (int i = 0; i < bd; ++i)
            if (d.shape.dims[i] == 1) pc[i] = "0";
        const string w4 = em.load_view4(fk.inputs[0], v, pc);
        if (!w4.empty()) {
            k << "    const uint gid = (blockIdx.x * 256u + threadIdx.x) * 4u;\n    if (gid >= " << S(n) << "u) return;\n";
            auto c = em.emit_coords(k, d.shape, "gid", "c");
            k << "    const int in_y = " << c[bd] << ", in_x = " << c[bd + 1] << ", in_c = " << c[bd + 2] << ";\n";
            k << "    const int group_index = in_c / " << S(group_nc) << ", group_c = in_c % " << S(group_nc) << ";\n";
            k << "    const int fbx = in_x % " << S(sw) << ", fby = in_y % " << S(sh) << ";\n";
            k << "    const int oxb = in_x / " << S(sw) << ", oyb = in_y / " << S(sh) << ";\n";
            k << "    float4 tmp = make_float4(0.f, 0.f, 0.f, 0.f);\n";
            k << "#pragma unroll\n    for (int iy = 0; iy < " << S((fh + sh - 1) / sh) << "; ++iy)\n";
            k << "#pragma unroll\n    for (int ix = 0; ix < " << S((fw + sw - 1) / sw) << "; ++ix) {\n";
            k << "        const int fx = fbx + " << S(sw) << " * ix, fy = fby + " << S(sh) << " * iy;\n";
            k << "        const int ox = oxb - ix, oy = oyb - iy;\n";
            k << "        const bool ok = fx < " << S(fw) << " && fy < " << S(fh) << " && ox >= 0 && ox < " << S(out_w) << " && oy >= 0 && oy < " << S(out_h) << ";\n";
            k << "        const int fxc = min(fx, " << S(fw - 1) << "), fyc = min(fy, " << S(fh - 1) << "), oxc = clampi(ox, 0, " << S(out_w - 1)
              << "), oyc = clampi(oy, 0, " << S(out_h - 1) << ");\n";
            k << "        const float4 w = " << w4 << ";\n";
            k << "        tmp.x += ok ? w.x : 0.f; tmp.y += ok ? w.y : 0.f; tmp.z += ok ? w.z : 0.f; tmp.w += ok ? w.w : 0.f;\n    }\n";
            k << "    " << ResultStore(em).four("tmp", "gid") << "\n}\n";
            out->grid = blocks_for(n / 4, 256);
            out->block = 256;
            out->source = k.str();
            out->note = fk.has_epilogue ? "windows_to_image x4 +epilogue" : "windows_to_image x4";
            return "";
        }
    }
    k << "    const uint gid = blockIdx.x * 256u + threadIdx.x;\n    if (gid >= " << S(n) << "u) return;\n";
    auto c = em.emit_coords(k, d.shape, "gid", "c");
    k << "    const int in_y = " << c[bd] << ", in_x = " << c[bd + 1] << ", in_c = " << c[bd + 2] << ";\n";
    k << "    const int group_index = in_c / " << S(group_nc) << ", group_c = in_c % " << S(group_nc) << ";\n";
    k << "    const int fbx = in_x % " << S(sw) << ", fby = in_y % " << S(sh) << ";\n";
    k << "    const int oxb = in_x / " << S(sw) << ", oyb = in_y / " << S(sh) << ";\n";
    k << "    float tmp = 0.f;\n";
    k << "#pragma unroll\n    for (int iy = 0; iy < " << S((fh + sh - 1) / sh) << "; ++iy)\n";
    k << "#pragma unroll\n    for (int ix = 0; ix < " << S((fw + sw - 1) / sw) << "; ++ix) {\n";
    k << "        const int fx = fbx + " << S(sw) << " * ix, fy = fby + " << S(sh) << " * iy;\n";
    k << "        const int ox = oxb - ix, oy = oyb - iy;\n";
    // the window must exist: the reference omits the ox/oy test (kernel.rs:775-776); the true adjoint needs it.
    // Taps without a window load a valid element instead and add zero, so that the loads of all taps are
    // independent of the tests and in flight together.
    k << "        const bool ok = fx < " << S(fw) << " && fy < " << S(fh) << " && ox >= 0 && ox < " << S(out_w) << " && oy >= 0 && oy < "
      << S(out_h) << ";\n";
    k << "        const int fxc = min(fx, " << S(fw - 1) << "), fyc = min(fy, " << S(fh - 1) << "), oxc = clampi(ox, 0, " << S(out_w - 1)
      << "), oyc = clampi(oy, 0, " << S(out_h - 1) << ");\n";
    std::vector<string> ic(r);
    for (int i = 0; i < bd; ++i) ic[i] = c[i];
    ic[bd] = "oyc"; ic[bd + 1] = "oxc"; ic[bd + 2] = "group_index"; ic[bd + 3] = "fyc"; ic[bd + 4] = "fxc"; ic[bd + 5] = "group_c";
    k << "        const float w = " << em.load_view(fk.inputs[0], v, ic) << ";\n";
    k << "        tmp += ok ? w : 0.f;\n    }\n";
    k << "    " << ResultStore(em).one("tmp", "gid") << "\n}\n";
    out->grid = blocks_for(n, 256);
    out->block = 256;
    out->source = k.str();
    out->note = fk.has_epilogue ? "windows_to_image +epilogue" : "windows_to_image";
    return "";
}

// Accumulators small enough for LDS that receive many values per entry (the coarse levels of a hash grid: half a
// million adds into a few hundred entries) are summed per workgroup in LDS first; the workgroup then adds its
// non-zero totals to memory.  Contention on the memory atomics drops by the number of values a workgroup folds.
bool scatter_privatised(const dsc_kernel_desc& d, int64_t* workgroups) {
    const int64_t table = element_count(d.shape), n = element_count(d.inputs[0].out_shape);
    if (table > 8192 || n < 16 * table || n < 65536) return false;
    // every workgroup ends with one memory atomic per non-zero entry: enough workgroups to fill the machine, few
    // enough that those closing atomics stay well below the values folded
    *workgroups = std::max<int64_t>(64, std::min<int64_t>(512, n / (2 * table)));
    return true;
}

// value, index and target of ScatterAdd element `gid` (names suffixed by `sfx`): value<sfx>, at<sfx>, ok<sfx>
void emit_scatter_element(Emitter& em, std::ostream& k, const string& gid, const string& sfx) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const dsc_view& vv = d.inputs[0];
    const dsc_view& vi = d.inputs[1];
    int64_t st[DSC_MAX_DIM];
    strides_of(d.shape, st);
    auto c = em.emit_coords(k, vv.out_shape, gid, "c" + sfx + "_");
    k << "    const float value" << sfx << " = " << em.load_view(fk.inputs[0], vv, c) << ";\n";
    k << "    const int si" << sfx << " = F2I(" << em.load_view(fk.inputs[1], vi, {c[d.axis]}) << ");\n";
    string idx = "0";
    for (int i = 0; i < d.shape.rank; ++i) idx += " + " + (i == d.axis ? "si" + sfx : c[i]) + "*" + S(st[i]);
    k << "    const int at" << sfx << " = " << idx << ";\n";
    // bounds: an index outside the accumulator would be a wild write; the reference has no check, here it is dropped
    k << "    const bool ok" << sfx << " = si" << sfx << " >= 0 && si" << sfx << " < " << S(d.shape.dims[d.axis]) << ";\n";
}

string gen_scatter_add(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const int64_t n = element_count(d.inputs[0].out_shape);
    int64_t wgs = 0;
    const bool priv = scatter_privatised(d, &wgs);
    const int64_t table = element_count(d.shape);
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(em.fk) << "(" << em.kernel_params_decl() << ") {\n    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    auto emit_element = [&](const string& gid, const string& sfx) { emit_scatter_element(em, k, gid, sfx); };
    if (priv) {
        const int U = 4;  // elements per thread and trip: their loads are all issued before the first LDS atomic
        // The sums are kept in double: on gfx950 ds_add_f64 runs seven times faster than ds_add_f32 (0.18 against
        // 1.27 ns per add and CU, measured with random targets), and the rounding of the partial sums goes away.
        k << "    __shared__ double acc[" << S(table) << "];\n";
        k << "    for (int i = threadIdx.x; i < " << S(table) << "; i += 256) acc[i] = 0.0;\n    __syncthreads();\n";
        k << "    for (uint g0 = blockIdx.x * 256u + threadIdx.x; g0 < " << S(n) << "u; g0 += " << S(wgs * 256 * U) << "u) {\n";
        for (int u = 0; u < U; ++u) {
            k << "    const uint gid" << u << " = min(g0 + " << S(u * wgs * 256) << "u, " << S(n - 1) << "u);\n";
            emit_element("gid" + to_string(u), to_string(u));
        }
        k << "    __builtin_amdgcn_sched_barrier(0);\n";
        for (int u = 0; u < U; ++u)
            k << "    if (ok" << u << " && g0 + " << S(u * wgs * 256) << "u < " << S(n) << "u) atomicAdd(&acc[at" << u << "], (double)value" << u << ");\n";
        k << "    }\n    __syncthreads();\n";
        k << "    for (int i = threadIdx.x; i < " << S(table) << "; i += 256) {\n        const float total = (float)acc[i];\n";
        k << "        if (total != 0.f) unsafeAtomicAdd(&b" << fk.outputs[0] << "[i], total);\n    }\n}\n";
    } else {
        k << "    const uint gid = blockIdx.x * 256u + threadIdx.x;\n    if (gid >= " << S(n) << "u) return;\n";
        emit_element("gid", "");
        k << "    if (ok) unsafeAtomicAdd(&b" << fk.outputs[0] << "[at], value);\n}\n";
    }
    out->grid = priv ? (unsigned)wgs : blocks_for(n, 256);
    out->block = 256;
    out->source = k.str();
    out->note = priv ? "scatter_add: per-workgroup sums in LDS (ds_add_f64), then global_atomic_add_f32" : "scatter_add: global_atomic_add_f32";
    return "";
}

// ---- row-fused kernel ---------------------------------------------------------------------------------

string gen_row_fused(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const int64_t m = fk.row_m, n = fk.row_n;
    if (m < 1 || n < 2 || n > 64) return "row-fused: bad row shape";
    int64_t G = pow2_ceil(n);
    // A MatMul as stage 0: the lanes of a row share its k range as in the dot-product kernel (B in LDS, blocks of four k
    // per lane, a shuffle butterfly), after which lane `col` keeps the sum of its column.
    const bool mm0 = !fk.row_stages.empty() && fk.row_stages[0].k.raw().kind == DSC_KERNEL_MATMUL;
    int64_t K = 0, kblocks = 0, J = 0;
    if (mm0) {
        const MatMulDims g = matmul_dims(fk.row_stages[0].k.raw());
        if (g.batch != 1 || g.chunks != 1 || g.m != m || g.n != n || g.k * g.n > 8192) return "row-fused: the MatMul stage does not match the rows";
        K = g.k;
        kblocks = (K + 3) / 4;
        int64_t L = 4;
        while (L < 64 && L * 2 < kblocks) L *= 2;
        G = std::max(G, L);
        J = (kblocks + G - 1) / G;
    }
    // (one wave per workgroup, to spread 1000 rows over four times as many compute units, measured slower: 13.9 us
    // against 10.1 for the ConvNet's head -- every workgroup stages B for itself)
    const int64_t BT = 256;
    const int64_t per_block = BT / G;
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(" << S(BT) << ") void " << entry_name(fk) << "(" << em.kernel_params_decl() << ") {\n";
    k << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    k << "    const int col = threadIdx.x % " << G << ";\n";
    k << "    const int row = blockIdx.x * " << per_block << " + threadIdx.x / " << G << ";\n";
    // lanes past the last row or column repeat a valid element's work (every lane takes part in the shuffles)
    // and store nothing
    k << "    const bool row_ok = row < " << S(m) << ", col_ok = col < " << S(n) << ";\n";
    k << "    const int rowc = min(row, " << S(m - 1) << "), colc = min(col, " << S(n - 1) << ");\n";
    k << "    const int wide_gid = rowc * " << S(n) << " + colc;\n";
    IndexForm wide, narrow;
    wide.valid = narrow.valid = true;
    wide.names = {"rowc", "colc"};
    wide.coefs = {n, 1};
    wide.extents = {m, n};
    narrow.names = {"rowc"};
    narrow.coefs = {1};
    narrow.extents = {m};
    // variable holding output `o` of stage `s`
    auto stage_var = [&](int s_idx, int o) {
        const dsc_kernel_desc& sd = fk.row_stages[s_idx].k.raw();
        if (sd.kind == DSC_KERNEL_REDUCE || sd.kind == DSC_KERNEL_MATMUL) return "s" + to_string(s_idx) + "_r";
        return "s" + to_string(s_idx) + "_t" + to_string(sd.outputs[o]);
    };
    auto stage_is_wide = [&](int s_idx) {
        const dsc_kernel_desc& sd = fk.row_stages[s_idx].k.raw();
        return sd.kind == DSC_KERNEL_PER_ELEMENT && sd.shape.dims[0] == m * n;
    };
    for (int si = 0; si < (int)fk.row_stages.size(); ++si) {
        const RowStage& st = fk.row_stages[si];
        const dsc_kernel_desc& sd = st.k.raw();
        const string pfx = "s" + to_string(si) + "_";
        k << "    // stage " << si << ": " << label_name(sd) << "\n";
        if (sd.kind == DSC_KERNEL_MATMUL) {
            if (si != 0 || !mm0) return "row-fused: a MatMul can only be the first stage";
            const string la = em.load_view(st.inputs[0], sd.inputs[0], {"cb", "cm", "ck"});
            em.funcs << "DSC_INLINE float rows_load_a(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la << ";\n}\n";
            const string lb = em.load_view(st.inputs[1], sd.inputs[1], {"cb", "ck", "cn"});
            em.funcs << "DSC_INLINE float rows_load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";
            k << "    __shared__ float sB[" << S(kblocks * 4 * n) << "];\n";
            k << "    for (int e = threadIdx.x; e < " << S(kblocks * 4 * n) << "; e += " << S(BT) << ") {\n";
            k << "        const int kk = e / " << S(n) << ", nn = e % " << S(n) << ";\n";
            k << "        const float v = rows_load_b(0, min(kk, " << S(K - 1) << "), nn, " << em.params_pass() << ");\n";
            k << "        sB[e] = kk < " << S(K) << " ? v : 0.f;\n    }\n";
            if (fk.row_tail.on) {
                const FusedKernel::RowTail& rt = fk.row_tail;
                const string lb2 = em.load_view(rt.b, rt.mm.raw().inputs[1], {"cb", "ck", "cn"});
                em.funcs << "DSC_INLINE float tail_load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb2 << ";\n}\n";
                k << "    __shared__ __attribute__((aligned(16))) float sB2[" << S(n * K) << "];\n";
                k << "    for (int e = threadIdx.x; e < " << S(n * K) << "; e += " << S(BT) << ") sB2[e] = tail_load_b(0, e / " << S(K) << ", e % " << S(K) << ", " << em.params_pass() << ");\n";
            }
            // every block of the lane requested before anything is used; beyond k the clamped loads meet zeros of B
            k << "    float mm_a[" << S(J) << "][4];\n";
            // a lane's block is four consecutive k: one evaluation of A's producers where they can be taken in quads
            const string la4 = st.inputs[0].virt >= 0 && K % 4 == 0 ? em.load_view4(st.inputs[0], sd.inputs[0], {"cb", "cm", "ck"}) : string();
            if (!la4.empty()) {
                em.funcs << "DSC_INLINE float4 rows_load_a4(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la4 << ";\n}\n";
                k << "#pragma unroll\n    for (int j = 0; j < " << S(J) << "; ++j) {\n";
                k << "        const float4 q = rows_load_a4(0, rowc, min(4 * (col + j * " << S(G) << "), " << S(K - 4) << "), " << em.params_pass() << ");\n";
                k << "        mm_a[j][0] = q.x; mm_a[j][1] = q.y; mm_a[j][2] = q.z; mm_a[j][3] = q.w;\n    }\n";
            } else {
            k << "#pragma unroll\n    for (int j = 0; j < " << S(J) << "; ++j)\n#pragma unroll\n        for (int i = 0; i < 4; ++i)\n";
            k << "            mm_a[j][i] = rows_load_a(0, rowc, min(4 * (col + j * " << S(G) << ") + i, " << S(K - 1) << "), " << em.params_pass() << ");\n";
            }
            if (st.store_a >= 0) {
                // A is evaluated here and nowhere else: the launches that read it later find it in memory
                int64_t ab = 0, ac[DSC_MAX_DIM];
                if (sd.inputs[0].out_shape.rank != 3 || !affine_form(sd.inputs[0], &ab, ac) || ab != 0 || ac[1] != K || ac[2] != 1)
                    return "row-fused: an A operand that is stored must be a plain [m, k] array";
                const string ap = "b" + to_string(fk.outputs[st.store_a]);
                k << "#pragma unroll\n    for (int j = 0; j < " << S(J) << "; ++j) {\n        const int kb = 4 * (col + j * " << S(G) << ");\n";
                if (K % 4 == 0)
                    k << "        if (row_ok && kb < " << S(K) << ") *(float4*)(" << ap << " + row * " << S(K) << " + kb) = make_float4(mm_a[j][0], mm_a[j][1], mm_a[j][2], mm_a[j][3]);\n    }\n";
                else
                    k << "#pragma unroll\n        for (int i = 0; i < 4; ++i)\n            if (row_ok && kb + i < " << S(K) << ") " << ap << "[row * " << S(K) << " + kb + i] = mm_a[j][i];\n    }\n";
            }
            k << "    __syncthreads();\n";
            k << "    float mm_acc[" << S(n) << "];\n#pragma unroll\n    for (int nn = 0; nn < " << S(n) << "; ++nn) mm_acc[nn] = 0.f;\n";
            k << "#pragma unroll\n    for (int j = 0; j < " << S(J) << "; ++j) {\n";
            k << "        const int blk = col + j * " << S(G) << ";\n        if (blk < " << S(kblocks) << ") {\n";
            k << "#pragma unroll\n            for (int i = 0; i < 4; ++i)\n#pragma unroll\n                for (int nn = 0; nn < " << S(n) << "; ++nn)\n";
            k << "                    mm_acc[nn] = fmaf(mm_a[j][i], sB[(4 * blk + i) * " << S(n) << " + nn], mm_acc[nn]);\n        }\n    }\n";
            k << "#pragma unroll\n    for (int nn = 0; nn < " << S(n) << "; ++nn)\n#pragma unroll\n        for (int sft = 1; sft < " << S(G) << "; sft *= 2) mm_acc[nn] += __shfl_xor(mm_acc[nn], sft, 64);\n";
            k << "    float " << pfx << "r = 0.f;\n#pragma unroll\n    for (int nn = 0; nn < " << S(n) << "; ++nn) if (col == nn) " << pfx << "r = mm_acc[nn];\n";
            if (st.outputs[0] >= 0) k << "    if (row_ok && col_ok) b" << fk.outputs[st.outputs[0]] << "[row * " << S(n) << " + col] = " << pfx << "r;\n";
        } else if (sd.kind == DSC_KERNEL_PER_ELEMENT) {
            const bool is_wide = stage_is_wide(si);
            if (!is_wide && sd.shape.dims[0] != m) return "row-fused: per-element stage of the wrong size";
            std::map<int, string> ov;
            for (int i = 0; i < sd.n_inputs; ++i)
                if (st.inputs[i].stage >= 0) ov[i] = stage_var(st.inputs[i].stage, st.inputs[i].stage_out);
            em.emit_pe(k, sd, st.inputs, is_wide ? "wide_gid" : "rowc", pfx, ov, is_wide ? &wide : &narrow);
            for (int o = 0; o < sd.n_outputs; ++o) {
                if (st.outputs[o] < 0) continue;
                const string ptr = "b" + to_string(fk.outputs[st.outputs[o]]);
                if (is_wide) k << "    if (row_ok && col_ok) " << ptr << "[row * " << S(n) << " + col] = " << stage_var(si, o) << ";\n";
                else k << "    if (row_ok && col == 0) " << ptr << "[row] = " << stage_var(si, o) << ";\n";
            }
        } else if (sd.kind == DSC_KERNEL_REDUCE) {
            const bool is_max = sd.reduce_op == DSC_REDUCE_MAX;
            const string init = is_max ? "U2F(0xff800000u)" : "0.f";
            string x;
            if (st.inputs[0].stage >= 0) x = stage_var(st.inputs[0].stage, st.inputs[0].stage_out);
            else x = em.load_view(st.inputs[0], sd.inputs[0], {"rowc", "colc"});
            k << "    float " << pfx << "r = col_ok ? " << x << " : " << init << ";\n";
            for (int64_t off = G / 2; off >= 1; off /= 2) {
                const string other = "__shfl_xor(" + pfx + "r, " + S(off) + ", 64)";
                k << "    " << pfx << "r = " << (is_max ? "glsl_max(" + pfx + "r, " + other + ")" : pfx + "r + " + other) << ";\n";
            }
            if (st.outputs[0] >= 0) k << "    if (row_ok && col == 0) b" << fk.outputs[st.outputs[0]] << "[row] = " << pfx << "r;\n";
        } else {
            return "row-fused: stage must be a per-element or reduce kernel";
        }
    }
    if (fk.row_tail.on) {
        const FusedKernel::RowTail& rt = fk.row_tail;
        const dsc_kernel_desc& td = rt.mm.raw();
        const MatMulDims tg = matmul_dims(td);
        if (!mm0 || tg.batch != 1 || tg.chunks != 1 || tg.m != m || tg.k != n || tg.n != K || K % 4 != 0 || rt.b.buffer < 0 || rt.x_stage < 0 ||
            rt.x_stage >= (int)fk.row_stages.size() || !stage_is_wide(rt.x_stage))
            return "row-fused: the trailing product does not match the rows";
        if (rt.epilogue_a_input >= 0 && fk.row_stages[0].store_a < 0) return "row-fused: the trailing product's consumer reads an operand that is not stored";
        k << "    // trailing product: [m, " << n << "] x [" << n << ", " << K << "], a lane's blocks of four columns as in stage 0\n";
        const string x = stage_var(rt.x_stage, rt.x_stage_out);
        k << "    const int tl_base = (threadIdx.x & 63) / " << S(G) << " * " << S(G) << ";\n";
        k << "    float tl_x[" << S(n) << "];\n#pragma unroll\n    for (int c = 0; c < " << S(n) << "; ++c) tl_x[c] = __shfl(" << x << ", tl_base + c, 64);\n";
        std::ostringstream body;
        int n_res = 1;
        if (rt.has_epilogue) {
            const dsc_kernel_desc& pe = rt.epilogue.raw();
            n_res = pe.n_outputs;
            std::map<int, string> ov;
            ov[rt.epilogue_product_input] = "product";
            if (rt.epilogue_a_input >= 0) ov[rt.epilogue_a_input] = "operand";
            em.emit_pe(body, pe, rt.epilogue_inputs, "gid", "e", ov);
            for (int o = 0; o < pe.n_outputs; ++o) body << "    result[" << o << "] = et" << pe.outputs[o] << ";\n";
            em.funcs << "DSC_INLINE void tail_epilogue(float product, float operand, int gid, float* result, " << em.params_decl() << ") {\n" << body.str() << "}\n";
        }
        if ((int)rt.outputs.size() != n_res) return "row-fused: trailing product output count";
        k << "#pragma unroll\n    for (int j = 0; j < " << S(J) << "; ++j) {\n        const int blk = col + j * " << S(G) << ";\n";
        k << "        if (blk < " << S(kblocks) << ") {\n            float acc[4] = {0.f, 0.f, 0.f, 0.f};\n";
        k << "#pragma unroll\n            for (int c = 0; c < " << S(n) << "; ++c) {\n                const float4 b4 = *(const float4*)&sB2[c * " << S(K) << " + 4 * blk];\n";
        k << "                acc[0] = fmaf(tl_x[c], b4.x, acc[0]); acc[1] = fmaf(tl_x[c], b4.y, acc[1]); acc[2] = fmaf(tl_x[c], b4.z, acc[2]); acc[3] = fmaf(tl_x[c], b4.w, acc[3]);\n            }\n";
        if (rt.has_epilogue) {
            k << "            float res[4][" << n_res << "];\n#pragma unroll\n            for (int i = 0; i < 4; ++i) tail_epilogue(acc[i], mm_a[j][i], rowc * " << S(K) << " + 4 * blk + i, res[i], " << em.params_pass() << ");\n";
            for (int o = 0; o < n_res; ++o)
                k << "            if (row_ok) *(float4*)(b" << fk.outputs[rt.outputs[o]] << " + row * " << S(K) << " + 4 * blk) = make_float4(res[0][" << o << "], res[1][" << o << "], res[2][" << o << "], res[3][" << o << "]);\n";
        } else {
            k << "            if (row_ok) *(float4*)(b" << fk.outputs[rt.outputs[0]] << " + row * " << S(K) << " + 4 * blk) = make_float4(acc[0], acc[1], acc[2], acc[3]);\n";
        }
        k << "        }\n    }\n";
    }
    k << "}\n";
    out->grid = blocks_for(m, (int)per_block);
    out->block = (unsigned)BT;
    out->source = k.str();
    out->note = string(fk.row_tail.on ? "row-fused with the first stage's data gradient behind the last: " : "row-fused: ") + S(G) + " lanes per row, " + to_string(fk.row_stages.size()) + " stages" + (mm0 ? ", the first a MatMul over k=" + S(K) + " shared by the row's lanes" : "");
    return "";
}

// ---- convolution data gradient ---------------------------------------------------------------------------

// Words per pixel of the forward kernel's LDS tile: 16 neighbouring pixels times four channels should fall into 64
// different banks, which they do when the pitch is an odd multiple of four words.
int64_t conv_fwd_pitch(int64_t c) { return (c % 4 == 0 && (c / 4) % 2 == 0) ? c + 4 : c; }

int64_t dgrad_pitch(int64_t k) { return k % 8 == 0 ? k + 4 : k; }  // keeps 16-byte reads of neighbouring pixels off one bank

int64_t dgrad_lds_floats(const FusedKernel::ConvDgrad& c, int64_t k) {
    const int64_t ph = c.oh + c.fh - 1, pw = c.ow + c.fw - 1;
    return std::max(c.oh * c.ow * dgrad_pitch(k), (c.pad_h || c.pad_w) ? ph * pw * c.c : 0);
}

// Workgroup -> (image, group) for the convolution kernels.  Consecutive workgroups go to consecutive XCDs (eight, each
// with its own L2), and the groups of one image share cache lines: a pixel's channels of all groups are one 64- or
// 128-byte run, in the input and in the output.  Workgroups b and b + 8 sit on the same XCD, so the groups of an
// image are 8 apart: the line is fetched into one L2 only and its pieces are written from one L2.
void emit_image_group_of_block(std::ostream& k, int64_t images, int64_t groups) {
    k << "    const int cb = (blockIdx.x / 8) % " << S(groups) << ", img = (blockIdx.x / " << S(8 * groups) << ") * 8 + blockIdx.x % 8;\n";
    if (images % 8 != 0) k << "    if (img >= " << S(images) << ") return;\n";
}
int64_t image_group_grid(int64_t images, int64_t groups) { return (images + 7) / 8 * 8 * groups; }

string gen_conv_dgrad(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const FusedKernel::ConvDgrad& cv = fk.dgrad;
    const MatMulDims g = matmul_dims(d);
    const int64_t K = g.k, G = cv.g, C = cv.c, FH = cv.fh, FW = cv.fw, OH = cv.oh, OW = cv.ow;
    if (g.batch != G || g.m != cv.img * OH * OW || g.n != FH * FW * C || g.chunks != 1) return "conv dgrad: geometry mismatch";
    const int64_t PH = OH + FH - 1, PW = OW + FW - 1;
    const int64_t GC = G * C, PITCH = dgrad_pitch(K);
    const int64_t H = PH - 2 * cv.pad_h, W = PW - 2 * cv.pad_w;
    const bool unpad = cv.pad_h > 0 || cv.pad_w > 0;
    if (H < 1 || W < 1 || K % 4 != 0) return "conv dgrad: unsupported geometry";
    const int64_t lds = dgrad_lds_floats(cv, K);
    if ((lds + PITCH + 4) * 4 > 64 * 1024) return "conv dgrad: image tile does not fit LDS";

    const string la = em.load_view(fk.inputs[0], d.inputs[0], {"cb", "cm", "ck"});
    em.funcs << "DSC_INLINE float load_a(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la << ";\n}\n";
    const string lb = em.load_view(fk.inputs[1], d.inputs[1], {"cb", "ck", "cn"});
    em.funcs << "DSC_INLINE float load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";

    std::ostringstream k;
    const string out_ptr = "b" + to_string(fk.outputs[0]);
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(fk) << "(" << em.kernel_params_decl() << ") {\n";
    k << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    // the last PITCH floats stay zero: a tap outside the output reads them instead of masking every value it loads
    const int64_t zero_at = (lds + 3) / 4 * 4;
    k << "    __shared__ __attribute__((aligned(16))) float lds[" << S(zero_at + PITCH) << "];\n";
    k << "    if (threadIdx.x < " << S(PITCH) << ") lds[" << S(zero_at) << " + threadIdx.x] = 0.f;\n";
    emit_image_group_of_block(k, cv.img, G);
    // 1. dC of this image and group: tile[oy][ox][oc].  (No halo: the taps that fall outside the output are
    // predicated below, which keeps the tile small enough for every workgroup of a ConvNet-sized launch to be
    // resident at once.)  Groups of 8 loads are issued before any of them is stored: one memory round trip per
    // group, not per element.
    const int64_t fill_n = OH * OW * K;
    k << "    for (int i0 = threadIdx.x; i0 < " << S(fill_n) << "; i0 += 2048) {\n        float v[8];\n";
    k << "#pragma unroll\n        for (int u = 0; u < 8; ++u) {\n";
    k << "            const int i = min(i0 + u * 256, " << S(fill_n - 1) << ");\n";
    k << "            v[u] = load_a(cb, img * " << S(OH * OW) << " + i / " << S(K) << ", i % " << S(K) << ", " << em.params_pass() << ");\n        }\n";
    k << "        __builtin_amdgcn_sched_barrier(0);\n";
    k << "#pragma unroll\n        for (int u = 0; u < 8; ++u) {\n";
    k << "            const int i = i0 + u * 256;\n";
    k << "            if (i < " << S(fill_n) << ") lds[(i / " << S(K) << ") * " << S(PITCH) << " + i % " << S(K) << "] = v[u];\n        }\n    }\n";
    k << "    __syncthreads();\n";
    // 2. one padded-image pixel per thread and pass: acc[c] over taps and output channels; the filter element is
    // the same for every lane, so it comes through the scalar unit.  The tap loop stays a loop and each block of
    // 8 channels is fenced: unrolled whole, the scheduler would hoist all the filter loads to the top and spill
    // the scalar registers holding them.
    const int64_t passes = (PH * PW + 255) / 256;
    const int64_t OCB = K % 8 == 0 ? 8 : 4;
    k << "    float acc[" << passes << "][" << S(C) << "];\n";
    k << "#pragma unroll\n    for (int ps = 0; ps < " << passes << "; ++ps) {\n";
    k << "        const int p = min(ps * 256 + (int)threadIdx.x, " << S(PH * PW - 1) << ");\n";
    k << "        const int py = p / " << S(PW) << ", px = p % " << S(PW) << ";\n";
    k << "#pragma unroll\n        for (int c = 0; c < " << S(C) << "; ++c) acc[ps][c] = 0.f;\n";
    k << "#pragma unroll 1\n        for (int tap = 0; tap < " << S(FH * FW) << "; ++tap) {\n";
    k << "            const int fy = tap / " << S(FW) << ", fx = tap % " << S(FW) << ";\n";
    k << "            const int oy = py - fy, ox = px - fx;\n";
    k << "            const bool inside = oy >= 0 && oy < " << S(OH) << " && ox >= 0 && ox < " << S(OW) << ";\n";
    k << "            const float* src = &lds[inside ? (oy * " << S(OW) << " + ox) * " << S(PITCH) << " : " << S(zero_at) << "];\n";
    k << "#pragma unroll\n            for (int oc = 0; oc < " << S(K) << "; oc += " << OCB << ") {\n";
    k << "                float a[" << OCB << "];\n";
    k << "#pragma unroll\n                for (int q = 0; q < " << OCB << "; q += 4) {\n";
    k << "                    const float4 a4 = *(const float4*)(src + oc + q);\n";
    k << "                    a[q] = a4.x; a[q + 1] = a4.y; a[q + 2] = a4.z; a[q + 3] = a4.w;\n                }\n";
    k << "#pragma unroll\n                for (int j = 0; j < " << OCB << "; ++j)\n";
    k << "#pragma unroll\n                    for (int c = 0; c < " << S(C) << "; ++c)\n";
    k << "                        acc[ps][c] = fmaf(a[j], load_b(cb, oc + j, tap * " << S(C) << " + c, " << em.params_pass() << "), acc[ps][c]);\n";
    k << "                __builtin_amdgcn_sched_barrier(0);\n";
    k << "            }\n        }\n    }\n";
    if (!unpad) {
        k << "#pragma unroll\n    for (int ps = 0; ps < " << passes << "; ++ps) {\n";
        k << "        const int p = ps * 256 + (int)threadIdx.x;\n        if (p < " << S(PH * PW) << ") {\n";
        k << "#pragma unroll\n            for (int c = 0; c < " << S(C) << "; ++c) " << out_ptr << "[(img * " << S(PH * PW) << " + p) * " << S(GC)
          << " + cb * " << S(C) << " + c] = acc[ps][c];\n        }\n    }\n}\n";
    } else {
        // 3. the padded-image gradient goes through LDS (the tile is dead by now); each pixel of the image then sums
        // the padded pixels that replicate it: itself, plus the border rows / columns for pixels on the edge
        k << "    __syncthreads();\n";
        k << "#pragma unroll\n    for (int ps = 0; ps < " << passes << "; ++ps) {\n";
        k << "        const int p = ps * 256 + (int)threadIdx.x;\n        if (p < " << S(PH * PW) << ") {\n";
        k << "#pragma unroll\n            for (int c = 0; c < " << S(C) << "; ++c) lds[p * " << S(C) << " + c] = acc[ps][c];\n        }\n    }\n";
        k << "    __syncthreads();\n";
        k << "    for (int i = threadIdx.x; i < " << S(H * W * C) << "; i += 256) {\n";
        k << "        const int c = i % " << S(C) << ", x = (i / " << S(C) << ") % " << S(W) << ", y = i / " << S(C * W) << ";\n";
        k << "        float sum = 0.f;\n";
        // candidate rows / columns: the pixel's own, and the border ones when it lies on the edge (as the Unpad
        // kernel: k_min = in - (coord == 0 ? pad : 0), k_max = in + (coord == last ? pad : 0))
        const string outer = cv.rows_first ? "jx" : "jy", inner = cv.rows_first ? "jy" : "jx";
        auto range = [&](const string& j) {
            const bool is_y = j == "jy";
            return "for (int " + j + " = " + S(-(is_y ? cv.pad_h : cv.pad_w)) + "; " + j + " <= " + S(is_y ? cv.pad_h : cv.pad_w) + "; ++" + j + ")";
        };
        if (H > 1 && W > 1) {
            // a pixel lies on at most one edge per axis, so it has at most pad + 1 candidates per axis, taken in rising
            // order: on the first edge the padded coordinates 0..pad, on the last one own..own + pad, else its own
            auto slots = [&](const string& q, bool is_y) {
                return "for (int " + q + " = 0; " + q + " <= " + S(is_y ? cv.pad_h : cv.pad_w) + "; ++" + q + ")";
            };
            const string qo = cv.rows_first ? "qx" : "qy", qi = cv.rows_first ? "qy" : "qx";
            k << "        const bool edge_y = y == 0 || y == " << S(H - 1) << ", edge_x = x == 0 || x == " << S(W - 1) << ";\n";
            k << "        const int base_y = y == 0 ? 0 : y + " << S(cv.pad_h) << ", base_x = x == 0 ? 0 : x + " << S(cv.pad_w) << ";\n";
            k << "#pragma unroll\n        " << slots(qo, !cv.rows_first) << " {\n            float part = 0.f;\n";
            k << "#pragma unroll\n            " << slots(qi, cv.rows_first) << " {\n";
            k << "                const bool ok = (edge_y || qy == 0) && (edge_x || qx == 0);\n";
            k << "                const int ky = base_y + (edge_y ? qy : 0), kx = base_x + (edge_x ? qx : 0);\n";
            k << "                const float w = lds[(ky * " << S(PW) << " + kx) * " << S(C) << " + c];\n";
            k << "                part += ok ? w : 0.f;\n            }\n            sum += part;\n        }\n";
        } else {
        k << "#pragma unroll\n        " << range(outer) << " {\n            float part = 0.f;\n";
        k << "#pragma unroll\n            " << range(inner) << " {\n";
        k << "                const bool ok_y = jy == 0 || (jy < 0 && y == 0) || (jy > 0 && y == " << S(H - 1) << ");\n";
        k << "                const bool ok_x = jx == 0 || (jx < 0 && x == 0) || (jx > 0 && x == " << S(W - 1) << ");\n";
        k << "                const int ky = clampi(y + " << S(cv.pad_h) << " + jy, 0, " << S(PH - 1) << "), kx = clampi(x + " << S(cv.pad_w)
          << " + jx, 0, " << S(PW - 1) << ");\n";
        k << "                const float w = lds[(ky * " << S(PW) << " + kx) * " << S(C) << " + c];\n";
        k << "                part += (ok_y && ok_x) ? w : 0.f;\n            }\n            sum += part;\n        }\n";
        }
        k << "        " << out_ptr << "[((img * " << S(H) << " + y) * " << S(W) << " + x) * " << S(GC) << " + cb * " << S(C) << " + c] = sum;\n    }\n}\n";
    }
    if (image_group_grid(cv.img, G) >= kMaxIndex) return "conv dgrad: grid too large";
    out->grid = (unsigned)image_group_grid(cv.img, G);
    out->block = 256;
    out->source = k.str();
    out->note = "conv data gradient: workgroup per image and group, tile in LDS, " + S(FH) + "x" + S(FW) + " taps x " + S(K) + " channels" +
                (unpad ? ", border folds fused" : "");
    return "";
}

// ---- convolution backward: data gradient and filter gradient in one kernel ---------------------------------

// Workgroup = (group, set of images).  Per image: dC of the image goes to LDS in *slots* -- slot oy * PW + ox with
// PW = ow + fw - 1 the width of the padded image, so that the slots of an output row are followed by fw - 1 slots
// that stay zero -- and the image's padded input tile goes to LDS as in the forward kernel.  The data gradient is
// then what the data-gradient kernel computes (one padded pixel per thread, taps x output channels, border folds
// through LDS).  The filter gradient is im2col^T x dC over the slots: with the padded pitch, the im2col element of
// slot q for tap (fy, fx) and channel c is one tile word at (q + fy * PW + fx) * pitch + c, so the A fragment of
// v_mfma_f32_16x16x4f32 (lane l: row kidx = 16 * mt + l % 16, slot 4 * s + l / 16) is a per-lane constant plus a
// per-step term, and the B fragment is dC[slot][oc].  Slots without a pixel multiply a zero, whatever the tile word
// beside them holds.  One im2col row of ones (kidx = fh * fw * c) makes row fh*fw*c of the product the column sums
// of dC: the bias gradient.  The accumulators live across the workgroup's images; the four waves take every fourth
// step and are summed through LDS at the end, one partial product per workgroup.
struct ConvBwdLayout {
    int64_t PH, PW, KD, PITCH, CP, SLP, steps, DC_AT, ZERO_AT, XT_AT, XT_FLOATS, ONE_AT, ZW_AT, GB_AT, TOTAL;
    int MT, NT;
    // data gradient on the matrix cores (see gen_conv_bwd): pixels per group, shifted taps per filter row, B fragments
    // per lane, groups per image row, groups, tiles of 16 groups, tiles per wave
    bool mfma_dgrad;
    int64_t P, TQ, GS, GPR, GROUPS, TILES, TPW;
};

ConvBwdLayout conv_bwd_layout(const FusedKernel::ConvDgrad& full, int64_t K, int64_t cp_override = 0) {
    FusedKernel::ConvDgrad c = full;
    if (c.wgrad_only && c.bands > 1) c.oh = full.oh / c.bands;  // the tiles hold one band of output rows
    ConvBwdLayout L{};
    L.PH = c.oh + c.fh - 1;
    L.PW = c.ow + c.fw - 1;
    L.KD = c.fh * c.fw * c.c;
    L.CP = cp_override > 0 ? cp_override : conv_fwd_pitch(c.c);
    L.MT = (int)((L.KD + (c.bias ? 1 : 0) + 15) / 16);
    L.NT = (int)((K + 15) / 16);
    L.P = (c.c == 4 || c.c == 8 || c.c == 16) ? 16 / c.c : 0;
    L.TQ = c.fw + L.P - 1;
    L.GS = L.P ? c.fh * L.TQ * K / 4 : 0;
    L.GPR = L.P ? (L.PW + L.P - 1) / L.P : 1;
    L.GROUPS = L.PH * L.GPR;
    L.TILES = (L.GROUPS + 15) / 16;
    L.TPW = (L.TILES + 3) / 4;
    L.mfma_dgrad = L.P > 0 && L.GS <= 96 && L.TPW <= 8 && !c.wgrad_only;
    // the FMA form reads 16-byte pieces of a slot; the filter gradient alone reads four consecutive slots' words
    // li .. li + 15, which K words per slot spread over all banks
    L.PITCH = c.wgrad_only ? K : dgrad_pitch(K);
    if (L.mfma_dgrad) {
        // words per slot: the one (from k to k + 8) that spreads an A fragment load of the data gradient -- lane l reads
        // word l / 16 of the slot of group l % 16 -- over the most of the 64 banks
        int best_worst = 1 << 30;
        for (int64_t pitch = K; pitch <= K + 8; ++pitch) {
            int lanes_on_bank[64] = {0};
            int worst = 0;
            for (int l = 0; l < 64; ++l) {
                const int64_t grp = l % 16, slot = (grp / L.GPR) * L.PW + (grp % L.GPR) * L.P;
                worst = std::max(worst, ++lanes_on_bank[(slot * pitch + l / 16) % 64]);
            }
            if (worst < best_worst) {
                best_worst = worst;
                L.PITCH = pitch;
            }
        }
    }
    L.SLP = (c.oh * L.PW + 3) / 4 * 4;
    L.steps = L.SLP / 4;
    // With the data gradient on the matrix cores the slots start behind fw - 1 slots that stay zero and the zero row is
    // as long as a filter row's taps reach: a lane's fragments of a filter row then lie at literal distances from one
    // address (a tap left of the image falls on the zero slots that end the row above, or on the head), and a filter
    // row outside the image takes that address to the zero row as a whole.
    L.DC_AT = L.mfma_dgrad ? ((c.fw - 1) * L.PITCH + 3) / 4 * 4 : 0;
    L.ZERO_AT = L.DC_AT + L.SLP * L.PITCH;
    L.XT_AT = (L.ZERO_AT + (L.mfma_dgrad ? (L.TQ - 1) * L.PITCH + K + 4 : L.PITCH) + 3) / 4 * 4;
    const int64_t pixels = std::max(L.PH * L.PW, L.SLP + (c.fh - 1) * L.PW + c.fw - 1);  // what a fragment load may address
    L.XT_FLOATS = (pixels * L.CP + 3) / 4 * 4;
    L.ONE_AT = L.XT_AT + L.XT_FLOATS;
    L.ZW_AT = L.ONE_AT + 1;
    // the data gradient's B fragments (one word per lane and step) stay in LDS: in registers they would cost the
    // kernel a wave of occupancy
    L.GB_AT = L.ONE_AT + 4;
    L.TOTAL = std::max<int64_t>(L.GB_AT + (L.mfma_dgrad ? L.GS * 64 : 0), (int64_t)4 * L.MT * L.NT * 256);
    // four workgroups per CU (160 KB of LDS) matter more than the input tile's bank spread
    if (cp_override == 0 && L.CP != c.c && L.TOTAL * 4 * 4 > 160 * 1024) {
        const ConvBwdLayout tight = conv_bwd_layout(full, K, c.c);
        if (tight.TOTAL * 4 * 4 <= 160 * 1024) return tight;
    }
    return L;
}

bool conv_bwd_fits_impl(const FusedKernel::ConvDgrad& c, int64_t k) {
    if (c.wgrad_only ? (k % 4 != 0 || c.g * c.c > 64) : !conv_dgrad_fits(c, k)) return false;
    const ConvBwdLayout L = conv_bwd_layout(c, k);
    if (c.bands < 1 || (c.bands > 1 && (!c.wgrad_only || c.oh % c.bands != 0))) return false;
    return L.TOTAL * 4 <= 64 * 1024 && L.MT * L.NT <= 8 && c.chunks >= 8 && c.chunks % 8 == 0;
}

// Whether the convolution backward kernel of this geometry runs with loader waves.  Without them a workgroup is one
// chain per image -- request the tiles, wait, store them to LDS, barrier, matrix phases, folds -- and the workgroups
// that share a CU walk it in step, so fill time and matrix time add up.  With them a workgroup has eight waves and two
// tile buffers: waves 4-7 only ever fill the buffer of the set's next image (their registers hold the loads in
// flight; they own no accumulators), waves 0-3 only ever run the matrix phases and the folds of the current one, and
// one barrier per image hands the buffers over.  Two such workgroups have to fit a CU's 160 KB of LDS.
bool conv_bwd_loader_waves_impl(const FusedKernel& fk) {
    const FusedKernel::ConvDgrad& cv = fk.dgrad;
    if (!cv.on || !cv.wgrad || cv.wgrad_only || fk.as_part) return false;
    if (const char* e = std::getenv("DSC_CONV_BWD_LOADERS"))
        if (e[0] == '0') return false;
    const MatMulDims g = matmul_dims(fk.main.raw());
    const ConvBwdLayout L = conv_bwd_layout(cv, g.k);
    const int64_t total = std::max<int64_t>(2 * L.ONE_AT + 4 + (L.mfma_dgrad ? L.GS * 64 : 0), (int64_t)4 * L.MT * L.NT * 256);
    return total * 4 <= 80 * 1024 && cv.img >= 2 * cv.chunks - cv.chunks / 2;  // most sets hold two images or more
}

string gen_conv_bwd(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const FusedKernel::ConvDgrad& cv = fk.dgrad;
    const MatMulDims g = matmul_dims(d);
    const bool wonly = cv.wgrad_only;
    const int64_t BANDS = wonly ? cv.bands : 1, OHF = cv.oh;  // OH below: the output rows a workgroup's tiles hold
    const int64_t K = wonly ? g.n : g.k, G = cv.g, C = cv.c, FH = cv.fh, FW = cv.fw, OH = OHF / BANDS, OW = cv.ow, IMG = cv.img;
    if (wonly ? (g.batch != G || g.k != IMG * OHF * OW || g.m != FH * FW * C) : (g.batch != G || g.m != IMG * OH * OW || g.n != FH * FW * C || g.chunks != 1))
        return "conv backward: geometry mismatch";
    if (fk.inputs.size() != 3 || fk.inputs[2].buffer < 0) return "conv backward: the image must be a buffer";
    if ((int)fk.outputs.size() != (wonly ? 1 : 2) + (cv.bias ? 1 : 0)) return "conv backward: output count";
    const int DC = wonly ? 1 : 0;  // which operand of `main` is dC: [g][(img, oy, ox)][oc] either way
    if (!conv_bwd_fits_impl(cv, K)) return "conv backward: geometry does not fit";
    const ConvBwdLayout L = conv_bwd_layout(cv, K);
    const int64_t PH = L.PH, PW = L.PW, KD = L.KD, PITCH = L.PITCH, CP = L.CP, GC = G * C;
    const int64_t H = OHF + FH - 1 - 2 * cv.pad_h, W = PW - 2 * cv.pad_w;
    const bool unpad = cv.pad_h > 0 || cv.pad_w > 0;
    const int MT = L.MT, NT = L.NT;
    if (H < 1 || W < 1 || K % 4 != 0) return "conv backward: unsupported geometry";
    // Loader waves (see conv_bwd_loader_waves): 512 threads, the upper four waves fill the other of two tile buffers
    // with the set's next image while the lower four run the matrix phases of the current one.
    const bool spec = conv_bwd_loader_waves_impl(fk);
    const int64_t BLOCK = spec ? 512 : 256;
    const int64_t BUFSZ = L.ONE_AT;  // one buffer: dC slots, the zero row, the input tile
    const int64_t ONE_AT = spec ? 2 * BUFSZ : L.ONE_AT, ZW_AT = ONE_AT + 1, GB_AT = ONE_AT + 4;
    const int64_t TOTAL = spec ? std::max<int64_t>(GB_AT + (L.mfma_dgrad ? L.GS * 64 : 0), (int64_t)4 * MT * NT * 256) : L.TOTAL;

    const string la = em.load_view(fk.inputs[DC], d.inputs[DC], {"cb", "cm", "ck"});
    em.funcs << "DSC_INLINE float load_a(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la << ";\n}\n";
    // four consecutive output channels of a pixel from one evaluation of the producers, where they allow it
    const string la4 = fk.inputs[DC].virt >= 0 && K % 4 == 0 ? em.load_view4(fk.inputs[DC], d.inputs[DC], {"cb", "cm", "ck"}) : string();
    if (!la4.empty())
        em.funcs << "DSC_INLINE float4 load_a4(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la4 << ";\n}\n";
    if (!wonly) {
        const string lb = em.load_view(fk.inputs[1], d.inputs[1], {"cb", "ck", "cn"});
        em.funcs << "DSC_INLINE float load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";
    }

    std::ostringstream k;
    const string out_ptr = "b" + to_string(fk.outputs[0]), part_ptr = "b" + to_string(fk.outputs[wonly ? 0 : 1]);
    const string img_ptr = "b" + to_string(fk.inputs[2].buffer);
    k << "typedef float cb_float4 __attribute__((ext_vector_type(4)));\n";
    k << "extern \"C\" __global__ __launch_bounds__(" << S(BLOCK) << (spec ? ", 4" : "") << ") void " << entry_name(fk) << "(" << em.kernel_params_decl() << ") {\n";
    k << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    k << "    __shared__ __attribute__((aligned(16))) float smem[" << S(TOTAL) << "];\n";
    k << "    float* const lds = smem;\n    float* const xt = smem + " << S(L.XT_AT) << ";\n";
    // the groups of a set of images sit 8 workgroups apart: same XCD, same L2 (they share the lines of dC, of the
    // image and of the output)
    if (BANDS > 1)
        k << "    const int band = blockIdx.x / " << S(cv.chunks * G) << ", in_band = blockIdx.x % " << S(cv.chunks * G) << ";\n";
    else
        k << "    const int band = 0, in_band = blockIdx.x;\n";
    k << "    const int cb = (in_band / 8) % " << S(G) << ", chunk = (in_band / " << S(8 * G) << ") * 8 + in_band % 8;\n";
    // tid / wave: a thread's place among the 256 that share a role (all of them without loader waves)
    // (the role comes through readfirstlane: a branch the compiler knows to be uniform is a scalar branch, so no wave
    // ever walks the other role's barriers with an empty execution mask)
    if (spec) k << "    const int tid = threadIdx.x & 255;\n    const bool loader = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 8)) != 0;\n";
    else k << "    const int tid = threadIdx.x;\n";
    k << "    const int lane = tid & 63, wave = " << (spec ? "__builtin_amdgcn_readfirstlane(tid >> 6)" : "tid >> 6") << ", li = lane & 15, lk = lane >> 4;\n";
    // what stays zero for the whole kernel: slots without a pixel, the zero row, the tile words behind the last pixel
    if (spec) {
        // (with loader waves no barrier stands between this and the first image's fills: only the words no fill writes
        // and a fragment may read are cleared -- the head, the slots right of the output's columns, the slots behind
        // its last row with the zero row, the tile words behind the last pixel)
        const int64_t RB = (PW - OW) * PITCH;
        auto clear_range = [&](int64_t from, int64_t to) {
            for (int64_t b2 = 0; b2 < 2; ++b2)
                if (to > from)
                    k << "    for (int i = threadIdx.x; i < " << S(to - from) << "; i += " << S(BLOCK) << ") smem[" << S(b2 * BUFSZ + from) << " + i] = 0.f;\n";
        };
        clear_range(0, L.DC_AT);
        clear_range(L.DC_AT + OH * PW * PITCH, L.XT_AT);
        clear_range(L.XT_AT + PH * PW * CP, BUFSZ);
        if (RB > 0) {
            k << "    for (int i = threadIdx.x; i < " << S(2 * OH * RB) << "; i += " << S(BLOCK) << ") {\n";
            k << "        const int r = i % " << S(OH * RB) << ";\n";
            k << "        smem[(i / " << S(OH * RB) << ") * " << S(BUFSZ) << " + " << S(L.DC_AT) << " + ((r / " << S(RB) << ") * " << S(PW) << " + " << S(OW) << ") * " << S(PITCH) << " + r % " << S(RB) << "] = 0.f;\n    }\n";
        }
    } else {
        k << "    for (int i = threadIdx.x; i < " << S(ONE_AT) << "; i += " << S(BLOCK) << ") smem[i] = 0.f;\n";
    }
    k << "    if (threadIdx.x == 0) { smem[" << S(ONE_AT) << "] = 1.f; smem[" << S(ZW_AT) << "] = 0.f; }\n";
    // fragment addresses of this lane: a constant, plus the step's slot term where the mask says so
    k << "    int a_off[" << MT << "], a_msk[" << MT << "], b_off[" << NT << "], b_msk[" << NT << "];\n";
    k << "#pragma unroll\n    for (int mt = 0; mt < " << MT << "; ++mt) {\n";
    k << "        const int kidx = mt * 16 + li, tap = kidx / " << S(C) << ";\n";
    k << "        const bool real = kidx < " << S(KD) << ";\n";
    k << "        a_off[mt] = real ? " << S(L.XT_AT) << " + ((tap / " << S(FW) << ") * " << S(PW) << " + tap % " << S(FW) << ") * " << S(CP) << " + kidx % " << S(C)
      << " : (" << (cv.bias ? "kidx == " + S(KD) : string("false")) << " ? " << S(ONE_AT) << " : " << S(ZW_AT) << ");\n";
    k << "        a_msk[mt] = real ? -1 : 0;\n    }\n";
    k << "#pragma unroll\n    for (int nt = 0; nt < " << NT << "; ++nt) {\n";
    k << "        const int oc = nt * 16 + li;\n";
    k << "        b_off[nt] = oc < " << S(K) << " ? " << S(L.DC_AT) << " + oc : " << S(L.ZERO_AT) << ";\n        b_msk[nt] = oc < " << S(K) << " ? -1 : 0;\n    }\n";
    k << "    cb_float4 wacc[" << MT << "][" << NT << "];\n";
    k << "#pragma unroll\n    for (int mt = 0; mt < " << MT << "; ++mt)\n#pragma unroll\n        for (int nt = 0; nt < " << NT
      << "; ++nt) wacc[mt][nt] = (cb_float4){0.f, 0.f, 0.f, 0.f};\n";
    // Data gradient on the matrix cores.  With few channels a 16-wide MFMA column block would be mostly empty, so a
    // row of the product is a *group* of P = 16 / c neighbouring pixels of the padded image and a column is (pixel of
    // the group, channel): dX[y][x0 + par][c] = sum over (ty, tq, oc) of dC[y - ty][x0 - tq][oc] * W'[ty][tq][oc][(par, c)]
    // with tq = tx - par running over fw + P - 1 values and W' = W[oc][ty][tq + par][c] where that tap exists, else 0.
    // The A fragment (lane l: group l % 16, k = 4 s + l / 16) is then dC of one slot for all four k of a step, and
    // the B fragments are the same for every group: they stay in registers for the whole kernel.
    const int64_t P = L.P, TQ = L.TQ, GS = L.GS, GPR = L.GPR, GROUPS = L.GROUPS, TPW = L.TPW;
    const bool mfma_dgrad = L.mfma_dgrad;
    // the geometry whose border folds are lane exchanges (below): pairs of 8 channels, 8 pairs per padded row (two rows
    // per tile of 16 pairs), one replicated pixel on every side
    const bool reg_fold = mfma_dgrad && !wonly && C == 8 && PW == 16 && PH % 2 == 0 && cv.pad_h == 1 && cv.pad_w == 1 && H > 1 && W > 1 &&
                          !(std::getenv("DSC_CONV_BWD_REGFOLD") && std::getenv("DSC_CONV_BWD_REGFOLD")[0] == '0');
    if (mfma_dgrad && spec) {
        // this lane's pixel group in each of the wave's tiles: its row, and the word of its first tap in filter row 0
        k << "    int dgy[" << S(TPW) << "], dbase[" << S(TPW) << "];\n";
        k << "#pragma unroll\n    for (int t = 0; t < " << S(TPW) << "; ++t) {\n";
        k << "        const int grp = (t * 4 + wave) * 16 + li;\n        dgy[t] = grp / " << S(GPR) << ";\n";
        k << "        dbase[t] = " << S(L.DC_AT) << " + (dgy[t] * " << S(PW) << " + (grp % " << S(GPR) << ") * " << S(P) << " - " << S(FW - 1) << ") * " << S(PITCH) << " + lk;\n    }\n";
    }
    // (with loader waves the four matrix waves take a quarter of the fragments each, while the loader waves already
    // have the set's first image requested: one round trip to memory before the first product, not two)
    auto emit_b_fragments = [&](bool shared_out) {
        k << "    {\n";
        k << "        const int par = li / " << S(C) << ", gc = li % " << S(C) << ";\n";
        for (int64_t w4 = 0; w4 < (shared_out ? 4 : 1); ++w4) {
            if (shared_out) k << "        " << (w4 ? "else " : "") << "if (wave == " << S(w4) << ") {\n";
            for (int64_t s = shared_out ? w4 : 0; s < GS; s += shared_out ? 4 : 1) {
                const int64_t oc0 = (4 * s) % K, tt = (4 * s) / K, ty = tt / TQ, tq = tt % TQ - (P - 1);
                k << "        { const int tx = " << S(tq) << " + par; const float w = load_b(cb, " << S(oc0) << " + lk, (" << S(ty * FW) << " + clampi(tx, 0, " << S(FW - 1)
                  << ")) * " << S(C) << " + gc, " << em.params_pass() << "); smem[" << S(GB_AT + s * 64) << " + lane] = (tx >= 0 && tx < " << S(FW) << ") ? w : 0.f; }\n";
            }
            if (shared_out) k << "        }\n";
        }
        k << "    }\n";
    };
    if (mfma_dgrad && !spec) emit_b_fragments(false);
    // Fills.  The loads of an image -- dC of the image and group, and the image's padded input tile,
    // xt[py][px][c] = image[clamp(py - pad_h)][clamp(px - pad_w)][c] -- are all issued before the first of them is
    // stored to LDS: one round trip to memory per image.  (Requesting the next image's loads before the matrix phases
    // of the current one, to have them in flight meanwhile, measured slower: 45.8 us against 42.2 for the ConvNet's
    // second convolution -- the registers that hold them cost a wave of occupancy.)
    // dC in 16-byte pieces when the operand is a buffer whose k runs along memory
    int64_t dc_base = 0, dc_coef[DSC_MAX_DIM] = {0};
    const bool vec_dc = fk.inputs[DC].buffer >= 0 && K % 4 == 0 && affine_form(d.inputs[DC], &dc_base, dc_coef) && dc_coef[2] == 1 && dc_base % 4 == 0 &&
                        dc_coef[1] % 4 == 0 && (G == 1 || dc_coef[0] % 4 == 0);
    // Four consecutive output channels of a pixel per thread also when dC is a fused producer: the producers' index
    // arithmetic (divisions by the extents of every view on the way) is then shared by the four evaluations, whose
    // element ids differ in their two lowest bits only.
    const bool quad_dc = K % 4 == 0;
    // dC read off the pooling windows' words (ConvDgrad::PoolMasks): a word and the window's four dP values per quad
    const bool pmask = cv.pm.on;
    if (pmask && (K % 4 != 0 || OHF % 2 != 0 || OW % 2 != 0 || fk.inputs[DC].buffer < 0 || cv.pm.masks.buffer < 0))
        return "conv backward: pooling words need channel quads, even extents and buffers";
    const string pm_leak = "U2F(0x" + [&] { char b[16]; std::snprintf(b, sizeof b, "%08x", cv.pm.leak_bits); return string(b); }() + "u)";
    const int64_t dunit = quad_dc ? 4 : 1;
    const int64_t fill_n = OH * OW * K / dunit, NC = (fill_n + 255) / 256;
    const bool vec_fill = C % 4 == 0;
    const int64_t unit = vec_fill ? 4 : 1, xn = PH * PW * C / unit, NX = (xn + 255) / 256;
    const string vt = vec_fill ? "float4" : "float", dvt = quad_dc ? "float4" : "float";
    auto emit_issue = [&](const string& img, const string& ind) {
        k << "#pragma unroll\n" << ind << "for (int u = 0; u < " << S(NC) << "; ++u) {\n";
        k << ind << "    const int i = min(tid + u * 256, " << S(fill_n - 1) << ") * " << S(dunit) << ";\n";
        if (pmask) {
            k << ind << "    const int pi = i / " << S(K) << ", oc = i % " << S(K) << ", wy = (band * " << S(OH) << " + pi / " << S(OW) << ") >> 1, wx = (pi % " << S(OW) << ") >> 1;\n";
            k << ind << "    pw[u] = ((const uint*)b" << cv.pm.masks.buffer << ")[((cb * " << S(IMG) << " + " << img << ") * " << S((OHF / 2) * (OW / 2)) << " + wy * " << S(OW / 2)
              << " + wx) * " << S(K / 4) << " + (oc >> 2)];\n";
            k << ind << "    pv[u] = *(const float4*)(b" << fk.inputs[DC].buffer << " + ((" << img << " * " << S(OHF / 2) << " + wy) * " << S(OW / 2) << " + wx) * " << S(G * K)
              << " + cb * " << S(K) << " + oc);\n" << ind << "}\n";
        } else if (vec_dc)
            k << ind << "    pv[u] = *(const float4*)(b" << fk.inputs[DC].buffer << " + " << S(dc_base) << " + cb * " << S(G == 1 ? 0 : dc_coef[0]) << " + (" << img << " * "
              << S(OHF * OW) << " + band * " << S(OH * OW) << " + i / " << S(K) << ") * " << S(dc_coef[1]) << " + i % " << S(K) << ");\n" << ind << "}\n";
        else if (quad_dc && !la4.empty()) {
            k << ind << "    const int pix = " << img << " * " << S(OHF * OW) << " + band * " << S(OH * OW) << " + i / " << S(K) << ", oc = i % " << S(K) << ";\n";
            k << ind << "    pv[u] = load_a4(cb, pix, oc, " << em.params_pass() << ");\n" << ind << "}\n";
        } else if (quad_dc) {
            k << ind << "    const int pix = " << img << " * " << S(OHF * OW) << " + band * " << S(OH * OW) << " + i / " << S(K) << ", oc = i % " << S(K) << ";\n";
            k << ind << "    pv[u] = make_float4(load_a(cb, pix, oc, " << em.params_pass() << "), load_a(cb, pix, oc + 1, " << em.params_pass() << "), load_a(cb, pix, oc + 2, "
              << em.params_pass() << "), load_a(cb, pix, oc + 3, " << em.params_pass() << "));\n" << ind << "}\n";
        } else
            k << ind << "    pv[u] = load_a(cb, " << img << " * " << S(OHF * OW) << " + band * " << S(OH * OW) << " + i / " << S(K) << ", i % " << S(K) << ", " << em.params_pass() << ");\n" << ind << "}\n";
        k << "#pragma unroll\n" << ind << "for (int u = 0; u < " << S(NX) << "; ++u) {\n";
        k << ind << "    const int e = min(tid + u * 256, " << S(xn - 1) << ") * " << S(unit) << ";\n";
        k << ind << "    const int ch = e % " << S(C) << ", px = (e / " << S(C) << ") % " << S(PW) << ", py = e / " << S(C * PW) << ";\n";
        k << ind << "    const int sy = clampi(py + band * " << S(OH) << " - " << S(cv.pad_h) << ", 0, " << S(H - 1) << "), sx = clampi(px - " << S(cv.pad_w) << ", 0, " << S(W - 1) << ");\n";
        k << ind << "    xv[u] = *(const " << vt << "*)(" << img_ptr << " + ((" << img << " * " << S(H) << " + sy) * " << S(W) << " + sx) * " << S(GC) << " + cb * " << S(C)
          << " + ch);\n" << ind << "}\n";
        k << ind << "__builtin_amdgcn_sched_barrier(0);\n";
    };
    auto emit_tile_stores = [&](const string& ind, const string& buf) {
        k << "#pragma unroll\n" << ind << "for (int u = 0; u < " << S(NC) << "; ++u) {\n";
        k << ind << "    const int i = (tid + u * 256) * " << S(dunit) << ", pi = i / " << S(K) << ";\n";
        if (pmask) {
            k << ind << "    {\n" << ind << "        const uint bits = pw[u] >> (8 * (((pi % " << S(OW) << ") & 1) | (((band * " << S(OH) << " + pi / " << S(OW) << ") & 1) << 1)));\n";
            const char* comp[4] = {"x", "y", "z", "w"};
            for (int j = 0; j < 4; ++j)
                k << ind << "        { const float v = (bits & " << (1u << (2 * j)) << "u) ? pv[u]." << comp[j] << " : 0.f; pv[u]." << comp[j] << " = (bits & " << (2u << (2 * j))
                  << "u) ? v : v * " << pm_leak << "; }\n";
            k << ind << "    }\n";
        }
        k << ind << "    float* const at = lds + " << buf << " + " << S(L.DC_AT) << " + ((pi / " << S(OW) << ") * " << S(PW) << " + pi % " << S(OW) << ") * " << S(PITCH) << " + i % " << S(K) << ";\n";
        if (quad_dc && PITCH % 4 == 0)
            k << ind << "    if (tid + u * 256 < " << S(fill_n) << ") *(float4*)at = pv[u];\n" << ind << "}\n";
        else if (quad_dc)
            k << ind << "    if (tid + u * 256 < " << S(fill_n) << ") { at[0] = pv[u].x; at[1] = pv[u].y; at[2] = pv[u].z; at[3] = pv[u].w; }\n" << ind << "}\n";
        else
            k << ind << "    if (tid + u * 256 < " << S(fill_n) << ") at[0] = pv[u];\n" << ind << "}\n";
        k << "#pragma unroll\n" << ind << "for (int u = 0; u < " << S(NX) << "; ++u) {\n";
        k << ind << "    const int e = (tid + u * 256) * " << S(unit) << ";\n";
        k << ind << "    if (tid + u * 256 < " << S(xn) << ") *(" << vt << "*)(xt + " << buf << " + (e / " << S(C) << ") * " << S(CP) << " + e % " << S(C) << ") = xv[u];\n"
          << ind << "}\n";
    };
    if (!spec) k << "    __syncthreads();\n";
    // Barriers the lower waves pass inside one image's matrix phases: the loader waves pass as many.
    int phase_syncs = 0;
    auto sync = [&]() {
        k << "        __syncthreads();\n";
        ++phase_syncs;
    };
    const string loop_head = "    int bo = 0;\n    for (int img = chunk; img < " + S(IMG) + "; img += " + S(cv.chunks) + ", bo ^= " + S(BUFSZ) + ") {\n";
    if (spec) {
        // The two roles are two loops, so that neither carries the other's registers (the accumulators and fragment
        // addresses of the matrix phases, the addresses the fills keep): the loader waves then have room to request
        // all of an image's loads in one go.  Both pass the same barriers.
        k << "    if (!loader) {\n";
        if (mfma_dgrad) emit_b_fragments(true);
        k << "    __syncthreads();\n" << loop_head;
    } else {
        k << "    constexpr int bo = 0;\n";
        k << "    for (int img = chunk; img < " << S(IMG) << "; img += " << S(cv.chunks) << ") {\n";
        k << "        {\n            " << dvt << " pv[" << S(NC) << "];\n            " << vt << " xv[" << S(NX) << "];\n";
        if (pmask) k << "            uint pw[" << S(NC) << "];\n";
        emit_issue("img", "            ");
        emit_tile_stores("            ", "0");
        k << "        }\n";
        k << "        __syncthreads();\n";
    }
    // 2a. filter gradient: this wave's steps of four slots
    {
        // With loader waves two waves per SIMD run these products (the other two are loader waves), so a wave has to
        // keep the matrix pipe busy by itself: the fragments of two steps are requested before the first product is issued.
        // The fragment addresses are running registers: a step is an add per fragment (none for the second step of
        // a pair in the tiles whose rows are all real: its distance is a literal in the read), where a slot term
        // computed from the step number cost two to three vector instructions per read -- and vector instructions
        // do not hide behind the products of the other wave on the SIMD, they take turns with them.
        auto full_a = [&](int mt) { return (int64_t)(mt + 1) * 16 <= KD; };
        auto full_b = [&](int nt) { return (int64_t)(nt + 1) * 16 <= K; };
        k << "        const char* const sbytes = (const char*)smem;\n        int aw[" << MT << "], bw[" << NT << "];  // in bytes\n";
        k << "#pragma unroll\n        for (int mt = 0; mt < " << MT << "; ++mt) aw[mt] = 4 * (a_off[mt] + ((((4 * wave + lk) * " << S(CP) << ") + bo) & a_msk[mt]));\n";
        k << "#pragma unroll\n        for (int nt = 0; nt < " << NT << "; ++nt) bw[nt] = 4 * (b_off[nt] + bo + (((4 * wave + lk) * " << S(PITCH) << ") & b_msk[nt]));\n";
        auto emit_reads = [&](const string& ind, int halves) {
            for (int h = 0; h < halves; ++h) {
                for (int mt = 0; mt < MT; ++mt)
                    k << ind << "fa[" << h << "][" << mt << "] = *(const float*)(sbytes + aw[" << mt << "]" << (h ? (full_a(mt) ? " + " + S(64 * CP) : " + (" + S(64 * CP) + " & a_msk[" + to_string(mt) + "])") : string()) << ");\n";
                for (int nt = 0; nt < NT; ++nt)
                    k << ind << "fb[" << h << "][" << nt << "] = *(const float*)(sbytes + bw[" << nt << "]" << (h ? (full_b(nt) ? " + " + S(64 * PITCH) : " + (" + S(64 * PITCH) + " & b_msk[" + to_string(nt) + "])") : string()) << ");\n";
            }
        };
        k << "        int s = wave;\n";
        k << "#pragma unroll 1\n        for (; s + 4 < " << S(L.steps) << "; s += 8) {\n";
        k << "            float fa[2][" << MT << "], fb[2][" << NT << "];\n";
        emit_reads("            ", 2);
        k << "            __builtin_amdgcn_sched_barrier(0);\n";
        k << "#pragma unroll\n            for (int h = 0; h < 2; ++h)\n#pragma unroll\n                for (int mt = 0; mt < " << MT << "; ++mt)\n#pragma unroll\n                    for (int nt = 0; nt < " << NT << "; ++nt)\n";
        k << "                        wacc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[h][mt], fb[h][nt], wacc[mt][nt], 0, 0, 0);\n";
        k << "            __builtin_amdgcn_sched_barrier(0);\n";
        for (int mt = 0; mt < MT; ++mt)
            k << "            aw[" << mt << "] += " << (full_a(mt) ? S(128 * CP) : "(" + S(128 * CP) + " & a_msk[" + to_string(mt) + "])") << ";\n";
        for (int nt = 0; nt < NT; ++nt)
            k << "            bw[" << nt << "] += " << (full_b(nt) ? S(128 * PITCH) : "(" + S(128 * PITCH) + " & b_msk[" + to_string(nt) + "])") << ";\n";
        k << "        }\n";
        // the wave's odd step, where it has one
        k << "        if (s < " << S(L.steps) << ") {\n";
        k << "            float fa[1][" << MT << "], fb[1][" << NT << "];\n";
        emit_reads("            ", 1);
        k << "#pragma unroll\n            for (int mt = 0; mt < " << MT << "; ++mt)\n#pragma unroll\n                for (int nt = 0; nt < " << NT << "; ++nt)\n";
        k << "                    wacc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[0][mt], fb[0][nt], wacc[mt][nt], 0, 0, 0);\n";
        k << "        }\n";
    }
    const int64_t passes = (PH * PW + 255) / 256;
    if (wonly) {
        k << "        __syncthreads();\n";  // the next image's fills overwrite what the fragments read
    } else if (mfma_dgrad) {
        // 2b. data gradient: every wave takes every fourth tile of 16 pixel groups
        k << "        cb_float4 dacc[" << S(TPW) << "];\n";
        if (spec) {
            // the wave's tiles side by side: independent accumulators, one B fragment serves all of them, and the
            // fragments of a filter row are all requested before its first product
            const int64_t K4 = K / 4, NF = TQ * K4;
            k << "#pragma unroll\n        for (int t = 0; t < " << S(TPW) << "; ++t) dacc[t] = (cb_float4){0.f, 0.f, 0.f, 0.f};\n";
            k << "#pragma unroll 1\n        for (int ty = 0; ty < " << S(FH) << "; ++ty) {\n";
            k << "            const float* const gbp = smem + " << S(GB_AT) << " + ty * " << S(NF * 64) << " + lane;\n";
            k << "            float fa[" << S(TPW) << "][" << S(NF) << "], fb[" << S(NF) << "];\n";
            k << "#pragma unroll\n            for (int i = 0; i < " << S(NF) << "; ++i) fb[i] = gbp[i * 64];\n";
            // one address per tile and filter row: the row's first tap of this lane's group, or the zero row
            k << "#pragma unroll\n            for (int t = 0; t < " << S(TPW) << "; ++t) {\n";
            k << "                const int oy = dgy[t] - ty;\n";
            k << "                const int at = bo + ((unsigned)oy < " << S(OH) << "u ? dbase[t] - ty * " << S(PW * PITCH) << " : " << S(L.ZERO_AT) << " + lk);\n";
            k << "#pragma unroll\n                for (int tqi = 0; tqi < " << S(TQ) << "; ++tqi)\n";
            k << "#pragma unroll\n                    for (int o4 = 0; o4 < " << S(K4) << "; ++o4) fa[t][tqi * " << S(K4) << " + o4] = lds[at + (" << S(TQ - 1) << " - tqi) * " << S(PITCH) << " + 4 * o4];\n";
            k << "            }\n";
            k << "            __builtin_amdgcn_sched_barrier(0);\n";
            k << "#pragma unroll\n            for (int i = 0; i < " << S(NF) << "; ++i)\n#pragma unroll\n                for (int t = 0; t < " << S(TPW) << "; ++t)\n";
            k << "                    dacc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[t][i], fb[i], dacc[t], 0, 0, 0);\n";
            k << "            __builtin_amdgcn_sched_barrier(0);\n";
            k << "        }\n";
        }
        if (!spec) {
        k << "#pragma unroll\n        for (int t = 0; t < " << S(TPW) << "; ++t) {\n";
        k << "            const int grp = (t * 4 + wave) * 16 + li, gy = grp / " << S(GPR) << ", gx0 = (grp % " << S(GPR) << ") * " << S(P) << ";\n";
        k << "            cb_float4 d = (cb_float4){0.f, 0.f, 0.f, 0.f};\n";
        // (the filter rows stay a loop: unrolled whole, the scheduler hoists every LDS load of a tile and the kernel
        // loses a wave of occupancy to the registers that hold them)
        k << "#pragma unroll 1\n            for (int ty = 0; ty < " << S(FH) << "; ++ty) {\n";
        k << "                const int oy = gy - ty;\n                const float* const gbp = smem + " << S(GB_AT) << " + ty * " << S(TQ * (K / 4) * 64) << " + lane;\n";
        for (int64_t tqi = 0; tqi < TQ; ++tqi) {
            const int64_t tq = tqi - (P - 1);
            k << "                {\n                    const int ox = gx0 - " << S(tq) << ";\n";
            k << "                    const int at = bo + ((oy >= 0 && oy < " << S(OH) << " && ox >= 0 && ox < " << S(OW) << ") ? " << S(L.DC_AT) << " + (oy * " << S(PW) << " + ox) * " << S(PITCH) << " : "
              << S(L.ZERO_AT) << ");\n";
            for (int64_t o4 = 0; o4 < K / 4; ++o4)
                k << "                    d = __builtin_amdgcn_mfma_f32_16x16x4f32(lds[at + " << S(4 * o4) << " + lk], gbp[" << S((tqi * (K / 4) + o4) * 64) << "], d, 0, 0, 0);\n";
            k << "                }\n";
        }
        k << "            }\n";
        k << "            dacc[t] = d;\n        }\n";
        }
        // register r of lane l is D[group 4 * (l / 16) + r][(pixel of the group, channel) = l % 16]
        auto emit_dacc_stores = [&](const string& target_of_p) {
            k << "#pragma unroll\n        for (int t = 0; t < " << S(TPW) << "; ++t)\n#pragma unroll\n            for (int r = 0; r < 4; ++r) {\n";
            k << "                const int grp = (t * 4 + wave) * 16 + 4 * lk + r, gy = grp / " << S(GPR) << ", gx = (grp % " << S(GPR) << ") * " << S(P) << " + li / " << S(C)
              << ", gc = li % " << S(C) << ";\n";
            k << "                const int p = gy * " << S(PW) << " + gx;\n";
            k << "                if (grp < " << S(GROUPS) << " && gx < " << S(PW) << ") " << target_of_p << " = dacc[t][r];\n            }\n";
        };
        if (!unpad) {
            emit_dacc_stores(out_ptr + "[(img * " + S(PH * PW) + " + p) * " + S(GC) + " + cb * " + S(C) + " + gc]");
        } else if (reg_fold) {
            // Border folds in registers.  Register r of lane (li, lk) of tile T is padded pixel row 2 T + lk / 2, pixel
            // pair 4 (lk % 2) + r, pixel li / 8 of the pair, channel li % 8: the two padded columns that replicate an
            // image's edge column are the two pixels of the row's first / last pair (lanes 8 apart), the two padded rows
            // that replicate an edge row are the two rows of the first / last tile (lanes 32 apart).  Sums in the order
            // of the Unpads; the lane whose padded pixel is the image's own stores.
            const string yfold = "                if (T == 0 || T == " + S(L.TILES - 1) + ") {\n#pragma unroll\n                    for (int r = 0; r < 4; ++r) v[r] += __shfl_xor(v[r], 32, 64);\n                }\n";
            const string xfold = "                {\n                    const float f0 = v[0] + dsc_lane_xor8(v[0]), f3 = v[3] + dsc_lane_xor8(v[3]);\n"
                                 "                    v[0] = (lk & 1) ? v[0] : f0;\n                    v[3] = (lk & 1) ? f3 : v[3];\n                }\n";
            k << "        {\n            const int par = li >> 3, gc = li & 7;\n";
            k << "#pragma unroll\n            for (int t = 0; t < " << S(TPW) << "; ++t) {\n";
            k << "                const int T = t * 4 + wave;\n                float v[4] = {dacc[t][0], dacc[t][1], dacc[t][2], dacc[t][3]};\n";
            k << (cv.rows_first ? yfold + xfold : xfold + yfold);
            k << "                const int gy = 2 * T + (lk >> 1);\n";
            k << "#pragma unroll\n                for (int r = 0; r < 4; ++r) {\n";
            k << "                    const int gx = 2 * (4 * (lk & 1) + r) + par;\n";
            k << "                    if (T < " << S(L.TILES) << " && gy >= 1 && gy <= " << S(PH - 2) << " && gx >= 1 && gx <= " << S(PW - 2) << ") " << out_ptr << "[((img * " << S(H)
              << " + gy - 1) * " << S(W) << " + gx - 1) * " << S(GC) << " + cb * " << S(C) << " + gc] = v[r];\n                }\n            }\n        }\n";
        } else {
            sync();
            emit_dacc_stores("xt[bo + p * " + S(C) + " + gc]");
            sync();
        }
    } else {
    // 2b. data gradient: one padded-image pixel per thread and pass, taps x output channels, the filter element
    // through the scalar unit (as the data-gradient kernel)
    const int64_t OCB = K % 8 == 0 ? 8 : 4;
    k << "        float acc[" << passes << "][" << S(C) << "];\n";
    k << "#pragma unroll\n        for (int ps = 0; ps < " << passes << "; ++ps) {\n";
    k << "            const int p = min(ps * 256 + tid, " << S(PH * PW - 1) << ");\n";
    k << "            const int py = p / " << S(PW) << ", px = p % " << S(PW) << ";\n";
    k << "#pragma unroll\n            for (int c = 0; c < " << S(C) << "; ++c) acc[ps][c] = 0.f;\n";
    k << "#pragma unroll 1\n            for (int tap = 0; tap < " << S(FH * FW) << "; ++tap) {\n";
    k << "                const int fy = tap / " << S(FW) << ", fx = tap % " << S(FW) << ";\n";
    k << "                const int oy = py - fy, ox = px - fx;\n";
    k << "                const bool inside = oy >= 0 && oy < " << S(OH) << " && ox >= 0 && ox < " << S(OW) << ";\n";
    k << "                const float* src = &lds[bo + (inside ? " << S(L.DC_AT) << " + (oy * " << S(PW) << " + ox) * " << S(PITCH) << " : " << S(L.ZERO_AT) << ")];\n";
    k << "#pragma unroll\n                for (int oc = 0; oc < " << S(K) << "; oc += " << OCB << ") {\n";
    k << "                    float a[" << OCB << "];\n";
    k << "#pragma unroll\n                    for (int q = 0; q < " << OCB << "; q += 4) {\n";
    k << "                        const float4 a4 = *(const float4*)(src + oc + q);\n";
    k << "                        a[q] = a4.x; a[q + 1] = a4.y; a[q + 2] = a4.z; a[q + 3] = a4.w;\n                    }\n";
    k << "#pragma unroll\n                    for (int j = 0; j < " << OCB << "; ++j)\n";
    k << "#pragma unroll\n                        for (int c = 0; c < " << S(C) << "; ++c)\n";
    k << "                            acc[ps][c] = fmaf(a[j], load_b(cb, oc + j, tap * " << S(C) << " + c, " << em.params_pass() << "), acc[ps][c]);\n";
    k << "                    __builtin_amdgcn_sched_barrier(0);\n";
    k << "                }\n            }\n        }\n";
    if (!unpad) {
        k << "#pragma unroll\n        for (int ps = 0; ps < " << passes << "; ++ps) {\n";
        k << "            const int p = ps * 256 + tid;\n            if (p < " << S(PH * PW) << ") {\n";
        k << "#pragma unroll\n                for (int c = 0; c < " << S(C) << "; ++c) " << out_ptr << "[(img * " << S(PH * PW) << " + p) * " << S(GC)
          << " + cb * " << S(C) << " + c] = acc[ps][c];\n            }\n        }\n";
    } else {
        // 3. the padded-image gradient goes through the input tile's memory (dead by now); each pixel of the image sums
        // the padded pixels that replicate it
        sync();
        k << "#pragma unroll\n        for (int ps = 0; ps < " << passes << "; ++ps) {\n";
        k << "            const int p = ps * 256 + tid;\n            if (p < " << S(PH * PW) << ") {\n";
        k << "#pragma unroll\n                for (int c = 0; c < " << S(C) << "; ++c) xt[bo + p * " << S(C) << " + c] = acc[ps][c];\n            }\n        }\n";
        sync();
    }
    }
    // (four channels of a pixel per evaluation where the layouts allow 16-byte pieces; the sums keep their order)
    const bool fold4 = unpad && !wonly && H > 1 && W > 1 && C % 4 == 0 && GC % 4 == 0 && L.XT_AT % 4 == 0 && BUFSZ % 4 == 0;
    if (reg_fold) {
        // (folded in registers above)
    } else if (fold4) {
        const int64_t CQ = C / 4;
        k << "        for (int i = tid; i < " << S(H * W * CQ) << "; i += 256) {\n";
        k << "            const int c = (i % " << S(CQ) << ") * 4, x = (i / " << S(CQ) << ") % " << S(W) << ", y = i / " << S(CQ * W) << ";\n";
        k << "            float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);\n";
        auto slots = [&](const string& q, bool is_y) {
            return "for (int " + q + " = 0; " + q + " <= " + S(is_y ? cv.pad_h : cv.pad_w) + "; ++" + q + ")";
        };
        const string qo = cv.rows_first ? "qx" : "qy", qi = cv.rows_first ? "qy" : "qx";
        k << "            const bool edge_y = y == 0 || y == " << S(H - 1) << ", edge_x = x == 0 || x == " << S(W - 1) << ";\n";
        k << "            const int base_y = y == 0 ? 0 : y + " << S(cv.pad_h) << ", base_x = x == 0 ? 0 : x + " << S(cv.pad_w) << ";\n";
        k << "#pragma unroll\n            " << slots(qo, !cv.rows_first) << " {\n                float4 part = make_float4(0.f, 0.f, 0.f, 0.f);\n";
        k << "#pragma unroll\n                " << slots(qi, cv.rows_first) << " {\n";
        k << "                    const bool ok = (edge_y || qy == 0) && (edge_x || qx == 0);\n";
        k << "                    const int ky = base_y + (edge_y ? qy : 0), kx = base_x + (edge_x ? qx : 0);\n";
        k << "                    const float4 w = *(const float4*)(xt + bo + (ky * " << S(PW) << " + kx) * " << S(C) << " + c);\n";
        k << "                    part.x += ok ? w.x : 0.f; part.y += ok ? w.y : 0.f; part.z += ok ? w.z : 0.f; part.w += ok ? w.w : 0.f;\n                }\n";
        k << "                sum.x += part.x; sum.y += part.y; sum.z += part.z; sum.w += part.w;\n            }\n";
        k << "            *(float4*)(" << out_ptr << " + ((img * " << S(H) << " + y) * " << S(W) << " + x) * " << S(GC) << " + cb * " << S(C) << " + c) = sum;\n        }\n";
    } else if (unpad && !wonly) {
        k << "        for (int i = tid; i < " << S(H * W * C) << "; i += 256) {\n";
        k << "            const int c = i % " << S(C) << ", x = (i / " << S(C) << ") % " << S(W) << ", y = i / " << S(C * W) << ";\n";
        k << "            float sum = 0.f;\n";
        const string outer = cv.rows_first ? "jx" : "jy", inner = cv.rows_first ? "jy" : "jx";
        auto range = [&](const string& j) {
            const bool is_y = j == "jy";
            return "for (int " + j + " = " + S(-(is_y ? cv.pad_h : cv.pad_w)) + "; " + j + " <= " + S(is_y ? cv.pad_h : cv.pad_w) + "; ++" + j + ")";
        };
        if (H > 1 && W > 1) {
            auto slots = [&](const string& q, bool is_y) {
                return "for (int " + q + " = 0; " + q + " <= " + S(is_y ? cv.pad_h : cv.pad_w) + "; ++" + q + ")";
            };
            const string qo = cv.rows_first ? "qx" : "qy", qi = cv.rows_first ? "qy" : "qx";
            k << "            const bool edge_y = y == 0 || y == " << S(H - 1) << ", edge_x = x == 0 || x == " << S(W - 1) << ";\n";
            k << "            const int base_y = y == 0 ? 0 : y + " << S(cv.pad_h) << ", base_x = x == 0 ? 0 : x + " << S(cv.pad_w) << ";\n";
            k << "#pragma unroll\n            " << slots(qo, !cv.rows_first) << " {\n                float part = 0.f;\n";
            k << "#pragma unroll\n                " << slots(qi, cv.rows_first) << " {\n";
            k << "                    const bool ok = (edge_y || qy == 0) && (edge_x || qx == 0);\n";
            k << "                    const int ky = base_y + (edge_y ? qy : 0), kx = base_x + (edge_x ? qx : 0);\n";
            k << "                    const float w = xt[bo + (ky * " << S(PW) << " + kx) * " << S(C) << " + c];\n";
            k << "                    part += ok ? w : 0.f;\n                }\n                sum += part;\n            }\n";
        } else {
            k << "#pragma unroll\n            " << range(outer) << " {\n                float part = 0.f;\n";
            k << "#pragma unroll\n                " << range(inner) << " {\n";
            k << "                    const bool ok_y = jy == 0 || (jy < 0 && y == 0) || (jy > 0 && y == " << S(H - 1) << ");\n";
            k << "                    const bool ok_x = jx == 0 || (jx < 0 && x == 0) || (jx > 0 && x == " << S(W - 1) << ");\n";
            k << "                    const int ky = clampi(y + " << S(cv.pad_h) << " + jy, 0, " << S(PH - 1) << "), kx = clampi(x + " << S(cv.pad_w)
              << " + jx, 0, " << S(PW - 1) << ");\n";
            k << "                    const float w = xt[bo + (ky * " << S(PW) << " + kx) * " << S(C) << " + c];\n";
            k << "                    part += (ok_y && ok_x) ? w : 0.f;\n                }\n                sum += part;\n            }\n";
        }
        k << "            " << out_ptr << "[((img * " << S(H) << " + y) * " << S(W) << " + x) * " << S(GC) << " + cb * " << S(C) << " + c] = sum;\n        }\n";
    }
    // the next image's fills overwrite what the matrix phases and the folds read (with loader waves: the buffer the
    // lower waves turn to next has been filled)
    if (!wonly) k << "        __syncthreads();\n";
    k << "    }\n";
    if (spec) {
        // the loader waves: the set's first image, then per image the next one into the other buffer and the
        // barriers of the matrix phases
        k << "    } else {\n";
        k << "    if (chunk < " << S(IMG) << ") {\n        " << dvt << " pv[" << S(NC) << "];\n        " << vt << " xv[" << S(NX) << "];\n";
        if (pmask) k << "        uint pw[" << S(NC) << "];\n";
        emit_issue("chunk", "        ");
        emit_tile_stores("        ", "0");
        k << "    }\n    __syncthreads();\n" << loop_head;
        k << "        const int nimg = img + " << S(cv.chunks) << ";\n";
        k << "        if (nimg < " << S(IMG) << ") {\n            " << dvt << " pv[" << S(NC) << "];\n            " << vt << " xv[" << S(NX) << "];\n";
        if (pmask) k << "            uint pw[" << S(NC) << "];\n";
        emit_issue("nimg", "            ");
        emit_tile_stores("            ", "(bo ^ " + S(BUFSZ) + ")");
        k << "        }\n";
        for (int i = 0; i < phase_syncs + 1; ++i) k << "        __syncthreads();\n";
        k << "    }\n    }\n";
    }
    // 4. the four waves' accumulators are summed through LDS; register r of lane l is D[4 * (l / 16) + r][l % 16]
    const int64_t R = (int64_t)MT * NT * 256;
    k << "#pragma unroll\n    for (int mt = 0; mt < " << MT << "; ++mt)\n#pragma unroll\n        for (int nt = 0; nt < " << NT
      << "; ++nt)\n#pragma unroll\n            for (int r = 0; r < 4; ++r) " << (spec ? "if (!loader) " : "") << "smem[wave * " << S(R) << " + (mt * " << NT << " + nt) * 256 + r * 64 + lane] = wacc[mt][nt][r];\n";
    k << "    __syncthreads();\n";
    k << "    for (int i = threadIdx.x; i < " << S(R) << "; i += " << S(BLOCK) << ") {\n";
    k << "        const float sum = (smem[i] + smem[" << S(R) << " + i]) + (smem[" << S(2 * R) << " + i] + smem[" << S(3 * R) << " + i]);\n";
    k << "        const int tile = i >> 8, r = (i >> 6) & 3, l = i & 63;\n";
    k << "        const int cm = (tile / " << NT << ") * 16 + 4 * (l >> 4) + r, cn = (tile % " << NT << ") * 16 + (l & 15);\n";
    k << "        if (cm < " << S(KD) << " && cn < " << S(K) << ") " << part_ptr << "[((band * " << S(cv.chunks) << " + chunk) * " << S(G) << " + cb) * " << S(KD * K) << " + cm * " << S(K) << " + cn] = sum;\n";
    if (cv.bias)
        k << "        if (cm == " << S(KD) << " && cn < " << S(K) << ") b" << fk.outputs[wonly ? 1 : 2] << "[((band * " << S(cv.chunks) << " + chunk) * " << S(G) << " + cb) * " << S(K) << " + cn] = sum;\n";
    k << "    }\n}\n";
    if (cv.chunks * G * BANDS >= kMaxIndex) return "conv backward: grid too large";
    out->grid = (unsigned)(cv.chunks * G * BANDS);
    out->block = (unsigned)BLOCK;
    out->source = k.str();
    out->note = "conv backward: workgroup per group and image set (" + S(cv.chunks) + " sets), dC and input tile in LDS, " + (pmask ? "dC read off the pooling windows' words, " : "") +
                (spec ? "loader waves fill the next image's tiles, " : "") +
                (wonly ? "no data gradient, " + S(BANDS) + " bands of " + S(OH) + " output rows" : "data gradient " + S(FH) + "x" + S(FW) + " taps x " + S(K) + " channels" + (unpad ? " with border folds" : "")) +
                ", filter gradient mfma 16x16x4 " + to_string(MT) + "x" + to_string(NT) + " tiles" + (cv.bias ? " +column sums of dC" : "");
    return "";
}

// ---- convolution forward ---------------------------------------------------------------------------------


// One workgroup per (image, group).  The group's channels of the image go to LDS once with replicate padding applied
// (a tile of (oh + fh - 1) x (ow + fw - 1) pixels), so that an im2col element is one LDS word at
// window origin + tap offset with no clamping left in the inner loop: an im2col row read from memory is fh*fw
// separate pieces, and a load instruction over 64 rows touches 64 cache lines.  Products run on
// v_mfma_f32_16x16x4f32 with the operands swapped (D^T = B^T A^T): a wave takes 16 output pixels at a time, lane l
// feeds the im2col value of pixel l % 16 at k = 4 s + l / 16 from LDS, holds B's K/4 fragments in registers for the
// whole kernel, and ends up with four consecutive output channels of its pixel: one 16-byte store per output.
// The kernel is bound by instruction issue, not by MFMA or memory, so everything per element is kept off the VALU:
// tap offsets are literals when the channel count is a multiple of four, and the fused consumer gets its
// coordinates instead of dividing an index.
string gen_conv_fwd(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const FusedKernel::ConvFwd& cv = fk.cfwd;
    const MatMulDims g = matmul_dims(d);
    const bool rows = d.output_mode == DSC_MATMUL_ROWS;
    const int64_t batch_stride = rows ? g.n : g.m * g.n, row_stride = rows ? g.batch * g.n : g.n;
    const int64_t K = g.k, C = cv.c, GC = cv.g * cv.c, PIX = cv.oh * cv.ow;
    if (g.batch != cv.g || g.m != cv.img * PIX || K != cv.fh * cv.fw * C || g.chunks != 1 || fk.inputs[0].buffer < 0 ||
        !conv_fwd_fits(cv, g.n))
        return "conv forward: geometry mismatch";
    const int64_t PH = cv.oh + cv.fh - 1, PW = cv.ow + cv.fw - 1;
    const int64_t CP = conv_fwd_pitch(C);  // words per pixel in LDS
    // with pooling a tile of 16 pixels is two image rows by eight columns, so that a pooling window's four pixels sit in
    // lanes l, l ^ 1, l ^ 8, l ^ 9 of one tile
    const bool pooled = fk.pool.on;
    const int64_t TPR = (cv.ow + 7) / 8, OH2 = cv.oh / 2, OW2 = cv.ow / 2;
    const int64_t steps = (K + 3) / 4, tiles = pooled ? OH2 * TPR : (PIX + 15) / 16;
    const int n_out = fk.has_epilogue ? fk.epilogue.raw().n_outputs : 1;
    const int n_pool_out = pooled && fk.pool.has_epilogue ? fk.pool.epilogue.raw().n_outputs : 0;
    if (pooled) {
        if (cv.oh % 2 || cv.ow % 2 || g.n % 4 || fk.pool.source < 0 || fk.pool.source >= n_out) return "conv forward: pooling needs even extents and whole 16-byte channel pieces";
        if ((int)fk.outputs.size() != n_out + n_pool_out + (fk.pool.store_pooled ? 1 : 0)) return "conv forward: pooled output count";
        if (fk.pool.has_epilogue) {
            const dsc_kernel_desc& pe = fk.pool.epilogue.raw();
            std::ostringstream body;
            std::map<int, string> ov;
            ov[fk.pool.epilogue_product_input] = "product";
            em.emit_pe(body, pe, fk.pool.epilogue_inputs, "gid", "q", ov);
            for (int o = 0; o < pe.n_outputs; ++o) body << "    result[" << o << "] = qt" << pe.outputs[o] << ";\n";
            em.funcs << "DSC_INLINE void pool_epilogue(float product, int gid, float* result, " << em.params_decl() << ") {\n" << body.str() << "}\n";
        }
    }
    const string lb = em.load_view(fk.inputs[1], d.inputs[1], {"cb", "ck", "cn"});
    em.funcs << "DSC_INLINE float load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";
    if (fk.has_epilogue) {
        const dsc_kernel_desc& pe = fk.epilogue.raw();
        std::ostringstream body;
        std::map<int, string> ov;
        ov[fk.epilogue_product_input] = "product";
        IndexForm form;
        form.valid = true;
        form.names = {"cb", "cm", "cn"};
        form.coefs = {batch_stride, row_stride, 1};
        form.extents = {g.batch, g.m, g.n};
        em.emit_pe(body, pe, fk.epilogue_inputs, "gid", "e", ov, &form);
        for (int o = 0; o < pe.n_outputs; ++o) body << "    result[" << o << "] = et" << pe.outputs[o] << ";\n";
        em.funcs << "DSC_INLINE void mm_epilogue(float product, int gid, int cb, int cm, int cn, float* result, " << em.params_decl() << ") {\n"
                 << body.str() << "}\n";
    }
    const string img_ptr = "b" + to_string(fk.inputs[0].buffer);
    const bool vec_fill = C % 4 == 0;                         // 16-byte pieces of a pixel's channels
    const bool literal_taps = C % 4 == 0;                     // then a k step's four values share one tap
    const bool vec_store = g.n % 4 == 0 && batch_stride % 4 == 0 && row_stride % 4 == 0;
    if (pooled && !vec_store) return "conv forward: pooling needs 16-byte stores";
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(fk) << "(" << em.kernel_params_decl() << ") {\n";
    k << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    k << "    typedef float cf_float4 __attribute__((ext_vector_type(4)));\n";
    const int64_t unit = vec_fill ? 4 : 1, fill_n = PH * PW * C / unit, per_thread = (fill_n + 255) / 256;
    const int64_t FU = std::min<int64_t>(per_thread, 8);
    k << "    __shared__ __attribute__((aligned(16))) float tile[" << S(PH * PW * CP) << "];\n";
    k << "    __shared__ float sB[" << S(steps * 64) << "];\n";
    // (placing the groups of an image on one XCD, as the data-gradient kernel does, measured slower here: 20.5 us
    // against 18.4 -- this kernel is bound by its stores, and neighbouring workgroups writing the two halves of a
    // line from two L2s spread that load)
    k << "    const int cb = blockIdx.x % " << S(cv.g) << ", img = blockIdx.x / " << S(cv.g) << ";\n";
    k << "    const int lane = threadIdx.x & 63, li = lane & 15, lk = lane >> 4;\n";
    // the 16-pixel tiles are dealt to the four waves in turn; which wave takes the odd ones out rotates with the
    // workgroup, so that no SIMD of a CU collects all of them
    // (through readfirstlane: the tile numbers and what the addresses take from them are then scalar arithmetic)
    k << "    const int wv = __builtin_amdgcn_readfirstlane((int)(((threadIdx.x >> 6) + blockIdx.x) & 3));\n";
    // 1. B goes through LDS: every wave needs all of it in MFMA fragment order, and when each wave of every
    // workgroup fetched its fragments itself (K/4 loads per lane, the same few cache lines for the whole grid) those
    // loads alone cost a third of the kernel.  Zero beyond k and n.
    const int64_t BU = (steps * 64 + 255) / 256;
    k << "    float bv[" << S(BU) << "];\n";
    k << "#pragma unroll\n    for (int u = 0; u < " << S(BU) << "; ++u) {\n";
    k << "        const int e = threadIdx.x + u * 256, kk = e >> 4, nn = e & 15;\n";
    k << "        const float v = load_b(cb, min(kk, " << S(K - 1) << "), min(nn, " << S(g.n - 1) << "), " << em.params_pass() << ");\n";
    k << "        bv[u] = (kk < " << S(K) << " && nn < " << S(g.n) << ") ? v : 0.f;\n    }\n";
    // 2. the padded tile: tile[py][px][c] = image[clamp(py - pad_h)][clamp(px - pad_w)][c]
    const string vt = vec_fill ? "float4" : "float";
    auto emit_fill_loads = [&](const string& ind) {
        k << "#pragma unroll\n" << ind << "for (int u = 0; u < " << S(FU) << "; ++u) {\n";
        k << ind << "    const int e = min(i0 + u * 256, " << S(fill_n - 1) << ") * " << S(unit) << ";\n";
        k << ind << "    const int ch = e % " << S(C) << ", px = (e / " << S(C) << ") % " << S(PW) << ", py = e / " << S(C * PW) << ";\n";
        k << ind << "    const int sy = clampi(py - " << S(cv.pad_h) << ", 0, " << S(cv.h - 1) << "), sx = clampi(px - " << S(cv.pad_w) << ", 0, " << S(cv.w - 1) << ");\n";
        k << ind << "    v[u] = *(const " << vt << "*)(" << img_ptr << " + ((img * " << S(cv.h) << " + sy) * " << S(cv.w) << " + sx) * " << S(GC) << " + cb * " << S(C)
          << " + ch);\n" << ind << "}\n";
    };
    auto emit_fill_stores = [&](const string& ind) {
        k << "#pragma unroll\n" << ind << "for (int u = 0; u < " << S(FU) << "; ++u)\n" << ind << "    if (i0 + u * 256 < " << S(fill_n) << ") *(" << vt << "*)(tile + "
          << (CP == C ? "(i0 + u * 256) * " + S(unit) : "((i0 + u * 256) * " + S(unit) + " / " + S(C) + ") * " + S(CP) + " + (i0 + u * 256) * " + S(unit) + " % " + S(C))
          << ") = v[u];\n";
    };
    k << "    " << vt << " v[" << S(FU) << "];\n";
    if (per_thread <= 8) {
        k << "    const int i0 = threadIdx.x;\n";
        emit_fill_loads("    ");
        emit_fill_stores("    ");
    } else {
        k << "    for (int i0 = threadIdx.x; i0 < " << S(fill_n) << "; i0 += " << S(256 * FU) << ") {\n";
        emit_fill_loads("        ");
        emit_fill_stores("        ");
        k << "    }\n";
    }
    k << "#pragma unroll\n    for (int u = 0; u < " << S(BU) << "; ++u)\n        if (threadIdx.x + u * 256 < " << S(steps * 64) << ") sB[threadIdx.x + u * 256] = bv[u];\n";
    k << "    __syncthreads();\n";
    // lane l holds B[k = 4 s + l / 16][n = l % 16]
    k << "    float fb[" << S(steps) << "];\n";
    k << "#pragma unroll\n    for (int s = 0; s < " << S(steps) << "; ++s) fb[s] = sB[s * 64 + lane];\n";
    // 3. offsets of the k steps inside a pixel's window
    if (literal_taps) {
        k << "    constexpr int KO[" << S(steps) << "] = {";
        for (int64_t s = 0; s < steps; ++s) {
            const int64_t tap = 4 * s / C, ch = 4 * s % C;
            k << (s ? ", " : "") << S(((tap / cv.fw) * PW + tap % cv.fw) * CP + ch);
        }
        k << "};\n";
    }
    auto emit_group = [&](int64_t TG, const string& q0, const string& ind) {
        k << ind << "int pb[" << S(TG) << "];\n" << ind << "cf_float4 acc[" << S(TG) << "];\n";
        k << "#pragma unroll\n" << ind << "for (int j = 0; j < " << S(TG) << "; ++j) {\n";
        if (pooled) {
            k << ind << "    const int t = (" << q0 << " + j) * 4 + wv;\n";
            k << ind << "    pb[j] = ((2 * (t / " << S(TPR) << ") + (li >> 3)) * " << S(PW) << " + min(8 * (t % " << S(TPR) << ") + (li & 7), " << S(cv.ow - 1) << ")) * " << S(CP)
              << (literal_taps ? " + lk" : "") << ";\n";
        } else {
            k << ind << "    const int p = min(((" << q0 << " + j) * 4 + wv) * 16 + li, " << S(PIX - 1) << ");\n";
            k << ind << "    pb[j] = ((p / " << S(cv.ow) << ") * " << S(PW) << " + p % " << S(cv.ow) << ") * " << S(CP) << (literal_taps ? " + lk" : "") << ";\n";
        }
        k << ind << "    acc[j] = (cf_float4){0.f, 0.f, 0.f, 0.f};\n" << ind << "}\n";
        k << "#pragma unroll\n" << ind << "for (int s = 0; s < " << S(steps) << "; ++s) {\n";
        if (literal_taps) {
            k << ind << "    const int ko = KO[s];\n";
        } else {
            // past the end of k the B fragment is zero, so the repeated value adds nothing
            k << ind << "    const int kk = min(4 * s + lk, " << S(K - 1) << "), tap = kk / " << S(C) << ";\n";
            k << ind << "    const int ko = ((tap / " << S(cv.fw) << ") * " << S(PW) << " + tap % " << S(cv.fw) << ") * " << S(C) << " + kk % " << S(C) << ";\n";
        }
        k << "#pragma unroll\n" << ind << "    for (int j = 0; j < " << S(TG) << "; ++j)\n";
        k << ind << "        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fb[s], tile[pb[j] + ko], acc[j], 0, 0, 0);\n" << ind << "}\n";
        // accumulator register i of lane l is D^T[column 4 * (l / 16) + i][pixel l % 16]
        k << "#pragma unroll\n" << ind << "for (int j = 0; j < " << S(TG) << "; ++j) {\n";
        if (pooled) {
            // every lane runs the consumer on a pixel that exists (the shuffles below need all lanes); only the lanes
            // whose own pixel and channels exist store
            k << ind << "    const int t = (" << q0 << " + j) * 4 + wv, yy = 2 * (t / " << S(TPR) << ") + (li >> 3), xr = 8 * (t % " << S(TPR) << ") + (li & 7);\n";
            k << ind << "    const bool valid = xr < " << S(cv.ow) << " && 4 * lk < " << S(g.n) << ";\n";
            k << ind << "    const int cm = img * " << S(PIX) << " + yy * " << S(cv.ow) << " + min(xr, " << S(cv.ow - 1) << "), cn = min(4 * lk, " << S(g.n - 4) << ");\n";
            k << ind << "    const int c_at = cb * " << S(batch_stride) << " + cm * " << S(row_stride) << " + cn;\n";
            k << ind << "    {\n";
        } else {
            k << ind << "    const int pp = ((" << q0 << " + j) * 4 + wv) * 16 + li, cm = img * " << S(PIX) << " + pp, cn = 4 * lk;\n";
            k << ind << "    const int c_at = cb * " << S(batch_stride) << " + cm * " << S(row_stride) << " + cn;\n";
            k << ind << "    if (pp < " << S(PIX) << " && cn < " << S(g.n) << ") {\n";
        }
        if (fk.has_epilogue) {
            k << ind << "        float res[4][" << n_out << "];\n";
            k << "#pragma unroll\n" << ind << "        for (int i = 0; i < 4; ++i) mm_epilogue(acc[j][i], c_at + i, cb, cm, min(cn + i, " << S(g.n - 1) << "), res[i], "
              << em.params_pass() << ");\n";
        }
        auto val = [&](int i, int o) { return fk.has_epilogue ? "res[" + to_string(i) + "][" + to_string(o) + "]" : "acc[j][" + to_string(i) + "]"; };
        for (int o = 0; o < n_out; ++o) {
            if (pooled && fk.pool.masks && o == fk.pool.source) continue;  // its readers take the window words below
            const string ptr = "b" + to_string(fk.outputs[o]);
            if (vec_store) {
                k << ind << "        " << (pooled ? "if (valid) " : "") << "*(float4*)(" << ptr << " + c_at) = make_float4(" << val(0, o) << ", " << val(1, o) << ", " << val(2, o) << ", "
                  << val(3, o) << ");\n";
            } else {
                for (int i = 0; i < 4; ++i)
                    k << ind << "        if (cn + " << i << " < " << S(g.n) << ") " << ptr << "[c_at + " << i << "] = " << val(i, o) << ";\n";
            }
        }
        if (pooled) {
            // the window's maximum: across the column pair, then across the row pair
            // (the four channels side by side, step by step: a lane exchange may not follow the instruction that wrote
            // its operand, and written channel by channel every exchange waited out that distance)
            k << ind << "        float pm[4];\n";
            k << ind << "        dsc_window_max4(" << val(0, fk.pool.source) << ", " << val(1, fk.pool.source) << ", " << val(2, fk.pool.source) << ", " << val(3, fk.pool.source) << ", pm);\n";
            const int64_t pbs = rows ? g.n : (int64_t)cv.img * OH2 * OW2 * g.n, prs = rows ? g.batch * g.n : g.n;
            if (fk.pool.masks) {
                // two bits per element: equals its window's maximum, is positive; the four pixels of a window meet in
                // one word per four channels (lanes l, l ^ 1, l ^ 8, l ^ 9)
                k << ind << "        uint mw = dsc_window_bits4(" << val(0, fk.pool.source) << ", " << val(1, fk.pool.source) << ", " << val(2, fk.pool.source) << ", " << val(3, fk.pool.source)
                  << ", pm[0], pm[1], pm[2], pm[3]);\n";
                k << ind << "        mw <<= 8 * ((li & 1) | ((li >> 3) << 1));\n";
                k << ind << "        mw |= (uint)dsc_lane_xor1((int)mw);\n" << ind << "        mw |= (uint)dsc_lane_xor8((int)mw);\n";
            }
            k << ind << "        const int p_at = cb * " << S(pbs) << " + (img * " << S(OH2 * OW2) << " + (t / " << S(TPR) << ") * " << S(OW2) << " + (xr >> 1)) * " << S(prs) << " + cn;\n";
            if (fk.pool.has_epilogue) {
                // the window's four lanes all hold its four maxima: each runs the consumer for one of the four channels
                // (all four in one lane, the other three idle, cost this issue-bound kernel four times the instructions)
                k << ind << "        const int wq = (li & 1) | ((li >> 3) << 1);\n";
                k << ind << "        float pmq = pm[0];\n";
                k << ind << "        pmq = wq == 1 ? pm[1] : pmq;\n" << ind << "        pmq = wq == 2 ? pm[2] : pmq;\n" << ind << "        pmq = wq == 3 ? pm[3] : pmq;\n";
                k << ind << "        if (valid) {\n";
                k << ind << "            float pres[" << n_pool_out << "];\n";
                k << ind << "            pool_epilogue(pmq, p_at + wq, pres, " << em.params_pass() << ");\n";
                for (int o = 0; o < n_pool_out; ++o) k << ind << "            b" << fk.outputs[n_out + o] << "[p_at + wq] = pres[" << o << "];\n";
                k << ind << "        }\n";
            }
            k << ind << "        if (valid && (li & 9) == 0) {\n";
            if (fk.pool.masks)
                k << ind << "            ((uint*)b" << fk.outputs[fk.pool.source] << ")[((cb * " << S(cv.img) << " + img) * " << S(OH2 * OW2) << " + (t / " << S(TPR) << ") * " << S(OW2)
                  << " + (xr >> 1)) * " << S(g.n / 4) << " + lk] = mw;\n";
            if (fk.pool.store_pooled)
                k << ind << "            *(float4*)(b" << fk.outputs[n_out + n_pool_out] << " + p_at) = make_float4(pm[0], pm[1], pm[2], pm[3]);\n";
            k << ind << "        }\n";
        }
        k << ind << "    }\n" << ind << "}\n";
    };
    // 4. every wave has `full` whole turns, taken TGMAX tiles at a time so that their MFMA chains interleave; the
    // waves with wv < rem have one more
    const int64_t full = tiles / 4, rem = tiles % 4, TGMAX = 8;
    const int64_t whole_groups = full / TGMAX, tail = full % TGMAX;
    if (whole_groups == 1) {
        k << "    {\n";
        emit_group(TGMAX, "0", "        ");
        k << "    }\n";
    } else if (whole_groups > 1) {
        k << "    for (int q0 = 0; q0 < " << S(whole_groups * TGMAX) << "; q0 += " << S(TGMAX) << ") {\n";
        emit_group(TGMAX, "q0", "        ");
        k << "    }\n";
    }
    if (tail) {
        k << "    {\n";
        emit_group(tail, S(whole_groups * TGMAX), "        ");
        k << "    }\n";
    }
    if (rem) {
        k << "    if (wv < " << S(rem) << ") {\n";
        emit_group(1, S(full), "        ");
        k << "    }\n";
    }
    k << "}\n";
    if (cv.img * cv.g >= kMaxIndex) return "conv forward: grid too large";
    out->grid = (unsigned)(cv.img * cv.g);
    out->block = 256;
    out->source = k.str();
    out->note = "conv forward: workgroup per image and group, padded image tile in LDS, mfma 16x16x4, " + S(cv.fh) + "x" + S(cv.fw) + " taps x " + S(C) +
                " channels" + (fk.has_epilogue ? " +epilogue" : "") +
                (pooled ? string(" +2x2 max-pool") + (fk.pool.has_epilogue ? " with its consumer" : "") + (fk.pool.masks ? ", window words in place of its source" : "") : string());
    return "";
}

// ---- matmul -------------------------------------------------------------------------------------------

struct MmConfig {
    int bm, bn, bk, wm, wn, group_m;
};

bool config_ok(const MmConfig& c) {
    if (c.bm <= 0 || c.bn <= 0 || c.bk <= 0 || c.wm <= 0 || c.wn <= 0 || c.group_m <= 0) return false;
    if (c.bk % 8) return false;
    if (c.bm % (32 * c.wm) || c.bn % (32 * c.wn)) return false;
    const int nt = 64 * c.wm * c.wn;
    if (nt > 1024) return false;
    if ((c.bm * c.bk) % 4 || (c.bn * c.bk) % 4) return false;
    const int lds = 2 * 4 * (std::max(c.bm * (c.bk + 4), c.bk * (c.bm + 8)) + std::max(c.bn * (c.bk + 4), c.bk * (c.bn + 8)));
    if (lds > 160 * 1024) return false;  // gfx950 LDS per workgroup
    const int acc = (c.bm / c.wm / 32) * (c.bn / c.wn / 32) * 16;
    return acc <= 256;
}

// The tile shape with the best predicted rate: how evenly its tiles deal out over the 256 CUs (the CU with the most
// tiles sets the time: 288 tiles of 256x128 on 3072^3 ran at 74.8 TFLOP/s, 2304 tiles of 64x64 at 105.4) times what
// the shape reaches on a CU, which grows with the number of tiles a CU works through (co-resident workgroups cover one
// another's barriers and first loads).  The two rates per shape are measurements on MI355X, TFLOP/s with exactly one
// tile per CU and with many: 256x256 144 / 144 (one workgroup fills a CU), 256x128 125 / 137, 128x128 108 / 134,
// 128x64 93 / 127, 64x64 78 / 117, 64x32 36 / 78, 32x32 30 / 77.  The prediction was within 5 % of the measurement on 2560^3, 3072^3, 5120^3 and
// 6144^3 for every shape (20 cases) and picks the fastest measured shape on each.
MmConfig pick_config(int64_t M, int64_t N, int64_t K /* per chunk */, int64_t groups /* batch * k-chunks */) {
    struct Rated { MmConfig c; double one, many; };
    static const Rated candidates[] = {
        {{256, 256, 16, 4, 4, 4}, 144, 144}, {{256, 128, 16, 4, 2, 4}, 125, 137}, {{128, 128, 16, 2, 2, 8}, 108, 134}, {{128, 64, 16, 2, 2, 8}, 93, 127},
        {{64, 64, 16, 2, 2, 8}, 78, 117},    {{64, 32, 16, 2, 1, 8}, 36, 78},     {{32, 32, 16, 1, 1, 8}, 30, 77},
    };
    auto tiles = [&](const MmConfig& c) { return ((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn) * groups; };
    MmConfig best = candidates[6].c;
    double best_rate = -1.0;
    for (const Rated& r : candidates) {
        const MmConfig& c = r.c;
        // do not pad an extent to more than twice its size
        if (c.bm > 32 && M * 2 <= c.bm) continue;
        if (c.bn > 32 && N * 2 <= c.bn) continue;
        const int64_t t = tiles(c), rounds = (t + 255) / 256;
        const double fill = (double)t / (double)(rounds * 256);
        // the work inside the padded tiles that is real
        const double real = ((double)M * (double)N) / ((double)((M + c.bm - 1) / c.bm * c.bm) * (double)((N + c.bn - 1) / c.bn * c.bn));
        const double rate = fill * real * (r.many - (r.many - r.one) / (double)rounds);
        if (rate > best_rate * 1.02) {  // a smaller tile has to win by more than the model's noise
            best_rate = rate;
            best = c;
        }
    }
    MmConfig c = best;
    // narrow outputs: keep all four waves along m
    if (c.bn == 32 && c.bm == 64) { c.wm = 2; c.wn = 1; }
    // Small tiles mean a small, latency-bound product: every k-tile costs one round trip to memory, so a 64x64 tile
    // over a long k takes it in 64-deep steps (more bytes in flight per step; LDS has room to spare at this size).
    // Measured on 1024^3 (256 tiles of 64x64): 40.2 -> 34.0 us.  DSC_MM_DEEP_K=0 switches it off, =1 also deepens the
    // 128x64 tile (32-deep), which did not pay on the shapes measured.
    {
        const char* e = std::getenv("DSC_MM_DEEP_K");
        const bool off = e && e[0] == '0', wide = e && e[0] != '0';
        const int deep = c.bm * c.bn <= 64 * 64 ? 64 : (wide && c.bm * c.bn <= 128 * 64 ? 32 : 16);
        if (!off && deep > c.bk && K >= (wide ? 2 * deep : 512)) c.bk = deep;
    }
    // tuning hook: DSC_MM_TILE="BM,BN,BK,WAVES_M,WAVES_N,GROUP_M" for products at least one tile large
    if (const char* env = std::getenv("DSC_MM_TILE")) {
        MmConfig e{};
        if (std::sscanf(env, "%d,%d,%d,%d,%d,%d", &e.bm, &e.bn, &e.bk, &e.wm, &e.wn, &e.group_m) == 6 && config_ok(e) &&
            M >= e.bm && N >= e.bn)
            c = e;
    }
    return c;
}

// Tall products with a few columns whose rows lie contiguous in memory and are long (the output layer of a coordinate
// network: 262144 x 256 -> 3) go to the dot-product kernel instead of the row-per-thread one: with a lane per row the
// 64 lanes of a load touch 64 different cache lines, eight loads before a line is used up, and a row of 1 KB per
// lane is more than L1 keeps.  With L lanes along a row every line is requested once.  Measured on MI355X:
// 262144 x 256 -> 3 77.4 -> 53 us, 262144 x 64 -> 3 23.6 -> 19.4 us.
bool dot_kernel_for_many_rows(const FusedKernel& fk, const MatMulDims& g) {
    if (const char* e = std::getenv("DSC_MM_DOT"))
        if (e[0] == '0') return false;
    if (g.chunks != 1 && !fk.sum_chunks) return false;
    if (fk.colsum_out >= 0 || fk.out_slice_width || fk.dgrad.on || fk.cfwd.on || fk.pool.on) return false;
    if (!(g.n <= 16 && g.k >= 64 && g.k <= 256 && g.k * g.n <= 4096 && g.m * g.batch >= 16384)) return false;
    int64_t base = 0, coef[DSC_MAX_DIM] = {0};
    return fk.inputs[0].buffer >= 0 && affine_form(fk.main.raw().inputs[0], &base, coef) && coef[2] == 1;
}

// Row-per-thread matmul for tall products with a narrow output (N <= 32, K <= 256): the HBM-bound GEMMs of the
// convolutions (N = 16, K = 9 / 72) and of the narrow output layers.  Every thread owns one row of C in
// registers.  B's address is the same for every lane of a wave, so the compiler fetches it with scalar loads
// and the FMAs take it as an SGPR operand: no LDS traffic, no barrier.  The k loop is unrolled, so everything
// in an operand's address that depends only on k (the filter tap of an im2col view) is a constant and only
// the row part (image, y, x) is computed per lane, once.  No MFMA: these products have 3-7 flop per byte.
bool rows_kernel_applies(const FusedKernel& fk, const MatMulDims& g) {
    if (const char* e = std::getenv("DSC_MM_ROWS"))
        if (e[0] == '0') return false;
    if (g.chunks != 1 && !fk.sum_chunks) return false;
    if (dot_kernel_for_many_rows(fk, g)) return false;
    return g.n <= 32 && g.k <= 256 && g.k * g.n <= 8192 && g.m * g.batch >= 16384;
}

// Products with a very short k (the three input coordinates or output channels of a coordinate network: k <= 16) are
// outer-product sums, bound by streaming C: one thread computes four adjacent columns of one row, A's k values
// and B's 16-byte pieces come from L1, and the fused consumer runs on the four results before one 16-byte store
// per output.  No LDS, no MFMA.
bool smallk_kernel_applies(const FusedKernel& fk, const MatMulDims& g) {
    if (const char* e = std::getenv("DSC_MM_SMALLK"))
        if (e[0] == '0') return false;
    if (g.chunks != 1 && !fk.sum_chunks) return false;
    const bool rows = fk.main.raw().output_mode == DSC_MATMUL_ROWS;
    const int64_t batch_stride = rows ? g.n : g.m * g.n, row_stride = rows ? g.batch * g.n : g.n;
    return g.k <= 16 && g.n >= 16 && g.n % 4 == 0 && batch_stride % 4 == 0 && row_stride % 4 == 0 && g.m * g.n * g.batch >= 65536;
}

string gen_matmul_smallk(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const MatMulDims g = matmul_dims(d);
    const bool rows = d.output_mode == DSC_MATMUL_ROWS;
    const int64_t batch_stride = rows ? g.n : g.m * g.n, row_stride = rows ? g.batch * g.n : g.n;
    const int n_out = fk.has_epilogue ? fk.epilogue.raw().n_outputs : 1;
    const string la = em.load_view(fk.inputs[0], d.inputs[0], {"cb", "cm", "ck"});
    em.funcs << "DSC_INLINE float load_a(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la << ";\n}\n";
    const string lb = em.load_view(fk.inputs[1], d.inputs[1], {"cb", "ck", "cn"});
    em.funcs << "DSC_INLINE float load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";
    if (fk.has_epilogue) {
        const dsc_kernel_desc& pe = fk.epilogue.raw();
        std::ostringstream body;
        std::map<int, string> ov;
        ov[fk.epilogue_product_input] = "product";
        IndexForm form;
        form.valid = true;
        form.names = {"cb", "cm", "cn"};
        form.coefs = {batch_stride, row_stride, 1};
        form.extents = {g.batch, g.m, g.n};
        em.emit_pe(body, pe, fk.epilogue_inputs, "gid", "e", ov, &form);
        for (int o = 0; o < pe.n_outputs; ++o) body << "    result[" << o << "] = et" << pe.outputs[o] << ";\n";
        em.funcs << "DSC_INLINE void mm_epilogue(float product, int gid, int cb, int cm, int cn, float* result, " << em.params_decl() << ") {\n"
                 << body.str() << "}\n";
    }
    const int64_t nq = g.n / 4, total = g.batch * g.m * nq;
    if (total >= kMaxIndex) return "matmul: too large";
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(fk) << "(" << em.kernel_params_decl() << ") {\n";
    k << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    k << "    const uint t = blockIdx.x * 256u + threadIdx.x;\n    if (t >= " << S(total) << "u) return;\n";
    k << "    const int cn = (int)(t % " << S(nq) << "u) * 4, cm = (int)((t / " << S(nq) << "u) % " << S(g.m) << "u), cb = (int)(t / " << S(nq * g.m) << "u);\n";
    k << "    float acc[4] = {0.f, 0.f, 0.f, 0.f};\n";
    k << "#pragma unroll\n    for (int ck = 0; ck < " << S(g.k) << "; ++ck) {\n";
    k << "        const float a = load_a(cb, cm, ck, " << em.params_pass() << ");\n";
    k << "#pragma unroll\n        for (int j = 0; j < 4; ++j) acc[j] = fmaf(a, load_b(cb, ck, cn + j, " << em.params_pass() << "), acc[j]);\n    }\n";
    k << "    const int c_at = cb * " << S(batch_stride) << " + cm * " << S(row_stride) << " + cn;\n";
    if (fk.has_epilogue) {
        k << "    float res[4][" << n_out << "];\n";
        k << "#pragma unroll\n    for (int j = 0; j < 4; ++j) mm_epilogue(acc[j], c_at + j, cb, cm, cn + j, res[j], " << em.params_pass() << ");\n";
        for (int o = 0; o < n_out; ++o)
            k << "    *(float4*)(b" << fk.outputs[o] << " + c_at) = make_float4(res[0][" << o << "], res[1][" << o << "], res[2][" << o << "], res[3]["
              << o << "]);\n";
    } else {
        k << "    *(float4*)(b" << fk.outputs[0] << " + c_at) = make_float4(acc[0], acc[1], acc[2], acc[3]);\n";
    }
    k << "}\n";
    out->grid = blocks_for(total, 256);
    out->block = 256;
    out->source = k.str();
    out->note = string("short-k fma, four columns per thread") + (fk.has_epilogue ? " +epilogue" : "");
    return "";
}

// The short-k kernel of a layer's data gradient that computes the layer's weight gradient as well (see
// FusedKernel::GradPair).  256 threads = n/4 column quads x (1024 / n) row lanes; a workgroup owns `chunk_rows` rows.
// Per row a thread loads dY's k values, 16 bytes of X and computes what the short-k kernel computes, with X handed
// to the consumer as a value; X times dY goes into 4k accumulators, which meet in LDS at the end.  Up to eight rows
// are requested before the first is used.
string gen_matmul_smallk_pair(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const MatMulDims g = matmul_dims(d);
    const dsc_kernel_desc& pe = fk.epilogue.raw();
    const int n_out = pe.n_outputs;
    const int64_t N = g.n, KS = g.k, NQ = N / 4, RL = 256 / NQ, R = fk.pair.chunk_rows, C = fk.pair.chunks;
    if (!fk.has_epilogue || g.batch != 1 || KS > 4 || N % 4 != 0 || NQ > 256 || 256 % NQ != 0 || R < 1 || C < 1 || (C - 1) * R >= g.m || C * R < g.m ||
        C >= kMaxIndex || fk.pair.x_buffer < 0 || fk.pair.out < 0)
        return "matmul: not a data/weight gradient pair";
    // rows in flight per thread (262144 x 256, k = 3, 1024 workgroups: 2 rows 105.6 us, 4 103.5, 8 97.7, 16 96.1)
    const int U = (int)std::max<int64_t>(1, std::min<int64_t>(8, R / RL));
    const string la = em.load_view(fk.inputs[0], d.inputs[0], {"cb", "cm", "ck"});
    em.funcs << "DSC_INLINE float load_a(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la << ";\n}\n";
    const string lb = em.load_view(fk.inputs[1], d.inputs[1], {"cb", "ck", "cn"});
    em.funcs << "DSC_INLINE float load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";
    {
        std::ostringstream body;
        std::map<int, string> ov;
        ov[fk.epilogue_product_input] = "product";
        for (int i = 0; i < pe.n_inputs; ++i)
            if (i != fk.epilogue_product_input && fk.epilogue_inputs[i].buffer == fk.pair.x_buffer && is_identity(pe.inputs[i]) &&
                element_count(pe.inputs[i].out_shape) == g.m * N)
                ov[i] = "xval";
        IndexForm form;
        form.valid = true;
        form.names = {"cb", "cm", "cn"};
        form.coefs = {g.m * N, N, 1};
        form.extents = {g.batch, g.m, g.n};
        em.emit_pe(body, pe, fk.epilogue_inputs, "gid", "e", ov, &form);
        for (int o = 0; o < pe.n_outputs; ++o) body << "    result[" << o << "] = et" << pe.outputs[o] << ";\n";
        em.funcs << "DSC_INLINE void mm_epilogue(float product, float xval, int gid, int cb, int cm, int cn, float* result, " << em.params_decl() << ") {\n"
                 << body.str() << "}\n";
    }
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(fk) << "(" << em.kernel_params_decl() << ") {\n";
    k << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    k << "    __shared__ float red[" << S(RL * N * KS) << "];\n";
    k << "    const int q = threadIdx.x % " << S(NQ) << ", rl = threadIdx.x / " << S(NQ) << ", cn = q * 4, cb = 0;\n";
    k << "    const int row_begin = blockIdx.x * " << S(R) << ", row_end = min(row_begin + " << S(R) << ", " << S(g.m) << ");\n";
    k << "    float bq[" << S(KS) << "][4], wg[" << S(KS) << "][4];\n";
    k << "#pragma unroll\n    for (int ck = 0; ck < " << S(KS) << "; ++ck)\n#pragma unroll\n        for (int j = 0; j < 4; ++j) {\n";
    k << "            bq[ck][j] = load_b(cb, ck, cn + j, " << em.params_pass() << ");\n            wg[ck][j] = 0.f;\n        }\n";
    k << "    for (int r0 = row_begin + rl; r0 < row_end; r0 += " << S(RL * U) << ") {\n";
    k << "        float a[" << U << "][" << S(KS) << "];\n        float4 x[" << U << "];\n";
    // rows past the chunk's end repeat its last row's loads and take no part in the sums or the stores
    k << "#pragma unroll\n        for (int u = 0; u < " << U << "; ++u) {\n";
    k << "            const int cm = min(r0 + u * " << S(RL) << ", row_end - 1);\n";
    k << "#pragma unroll\n            for (int ck = 0; ck < " << S(KS) << "; ++ck) a[u][ck] = load_a(cb, cm, ck, " << em.params_pass() << ");\n";
    k << "            x[u] = *(const float4*)(b" << fk.pair.x_buffer << " + (cm * " << S(N) << " + cn));\n        }\n";
    k << "#pragma unroll\n        for (int u = 0; u < " << U << "; ++u) {\n";
    k << "            const int cm = r0 + u * " << S(RL) << ";\n            if (cm < row_end) {\n";
    k << "                const float xs[4] = {x[u].x, x[u].y, x[u].z, x[u].w};\n";
    k << "                const int c_at = cm * " << S(N) << " + cn;\n";
    k << "                float res[4][" << n_out << "];\n";
    k << "#pragma unroll\n                for (int j = 0; j < 4; ++j) {\n                    float acc = 0.f;\n";
    k << "#pragma unroll\n                    for (int ck = 0; ck < " << S(KS) << "; ++ck) acc = fmaf(a[u][ck], bq[ck][j], acc);\n";
    k << "                    mm_epilogue(acc, xs[j], c_at + j, cb, cm, cn + j, res[j], " << em.params_pass() << ");\n";
    k << "#pragma unroll\n                    for (int ck = 0; ck < " << S(KS) << "; ++ck) wg[ck][j] = fmaf(xs[j], a[u][ck], wg[ck][j]);\n                }\n";
    for (int o = 0; o < n_out; ++o)
        k << "                *(float4*)(b" << fk.outputs[o] << " + c_at) = make_float4(res[0][" << o << "], res[1][" << o << "], res[2][" << o << "], res[3]["
          << o << "]);\n";
    k << "            }\n        }\n    }\n";
    // partial[chunk][column][k]: the row lanes' sums meet in LDS
    k << "#pragma unroll\n    for (int j = 0; j < 4; ++j)\n#pragma unroll\n        for (int ck = 0; ck < " << S(KS) << "; ++ck) red[rl * " << S(N * KS)
      << " + (cn + j) * " << S(KS) << " + ck] = wg[ck][j];\n";
    k << "    __syncthreads();\n";
    k << "    for (int i = threadIdx.x; i < " << S(N * KS) << "; i += 256) {\n        float sum = red[i];\n";
    k << "        for (int r = 1; r < " << S(RL) << "; ++r) sum += red[r * " << S(N * KS) << " + i];\n";
    k << "        b" << fk.pair.out << "[blockIdx.x * " << S(N * KS) << " + i] = sum;\n    }\n}\n";
    out->grid = (unsigned)C;
    out->block = 256;
    out->source = k.str();
    out->note = "short-k fma, four columns per thread +epilogue, +the weight gradient X^T A over " + S(C) + " chunks of " + S(R) + " rows";
    return "";
}

// Dot-product kernel for products with few columns and not many rows (a classifier head: 1000 x 128 -> 10): too
// small to fill the MFMA template's tiles -- a 32x32 tile grid of such a product is a few dozen single-wave
// workgroups, each walking k in eight sequential load -> LDS -> MFMA round trips.  Here L lanes share one row: lane l
// takes the 16-byte blocks l, l + L, ... of the row's k range (consecutive lanes read consecutive memory), multiplies
// them with B from LDS (the whole of B is a few KB), and the lanes' partial sums meet in a shuffle butterfly.  All
// loads of a lane are independent, so the kernel is one memory round trip deep.
bool dot_shape(const MatMulDims& g) {
    // B is staged by every workgroup, for the 256 / L rows it holds: beyond a few KB that costs more than the k
    // re-split + MFMA path (1000 x 784 -> 10: 14.6 us against 9.1 + a reduce that rides in the consumer)
    return g.chunks == 1 && g.n <= 16 && g.k >= 32 && g.k * g.n <= 4096 && g.m * g.batch >= 64 && g.m * g.batch < 16384;
}

bool dot_kernel_applies(const FusedKernel& fk, const MatMulDims& g) {
    if (const char* e = std::getenv("DSC_MM_DOT"))
        if (e[0] == '0') return false;
    MatMulDims whole = g;
    if (fk.sum_chunks) whole.chunks = 1;  // one full sum over k is what this kernel computes anyway
    return fk.colsum_out < 0 && (dot_shape(whole) || dot_kernel_for_many_rows(fk, g));
}

}  // namespace

bool matmul_fits_row_stage(const FusedKernel& fk) {
    const dsc_kernel_desc& d = fk.main.raw();
    if (d.kind != DSC_KERNEL_MATMUL || d.output_mode != DSC_MATMUL_BATCHES || fk.colsum_out >= 0 || fk.dgrad.on || fk.cfwd.on || fk.out_slice_width) return false;
    const MatMulDims g = matmul_dims(d);
    return g.batch == 1 && g.chunks == 1 && g.n >= 2 && dot_kernel_applies(fk, g);
}

namespace {
string gen_matmul_dot(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const MatMulDims g = matmul_dims(d);
    const bool rows = d.output_mode == DSC_MATMUL_ROWS;
    const int64_t batch_stride = rows ? g.n : g.m * g.n, row_stride = rows ? g.batch * g.n : g.n;
    const int n_out = fk.has_epilogue ? fk.epilogue.raw().n_outputs : 1;
    const int64_t N = g.n, K = g.k, blocks = (K + 3) / 4;
    int64_t L = 4;
    while (L < 64 && L * 2 < blocks) L *= 2;  // about two blocks per lane
    const int64_t J = (blocks + L - 1) / L, RPW = 256 / L, total_rows = g.m * g.batch;
    const string la = em.load_view(fk.inputs[0], d.inputs[0], {"cb", "cm", "ck"});
    em.funcs << "DSC_INLINE float load_a(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la << ";\n}\n";
    const string lb = em.load_view(fk.inputs[1], d.inputs[1], {"cb", "ck", "cn"});
    em.funcs << "DSC_INLINE float load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";
    if (fk.has_epilogue) {
        const dsc_kernel_desc& pe = fk.epilogue.raw();
        std::ostringstream body;
        std::map<int, string> ov;
        ov[fk.epilogue_product_input] = "product";
        IndexForm form;
        form.valid = true;
        form.names = {"cb", "cm", "cn"};
        form.coefs = {batch_stride, row_stride, 1};
        form.extents = {g.batch, g.m, g.n};
        em.emit_pe(body, pe, fk.epilogue_inputs, "gid", "e", ov, &form);
        for (int o = 0; o < pe.n_outputs; ++o) body << "    result[" << o << "] = et" << pe.outputs[o] << ";\n";
        em.funcs << "DSC_INLINE void mm_epilogue(float product, int gid, int cb, int cm, int cn, float* result, " << em.params_decl() << ") {\n"
                 << body.str() << "}\n";
    }
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(fk) << "(" << em.kernel_params_decl() << ") {\n";
    k << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    // B of this workgroup's batch: [k][n], zero beyond k (a workgroup's rows may straddle two batches only when
    // the batch has fewer rows than a workgroup, which the row -> batch split below rules out by using one batch
    // per workgroup)
    // Many rows: a workgroup walks T groups of RPW rows with B staged once, the next group's A requested before the
    // current one is multiplied.
    const int64_t T = total_rows >= 16384 ? 8 : 1;
    const int64_t wgs_per_batch = (g.m + RPW * T - 1) / (RPW * T);
    k << "    __shared__ float sB[" << S(blocks * 4 * N) << "];\n";
    k << "    const int cb = blockIdx.x / " << S(wgs_per_batch) << ", row0 = (blockIdx.x % " << S(wgs_per_batch) << ") * " << S(RPW * T) << ";\n";
    k << "    for (int e = threadIdx.x; e < " << S(blocks * 4 * N) << "; e += 256) {\n";
    k << "        const int kk = e / " << S(N) << ", nn = e % " << S(N) << ";\n";
    k << "        const float v = load_b(cb, min(kk, " << S(K - 1) << "), nn, " << em.params_pass() << ");\n";
    k << "        sB[e] = kk < " << S(K) << " ? v : 0.f;\n    }\n";
    k << "    const int lg = threadIdx.x % " << S(L) << ", rl = row0 + threadIdx.x / " << S(L) << ";\n";
    // A: every block of the lane requested before anything is used; beyond k the clamped loads repeat valid
    // elements, which meet zeros of B
    k << "    float a[" << S(J) << "][4], an[" << S(J) << "][4];\n";
    auto load_group = [&](const char* dst, const string& row) {
        k << "#pragma unroll\n    for (int j = 0; j < " << S(J) << "; ++j)\n#pragma unroll\n        for (int i = 0; i < 4; ++i)\n";
        k << "            " << dst << "[j][i] = load_a(cb, min(" << row << ", " << S(g.m - 1) << "), min(4 * (lg + j * " << S(L) << ") + i, " << S(K - 1) << "), "
          << em.params_pass() << ");\n";
    };
    load_group("a", "rl");
    k << "    __syncthreads();\n";
    k << "#pragma unroll\n    for (int it = 0; it < " << S(T) << "; ++it) {\n";
    k << "    const int cm = rl + it * " << S(RPW) << ";\n";
    if (T > 1) {
        k << "    if (it + 1 < " << S(T) << ") {\n";
        load_group("an", "cm + " + S(RPW));
        k << "    }\n";
    }
    k << "    float acc[" << S(N) << "];\n#pragma unroll\n    for (int n = 0; n < " << S(N) << "; ++n) acc[n] = 0.f;\n";
    k << "#pragma unroll\n    for (int j = 0; j < " << S(J) << "; ++j) {\n";
    k << "        const int blk = lg + j * " << S(L) << ";\n";
    k << "        if (blk < " << S(blocks) << ") {\n";
    k << "#pragma unroll\n            for (int i = 0; i < 4; ++i)\n#pragma unroll\n                for (int n = 0; n < " << S(N) << "; ++n)\n";
    k << "                    acc[n] = fmaf(a[j][i], sB[(4 * blk + i) * " << S(N) << " + n], acc[n]);\n        }\n    }\n";
    k << "#pragma unroll\n    for (int n = 0; n < " << S(N) << "; ++n)\n#pragma unroll\n        for (int s = 1; s < " << S(L) << "; s *= 2) acc[n] += __shfl_xor(acc[n], s);\n";
    // every lane of the group now holds the row's sums; lane lg stores columns lg, lg + L, ...
    k << "    if (cm < " << S(g.m) << ") {\n";
    k << "#pragma unroll\n        for (int n = 0; n < " << S(N) << "; ++n)\n            if (n % " << S(L) << " == lg) {\n";
    k << "                const int c_at = cb * " << S(batch_stride) << " + cm * " << S(row_stride) << " + n;\n";
    if (fk.has_epilogue) {
        k << "                float res[" << n_out << "];\n                mm_epilogue(acc[n], c_at, cb, cm, n, res, " << em.params_pass() << ");\n";
        for (int o = 0; o < n_out; ++o) k << "                b" << fk.outputs[o] << "[c_at] = res[" << o << "];\n";
    } else {
        k << "                b" << fk.outputs[0] << "[c_at] = acc[n];\n";
    }
    k << "            }\n    }\n";
    if (T > 1) k << "#pragma unroll\n    for (int j = 0; j < " << S(J) << "; ++j)\n#pragma unroll\n        for (int i = 0; i < 4; ++i) a[j][i] = an[j][i];\n";
    k << "    }\n}\n";
    (void)total_rows;
    if (wgs_per_batch * g.batch >= kMaxIndex) return "matmul: grid too large";
    out->grid = (unsigned)(wgs_per_batch * g.batch);
    out->block = 256;
    out->source = k.str();
    out->note = "dot products: " + S(L) + " lanes per row, " + (T > 1 ? S(T) + " row groups per workgroup, " : string()) + "B in LDS" + (fk.has_epilogue ? " +epilogue" : "");
    return "";
}

string gen_matmul_rows(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const MatMulDims g = matmul_dims(d);
    const dsc_view& va = d.inputs[0];
    const dsc_view& vb = d.inputs[1];
    const bool rows = d.output_mode == DSC_MATMUL_ROWS;
    const int64_t batch_stride = rows ? g.n : g.m * g.n, row_stride = rows ? g.batch * g.n : g.n;
    // Measured on MI355X on the ConvNet's k=72 product (196000 x 2 x 16): one row per thread, k unrolled by 8 and B
    // through the scalar unit 35 us; B in LDS 40 us; two / four rows per thread 41 / 46 us.  The slower variants stay
    // in the generator (R, b_in_lds) because other shapes may want them; nothing selects them today.
    const int R = 1;  // rows per thread
    const int unroll = g.k <= 16 ? (int)g.k : 8;
    const int64_t blocks_per_batch = (g.m + 256 * R - 1) / (256 * R);
    const bool b_in_lds = false;
    const int n_out = fk.has_epilogue ? fk.epilogue.raw().n_outputs : 1;

    const string la = em.load_view(fk.inputs[0], va, {"cb", "cm", "ck"});
    em.funcs << "DSC_INLINE float load_a(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la << ";\n}\n";
    const string lb = em.load_view(fk.inputs[1], vb, {"cb", "ck", "cn"});
    em.funcs << "DSC_INLINE float load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";
    if (fk.has_epilogue) {
        const dsc_kernel_desc& pe = fk.epilogue.raw();
        std::ostringstream body;
        std::map<int, string> ov;
        ov[fk.epilogue_product_input] = "product";
        em.emit_pe(body, pe, fk.epilogue_inputs, "gid", "e", ov);
        for (int o = 0; o < pe.n_outputs; ++o) body << "    result[" << o << "] = et" << pe.outputs[o] << ";\n";
        em.funcs << "DSC_INLINE void mm_epilogue(float product, int gid, float* result, " << em.params_decl() << ") {\n"
                 << body.str() << "}\n";
    }

    // 16-byte stores when four consecutive columns are four consecutive, aligned words
    const bool vec_store = g.n % 4 == 0 && batch_stride % 4 == 0 && row_stride % 4 == 0;
    std::ostringstream k;
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(fk) << "(" << em.kernel_params_decl() << ") {\n";
    k << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    // A depthwise product (one column per batch, the batches innermost in memory: [m][batch][1], the channels of an
    // image) with consecutive lanes on consecutive batches of a row: the loads of A and the store then walk memory,
    // where a lane per row of one batch reads and writes words `batch` apart (measured on a 3x3 blur of [1000, 27,
    // 27, 16]: 134 us with a lane per row).  B is then a vector load per lane, from a few cache lines.
    const bool batch_lanes = rows && g.n == 1 && g.batch > 1 && g.batch * g.m < kMaxIndex && R == 1 && !b_in_lds && !fk.out_slice_width;
    // (the filters, read per lane here, stay in memory: staged in LDS -- a fill and a barrier per workgroup -- the blur of
    // [1000, 27, 27, 16] took 16.2 us against 14.0; and four batches per thread, A's four read with one 16-byte load,
    // took 14.1 us: the kernel is not bound by its load instructions)
    if (batch_lanes) {
        k << "    const int flat = min((int)(blockIdx.x * 256u + threadIdx.x), " << S(g.batch * g.m - 1) << ");\n";
        k << "    const int cb = flat % " << S(g.batch) << ";\n";
        k << "    const int row0 = blockIdx.x * 256u + threadIdx.x < " << S(g.batch * g.m) << "u ? flat / " << S(g.batch) << " : " << S(g.m) << ";\n";
    } else {
    k << "    const int cb = blockIdx.x / " << S(blocks_per_batch) << ";\n";
    k << "    const int row0 = (blockIdx.x % " << S(blocks_per_batch) << ") * " << S(256 * R) << " + threadIdx.x;\n";
    }
    if (b_in_lds) {
        k << "    __shared__ __attribute__((aligned(16))) float sB[" << S(g.k * g.n) << "];\n";
        k << "    for (int i = threadIdx.x; i < " << S(g.k * g.n) << "; i += 256) sB[i] = load_b(cb, i / " << S(g.n) << ", i % " << S(g.n)
          << ", " << em.params_pass() << ");\n";
        k << "    __syncthreads();\n";
    }
    const int Q = (int)(g.n / 4);  // 16-byte pieces per row
    const int64_t W = fk.out_slice_width;  // slice-major store: a lane writes w floats of every slice, lanes on consecutive rows
    if (W && (g.n % W != 0 || g.batch != 1 || fk.has_epilogue || rows)) return "matmul rows: slice-major store needs one batch, no epilogue and whole slices";
    const bool transposed_store = !W && vec_store && (Q == 1 || Q == 2 || Q == 4 || Q == 8);
    // With at most 16 columns and a k of some length the products go through v_mfma_f32_16x16x4f32 instead of
    // scalar-operand FMAs (twice the fp32 rate with packed math off): a wave takes its 64 rows as four 16-row tiles,
    // lane l feeds A[row l % 16][k = 4 s + l / 16] straight from memory (the same generated load, so an im2col view
    // costs what it costs the FMA path) and keeps B's K/4 fragments in registers; the results land in the LDS
    // staging buffer of the store below in row order.
    bool use_mfma = transposed_store && g.n <= 16 && g.k >= 16 && g.k % 4 == 0 && R == 1 && !b_in_lds;
    if (const char* e = std::getenv("DSC_ROWS_MFMA"))
        if (e[0] == '0') use_mfma = false;
    if (use_mfma) {
        // k is taken in blocks of four consecutive values (one 16-byte piece of an im2col row: four channels of one
        // tap), block q * J + j going to lane group q = l / 16: a lane then computes one address per block, not per
        // k, and feeds the four values to four MFMA steps.  A and B use the same order of k, so the sum is the same.
        const int64_t blocks = g.k / 4;
        const int64_t J = (blocks + 3) / 4;
        k << "    typedef float rm_float4 __attribute__((ext_vector_type(4)));\n";
        k << "    const int lane = threadIdx.x & 63, li = lane & 15, lk = lane >> 4;\n";
        k << "    const int wave_row0 = row0 - lane;\n";
        k << "    float fb[" << S(J) << "][4];\n";
        k << "#pragma unroll\n    for (int j = 0; j < " << S(J) << "; ++j) {\n";
        k << "        const int blk = lk * " << S(J) << " + j;\n";
        k << "#pragma unroll\n        for (int i = 0; i < 4; ++i) {\n";
        k << "            const float v = load_b(cb, min(4 * blk + i, " << S(g.k - 1) << "), min(li, " << S(g.n - 1) << "), " << em.params_pass() << ");\n";
        k << "            fb[j][i] = (blk < " << S(blocks) << " && li < " << S(g.n) << ") ? v : 0.f;\n        }\n    }\n";
        k << "    int cmt[4];\n#pragma unroll\n    for (int t = 0; t < 4; ++t) cmt[t] = min(wave_row0 + t * 16 + li, " << S(g.m - 1) << ");\n";
        k << "    rm_float4 acc4[4];\n#pragma unroll\n    for (int t = 0; t < 4; ++t) acc4[t] = (rm_float4){0.f, 0.f, 0.f, 0.f};\n";
        // the A loads of JG blocks are issued before their MFMAs.  Measured on the ConvNet's second convolution
        // (392000 rows, k = 72): JG 1 / 2 / 3 / 5 = 24.9 / 23.6 / 23.8 / 27.4 us against 25.4 for the FMA path -- the
        // kernel is bound by the 64 cache lines that every 16-byte load instruction of an im2col row block touches,
        // not by either arithmetic pipe.
        const int64_t JG = std::min<int64_t>(2, J);
        k << "#pragma unroll\n    for (int j0 = 0; j0 < " << S(J) << "; j0 += " << S(JG) << ") {\n";
        k << "        float fa[" << S(JG) << "][4][4];\n";
        k << "#pragma unroll\n        for (int jj = 0; jj < " << S(JG) << "; ++jj) {\n";
        k << "            const int blk = min(lk * " << S(J) << " + min(j0 + jj, " << S(J - 1) << "), " << S(blocks - 1) << ");\n";
        k << "#pragma unroll\n            for (int t = 0; t < 4; ++t)\n#pragma unroll\n                for (int i = 0; i < 4; ++i) fa[jj][t][i] = load_a(cb, cmt[t], 4 * blk + i, "
          << em.params_pass() << ");\n        }\n";
        k << "        __builtin_amdgcn_sched_barrier(0);\n";
        // B is zero for the blocks past the end, so whatever A repeats there adds nothing
        k << "#pragma unroll\n        for (int jj = 0; jj < " << S(JG) << "; ++jj)\n            if (j0 + jj < " << S(J) << ")\n";
        k << "#pragma unroll\n                for (int i = 0; i < 4; ++i)\n#pragma unroll\n                    for (int t = 0; t < 4; ++t)\n";
        k << "                        acc4[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[jj][t][i], fb[j0 + jj][i], acc4[t], 0, 0, 0);\n";
        k << "    }\n";
    } else {
    // rows past the end repeat the last row's loads (no divergent loads) and skip the store
    k << "    int cml[" << R << "];\n";
    k << "#pragma unroll\n    for (int r = 0; r < " << R << "; ++r) cml[r] = min(row0 + r * 256, " << S(g.m - 1) << ");\n";
    // R rows per thread (256 apart, so lanes stay on consecutive rows): each B word feeds R FMAs
    k << "    float acc[" << R << "][" << S(g.n) << "];\n";
    k << "#pragma unroll\n    for (int r = 0; r < " << R << "; ++r)\n#pragma unroll\n        for (int n = 0; n < " << S(g.n) << "; ++n) acc[r][n] = 0.f;\n";
    k << "#pragma unroll " << unroll << "\n    for (int ck = 0; ck < " << S(g.k) << "; ++ck) {\n";
    k << "        float a[" << R << "];\n";
    k << "#pragma unroll\n        for (int r = 0; r < " << R << "; ++r) a[r] = load_a(cb, cml[r], ck, " << em.params_pass() << ");\n";
    k << "#pragma unroll\n        for (int n = 0; n < " << S(g.n) << "; ++n) {\n";
    if (b_in_lds)
        k << "            const float bv = sB[ck * " << S(g.n) << " + n];\n";
    else  // the address is the same for every lane: the compiler reads B through the scalar unit into SGPRs
        k << "            const float bv = load_b(cb, ck, n, " << em.params_pass() << ");\n";
    k << "#pragma unroll\n            for (int r = 0; r < " << R << "; ++r) acc[r][n] = fmaf(a[r], bv, acc[r][n]);\n        }\n";
    k << "    }\n";
    }
    if (transposed_store) {
        // A thread holds one whole row, so storing it directly makes every lane of a store instruction write 16
        // bytes of a different row (N*4 bytes apart).  Instead each wave passes its 64 rows through LDS and reads
        // them back so that Q consecutive lanes hold one row: a store instruction then writes 1 KiB of
        // consecutive memory, and the epilogue's own loads are consecutive too.
        const int pitch = (int)g.n + 4;
        k << "    __shared__ __attribute__((aligned(16))) float tr[4][" << 64 * pitch << "];\n";
        k << "    float* my = tr[threadIdx.x >> 6];\n";
        if (!use_mfma) k << "    const int lane = threadIdx.x & 63;\n    const int wave_row0 = row0 - lane;\n";
        k << "#pragma unroll\n    for (int r = 0; r < " << R << "; ++r) {\n";
        if (R > 1) k << "        __syncthreads();\n";
        if (use_mfma) {
            // accumulator register i of lane l is D[4 * (l / 16) + i][l % 16] of its tile
            k << "#pragma unroll\n        for (int t = 0; t < 4; ++t)\n#pragma unroll\n            for (int i = 0; i < 4; ++i)\n";
            k << "                if (li < " << S(g.n) << ") my[(t * 16 + 4 * lk + i) * " << pitch << " + li] = acc4[t][i];\n";
        } else {
        k << "#pragma unroll\n        for (int n = 0; n < " << S(g.n) << "; n += 4) *(float4*)&my[lane * " << pitch
          << " + n] = make_float4(acc[r][n], acc[r][n + 1], acc[r][n + 2], acc[r][n + 3]);\n";
        }
        k << "        __syncthreads();\n";
        k << "#pragma unroll\n        for (int s = 0; s < " << Q << "; ++s) {\n";
        k << "            const int rl = s * " << 64 / Q << " + lane / " << Q << ", q = lane % " << Q << ";\n";
        k << "            const int cm = wave_row0 + r * 256 + rl;\n";
        k << "            const float4 p = *(const float4*)&my[rl * " << pitch << " + q * 4];\n";
        k << "            if (cm < " << S(g.m) << ") {\n";
        k << "                const int c_at = cb * " << S(batch_stride) << " + cm * " << S(row_stride) << " + q * 4;\n";
        if (fk.has_epilogue) {
            k << "                const float pv[4] = {p.x, p.y, p.z, p.w};\n                float res[4][" << n_out << "];\n";
            k << "#pragma unroll\n                for (int j = 0; j < 4; ++j) mm_epilogue(pv[j], c_at + j, res[j], " << em.params_pass() << ");\n";
            for (int o = 0; o < n_out; ++o)
                k << "                *(float4*)(b" << fk.outputs[o] << " + c_at) = make_float4(res[0][" << o << "], res[1][" << o << "], res[2][" << o
                  << "], res[3][" << o << "]);\n";
        } else {
            k << "                *(float4*)(b" << fk.outputs[0] << " + c_at) = p;\n";
        }
        k << "            }\n        }\n    }\n}\n";
    } else {
    k << "#pragma unroll\n    for (int r = 0; r < " << R << "; ++r) {\n";
    k << "    const int cm = row0 + r * 256;\n    if (cm < " << S(g.m) << ") {\n";
    k << "    const int c_row = cb * " << S(batch_stride) << " + cm * " << S(row_stride) << ";\n";
    if (W) {
        for (int64_t sl = 0; sl < g.n / W; ++sl) {
            const string at = "b" + to_string(fk.outputs[0]) + " + (" + S(sl * g.m) + " + cm) * " + S(W);
            const string a0 = "acc[r][" + S(sl * W) + "]";
            if (W == 2) k << "    *(float2*)(" << at << ") = make_float2(acc[r][" << S(sl * W) << "], acc[r][" << S(sl * W + 1) << "]);\n";
            else if (W == 4)
                k << "    *(float4*)(" << at << ") = make_float4(acc[r][" << S(sl * W) << "], acc[r][" << S(sl * W + 1) << "], acc[r][" << S(sl * W + 2) << "], acc[r][" << S(sl * W + 3) << "]);\n";
            else
                for (int64_t j = 0; j < W; ++j) k << "    (" << at << ")[" << S(j) << "] = acc[r][" << S(sl * W + j) << "];\n";
        }
        k << "    (void)c_row;\n";
    } else if (vec_store) {
        k << "#pragma unroll\n    for (int n = 0; n < " << S(g.n) << "; n += 4) {\n";
        if (fk.has_epilogue) {
            k << "        float res[4][" << n_out << "];\n";
            k << "#pragma unroll\n        for (int j = 0; j < 4; ++j) mm_epilogue(acc[r][n + j], c_row + n + j, res[j], " << em.params_pass() << ");\n";
            for (int o = 0; o < n_out; ++o)
                k << "        *(float4*)(b" << fk.outputs[o] << " + c_row + n) = make_float4(res[0][" << o << "], res[1][" << o << "], res[2][" << o
                  << "], res[3][" << o << "]);\n";
        } else {
            k << "        *(float4*)(b" << fk.outputs[0] << " + c_row + n) = make_float4(acc[r][n], acc[r][n + 1], acc[r][n + 2], acc[r][n + 3]);\n";
        }
        k << "    }\n";
    } else {
        k << "#pragma unroll\n    for (int n = 0; n < " << S(g.n) << "; ++n) {\n";
        if (fk.has_epilogue) {
            k << "        float res[" << n_out << "];\n        mm_epilogue(acc[r][n], c_row + n, res, " << em.params_pass() << ");\n";
            for (int o = 0; o < n_out; ++o) k << "        b" << fk.outputs[o] << "[c_row + n] = res[" << o << "];\n";
        } else {
            k << "        b" << fk.outputs[0] << "[c_row + n] = acc[r][n];\n";
        }
        k << "    }\n";
    }
    k << "    }\n    }\n}\n";
    }
    out->grid = batch_lanes ? (unsigned)((g.batch * g.m + 255) / 256) : (unsigned)(blocks_per_batch * g.batch);
    out->block = 256;
    out->source = k.str();
    out->note = (use_mfma ? string("row-per-thread store, mfma 16x16x4 from memory, B in registers")
                 : batch_lanes ? string("row-per-thread fma, lanes along the batches of a row")
                          : string("row-per-thread fma, B ") + (b_in_lds ? "in LDS" : "in SGPRs")) +
                (fk.has_epilogue ? " +epilogue" : "") + (W ? ", product stored as " + S(g.n / W) + " column slices of width " + S(W) : string());
    return "";
}

// k range of one chunk of a MatMul descriptor: the reference writes `chunks` partial products of
// chunk_tiles * 16 k each (src/kernel.rs:436)
int64_t chunk_k_of(const MatMulDims& g) {
    const int64_t k_tiles = (g.k + 15) / 16;
    return ((k_tiles + g.chunks - 1) / g.chunks) * 16;
}

// Tall-k matmul: a small output (at most 16 tiles of 16x16) summed over a very long k that is already split
// into many chunks -- the weight gradients of the convolutions (72x16 and 9x16 outputs, k = batch * pixels)
// and of narrow dense layers.  There is nothing to reuse between workgroups, so the operands skip LDS: every
// wave takes its own k steps, loads the 16x4 / 4x16 MFMA fragments straight from memory (several steps in
// flight) and keeps the whole output in accumulators; the four waves of a workgroup are summed through LDS at
// the end.  One workgroup per (chunk, batch).
bool tallk_shape_impl(const MatMulDims& g) {
    if (const char* e = std::getenv("DSC_MM_TALLK"))
        if (e[0] == '0') return false;
    const int64_t tiles = ((g.m + 15) / 16) * ((g.n + 15) / 16);
    return tiles <= 16 && g.chunks > 1 && chunk_k_of(g) >= 128 && g.batch * g.chunks >= 128;
}

bool tallk_kernel_applies(const FusedKernel& fk, const MatMulDims& g) {
    return !fk.has_epilogue && !fk.sum_chunks && tallk_shape_impl(g);
}

string gen_matmul_tallk(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const MatMulDims g = matmul_dims(d);
    const bool rows = d.output_mode == DSC_MATMUL_ROWS;
    const int64_t batch_stride = rows ? g.n : g.m * g.n, row_stride = rows ? g.batch * g.n : g.n;
    const int64_t chunk_k = chunk_k_of(g);
    const int MT = (int)((g.m + 15) / 16), NT = (int)((g.n + 15) / 16);
    const int U = std::max(1, std::min(8, 24 / (MT + NT)));  // k steps of 4 in flight per wave

    const string la = em.load_view(fk.inputs[0], d.inputs[0], {"cb", "cm", "ck"});
    em.funcs << "DSC_INLINE float load_a(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la << ";\n}\n";
    const string lb = em.load_view(fk.inputs[1], d.inputs[1], {"cb", "ck", "cn"});
    em.funcs << "DSC_INLINE float load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";

    std::ostringstream k;
    k << "typedef float tk_float4 __attribute__((ext_vector_type(4)));\n";
    k << "extern \"C\" __global__ __launch_bounds__(256) void " << entry_name(fk) << "(" << em.kernel_params_decl() << ") {\n";
    k << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    k << "    __shared__ float red[4][" << MT * NT * 256 << "];\n";
    const bool colsum = fk.colsum_out >= 0;
    if (colsum) {
        k << "    __shared__ float cs_red[4][" << NT * 16 << "];\n";
        k << "    float cs[" << NT << "];\n#pragma unroll\n    for (int nt = 0; nt < " << NT << "; ++nt) cs[nt] = 0.f;\n";
    }
    k << "    const int chunk = blockIdx.x % " << S(g.chunks) << ", cb = blockIdx.x / " << S(g.chunks) << ";\n";
    k << "    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;\n";
    k << "    const int li = lane & 15, lk = lane >> 4;\n";
    k << "    const int k_begin = chunk * " << S(chunk_k) << ", k_end = min(k_begin + " << S(chunk_k) << ", " << S(g.k) << ");\n";
    k << "    tk_float4 acc[" << MT << "][" << NT << "];\n";
    k << "#pragma unroll\n    for (int mt = 0; mt < " << MT << "; ++mt)\n#pragma unroll\n        for (int nt = 0; nt < " << NT
      << "; ++nt) acc[mt][nt] = (tk_float4){0.f, 0.f, 0.f, 0.f};\n";
    // A fragment of v_mfma_f32_16x16x4f32: lane l holds A[l % 16][l / 16]; B fragment: B[l / 16][l % 16]
    k << "    for (int k0 = k_begin + wave * " << 4 * U << "; k0 < k_end; k0 += " << 16 * U << ") {\n";
    k << "        float fa[" << U << "][" << MT << "], fb[" << U << "][" << NT << "];\n";
    // out-of-range rows, columns and k repeat a valid element's load (no divergent loads) and are zeroed after
    // the fence below.  Nothing before the fence consumes a loaded value, so every load of the iteration is in
    // flight before the first wait (left alone, the compiler's schedule waits right after each load).
    k << "#pragma unroll\n        for (int u = 0; u < " << U << "; ++u) {\n";
    k << "            const int ckc = min(k0 + 4 * u + lk, " << S(g.k - 1) << ");\n";
    k << "#pragma unroll\n            for (int mt = 0; mt < " << MT << "; ++mt) fa[u][mt] = load_a(cb, min(mt * 16 + li, " << S(g.m - 1)
      << "), ckc, " << em.params_pass() << ");\n";
    k << "#pragma unroll\n            for (int nt = 0; nt < " << NT << "; ++nt) fb[u][nt] = load_b(cb, ckc, min(nt * 16 + li, " << S(g.n - 1)
      << "), " << em.params_pass() << ");\n";
    k << "        }\n";
    k << "        __builtin_amdgcn_sched_barrier(0);\n";
    k << "#pragma unroll\n        for (int u = 0; u < " << U << "; ++u) {\n";
    k << "            const bool k_ok = k0 + 4 * u + lk < k_end;\n";
    k << "#pragma unroll\n            for (int mt = 0; mt < " << MT << "; ++mt) fa[u][mt] = (k_ok && mt * 16 + li < " << S(g.m)
      << ") ? fa[u][mt] : 0.f;\n";
    k << "#pragma unroll\n            for (int nt = 0; nt < " << NT << "; ++nt) fb[u][nt] = (k_ok && nt * 16 + li < " << S(g.n)
      << ") ? fb[u][nt] : 0.f;\n";
    k << "        }\n";
    // column sums of B (a bias gradient riding on the weight gradient): the B fragments are summed per lane here,
    // over the lane groups and waves after the loop
    if (colsum)
        k << "#pragma unroll\n        for (int u = 0; u < " << U << "; ++u)\n#pragma unroll\n            for (int nt = 0; nt < " << NT
          << "; ++nt) cs[nt] += fb[u][nt];\n";
    k << "#pragma unroll\n        for (int u = 0; u < " << U << "; ++u)\n#pragma unroll\n            for (int mt = 0; mt < " << MT
      << "; ++mt)\n#pragma unroll\n                for (int nt = 0; nt < " << NT << "; ++nt)\n"
      << "                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[u][mt], fb[u][nt], acc[mt][nt], 0, 0, 0);\n";
    k << "    }\n";
    k << "#pragma unroll\n    for (int mt = 0; mt < " << MT << "; ++mt)\n#pragma unroll\n        for (int nt = 0; nt < " << NT
      << "; ++nt)\n#pragma unroll\n            for (int r = 0; r < 4; ++r) red[wave][(mt * " << NT << " + nt) * 256 + r * 64 + lane] = acc[mt][nt][r];\n";
    if (colsum) {
        k << "#pragma unroll\n    for (int nt = 0; nt < " << NT << "; ++nt) {\n";
        k << "        float t = cs[nt];\n        t += __shfl_xor(t, 16, 64);\n        t += __shfl_xor(t, 32, 64);\n";
        k << "        if (lk == 0) cs_red[wave][nt * 16 + li] = t;\n    }\n";
    }
    k << "    __syncthreads();\n";
    if (colsum) {
        k << "    if (threadIdx.x < " << NT * 16 << " && threadIdx.x < " << S(g.n) << ")\n";
        k << "        b" << fk.colsum_out << "[(chunk * " << S(g.batch) << " + cb) * " << S(g.n) << " + threadIdx.x] = (cs_red[0][threadIdx.x] + cs_red[1][threadIdx.x]) + (cs_red[2][threadIdx.x] + cs_red[3][threadIdx.x]);\n";
    }
    // accumulator register r of lane l is D[4 * (l / 16) + r][l % 16]
    k << "    for (int i = threadIdx.x; i < " << MT * NT * 256 << "; i += 256) {\n";
    k << "        const float sum = (red[0][i] + red[1][i]) + (red[2][i] + red[3][i]);\n";
    k << "        const int tile = i >> 8, r = (i >> 6) & 3, l = i & 63;\n";
    k << "        const int cm = (tile / " << NT << ") * 16 + 4 * (l >> 4) + r, cn = (tile % " << NT << ") * 16 + (l & 15);\n";
    k << "        if (cm < " << S(g.m) << " && cn < " << S(g.n) << ") b" << fk.outputs[0] << "[chunk * " << S(g.batch * g.m * g.n) << " + cb * "
      << S(batch_stride) << " + cm * " << S(row_stride) << " + cn] = sum;\n";
    k << "    }\n}\n";
    const int64_t grid = g.batch * g.chunks;
    if (grid >= kMaxIndex) return "matmul: grid too large";
    out->grid = (unsigned)grid;
    out->block = 256;
    out->source = k.str();
    char note[160];
    std::snprintf(note, sizeof note, "tall-k mfma 16x16x4, %dx%d tiles, operands from memory, %d steps in flight, chunks %lld%s", MT, NT, U,
                  (long long)g.chunks, colsum ? " +column sums of B" : "");
    out->note = note;
    return "";
}

// k split inside the workgroup: a product whose output is small (a few hundred 16x16 tiles) and whose k is a few
// hundred to a few thousand long -- the first layer of a classifier at batch 1000, 1000 x 784 -> 128.  Tiled for the
// MFMA template it is a few dozen workgroups walking k in sequential load -> LDS -> multiply round trips; split over k
// into partial products it is two launches and a pass over the partials.  Here a workgroup owns a block of 16 rows x
// NTB*16 columns for the WHOLE k: its waves take a slice of k each, load the 16x4 / 4x16 fragments of
// v_mfma_f32_16x16x4f32 straight from memory (A in 16-byte pieces along k, B a word per lane and row, a batch of
// k blocks requested before the first product), and meet in LDS, where the per-element consumer is applied before
// the one store.  One launch, no partials in memory.
struct KsplitPlan {
    int ntb = 0, waves = 0;
    int64_t blocks_m = 0, blocks_n = 0;
};
bool ksplit_plan(const FusedKernel& fk, const MatMulDims& g, KsplitPlan* p) {
    if (const char* e = std::getenv("DSC_MM_KSPLIT"))
        if (e[0] == '0') return false;
    if (!(fk.sum_chunks || g.chunks == 1) || fk.colsum_out >= 0 || fk.out_slice_width || fk.pair.on || fk.dgrad.on || fk.cfwd.on) return false;
    if (g.k < 512 || g.k > 2048 || g.m < 64 || g.n < 32 || g.n > 256) return false;
    {
        // both operands plain arrays, A's k along memory (16-byte pieces): a transposed or generated A would be
        // fetched a word at a time by every one of the block's column workgroups
        const dsc_kernel_desc& d = fk.main.raw();
        int64_t ab = 0, ac[DSC_MAX_DIM] = {0};
        if (fk.inputs.size() < 2 || fk.inputs[0].buffer < 0 || fk.inputs[1].buffer < 0 || d.inputs[0].out_shape.rank != 3 || !affine_form(d.inputs[0], &ab, ac) ||
            ac[2] != 1 || ab % 4 != 0 || ac[1] % 4 != 0 || (g.batch > 1 && ac[0] % 4 != 0) || g.k % 4 != 0)
            return false;
    }
    const int64_t bm = (g.m + 15) / 16;
    // columns per workgroup: the widest block that still leaves about one workgroup per compute unit
    int best = 0;
    for (int ntb : {4, 2, 1}) {
        if (16 * ntb > (g.n + 15) / 16 * 16) continue;  // no block wider than the product
        const int64_t wgs = bm * ((g.n + 16 * ntb - 1) / (16 * ntb)) * g.batch;
        if (wgs >= 192 && wgs <= 1024) { best = ntb; break; }
    }
    if (!best) return false;
    // the MFMA template's tiles must be few for this to pay: otherwise its reuse of operands through LDS wins
    if (((g.m + 63) / 64) * ((g.n + 63) / 64) * g.batch >= 128) return false;
    p->ntb = best;
    // (sixteen waves, one batch of loads each, measured the same as eight with two: 1000 x 128 over k = 784 8.6 us
    // either way -- the 38 MB the 252 blocks pull out of L2 between them is what bounds it, not the round trips)
    p->waves = 8;
    p->blocks_m = bm;
    p->blocks_n = (g.n + 16 * best - 1) / (16 * best);
    return true;
}
bool ksplit_kernel_applies(const FusedKernel& fk, const MatMulDims& g) {
    KsplitPlan p;
    return ksplit_plan(fk, g, &p);
}

string gen_matmul_ksplit(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const MatMulDims g = matmul_dims(d);
    KsplitPlan p;
    if (!ksplit_plan(fk, g, &p)) return "matmul k-split: shape does not apply";
    const bool rows = d.output_mode == DSC_MATMUL_ROWS;
    const int64_t batch_stride = rows ? g.n : g.m * g.n, row_stride = rows ? g.batch * g.n : g.n;
    const int NTB = p.ntb, W = p.waves;
    const int64_t kw = ((g.k + W - 1) / W + 15) / 16 * 16;  // k per wave, whole blocks of 16
    const int64_t nblk = kw / 16;
    const int U = (int)std::min<int64_t>(nblk, NTB >= 4 ? 3 : 4);  // blocks of 16 k requested together

    const string la = em.load_view(fk.inputs[0], d.inputs[0], {"cb", "cm", "ck"});
    em.funcs << "DSC_INLINE float load_a(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la << ";\n}\n";
    const string lb = em.load_view(fk.inputs[1], d.inputs[1], {"cb", "ck", "cn"});
    em.funcs << "DSC_INLINE float load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";
    // A in 16-byte pieces where k runs along memory
    int64_t ab = 0, ac[DSC_MAX_DIM] = {0};
    const bool a_vec = fk.inputs[0].buffer >= 0 && d.inputs[0].out_shape.rank == 3 && affine_form(d.inputs[0], &ab, ac) && ac[2] == 1 && ab % 4 == 0 &&
                       ac[1] % 4 == 0 && (g.batch == 1 || ac[0] % 4 == 0) && g.k % 4 == 0;
    int n_out = 1;
    if (fk.has_epilogue) {
        const dsc_kernel_desc& pe = fk.epilogue.raw();
        n_out = pe.n_outputs;
        std::ostringstream body;
        std::map<int, string> ov;
        ov[fk.epilogue_product_input] = "product";
        em.emit_pe(body, pe, fk.epilogue_inputs, "gid", "e", ov);
        for (int o = 0; o < pe.n_outputs; ++o) body << "    result[" << o << "] = et" << pe.outputs[o] << ";\n";
        em.funcs << "DSC_INLINE void mm_epilogue(float product, int gid, float* result, " << em.params_decl() << ") {\n" << body.str() << "}\n";
    }
    std::ostringstream k;
    k << "typedef float ks_float4 __attribute__((ext_vector_type(4)));\n";
    k << "extern \"C\" __global__ __launch_bounds__(" << 64 * W << ") void " << entry_name(fk) << "(" << em.kernel_params_decl() << ") {\n";
    k << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    k << "    __shared__ float red[" << W << "][" << NTB * 256 << "];\n";
    // Consecutive workgroup ids go to consecutive XCDs: the column blocks of a row block (which read the same rows of
    // A) get ids 8 apart, so that they share one L2 (measured for 1000x128x1568: 26.8 MB fetched from memory per launch
    // with neighbouring ids, for 7.1 MB of operands).
    const int64_t ks_total = p.blocks_n * p.blocks_m * g.batch, ks_per_xcd = (ks_total + 7) / 8;
    k << "    const int ks_block = (int)(blockIdx.x & 7u) * " << S(ks_per_xcd) << " + (int)(blockIdx.x >> 3);\n";
    k << "    if (ks_block >= " << S(ks_total) << ") return;\n";
    k << "    const int bn = ks_block % " << S(p.blocks_n) << ", bm = (ks_block / " << S(p.blocks_n) << ") % " << S(p.blocks_m) << ", cb = ks_block / " << S(p.blocks_n * p.blocks_m) << ";\n";
    k << "    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), li = lane & 15, lk = lane >> 4;\n";
    k << "    const int row = min(bm * 16 + li, " << S(g.m - 1) << ");\n";
    k << "    const int k_begin = wave * " << S(kw) << ", k_end = min(k_begin + " << S(kw) << ", " << S(g.k) << ");\n";
    k << "    ks_float4 acc[" << NTB << "];\n#pragma unroll\n    for (int nt = 0; nt < " << NTB << "; ++nt) acc[nt] = (ks_float4){0.f, 0.f, 0.f, 0.f};\n";
    k << "    for (int k0 = k_begin; k0 < k_end; k0 += " << 16 * U << ") {\n";
    k << "        float fa[" << U << "][4], fb[" << U << "][" << NTB << "][4];\n";
    // a lane's four k of a block: 16 * u + 4 * lk + j.  Out-of-range k repeat a valid element's load and are zeroed
    // after the fence; nothing before the fence consumes a loaded value, so the whole batch is in flight at once.
    k << "#pragma unroll\n        for (int u = 0; u < " << U << "; ++u) {\n            const int kq = k0 + 16 * u + 4 * lk;\n";
    if (a_vec) {
        k << "            { const float4 q = *(const float4*)(b" << fk.inputs[0].buffer << " + " << S(ab) << " + cb * " << S(g.batch == 1 ? 0 : ac[0]) << " + row * " << S(ac[1])
          << " + min(kq, " << S(g.k - 4) << ")); fa[u][0] = q.x; fa[u][1] = q.y; fa[u][2] = q.z; fa[u][3] = q.w; }\n";
    } else {
        k << "#pragma unroll\n            for (int j = 0; j < 4; ++j) fa[u][j] = load_a(cb, row, min(kq + j, " << S(g.k - 1) << "), " << em.params_pass() << ");\n";
    }
    k << "#pragma unroll\n            for (int nt = 0; nt < " << NTB << "; ++nt)\n#pragma unroll\n                for (int j = 0; j < 4; ++j)\n";
    k << "                    fb[u][nt][j] = load_b(cb, min(kq + j, " << S(g.k - 1) << "), min((bn * " << NTB << " + nt) * 16 + li, " << S(g.n - 1) << "), " << em.params_pass() << ");\n";
    k << "        }\n        __builtin_amdgcn_sched_barrier(0);\n";
    k << "#pragma unroll\n        for (int u = 0; u < " << U << "; ++u)\n#pragma unroll\n            for (int j = 0; j < 4; ++j) {\n";
    k << "                const bool k_ok = k0 + 16 * u + 4 * lk + j < k_end;\n";
    if (a_vec) k << "                const float a = (k_ok && k0 + 16 * u + 4 * lk <= " << S(g.k - 4) << ") ? fa[u][j] : 0.f;\n";
    else k << "                const float a = k_ok ? fa[u][j] : 0.f;\n";
    k << "#pragma unroll\n                for (int nt = 0; nt < " << NTB << "; ++nt)\n";
    k << "                    acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, k_ok ? fb[u][nt][j] : 0.f, acc[nt], 0, 0, 0);\n            }\n";
    k << "    }\n";
    // the waves' partial blocks meet in LDS; register r of lane l is D[4 * (l / 16) + r][l % 16]
    k << "#pragma unroll\n    for (int nt = 0; nt < " << NTB << "; ++nt)\n#pragma unroll\n        for (int r = 0; r < 4; ++r) red[wave][nt * 256 + r * 64 + lane] = acc[nt][r];\n";
    k << "    __syncthreads();\n";
    k << "    for (int i = threadIdx.x; i < " << NTB * 256 << "; i += " << 64 * W << ") {\n        float sum = red[0][i];\n";
    k << "#pragma unroll\n        for (int w = 1; w < " << W << "; ++w) sum += red[w][i];\n";
    k << "        const int nt = i >> 8, r = (i >> 6) & 3, l = i & 63;\n";
    k << "        const int cm = bm * 16 + 4 * (l >> 4) + r, cn = (bn * " << NTB << " + nt) * 16 + (l & 15);\n";
    k << "        if (cm < " << S(g.m) << " && cn < " << S(g.n) << ") {\n            const int gid = cb * " << S(batch_stride) << " + cm * " << S(row_stride) << " + cn;\n";
    if (fk.has_epilogue) {
        k << "            float res[" << n_out << "];\n            mm_epilogue(sum, gid, res, " << em.params_pass() << ");\n";
        for (int o = 0; o < n_out; ++o) k << "            b" << fk.outputs[o] << "[gid] = res[" << o << "];\n";
    } else {
        k << "            b" << fk.outputs[0] << "[gid] = sum;\n";
    }
    k << "        }\n    }\n}\n";
    const int64_t grid = ks_per_xcd * 8;
    if (grid >= kMaxIndex) return "matmul: grid too large";
    out->grid = (unsigned)grid;
    out->block = (unsigned)(64 * W);
    out->source = k.str();
    char note[200];
    std::snprintf(note, sizeof note, "k split over the %d waves of a workgroup, mfma 16x16x4 on a 16x%d block, operands from memory, %d blocks of 16 k in flight%s",
                  W, 16 * NTB, U, fk.has_epilogue ? " +epilogue" : "");
    out->note = note;
    return "";
}

// Tile configuration, k chunking and grid of the MFMA template for one product.
struct MmPlan {
    MmConfig c;
    int64_t kchunks = 1, chunk_k = 0, grid = 0;
};

bool plan_mfma(const FusedKernel& fk, const MatMulDims& g, MmPlan* plan, bool as_part) {
    const bool split = !fk.sum_chunks && g.chunks > 1;
    MmConfig c = pick_config(g.m, g.n, split ? chunk_k_of(g) : g.k, g.batch * (split ? g.chunks : 1));
    // inside a multi-part launch every part runs four waves: the one- and two-wave choices become 128x32 (narrow
    // outputs) or 64x64 tiles
    if (as_part && c.wm * c.wn < 4) c = g.n <= 32 ? MmConfig{128, 32, 16, 4, 1, 8} : MmConfig{64, 64, 16, 2, 2, 8};
    // k chunking: the reference writes `chunks` partial products of chunk_tiles*16 k each (kernel.rs:436)
    int64_t kchunks = 1, chunk_k = ((g.k + c.bk - 1) / c.bk) * c.bk;
    if (split) {
        const int64_t k_tiles = (g.k + 15) / 16;
        const int64_t chunk_tiles = (k_tiles + g.chunks - 1) / g.chunks;
        chunk_k = chunk_tiles * 16;
        kchunks = g.chunks;
        while (chunk_k % c.bk) c.bk /= 2;
    }
    if (!config_ok(c)) return false;
    plan->c = c;
    plan->kchunks = kchunks;
    plan->chunk_k = chunk_k;
    plan->grid = ((g.m + c.bm - 1) / c.bm) * ((g.n + c.bn - 1) / c.bn) * g.batch * kchunks;
    return true;
}

string gen_matmul(Emitter& em, Generated* out) {
    const FusedKernel& fk = em.fk;
    const dsc_kernel_desc& d = fk.main.raw();
    const MatMulDims g = matmul_dims(d);
    const dsc_view& va = d.inputs[0];
    const dsc_view& vb = d.inputs[1];
    const bool rows = d.output_mode == DSC_MATMUL_ROWS;
    if (fk.colsum_out >= 0 && (rows_kernel_applies(fk, g) || smallk_kernel_applies(fk, g)))
        return "matmul: column sums need the MFMA template or the tall-k kernel";
    if (fk.out_slice_width && (!rows_kernel_applies(fk, g) || fk.dgrad.on || fk.cfwd.on)) return "matmul: only the row-per-thread kernel stores slice-major";
    // (a gradient pair is a short-k kernel whatever else the product's shape would allow)
    if (fk.pair.on) return smallk_kernel_applies(fk, g) && !fk.out_slice_width ? gen_matmul_smallk_pair(em, out) : string("matmul: a gradient pair needs the short-k kernel");
    // (sign bytes are written and read by the MFMA template's 16-byte store path only)
    if ((fk.sign_out >= 0 || fk.epilogue_sign_input >= 0) &&
        (rows_kernel_applies(fk, g) || smallk_kernel_applies(fk, g) || tallk_kernel_applies(fk, g) || dot_kernel_applies(fk, g) || ksplit_kernel_applies(fk, g)))
        return "matmul: sign bytes need the MFMA kernel";
    if (rows_kernel_applies(fk, g)) return gen_matmul_rows(em, out);
    if (smallk_kernel_applies(fk, g)) return gen_matmul_smallk(em, out);
    if (tallk_kernel_applies(fk, g)) return gen_matmul_tallk(em, out);
    if (dot_kernel_applies(fk, g)) return gen_matmul_dot(em, out);
    if (ksplit_kernel_applies(fk, g)) return gen_matmul_ksplit(em, out);
    MmPlan plan;
    if (!plan_mfma(fk, g, &plan, fk.as_part)) return "matmul: invalid tile configuration";
    MmConfig c = plan.c;
    const int64_t kchunks = plan.kchunks, chunk_k = plan.chunk_k;
    if (fk.as_part && 64 * c.wm * c.wn != 256) return "matmul: a part of a multi-part launch runs 256 threads";

    // operand addressing
    int a_mode = 0, b_mode = 0;
    int64_t a_base = 0, a_coef[DSC_MAX_DIM] = {0}, b_base = 0, b_coef[DSC_MAX_DIM] = {0};
    const bool a_aff = fk.inputs[0].buffer >= 0 && affine_form(va, &a_base, a_coef);
    const bool b_aff = fk.inputs[1].buffer >= 0 && affine_form(vb, &b_base, b_coef);
    auto mult4 = [](int64_t x) { return x % 4 == 0; };
    if (a_aff && mult4(a_base) && (g.batch == 1 || mult4(a_coef[0]))) {
        if (a_coef[2] == 1 && mult4(g.k) && mult4(a_coef[1]) && chunk_k % 4 == 0) a_mode = 1;
        else if (a_coef[1] == 1 && mult4(g.m) && mult4(a_coef[2])) a_mode = 2;
    }
    if (b_aff && mult4(b_base) && (g.batch == 1 || mult4(b_coef[0]))) {
        if (b_coef[2] == 1 && mult4(g.n) && mult4(b_coef[1])) b_mode = 1;
        else if (b_coef[1] == 1 && mult4(g.k) && mult4(b_coef[2]) && chunk_k % 4 == 0) b_mode = 2;
    }

    std::ostringstream k;
    k << "#define MM_B " << S(g.batch) << "\n#define MM_M " << S(g.m) << "\n#define MM_N " << S(g.n) << "\n#define MM_K "
      << S(g.k) << "\n";
    k << "#define MM_KCHUNKS " << S(kchunks) << "\n#define MM_CHUNK_K " << S(chunk_k) << "\n";
    // k-tiles straight from memory into LDS (see MM_DIRECT in the template) wherever a product consists of whole tiles.
    // Measured on MI355X with two tile buffers against the pass through registers (TFLOP/s): 1024^3 (64x64x64 tiles)
    // 64.9 -> 78.4, 2048^3 (128x128x16) 92.0 -> 101.2, 2048x4096x1024 101.6 -> 107.2 and 4096x2048x4096 116.5 -> 120.1
    // (256x128x16), 262144x256x256 101.9 -> 103.5, 4096^3 131.9 -> 131.9, 8192^3 138.2 -> 138.6 (256x256x16).  A third
    // buffer (two tiles requested ahead) measured 1-2 % below two.
    // DSC_MM_DIRECT_LDS=0 switches the path off, =2 / =3 choose the number of buffers.
    auto direct_buffers = [&](const MmConfig& t) {
        const char* e = std::getenv("DSC_MM_DIRECT_LDS");
        const int nt = 64 * t.wm * t.wn;
        const int nbuf = !e ? 2 : e[0] == '2' ? 2 : e[0] == '3' ? 3 : 0;
        // every k range whole k-tiles; a tile may reach past M or N (it repeats the last row / the last four columns),
        // as long as the product is at least one piece wide and tall
        // (a descriptor may name more chunks than k has tiles for: the last chunks then start at or past k and the
        // reference writes zero partials for them; this path does not clamp k, so they stay on the register path)
        const bool whole = chunk_k % t.bk == 0 && kchunks * chunk_k == g.k && g.m >= 4 && g.n >= 4;
        const bool even = (t.bm * t.bk / 4) % nt == 0 && (t.bn * t.bk / 4) % nt == 0 && (t.bk & (t.bk - 1)) == 0;
        // (column sums are combined through the one free tile buffer: a 16-byte partial per thread has to fit it)
        // (weight gradients with their bias sums: 1024x1024 grid, layers of 256, 309 -> 318 steps/s)
        const bool sums_fit = fk.colsum_out < 0 || (int64_t)nt * 4 <= (int64_t)(t.bm + t.bn) * t.bk;
        if (nbuf && a_mode && b_mode && sums_fit && whole && even && chunk_k / t.bk >= nbuf &&
            (int64_t)nbuf * (t.bm + t.bn) * t.bk * 4 <= 160 * 1024)
            return nbuf;
        return 0;
    };
    // Without padding two buffers of a 32-deep 256x256 tile are 128 KiB: half the barriers per product.  8192^3
    // 137.9 -> 144.2 TFLOP/s (91.7 % of peak), 4096^3 131.8 -> 135.4, 262144x256x256 101.9 -> 103.6; eight waves on
    // the same tile 142.7, the 256x128 and 128x128 tiles gained nothing from 32-deep steps.
    // (a unit of two 32-deep tiles lost: 262144x256x64 124 us against 117.5, so k ranges under 128 keep 16-deep steps)
    // The smaller tiles gain from 32-deep steps as well: 128x128 on 2048^3 100.6 -> 106-108, 256x128 on 4096x2048x4096
    // 121.7 -> 124.5, 128x64 on 3072^3 97.2 -> 103.4 and on 2048x1024x2048 84.8 -> 92.6.
    if (c.bm * c.bn >= 128 * 64 && c.bk == 16 && chunk_k >= 128 && !std::getenv("DSC_MM_TILE")) {
        MmConfig deep = c;
        deep.bk = 32;
        if (c.bm == 256 && c.bn == 256) deep.group_m = 8;
        if (direct_buffers(deep) == 2) c = deep;
    }
    const int direct = direct_buffers(c);
    k << "#define BM " << c.bm << "\n#define BN " << c.bn << "\n#define BK " << c.bk << "\n#define WAVES_M " << c.wm
      << "\n#define WAVES_N " << c.wn << "\n#define GROUP_M " << c.group_m << "\n";
    k << "#define A_MODE " << a_mode << "\n#define B_MODE " << b_mode << "\n";
    if (a_mode) {
        k << "#define A_PTR b" << fk.inputs[0].buffer << "\n#define A_BASE " << S(a_base) << "\n#define A_SB "
          << S(g.batch == 1 ? 0 : a_coef[0]) << "\n#define A_SM " << S(a_coef[1]) << "\n#define A_SK " << S(a_coef[2]) << "\n";
    } else {
        const string la = em.load_view(fk.inputs[0], va, {"cb", "cm", "ck"});
        em.funcs << "DSC_INLINE float load_a(int cb, int cm, int ck, " << em.params_decl() << ") {\n    return " << la << ";\n}\n";
        k << "#define LOAD_A(b, m, k) load_a(b, m, k, " << em.params_pass() << ")\n";
    }
    if (b_mode) {
        k << "#define B_PTR b" << fk.inputs[1].buffer << "\n#define B_BASE " << S(b_base) << "\n#define B_SB "
          << S(g.batch == 1 ? 0 : b_coef[0]) << "\n#define B_SK " << S(b_coef[1]) << "\n#define B_SN " << S(b_coef[2]) << "\n";
    } else {
        const string lb = em.load_view(fk.inputs[1], vb, {"cb", "ck", "cn"});
        em.funcs << "DSC_INLINE float load_b(int cb, int ck, int cn, " << em.params_decl() << ") {\n    return " << lb << ";\n}\n";
        k << "#define LOAD_B(b, k, n) load_b(b, k, n, " << em.params_pass() << ")\n";
    }
    const int64_t batch_stride = rows ? g.n : g.m * g.n, row_stride = rows ? g.batch * g.n : g.n;
    k << "#define C_CHUNK_STRIDE " << S(g.batch * g.m * g.n) << "\n#define C_BATCH_STRIDE " << S(batch_stride)
      << "\n#define C_ROW_STRIDE " << S(row_stride) << "\n";
    k << "#define MM_PARAMS " << em.kernel_params_decl() << "\n#define MM_ENTRY " << entry_name(fk) << "\n";
    k << "#define MM_AS_PART " << (fk.as_part ? 1 : 0) << "\n#define MM_GRID " << S(plan.grid) << "\n";
    if (fk.colsum_out >= 0) {
        // the column sums are written as float4: n and the row of partials must be 16-byte aligned
        if (b_mode != 1 || g.n % 4 != 0 || (64 * c.wm * c.wn) % (c.bn / 4) != 0) return "matmul: column sums need B contiguous along n";
        k << "#define MM_COLSUM 1\n#define CS_PTR b" << fk.colsum_out << "\n";
    } else {
        k << "#define MM_COLSUM 0\n";
    }

    k << "#define MM_DIRECT " << direct << "\n";

    // results leave through LDS as 16-byte row pieces when the output allows it
    bool vec_store = g.n % 4 == 0 && batch_stride % 4 == 0 && row_stride % 4 == 0 && (g.batch * g.m * g.n) % 4 == 0;
    if (direct) {
        // every wave's corner (eight rows of a block) has to fit the one tile buffer that is free at the end of a unit
        if ((int64_t)c.wm * c.wn * 8 * 40 > (int64_t)(c.bm + c.bn) * c.bk) vec_store = false;
        if (const char* e = std::getenv("DSC_MM_VEC_STORE"))
            if (e[0] == '0') vec_store = false;
    } else {
        const int64_t sa = a_mode == 1 ? c.bm * (c.bk + 4) : c.bk * (c.bm + 8), sb = b_mode == 2 ? c.bn * (c.bk + 4) : c.bk * (c.bn + 8);
        const int64_t per_wave = 32 * 36, waves = (int64_t)c.wm * c.wn;
        const int64_t in_a = std::min(waves, 2 * sa / per_wave);
        if ((waves - in_a) * per_wave > 2 * sb) vec_store = false;
        if (const char* e = std::getenv("DSC_MM_VEC_STORE"))
            if (e[0] == '0') vec_store = false;
    }
    k << "#define MM_VEC_STORE " << (vec_store ? 1 : 0) << "\n";
    bool long_epilogue = false;
    {
        if (fk.has_epilogue) {
            const dsc_kernel_desc& pe = fk.epilogue.raw();
            for (int o = 0; o < pe.n_ops; ++o) {
                const dsc_pe_op& op = pe.ops[o];
                if (op.kind == DSC_PE_UNARY && (op.op == DSC_UN_SIN || op.op == DSC_UN_COS || op.op == DSC_UN_EXP || op.op == DSC_UN_LOG)) long_epilogue = true;
                if (op.kind == DSC_PE_BINARY && op.op == DSC_BIN_POW) long_epilogue = true;
                if (op.kind == DSC_PE_RAND || op.kind == DSC_PE_GATHER) long_epilogue = true;
            }
            if (pe.n_ops > 24 || !fk.virtuals.empty()) long_epilogue = true;
        }
        k << "#define MM_LONG_EPILOGUE " << (long_epilogue ? 1 : 0) << "\n";
    }
    if (fk.has_epilogue) {
        const dsc_kernel_desc& pe = fk.epilogue.raw();
        std::ostringstream body;
        std::map<int, string> ov;
        ov[fk.epilogue_product_input] = "product";
        // the element id as (batch, row, column): what the epilogue reads per column only (a bias) or per row
        // only is then addressed without dividing the id, and is loop-invariant along the other coordinate
        IndexForm form;
        form.valid = true;
        form.names = {"cb", "cm", "cn"};
        form.coefs = {batch_stride, row_stride, 1};
        form.extents = {g.batch, g.m, g.n};
        em.emit_pe(body, pe, fk.epilogue_inputs, "gid", "e", ov, &form);
        for (int o = 0; o < pe.n_outputs; ++o) body << "    result[" << o << "] = et" << pe.outputs[o] << ";\n";
        em.funcs << "DSC_INLINE void mm_epilogue(float product, int gid, int cb, int cm, int cn, float* result, " << em.params_decl() << ") {\n"
                 << body.str() << "}\n";
        std::ostringstream one, four;
        one << "DSC_INLINE void mm_store(float product, int gid, int cb, int cm, int cn, " << em.params_decl() << ") {\n";
        one << "    float res[" << pe.n_outputs << "];\n    mm_epilogue(product, gid, cb, cm, cn, res, " << em.params_pass() << ");\n";
        for (int o = 0; o < pe.n_outputs; ++o) one << "    b" << fk.outputs[o] << "[gid] = res[" << o << "];\n";
        one << "}\n";
        four << "DSC_INLINE void mm_store4(float4 p, int gid, int cb, int cm, int cn, " << em.params_decl() << ") {\n";
        four << "    const float pv[4] = {p.x, p.y, p.z, p.w};\n    float res[4][" << pe.n_outputs << "];\n";
        four << "#pragma unroll\n    for (int j = 0; j < 4; ++j) mm_epilogue(pv[j], gid + j, cb, cm, cn + j, res[j], " << em.params_pass() << ");\n";
        for (int o = 0; o < pe.n_outputs; ++o)
            four << "    *(float4*)(b" << fk.outputs[o] << " + gid) = make_float4(res[0][" << o << "], res[1][" << o << "], res[2][" << o
                 << "], res[3][" << o << "]);\n";
        const string sign_store = fk.sign_out < 0 ? string() :
            "    ((unsigned char*)b" + to_string(fk.sign_out) + ")[gid >> 2] = (unsigned char)((res[0][" + to_string(fk.sign_source) + "] > 0.f ? 1 : 0) | (res[1][" +
            to_string(fk.sign_source) + "] > 0.f ? 2 : 0) | (res[2][" + to_string(fk.sign_source) + "] > 0.f ? 4 : 0) | (res[3][" + to_string(fk.sign_source) + "] > 0.f ? 8 : 0));\n";
        four << sign_store;
        four << "}\n";
        em.funcs << one.str() << four.str();
        k << "#define MM_STORE(v, idx, b, m, n) mm_store(v, idx, b, m, n, " << em.params_pass() << ")\n";
        k << "#define MM_STORE4(v, idx, b, m, n) mm_store4(v, idx, b, m, n, " << em.params_pass() << ")\n";
        if ((fk.sign_out >= 0 || fk.epilogue_sign_input >= 0) && !(direct && vec_store && !long_epilogue && g.n % 4 == 0))
            return "matmul: sign bytes need the 16-byte store path over whole tiles";
        // Operands of the epilogue that the 16-byte store path can request ahead of the staging rounds (each round's
        // own load would wait on vmcnt(0), i.e. also for the previous round's store to be acknowledged): a
        // per-column operand (a bias: the view reads element base + column) once per block column, a per-element
        // operand (an activation the gradient is masked with: an identity view) one block ahead.
        std::vector<int> pre_col, pre_elem;
        std::vector<int64_t> pre_col_base;
        if (direct && vec_store && !long_epilogue) {
            for (int i = 0; i < pe.n_inputs; ++i) {
                if (i == fk.epilogue_product_input || fk.epilogue_inputs[i].buffer < 0) continue;
                const dsc_view& v = pe.inputs[i];
                int loads = 0;
                for (int o = 0; o < pe.n_ops; ++o)
                    if (pe.ops[o].kind == DSC_PE_LOAD && pe.ops[o].input_index == i) ++loads;
                    else if (pe.ops[o].kind == DSC_PE_GATHER && pe.ops[o].input_index == i) loads = -100;
                if (loads < 1) continue;
                int64_t base = 0, coef[DSC_MAX_DIM];
                if (is_identity(v) && element_count(v.out_shape) == g.batch * g.m * g.n) {
                    if (pre_elem.size() < 2) pre_elem.push_back(i);
                    continue;
                }
                if (i == fk.epilogue_sign_input) return "matmul: the sign bytes stand for an operand read element for element";
                const int last = v.out_shape.rank - 1;
                if (last < 0 || !affine_form(v, &base, coef) || v.out_shape.dims[last] != g.n || coef[last] != 1 || base % 4 != 0) continue;
                bool column_only = element_count(v.out_shape) == g.batch * g.m * g.n;
                for (int ax = 0; ax < last; ++ax)
                    if (v.out_shape.dims[ax] > 1 && coef[ax] != 0) column_only = false;
                if (column_only && pre_col.size() < 2) {
                    pre_col.push_back(i);
                    pre_col_base.push_back(base);
                }
            }
        }
        if (!pre_col.empty() || !pre_elem.empty()) {
            std::ostringstream pb, fn;
            std::map<int, string> pov;
            pov[fk.epilogue_product_input] = "product";
            string scalars, scalar_args[4];
            for (size_t q = 0; q < pre_col.size(); ++q) {
                pov[pre_col[q]] = "pc" + to_string(q);
                scalars += "float pc" + to_string(q) + ", ";
            }
            for (size_t q = 0; q < pre_elem.size(); ++q) {
                pov[pre_elem[q]] = "pe" + to_string(q);
                scalars += "float pe" + to_string(q) + ", ";
            }
            em.emit_pe(pb, pe, fk.epilogue_inputs, "gid", "e", pov, &form);
            for (int o = 0; o < pe.n_outputs; ++o) pb << "    result[" << o << "] = et" << pe.outputs[o] << ";\n";
            em.funcs << "DSC_INLINE void mm_epilogue_pre(float product, int gid, int cb, int cm, int cn, float* result, " << scalars << em.params_decl() << ") {\n"
                     << pb.str() << "}\n";
            fn << "DSC_INLINE void mm_store4_pre(float4 p, int gid, int cb, int cm, int cn, const float4* colv, const float4* elv, " << em.params_decl() << ") {\n";
            fn << "    const float pv[4] = {p.x, p.y, p.z, p.w};\n    float res[4][" << pe.n_outputs << "];\n";
            for (size_t q = 0; q < pre_col.size(); ++q) fn << "    const float c" << q << "[4] = {colv[" << q << "].x, colv[" << q << "].y, colv[" << q << "].z, colv[" << q << "].w};\n";
            for (size_t q = 0; q < pre_elem.size(); ++q) {
                if (pre_elem[q] == fk.epilogue_sign_input)  // a byte of four sign bits: the selects see +1 or -1
                    fn << "    const uint sb" << q << " = F2U(elv[" << q << "].x);\n    const float e" << q << "[4] = {(sb" << q << " & 1u) ? 1.f : -1.f, (sb" << q << " & 2u) ? 1.f : -1.f, (sb" << q
                       << " & 4u) ? 1.f : -1.f, (sb" << q << " & 8u) ? 1.f : -1.f};\n";
                else
                    fn << "    const float e" << q << "[4] = {elv[" << q << "].x, elv[" << q << "].y, elv[" << q << "].z, elv[" << q << "].w};\n";
            }
            fn << "#pragma unroll\n    for (int j = 0; j < 4; ++j) mm_epilogue_pre(pv[j], gid + j, cb, cm, cn + j, res[j], ";
            for (size_t q = 0; q < pre_col.size(); ++q) fn << "c" << q << "[j], ";
            for (size_t q = 0; q < pre_elem.size(); ++q) fn << "e" << q << "[j], ";
            fn << em.params_pass() << ");\n";
            for (int o = 0; o < pe.n_outputs; ++o)
                fn << "    *(float4*)(b" << fk.outputs[o] << " + gid) = make_float4(res[0][" << o << "], res[1][" << o << "], res[2][" << o
                   << "], res[3][" << o << "]);\n";
            fn << sign_store;
            fn << "}\n";
            em.funcs << fn.str();
            k << "#define MM_NPRE_COL " << pre_col.size() << "\n#define MM_NPRE_ELEM " << pre_elem.size() << "\n";
            k << "#define MM_LOAD_COL4(dst, cn) {";
            for (size_t q = 0; q < pre_col.size(); ++q)
                k << " (dst)[" << q << "] = *(const float4*)(b" << fk.epilogue_inputs[pre_col[q]].buffer << " + " << S(pre_col_base[q]) << " + (cn));";
            k << " }\n#define MM_LOAD_ELEM4(dst, gid) {";
            bool all_signs = !pre_elem.empty();
            for (size_t q = 0; q < pre_elem.size(); ++q) {
                if (pre_elem[q] == fk.epilogue_sign_input)
                    k << " (dst)[" << q << "].x = U2F((uint)((const unsigned char*)b" << fk.epilogue_inputs[pre_elem[q]].buffer << ")[(gid) >> 2]);";
                else {
                    k << " (dst)[" << q << "] = *(const float4*)(b" << fk.epilogue_inputs[pre_elem[q]].buffer << " + (gid));";
                    all_signs = false;
                }
            }
            // (a byte per round: all of a unit's rounds are requested before the first)
            k << " }\n#define MM_PRE_ALL " << (all_signs ? 1 : 0) << "\n";
            k << "#define MM_STORE4P(v, idx, b, m, n, colv, elv) mm_store4_pre(v, idx, b, m, n, colv, elv, " << em.params_pass() << ")\n";
        } else {
            k << "#define MM_NPRE_COL 0\n#define MM_NPRE_ELEM 0\n#define MM_PRE_ALL 0\n";
            if (fk.epilogue_sign_input >= 0) return "matmul: the sign bytes' operand is not requested ahead";
        }
    } else {
        k << "#define MM_STORE(v, idx, b, m, n) b" << fk.outputs[0] << "[idx] = (v)\n";
        k << "#define MM_STORE4(v, idx, b, m, n) *(float4*)(b" << fk.outputs[0] << " + (idx)) = (v)\n";
        k << "#define MM_NPRE_COL 0\n#define MM_NPRE_ELEM 0\n#define MM_PRE_ALL 0\n";
    }
    k << kMatmulMfmaSource;

    const int64_t grid = plan.grid;
    if (grid >= kMaxIndex) return "matmul: grid too large";
    out->grid = (unsigned)grid;
    out->block = 64 * c.wm * c.wn;
    out->source = k.str();
    {
        const char* e = std::getenv("DSC_MM_PERSISTENT");
        out->persistent_ok = !(e && e[0] == '0') && !fk.as_part && grid > 256 && chunk_k / c.bk <= 128;
    }
    char note[224];
    std::snprintf(note, sizeof note, "mfma 32x32x2 tile %dx%dx%d waves %dx%d A%d B%d chunks %lld%s%s%s%s", c.bm, c.bn, c.bk, c.wm, c.wn,
                  a_mode, b_mode, (long long)kchunks, fk.has_epilogue ? " +epilogue" : "", fk.colsum_out >= 0 ? " +column sums of B" : "",
                  out->persistent_ok ? " persistent" : "", direct == 3 ? " tiles straight into LDS x3" : direct == 2 ? " tiles straight into LDS x2" : "");
    out->note = note;
    if (fk.sign_out >= 0) out->note += ", writes its output's sign bytes";
    if (fk.epilogue_sign_input >= 0) out->note += ", masks by sign bytes";
    return "";
}

// Algorithmic bytes and flops of one launch (see Generated).
void count_work(const FusedKernel& fk, Generated* g) {
    const dsc_kernel_desc& d = fk.main.raw();
    std::vector<double> touched(fk.n_buffers, 0.0), extent(fk.n_buffers, 0.0);
    auto read = [&](const Source& s, const dsc_view& v, double elements) {
        if (s.buffer < 0) return;
        touched[s.buffer] += elements;
        extent[s.buffer] = std::max(extent[s.buffer], (double)element_count(v.in_shape));
    };
    auto read_desc = [&](const dsc_kernel_desc& k, const std::vector<Source>& srcs, int skip) {
        for (int i = 0; i < k.n_inputs && i < (int)srcs.size(); ++i) {
            if (i == skip) continue;
            double elements = (double)element_count(k.inputs[i].out_shape);
            if (k.kind == DSC_KERNEL_PER_ELEMENT)
                for (int o = 0; o < k.n_ops; ++o)
                    if (k.ops[o].kind == DSC_PE_GATHER && k.ops[o].input_index == i) elements = (double)element_count(k.ops[o].gather_shape);
            read(srcs[i], k.inputs[i], elements);
        }
    };
    if (fk.row_stages.empty()) read_desc(d, fk.inputs, -1);
    for (auto& st : fk.row_stages) read_desc(st.k.raw(), st.inputs, -1);
    for (auto& v : fk.virtuals) read_desc(v.pe.raw(), v.inputs, -1);
    if (fk.has_epilogue) read_desc(fk.epilogue.raw(), fk.epilogue_inputs, fk.epilogue_product_input);
    if (fk.pool.on && fk.pool.has_epilogue) read_desc(fk.pool.epilogue.raw(), fk.pool.epilogue_inputs, fk.pool.epilogue_product_input);
    // the convolution kernel reads the image itself, not the window copy its MatMul descriptor speaks of
    if (fk.cfwd.on && fk.inputs[0].buffer >= 0)
        touched[fk.inputs[0].buffer] = extent[fk.inputs[0].buffer] = (double)(fk.cfwd.img * fk.cfwd.h * fk.cfwd.w * fk.cfwd.g * fk.cfwd.c);
    double elements = 0;
    for (int i = 0; i < fk.n_buffers; ++i)
        if (!fk.buffer_is_output[i]) elements += std::min(touched[i], extent[i]);
    double out_each = (double)element_count(d.shape);
    if (d.kind == DSC_KERNEL_MATMUL) {
        const MatMulDims m = matmul_dims(d);
        out_each = (double)(m.batch * m.m * m.n) * (double)(fk.sum_chunks ? 1 : m.chunks);
        g->algo_flops = 2.0 * (double)m.batch * (double)m.m * (double)m.n * (double)m.k;
    }
    if (fk.dgrad.on && fk.dgrad.wgrad_only) {
        // dC and the image in (both counted above: dC through its view, the image through the im2col view, capped at
        // its size), one partial product and one row of column sums per image set out
        const FusedKernel::ConvDgrad& c = fk.dgrad;
        const MatMulDims m = matmul_dims(d);
        out_each = 0;
        elements += (double)(c.chunks * c.bands) * (double)c.g * ((double)(c.fh * c.fw * c.c) * (double)m.n + (c.bias ? (double)m.n : 0.0));
        g->algo_flops = 2.0 * (double)c.g * (double)(c.fh * c.fw * c.c) * (double)m.n * (double)(c.img * c.oh * c.ow);
    } else if (fk.dgrad.on) {
        const FusedKernel::ConvDgrad& c = fk.dgrad;
        const MatMulDims m = matmul_dims(d);
        const double ph = (double)(c.oh + c.fh - 1), pw = (double)(c.ow + c.fw - 1);
        out_each = (double)c.img * (ph - 2.0 * c.pad_h) * (pw - 2.0 * c.pad_w) * (double)(c.g * c.c);
        g->algo_flops = 2.0 * (double)c.g * (double)c.img * ph * pw * (double)(c.fh * c.fw * m.k) * (double)c.c;
        if (c.wgrad) {
            // the image is read as well; the filter gradient's flops are those of the MatMul it stands for
            // (k = images x output pixels), its partials and column sums are written once per image set
            elements += out_each;  // the image has the size of its gradient
            g->algo_flops += 2.0 * (double)c.g * (double)(c.fh * c.fw * c.c) * (double)m.k * (double)(c.img * c.oh * c.ow);
            elements += (double)c.chunks * (double)c.g * ((double)(c.fh * c.fw * c.c) * (double)m.k + (c.bias ? (double)m.k : 0.0));
            elements -= out_each * (double)(fk.outputs.size() - 1);  // only the first output has the image's size
        }
    }
    if (fk.dgrad.on && fk.dgrad.pm.on) {
        // dC was counted through its view at the convolution's output size: what is read is the pooled gradient (a
        // quarter of that) and one word per window and four channels
        const FusedKernel::ConvDgrad& c = fk.dgrad;
        const MatMulDims m = matmul_dims(d);
        const double dc = (double)c.img * (double)c.oh * (double)c.ow * (double)c.g * (double)(c.wgrad_only ? m.n : m.k);
        elements -= dc * (1.0 - 0.25 - 1.0 / 16.0);
    }
    if (fk.pool.on) {
        // the pooled array and what its consumer writes have a quarter of the convolution's elements
        const double extra = (double)((fk.pool.has_epilogue ? fk.pool.epilogue.raw().n_outputs : 0) + (fk.pool.store_pooled ? 1 : 0));
        elements -= out_each * extra * 0.75;
        // one word per window and four channels in place of the source array
        if (fk.pool.masks) elements -= out_each * (1.0 - 1.0 / 16.0);
    }
    if (d.kind == DSC_KERNEL_SCATTER_ADD)  // read-modify-write of the entries that receive a value
        out_each = 2.0 * std::min((double)element_count(d.shape), (double)element_count(d.inputs[0].out_shape));
    if (fk.row_stages.empty()) elements += out_each * (double)fk.outputs.size();
    // a byte per four elements written beside the activation / read in place of it
    if (fk.sign_out >= 0) elements -= out_each * (15.0 / 16.0);
    if (fk.epilogue_sign_input >= 0) elements -= out_each * (15.0 / 16.0);
    if (fk.pair.on) {
        // the last output is the weight gradient's partials, and its flops are those of the MatMul it stands for
        const MatMulDims m = matmul_dims(d);
        elements += (double)(fk.pair.chunks * m.n * m.k) - out_each;
        g->algo_flops *= 2.0;
    }
    for (auto& st : fk.row_stages) {
        for (int o : st.outputs)
            if (o >= 0) elements += (double)element_count(st.k.raw().shape);
        if (st.store_a >= 0) elements += (double)element_count(st.k.raw().inputs[0].out_shape);
    }
    if (fk.row_tail.on) {
        const MatMulDims tg = matmul_dims(fk.row_tail.mm.raw());
        elements += (double)(tg.k * tg.n) + (double)(tg.m * tg.n) * (double)fk.row_tail.outputs.size();
        g->algo_flops += 2.0 * (double)tg.m * (double)tg.n * (double)tg.k;
    }
    g->algo_bytes = 4.0 * elements;
}

}  // namespace

bool tallk_shape(const MatMulDims& g) { return tallk_shape_impl(g); }

bool grad_pair_shapes(const FusedKernel& s, const FusedKernel& t, int64_t* chunk_rows, int64_t* chunks) {
    const dsc_kernel_desc& sd = s.main.raw();
    const dsc_kernel_desc& td = t.main.raw();
    if (sd.kind != DSC_KERNEL_MATMUL || td.kind != DSC_KERNEL_MATMUL || sd.output_mode != DSC_MATMUL_BATCHES || td.output_mode != DSC_MATMUL_BATCHES) return false;
    auto plain = [](const FusedKernel& f) {
        return f.virtuals.empty() && f.colsum_out < 0 && !f.dgrad.on && !f.cfwd.on && !f.pool.on && !f.out_slice_width && f.parts.empty() &&
               f.row_stages.empty() && !f.pair.on && f.inputs.size() >= 2 && f.inputs[0].buffer >= 0 && f.inputs[1].buffer >= 0;
    };
    if (!plain(s) || !plain(t) || !s.has_epilogue || t.has_epilogue || t.sum_chunks) return false;
    const MatMulDims gs = matmul_dims(sd), gt = matmul_dims(td);
    if (!smallk_kernel_applies(s, gs) || !tallk_kernel_applies(t, gt)) return false;
    if (gs.batch != 1 || gt.batch != 1 || gs.k > 4 || gs.n > 1024 || 256 % (gs.n / 4) != 0) return false;
    if (gt.m != gs.n || gt.n != gs.k || gt.k != gs.m) return false;
    int64_t base = 0, coef[DSC_MAX_DIM] = {0};
    // dY [m, k] in order, as the short-k product's A and as the tall-k product's B
    if (!affine_form(sd.inputs[0], &base, coef) || base != 0 || coef[1] != gs.k || coef[2] != 1) return false;
    if (!affine_form(td.inputs[1], &base, coef) || base != 0 || coef[1] != gs.k || coef[2] != 1) return false;
    // X [m, n] in order, transposed by the tall-k product's view
    if (!affine_form(td.inputs[0], &base, coef) || base != 0 || coef[1] != 1 || coef[2] != gs.n) return false;
    *chunk_rows = chunk_k_of(gt);
    *chunks = gt.chunks;
    return (*chunks - 1) * *chunk_rows < gt.k && *chunks * *chunk_rows >= gt.k;
}
bool ksplit_kernel_shape(const FusedKernel& fk) {
    FusedKernel probe = fk;
    probe.sum_chunks = true;  // the planner asks before it has folded the sum over the reference's chunks in
    return ksplit_kernel_applies(probe, matmul_dims(fk.main.raw()));
}

bool dot_kernel_shape(const MatMulDims& g) {
    const char* e = std::getenv("DSC_MM_DOT");
    return !(e && e[0] == '0') && dot_shape(g);
}

FusedKernel FusedKernel::plain(const dsc_kernel_desc& d) {
    FusedKernel fk;
    fk.main = KernelDesc(d);
    const int n_in = fk.main.raw().n_inputs;
    int n_out = 1;
    if (d.kind == DSC_KERNEL_PER_ELEMENT) n_out = d.n_outputs;
    for (int i = 0; i < n_in; ++i) {
        Source s;
        s.buffer = i;
        fk.inputs.push_back(s);
    }
    for (int o = 0; o < n_out; ++o) fk.outputs.push_back(n_in + o);
    fk.n_buffers = n_in + n_out;
    fk.buffer_is_output.assign(fk.n_buffers, false);
    for (int o : fk.outputs) fk.buffer_is_output[o] = true;
    return fk;
}

std::string FusedKernel::key() const {
    std::string s = main.key();
    auto put_src = [&](const Source& x) {
        s.append(reinterpret_cast<const char*>(&x.buffer), 4);
        s.append(reinterpret_cast<const char*>(&x.virt), 4);
    };
    s += "|I";
    for (auto& x : inputs) put_src(x);
    for (auto& v : virtuals) {
        s += "|V" + v.pe.key();
        s.append(reinterpret_cast<const char*>(&v.out_op), 4);
        for (auto& x : v.inputs) put_src(x);
    }
    if (has_epilogue) {
        s += epilogue_permuted ? "|EP" : "|E";
        if (epilogue_keeps_product) s += "K";
        s += epilogue.key();
        s.append(reinterpret_cast<const char*>(&epilogue_product_input), 4);
        for (auto& x : epilogue_inputs) put_src(x);
    }
    for (auto& st : row_stages) {
        s += "|R" + st.k.key();
        for (auto& x : st.inputs) {
            put_src(x);
            s.append(reinterpret_cast<const char*>(&x.stage), 4);
            s.append(reinterpret_cast<const char*>(&x.stage_out), 4);
        }
        for (int o : st.outputs) s.append(reinterpret_cast<const char*>(&o), 4);
        s.append(reinterpret_cast<const char*>(&st.store_a), 4);
    }
    if (!row_stages.empty()) {
        s.append(reinterpret_cast<const char*>(&row_m), 8);
        s.append(reinterpret_cast<const char*>(&row_n), 8);
    }
    if (row_tail.on) {
        s += "|RT" + row_tail.mm.key();
        put_src(row_tail.b);
        for (int v : {row_tail.x_stage, row_tail.x_stage_out, row_tail.epilogue_product_input, row_tail.epilogue_a_input}) s.append(reinterpret_cast<const char*>(&v), 4);
        if (row_tail.has_epilogue) {
            s += "E" + row_tail.epilogue.key();
            for (auto& x : row_tail.epilogue_inputs) put_src(x);
        }
        for (int o : row_tail.outputs) s.append(reinterpret_cast<const char*>(&o), 4);
    }
    if (dgrad.on) {
        s += "|D";
        for (int64_t v : {dgrad.img, dgrad.oh, dgrad.ow, dgrad.g, dgrad.fh, dgrad.fw, dgrad.c, dgrad.pad_h, dgrad.pad_w, (int64_t)dgrad.rows_first,
                          (int64_t)dgrad.wgrad, (int64_t)dgrad.bias, dgrad.chunks})
            s.append(reinterpret_cast<const char*>(&v), 8);
        if (dgrad.pm.on) {
            s += "|PM";
            put_src(dgrad.pm.masks);
            s.append(reinterpret_cast<const char*>(&dgrad.pm.leak_bits), 4);
        }
    }
    if (cfwd.on) {
        s += "|CF";
        for (int64_t v : {cfwd.img, cfwd.h, cfwd.w, cfwd.g, cfwd.c, cfwd.fh, cfwd.fw, cfwd.oh, cfwd.ow, cfwd.pad_h, cfwd.pad_w})
            s.append(reinterpret_cast<const char*>(&v), 8);
    }
    if (pool.on) {
        s += "|PL";
        s.append(reinterpret_cast<const char*>(&pool.source), 4);
        s += pool.store_pooled ? "S" : "-";
        s += pool.masks ? "M" : "-";
        if (pool.has_epilogue) {
            s += "E" + pool.epilogue.key();
            s.append(reinterpret_cast<const char*>(&pool.epilogue_product_input), 4);
            for (auto& x : pool.epilogue_inputs) put_src(x);
        }
    }
    if (shared_scatter) s += "|SS";
    if (binned_pairs) s += "|BP";
    if (chain_group) s += "|CG";
    if (dgrad.wgrad_only) s += "|WO" + to_string((long long)dgrad.bands);
    if (binned_stage) s += "|BS" + to_string(binned_stage) + "," + to_string((long long)binned_table) + "," + to_string((long long)binned_total);
    for (size_t i = 0; i < parts.size(); ++i) {
        s += "|P{" + parts[i].key() + "}";
        for (int j : part_params[i]) s.append(reinterpret_cast<const char*>(&j), 4);
    }
    s += sum_chunks ? "|S1" : "|S0";
    if (out_slice_width) s += "|OSW" + to_string((long long)out_slice_width);
    if (row_width) s += "|RW" + to_string((long long)row_width);
    if (as_part) s += "|AP";
    if (colsum_out >= 0) s += "|CS" + to_string(colsum_out);
    if (sign_out >= 0) s += "|SG" + to_string(sign_out) + "," + to_string(sign_source);
    if (epilogue_sign_input >= 0) s += "|SI" + to_string(epilogue_sign_input);
    if (pair.on) s += "|GP" + to_string(pair.x_buffer) + "," + to_string(pair.out) + "," + to_string((long long)pair.chunk_rows) + "," + to_string((long long)pair.chunks);
    s += "|O";
    for (int o : outputs) s.append(reinterpret_cast<const char*>(&o), 4);
    s.append(reinterpret_cast<const char*>(&n_buffers), 4);
    if (const char* env = std::getenv("DSC_MM_TILE"))
        if (main.raw().kind == DSC_KERNEL_MATMUL) s += string("|T") + env;
    for (const char* name : {"DSC_MM_SMALLK", "DSC_MM_VEC_STORE", "DSC_MM_PERSISTENT", "DSC_MM_DEEP_K", "DSC_MM_DIRECT_LDS", "DSC_MM_ROWS", "DSC_MM_DOT", "DSC_ROWS_MFMA", "DSC_MM_TALLK", "DSC_MM_KSPLIT"})
        if (const char* env = std::getenv(name))
            if (main.raw().kind == DSC_KERNEL_MATMUL) s += string("|") + name + env;
    if (dgrad.on && dgrad.wgrad && !dgrad.wgrad_only)
        if (const char* env = std::getenv("DSC_CONV_BWD_LOADERS")) s += string("|LW") + env;
    return s;
}

namespace {
string generate_multi(const FusedKernel& fk, Generated* out);
string generate_scatter_chain(const FusedKernel& fk, Generated* out);
// threads of a first-stage workgroup; measured on the hash grid's eleven binned levels: 1024 88.8 us, 512 82.0, 256 85.9
int scatter_bin_threads() { return 512; }
string generate_scatter_bin(const FusedKernel& fk, Generated* out);
string generate_scatter_sum(const FusedKernel& fk, Generated* out);
string generate_chain_group(const FusedKernel& fk, Generated* out);
}

bool conv_fwd_fits(const FusedKernel::ConvFwd& c, int64_t n) {
    const int64_t k = c.fh * c.fw * c.c;
    const int64_t lds_bytes = (c.oh + c.fh - 1) * (c.ow + c.fw - 1) * conv_fwd_pitch(c.c) * 4 + (k + 3) / 4 * 256;  // image tile + B fragments
    return lds_bytes <= 60 * 1024 && n <= 16 && k >= 4 && k <= 512 && c.oh * c.ow >= 16;
}

bool conv_dgrad_fits(const FusedKernel::ConvDgrad& c, int64_t k) {
    if (k % 4 != 0 || c.g * c.c > 64 || c.fh * c.fw * k * c.g * c.c > 8192) return false;
    return (dgrad_lds_floats(c, k) + dgrad_pitch(k) + 4) * 4 <= 64 * 1024 && c.oh + c.fh - 1 > 2 * c.pad_h && c.ow + c.fw - 1 > 2 * c.pad_w;
}

bool conv_bwd_fits(const FusedKernel::ConvDgrad& c, int64_t k) { return conv_bwd_fits_impl(c, k); }
bool conv_bwd_loader_waves(const FusedKernel& fk) { return conv_bwd_loader_waves_impl(fk); }

bool can_be_part(const FusedKernel& fk) {
    if (!fk.parts.empty() || fk.binned_stage || fk.chain_group) return false;
    if (fk.dgrad.on && conv_bwd_loader_waves_impl(fk)) return false;  // 512 threads per workgroup
    if (fk.dgrad.on || fk.cfwd.on || !fk.row_stages.empty()) return true;
    if (fk.main.raw().kind != DSC_KERNEL_MATMUL) return true;
    // of the MatMul kernels, the row-per-thread, short-k and tall-k ones run 256 threads addressed by blockIdx.x
    const MatMulDims g = matmul_dims(fk.main.raw());
    if (rows_kernel_applies(fk, g) || smallk_kernel_applies(fk, g) || tallk_kernel_applies(fk, g) || dot_kernel_applies(fk, g)) return true;
    if (ksplit_kernel_applies(fk, g)) return false;  // eight waves per workgroup
    if (fk.colsum_out >= 0) return false;
    // the MFMA template, when its tile choice runs four waves: small products only (large ones want their
    // workgroups persistent and the CU's whole LDS, which a shared launch cannot give them)
    MmPlan plan;
    return plan_mfma(fk, g, &plan, true) && 64 * plan.c.wm * plan.c.wn == 256 && plan.grid <= 1024;
}

static std::string generate_one(const FusedKernel& fk, Generated* out, bool with_prelude);

std::string generate(const FusedKernel& fk, Generated* out) {
    if (fk.chain_group) return generate_chain_group(fk, out);
    if (fk.binned_stage == 1) return generate_scatter_bin(fk, out);
    if (fk.binned_stage == 2) return generate_scatter_sum(fk, out);
    if (!fk.parts.empty() && fk.shared_scatter) return generate_scatter_chain(fk, out);
    if (!fk.parts.empty()) return generate_multi(fk, out);
    return generate_one(fk, out, true);
}

static std::string generate_one(const FusedKernel& fk, Generated* out, bool with_prelude) {
    string err = validate(fk.main.raw());
    if (!err.empty()) return err;
    for (auto& v : fk.virtuals) {
        err = validate(v.pe.raw());
        if (!err.empty()) return "fused producer: " + err;
        const int vk = v.pe.raw().kind;
        if (vk != DSC_KERNEL_PER_ELEMENT && vk != DSC_KERNEL_REDUCE && vk != DSC_KERNEL_UNPAD && vk != DSC_KERNEL_WINDOWS_TO_IMAGE && vk != DSC_KERNEL_MATMUL)
            return "fused producer must be a per-element, reduce, unpad, windows-to-image or short matmul kernel";
        if (vk == DSC_KERNEL_MATMUL && (matmul_dims(v.pe.raw()).chunks != 1 || matmul_dims(v.pe.raw()).k > 4))
            return "fused producer: a matmul evaluated on demand has one chunk of at most four k";
        if ((int)v.inputs.size() != v.pe.raw().n_inputs) return "fused producer: input binding count";
    }
    if (fk.has_epilogue) {
        err = validate(fk.epilogue.raw());
        if (!err.empty()) return "epilogue: " + err;
        const int mk = fk.main.raw().kind;
        if (mk != DSC_KERNEL_MATMUL && mk != DSC_KERNEL_REDUCE && mk != DSC_KERNEL_WINDOWS_TO_IMAGE && mk != DSC_KERNEL_UNPAD)
            return "this kernel kind takes no epilogue";
        if (fk.epilogue_permuted && mk != DSC_KERNEL_REDUCE) return "only a Reduce takes an epilogue through a permuting view";
        if (fk.epilogue_keeps_product && (mk == DSC_KERNEL_MATMUL || fk.epilogue_permuted)) return "this epilogue cannot keep its product";
        if (!fk.pool.on && (int)fk.outputs.size() != fk.epilogue.raw().n_outputs + (fk.epilogue_keeps_product ? 1 : 0) + (fk.pair.on ? 1 : 0) + (fk.sign_out >= 0 ? 1 : 0)) return "epilogue output count";
    }
    if (fk.pool.on) {
        if (!fk.cfwd.on) return "pooling rides on the convolution-forward kernel only";
        if (fk.pool.has_epilogue) {
            err = validate(fk.pool.epilogue.raw());
            if (!err.empty()) return "pool consumer: " + err;
            if ((int)fk.pool.epilogue_inputs.size() != fk.pool.epilogue.raw().n_inputs) return "pool consumer: input binding count";
        }
    }
    for (auto& st : fk.row_stages) {
        err = validate(st.k.raw());
        if (!err.empty()) return "row stage: " + err;
        if ((int)st.inputs.size() != st.k.raw().n_inputs) return "row stage: input binding count";
        const int n_out = st.k.raw().kind == DSC_KERNEL_PER_ELEMENT ? st.k.raw().n_outputs : 1;
        if ((int)st.outputs.size() != n_out) return "row stage: output binding count";
    }
    if (fk.row_tail.on) {
        err = validate(fk.row_tail.mm.raw());
        if (!err.empty()) return "row tail: " + err;
        if (fk.row_tail.has_epilogue) {
            err = validate(fk.row_tail.epilogue.raw());
            if (!err.empty()) return "row tail consumer: " + err;
            if ((int)fk.row_tail.epilogue_inputs.size() != fk.row_tail.epilogue.raw().n_inputs) return "row tail consumer: input binding count";
        }
    }
    if (fk.row_stages.empty() && (int)fk.inputs.size() != fk.main.raw().n_inputs + (fk.dgrad.on && fk.dgrad.wgrad ? 1 : 0)) return "input binding count";
    if ((int)fk.buffer_is_output.size() != fk.n_buffers) return "buffer table size";
    err = check_sizes(fk);
    if (!err.empty()) return err;

    Emitter em(fk);
    Generated g;
    if (!fk.row_stages.empty()) {
        err = gen_row_fused(em, &g);
    } else if (fk.dgrad.on) {
        if (fk.main.raw().kind != DSC_KERNEL_MATMUL || fk.has_epilogue) return "conv dgrad: needs a plain MatMul";
        err = fk.dgrad.wgrad ? gen_conv_bwd(em, &g) : gen_conv_dgrad(em, &g);
    } else if (fk.cfwd.on) {
        if (fk.main.raw().kind != DSC_KERNEL_MATMUL) return "conv forward: needs a MatMul";
        err = gen_conv_fwd(em, &g);
    } else
    switch (fk.main.raw().kind) {
    case DSC_KERNEL_FILL: err = gen_fill(em, &g); break;
    case DSC_KERNEL_PER_ELEMENT: err = gen_per_element(em, &g); break;
    case DSC_KERNEL_REDUCE: err = gen_reduce(em, &g); break;
    case DSC_KERNEL_MATMUL: err = gen_matmul(em, &g); break;
    case DSC_KERNEL_UNPAD: err = gen_unpad(em, &g); break;
    case DSC_KERNEL_WINDOWS_TO_IMAGE: err = gen_windows_to_image(em, &g); break;
    case DSC_KERNEL_SCATTER_ADD: err = gen_scatter_add(em, &g); break;
    default: err = "unknown kernel kind";
    }
    if (!err.empty()) return err;
    g.source = (with_prelude ? string(kPreludeSource) + "\n" : string()) + em.funcs.str() + "\n" + g.source;
    g.n_buffers = fk.n_buffers;
    g.entry = entry_name(fk);
    count_work(fk, &g);
    *out = g;
    return "";
}

namespace {
// ScatterAdds chained through one accumulator that fits LDS (see FusedKernel::shared_scatter).  1024 threads per
// workgroup, one accumulator copy per workgroup: with tables of tens of kilobytes only one workgroup fits a CU, so
// the waves that hide the value / index loads have to come from inside it.
string generate_scatter_chain(const FusedKernel& fk, Generated* out) {
    const dsc_kernel_desc& first = fk.parts[0].main.raw();
    const int64_t table = element_count(first.shape);
    int64_t total = 0;
    for (auto& part : fk.parts) {
        const dsc_kernel_desc& d = part.main.raw();
        if (d.kind != DSC_KERNEL_SCATTER_ADD || !same_shape(d.shape, first.shape)) return "scatter chain: parts differ";
        total += element_count(d.inputs[0].out_shape);
    }
    if (table * 8 > 144 * 1024) return "scatter chain: accumulator does not fit LDS";
    // Up to one workgroup per CU.  A thread fetches U values of every link before it adds any (one memory round trip
    // per trip, not one per link).
    int64_t nmax = 0;
    for (auto& part : fk.parts) nmax = std::max(nmax, element_count(part.main.raw().inputs[0].out_shape));
    const int U = 2;
    // Every workgroup ends by adding its whole copy to memory, so an accumulator that is large against the values it
    // receives gets fewer workgroups: at least sixteen values per element and workgroup.
    const int64_t wgs = std::max<int64_t>(64, std::min<int64_t>(std::min<int64_t>(256, total / (16 * table)), (nmax + 1024 * U - 1) / (1024 * U)));
    Generated g;
    std::ostringstream src, fetches, adds;
    if (!fk.as_part) src << kPreludeSource << "\n";
    const string block_id = fk.as_part ? "dsc_block" : "blockIdx.x";
    int out_param = -1;
    for (size_t i = 0; i < fk.parts.size(); ++i) {
        const FusedKernel& part = fk.parts[i];
        if ((int)fk.part_params[i].size() != part.n_buffers) return "scatter chain: part parameter count";
        Emitter em(part);
        const int64_t n = element_count(part.main.raw().inputs[0].out_shape);
        std::ostringstream fn;
        fn << "DSC_INLINE void fetch(const uint gid, float* out_value, int* out_at, bool* out_ok, " << em.params_decl() << ") {\n";
        emit_scatter_element(em, fn, "gid", "");
        fn << "    *out_value = value;\n    *out_at = at;\n    *out_ok = ok;\n}\n";
        src << "namespace part" << i << " {\n" << em.funcs.str() << fn.str() << "}  // namespace part" << i << "\n\n";
        for (int u = 0; u < U; ++u) {
            const string id = "p" + to_string(i) + "u" + to_string(u);
            const string gid = "g0 + " + S(u * wgs * 1024) + "u";
            fetches << "        float v" << id << "; int a" << id << "; bool k" << id << ";\n";
            fetches << "        part" << i << "::fetch(min(" << gid << ", " << S(n - 1) << "u), &v" << id << ", &a" << id << ", &k" << id;
            for (int j : fk.part_params[i]) fetches << ", b" << j;
            fetches << ", rand_seed);\n";
            adds << "        if (k" << id << " && " << gid << " < " << S(n) << "u) atomicAdd(&acc[a" << id << "], (double)v" << id << ");\n";
        }
        out_param = fk.part_params[i][part.outputs[0]];
        Generated pg;  // for the work figures only
        if (generate_one(part, &pg, false).empty()) g.algo_bytes += pg.algo_bytes;
    }
    std::ostringstream body;
    body << "    for (uint g0 = " << block_id << " * 1024u + threadIdx.x; g0 < " << S(nmax) << "u; g0 += " << S(wgs * 1024 * U) << "u) {\n"
         << fetches.str() << "        __builtin_amdgcn_sched_barrier(0);\n" << adds.str() << "    }\n";
    Emitter em(fk);
    g.entry = "dsc_scatter_chain_l" + to_string(fk.parts.size()) + "_t" + S(table) + "_n" + S(total);
    if (fk.as_part) {
        src << "DSC_INLINE void part_entry(const uint dsc_block, char* dsc_lds, " << em.kernel_params_decl() << ") {\n";
        src << "    double* const acc = reinterpret_cast<double*>(dsc_lds);\n";
    } else {
        src << "extern \"C\" __global__ __launch_bounds__(1024) void " << g.entry << "(" << em.kernel_params_decl() << ") {\n";
        src << "    __shared__ double acc[" << S(table) << "];\n";
    }
    g.lds_bytes = (size_t)table * 8;
    src << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    src << "    for (int i = threadIdx.x; i < " << S(table) << "; i += 1024) acc[i] = 0.0;\n    __syncthreads();\n";
    src << body.str();
    src << "    __syncthreads();\n";
    src << "    for (int i = threadIdx.x; i < " << S(table) << "; i += 1024) {\n        const float sum = (float)acc[i];\n";
    src << "        if (sum != 0.f) unsafeAtomicAdd(&b" << out_param << "[i], sum);\n    }\n}\n";
    g.source = src.str();
    g.grid = (unsigned)wgs;
    g.block = 1024;
    g.n_buffers = fk.n_buffers;
    g.note = "scatter chain: " + to_string(fk.parts.size()) + " links into one accumulator of " + S(table) +
             " floats kept in LDS per workgroup (as doubles, ds_add_f64), then global_atomic_add_f32";
    *out = g;
    return "";
}

// Stage 1 of the two-launch ScatterAdd chain (FusedKernel::binned_stage): 1024 threads take 8192 values of one link,
// count them per accumulator segment in LDS (the add returns each record's rank inside its segment), turn the
// counts into offsets with one scan, reserve room in every segment's bin with one counter add per segment, order
// the records by segment in LDS and copy them out: consecutive LDS slots of one segment land on consecutive
// addresses, so the stores of a wave fall into a few runs instead of 64 places.
string generate_scatter_bin(const FusedKernel& fk, Generated* out) {
    const dsc_kernel_desc& first = fk.parts[0].main.raw();
    const int64_t table = element_count(first.shape);
    int64_t total = 0;
    for (auto& part : fk.parts) {
        const dsc_kernel_desc& d = part.main.raw();
        if (d.kind != DSC_KERNEL_SCATTER_ADD || !same_shape(d.shape, first.shape)) return "binned scatter: parts differ";
        total += element_count(d.inputs[0].out_shape);
    }
    if (table != fk.binned_table || total != fk.binned_total || fk.outputs.size() != 3) return "binned scatter: geometry differs from the plan";
    const bool pairs = fk.binned_pairs;
    if (pairs)
        for (auto& part : fk.parts)
            if (!scatter_rows_of_two(part.main.raw())) return "binned scatter: a link does not add rows of two";
    const BinnedScatterPlan bp = binned_scatter_plan(table, total, pairs);
    if (bp.nseg > 1024 || bp.nseg * bp.cap >= ((int64_t)1 << 31) || table >= ((int64_t)1 << 31)) return "binned scatter: accumulator too large";
    if (bp.nseg != 256) return "binned scatter: the kernels take 256 segments";
    // 8192 values per workgroup (runs of 16 records per segment on average) on 512 threads: a workgroup waits for
    // the round trip of its reservations, and three of these fit a CU where two of 1024 threads did
    const int NTH = scatter_bin_threads();
    const int U = (pairs ? 4096 : 8192) / NTH;  // records per thread
    const int64_t per_wg = (int64_t)NTH * U;     // records per workgroup
    const int rec = fk.outputs[0], cur = fk.outputs[1], acc = fk.outputs[2];
    Generated g;
    std::ostringstream src, fetches;
    if (!fk.as_part) src << kPreludeSource << "\n";
    const string block_id = fk.as_part ? "dsc_block" : "blockIdx.x";
    int64_t first_wg = 0;
    double rmw = 0;
    for (size_t i = 0; i < fk.parts.size(); ++i) {
        const FusedKernel& part = fk.parts[i];
        if ((int)fk.part_params[i].size() != part.n_buffers) return "binned scatter: part parameter count";
        Emitter em(part);
        const int64_t n = element_count(part.main.raw().inputs[0].out_shape);
        std::ostringstream fn;
        fn << "DSC_INLINE void fetch(const uint gid, float* out_value, int* out_at, bool* out_ok, " << em.params_decl() << ") {\n";
        emit_scatter_element(em, fn, "gid", "");
        fn << "    *out_value = value;\n    *out_at = at;\n    *out_ok = ok;\n}\n";
        src << "namespace part" << i << " {\n" << em.funcs.str() << fn.str() << "}  // namespace part" << i << "\n\n";
        const int64_t nrec = pairs ? n / 2 : n;  // records of this link
        const int64_t wgs = (nrec + per_wg - 1) / per_wg;
        fetches << "    " << (i ? "else " : "") << "if (" << block_id << " < " << S(first_wg + wgs) << "u) {\n";
        fetches << "        const uint g0 = (" << block_id << " - " << S(first_wg) << "u) * " << S(per_wg) << "u + tid;\n";
        for (int u = 0; u < U; ++u) {
            const string r = "min(g0 + " + S(u * NTH) + "u, " + S(nrec - 1) + "u)";
            if (pairs) {
                fetches << "        { int a_second; bool k_second;\n";
                fetches << "        part" << i << "::fetch(2u * " << r << ", &v" << u << ", &a" << u << ", &k" << u;
                for (int j : fk.part_params[i]) fetches << ", b" << j;
                fetches << ", rand_seed);\n";
                fetches << "        part" << i << "::fetch(2u * " << r << " + 1u, &w" << u << ", &a_second, &k_second";
                for (int j : fk.part_params[i]) fetches << ", b" << j;
                fetches << ", rand_seed); }\n";
            } else {
                fetches << "        part" << i << "::fetch(" << r << ", &v" << u << ", &a" << u << ", &k" << u;
                for (int j : fk.part_params[i]) fetches << ", b" << j;
                fetches << ", rand_seed);\n";
            }
            fetches << "        k" << u << " = k" << u << " && g0 + " << S(u * NTH) << "u < " << S(nrec) << "u;\n";
        }
        fetches << "    }\n";
        first_wg += wgs;
        Generated pg;  // for the work figures only
        if (generate_one(part, &pg, false).empty()) g.algo_bytes += pg.algo_bytes;
        rmw += 8.0 * (double)std::min(table, n);
    }
    g.algo_bytes = std::max(0.0, g.algo_bytes - rmw);  // the accumulator's read-modify-write is stage 2's work
    Emitter em(fk);
    g.entry = "dsc_scatter_bin_l" + to_string(fk.parts.size()) + "_t" + S(table) + "_n" + S(total);
    if (fk.as_part) {
        src << "DSC_INLINE void part_entry(const uint dsc_block, char* dsc_lds, " << em.kernel_params_decl() << ") {\n";
        src << "    float2* const stage = reinterpret_cast<float2*>(dsc_lds);\n";
        src << "    uint* const cnt = reinterpret_cast<uint*>(dsc_lds + " << S(per_wg * 8) << ");\n";
        src << "    uint* const lbase = cnt + " << S(bp.nseg) << ";\n    uint* const gbase = lbase + " << S(bp.nseg) << ";\n    uint* const wsum = gbase + " << S(bp.nseg) << ";\n";
        if (pairs) src << "    int* const stage_at = reinterpret_cast<int*>(wsum + 16);\n";
    } else {
        src << "extern \"C\" __global__ __launch_bounds__(" << NTH << ") void " << g.entry << "(" << em.kernel_params_decl() << ") {\n";
        src << "    __shared__ uint cnt[" << S(bp.nseg) << "], lbase[" << S(bp.nseg) << "], gbase[" << S(bp.nseg) << "], wsum[16];\n";
        src << "    __shared__ float2 stage[" << S(per_wg) << "];\n";
        if (pairs) src << "    __shared__ int stage_at[" << S(per_wg) << "];\n";
    }
    g.lds_bytes = (size_t)(per_wg * (pairs ? 12 : 8) + (3 * bp.nseg + 16) * 4);
    src << "    const uint rand_seed = seed_cell ? *seed_cell : seed_value;\n";
    src << "    const uint tid = threadIdx.x;\n";
    src << "    for (uint i = tid; i < " << S(bp.nseg) << "u; i += " << NTH << "u) cnt[i] = 0u;\n    __syncthreads();\n";
    for (int u = 0; u < U; ++u) src << "    float v" << u << " = 0.f, w" << u << " = 0.f; int a" << u << " = 0; bool k" << u << " = false;\n";
    src << fetches.str();
    src << "    __builtin_amdgcn_sched_barrier(0);\n";
    for (int u = 0; u < U; ++u) src << "    const uint r" << u << " = k" << u << " ? atomicAdd(&cnt[(a" << u << " >> 4) & 255], 1u) : 0u;\n";
    src << "    __syncthreads();\n";
    if (NTH < bp.nseg) return "binned scatter: fewer threads than segments";
    src << "    const uint c = tid < " << S(bp.nseg) << "u ? cnt[tid] : 0u;\n";
    src << "    uint incl = c;\n";
    src << "#pragma unroll\n    for (int d = 1; d < 64; d <<= 1) {\n        const uint up = __shfl_up(incl, d);\n        if ((int)(tid & 63u) >= d) incl += up;\n    }\n";
    src << "    if ((tid & 63u) == 63u) wsum[tid >> 6] = incl;\n    __syncthreads();\n";
    src << "    uint before = 0u, filled = 0u;\n";
    src << "#pragma unroll\n    for (uint w = 0; w < " << NTH / 64 << "u; ++w) {\n        const uint s = wsum[w];\n        if (w < (tid >> 6)) before += s;\n        filled += s;\n    }\n";
    src << "    uint* const cursor = reinterpret_cast<uint*>(b" << cur << ");\n";
    src << "    if (tid < " << S(bp.nseg) << "u) {\n        lbase[tid] = before + incl - c;\n        gbase[tid] = c ? atomicAdd(&cursor[tid * 16u], c) : 0u;\n    }\n";
    src << "    __syncthreads();\n";
    if (pairs) {
        // a record is a row: both values in one array, the target of the first in another behind it
        for (int u = 0; u < U; ++u)
            src << "    if (k" << u << ") { const uint at_slot = lbase[(a" << u << " >> 4) & 255] + r" << u << "; stage[at_slot] = make_float2(v" << u << ", w" << u
                << "); stage_at[at_slot] = a" << u << "; }\n";
        src << "    __syncthreads();\n";
        src << "    float2* const records = reinterpret_cast<float2*>(b" << rec << ");\n";
        src << "    int* const targets = reinterpret_cast<int*>(b" << rec << ") + " << S(2 * bp.nseg * bp.cap) << ";\n";
        src << "    for (uint slot = tid; slot < filled; slot += " << NTH << "u) {\n";
        src << "        const float2 r = stage[slot];\n        const int a = stage_at[slot];\n        const uint bin = ((uint)a >> 4) & 255u;\n";
        src << "        const uint pos = gbase[bin] + (slot - lbase[bin]);\n";
        src << "        if (pos < " << S(bp.cap) << "u) { records[bin * " << S(bp.cap) << "u + pos] = r; targets[bin * " << S(bp.cap) << "u + pos] = a; }\n";
        src << "        else { unsafeAtomicAdd(&b" << acc << "[a], r.x); unsafeAtomicAdd(&b" << acc << "[a + 1], r.y); }\n    }\n}\n";
    } else {
    for (int u = 0; u < U; ++u)
        src << "    if (k" << u << ") stage[lbase[(a" << u << " >> 4) & 255] + r" << u << "] = make_float2(__int_as_float(a" << u << "), v" << u << ");\n";
    src << "    __syncthreads();\n";
    src << "    float2* const records = reinterpret_cast<float2*>(b" << rec << ");\n";
    src << "    for (uint slot = tid; slot < filled; slot += " << NTH << "u) {\n";
    src << "        const float2 r = stage[slot];\n        const int a = __float_as_int(r.x);\n        const uint bin = ((uint)a >> 4) & 255u;\n";
    src << "        const uint pos = gbase[bin] + (slot - lbase[bin]);\n";
    src << "        if (pos < " << S(bp.cap) << "u) records[bin * " << S(bp.cap) << "u + pos] = r;\n";
    src << "        else unsafeAtomicAdd(&b" << acc << "[a], r.y);\n    }\n}\n";
    }
    g.source = src.str();
    g.grid = (unsigned)first_wg;
    g.block = NTH;
    g.n_buffers = fk.n_buffers;
    g.note = "scatter chain, stage 1 of 2: " + to_string(fk.parts.size()) + " links, " + (pairs ? "(target, two values)" : "(target, value)") + " records ordered by segment in LDS (" + S(bp.nseg) +
             " segments of " + S(bp.seg) + " floats, the accumulator's 64-byte lines dealt to them in turn), written in runs into bins of " + S(bp.cap) + " records";
    *out = g;
    return "";
}

// Stage 2: a workgroup sums the records of one segment (or of its slice of them) in LDS and adds the segment to the
// accumulator, lanes on consecutive addresses.
string generate_scatter_sum(const FusedKernel& fk, Generated* out) {
    const dsc_kernel_desc& d = fk.main.raw();
    const int64_t table = element_count(d.shape);
    if (d.kind != DSC_KERNEL_SCATTER_ADD || table != fk.binned_table || fk.inputs.size() != 2 || fk.outputs.size() != 1 || fk.n_buffers != 3 ||
        fk.inputs[0].buffer < 0 || fk.inputs[1].buffer < 0)
        return "binned scatter: stage 2 binds records, counters and the accumulator";
    const bool pairs = fk.binned_pairs;
    const BinnedScatterPlan bp = binned_scatter_plan(table, fk.binned_total, pairs);
    if (bp.nseg != 256 || bp.seg * 8 > 144 * 1024 || bp.nseg * bp.cap >= ((int64_t)1 << 31)) return "binned scatter: accumulator too large";
    const int rec = fk.inputs[0].buffer, cur = fk.inputs[1].buffer, acc = fk.outputs[0];
    const int U = 4;
    Emitter em(fk);
    Generated g;
    std::ostringstream src;
    if (!fk.as_part) src << kPreludeSource << "\n";
    g.entry = "dsc_scatter_sum_t" + S(table) + "_n" + S(fk.binned_total);
    src << "#ifndef LOCAL\n#define LOCAL(at) ((((at) >> 12) << 4) | ((at) & 15))\n#endif\n";
    if (fk.as_part) {
        src << "DSC_INLINE void part_entry(const uint dsc_block, char* dsc_lds, " << em.kernel_params_decl() << ") {\n";
        src << "    double* const seg = reinterpret_cast<double*>(dsc_lds);\n";
    } else {
        src << "extern \"C\" __global__ __launch_bounds__(1024) void " << g.entry << "(" << em.kernel_params_decl() << ") {\n";
        src << "    __shared__ double seg[" << S(bp.seg) << "];\n";
    }
    g.lds_bytes = (size_t)bp.seg * 8;
    src << "    const uint tid = threadIdx.x;\n";
    src << "    const uint s = " << (fk.as_part ? "dsc_block" : "blockIdx.x") << " / " << S(bp.slices) << "u, slice = " << (fk.as_part ? "dsc_block" : "blockIdx.x") << " % " << S(bp.slices) << "u;\n";
    src << "    for (uint i = tid; i < " << S(bp.seg) << "u; i += 1024u) seg[i] = 0.0;\n    __syncthreads();\n";
    src << "    const uint count = min(reinterpret_cast<const uint*>(b" << cur << ")[s * 16u], " << S(bp.cap) << "u);\n";
    src << "    const uint lo = (uint)((unsigned long long)count * slice / " << S(bp.slices) << "u), hi = (uint)((unsigned long long)count * (slice + 1u) / " << S(bp.slices) << "u);\n";
    src << "    const float2* const records = reinterpret_cast<const float2*>(b" << rec << ") + s * " << S(bp.cap) << "u;\n";
    src << "    uint i = lo + tid;\n";
    if (pairs) {
        // a row's two values sit side by side in one line of the accumulator, so side by side in the segment too
        src << "    const int* const targets = reinterpret_cast<const int*>(b" << rec << ") + " << S(2 * bp.nseg * bp.cap) << " + s * " << S(bp.cap) << "u;\n";
        src << "    for (; i + " << S((U - 1) * 1024) << "u < hi; i += " << S(U * 1024) << "u) {\n";
        for (int u = 0; u < U; ++u) src << "        const float2 r" << u << " = records[i + " << S(u * 1024) << "u]; const int t" << u << " = targets[i + " << S(u * 1024) << "u];\n";
        src << "        __builtin_amdgcn_sched_barrier(0);\n";
        for (int u = 0; u < U; ++u)
            src << "        { double* const at = &seg[LOCAL(t" << u << ")]; atomicAdd(at, (double)r" << u << ".x); atomicAdd(at + 1, (double)r" << u << ".y); }\n";
        src << "    }\n";
        src << "    for (; i < hi; i += 1024u) {\n        const float2 r = records[i];\n        double* const at = &seg[LOCAL(targets[i])];\n";
        src << "        atomicAdd(at, (double)r.x); atomicAdd(at + 1, (double)r.y);\n    }\n";
    } else {
    src << "    for (; i + " << S((U - 1) * 1024) << "u < hi; i += " << S(U * 1024) << "u) {\n";
    for (int u = 0; u < U; ++u) src << "        const float2 r" << u << " = records[i + " << S(u * 1024) << "u];\n";
    src << "        __builtin_amdgcn_sched_barrier(0);\n";
    for (int u = 0; u < U; ++u) src << "        atomicAdd(&seg[LOCAL(__float_as_int(r" << u << ".x))], (double)r" << u << ".y);\n";
    src << "    }\n";
    src << "    for (; i < hi; i += 1024u) {\n        const float2 r = records[i];\n        atomicAdd(&seg[LOCAL(__float_as_int(r.x))], (double)r.y);\n    }\n";
    }
    src << "    __syncthreads();\n";
    // local float j of segment s is float j % 16 of the accumulator's line (j / 16) * 256 + s
    src << "    for (uint j = tid; j < " << S(bp.seg) << "u; j += 1024u) {\n        const float sum = (float)seg[j];\n";
    src << "        const int at = (int)((((j >> 4) << 8) + s) << 4 | (j & 15u));\n";
    if (bp.slices == 1)  // the segment has one owner in this launch
        src << "        if (sum != 0.f && at < " << S(table) << ") b" << acc << "[at] += sum;\n    }\n}\n";
    else
        src << "        if (sum != 0.f && at < " << S(table) << ") unsafeAtomicAdd(&b" << acc << "[at], sum);\n    }\n}\n";
    g.source = src.str();
    g.grid = (unsigned)(bp.nseg * bp.slices);
    g.block = 1024;
    g.n_buffers = fk.n_buffers;
    g.algo_bytes = 8.0 * (double)std::min(table, fk.binned_total);
    g.note = "scatter chain, stage 2 of 2: a workgroup per segment (" + S(bp.nseg) + "), records summed in LDS (as doubles, ds_add_f64), the segment's lines added to the accumulator";
    *out = g;
    return "";
}

// Several chain kernels in one launch (FusedKernel::chain_group): each part is generated as a device function over
// the launch's one LDS block; workgroup ids [first, first + grid) of the launch run part i.
string generate_chain_group(const FusedKernel& fk, Generated* out) {
    if (fk.parts.size() != fk.part_params.size() || fk.parts.empty()) return "chain group: part tables differ";
    Generated g;
    std::ostringstream src, body;
    src << kPreludeSource << "\n";
    unsigned first = 0;
    size_t lds = 0;
    string kinds;
    for (size_t i = 0; i < fk.parts.size(); ++i) {
        FusedKernel part = fk.parts[i];
        if (!(part.binned_stage || (part.shared_scatter && !part.parts.empty())) || part.chain_group) return "chain group: a part is not a chain kernel";
        part.as_part = true;
        Generated pg;
        string err = generate(part, &pg);
        if (!err.empty()) return err;
        if ((pg.block != 1024 && pg.block != 512 && pg.block != 256) || pg.lds_bytes == 0 || (i && pg.block != g.block)) return "chain group: unexpected part form";
        g.block = pg.block;
        if ((int)fk.part_params[i].size() != part.n_buffers) return "chain group: part parameter count";
        src << "namespace chain" << i << " {\n" << pg.source << "}  // namespace chain" << i << "\n\n";
        body << "    if (blockIdx.x < " << first + pg.grid << "u) { chain" << i << "::part_entry(blockIdx.x - " << first << "u, dsc_lds";
        for (int j : fk.part_params[i]) body << ", b" << j;
        body << ", seed_cell, seed_value); return; }\n";
        first += pg.grid;
        lds = std::max(lds, pg.lds_bytes);
        g.algo_bytes += pg.algo_bytes;
        if (i == 0) kinds = pg.note;
    }
    Emitter em(fk);
    g.entry = string(fk.parts[0].binned_stage == 1 ? "dsc_scatter_bin" : fk.parts[0].binned_stage == 2 ? "dsc_scatter_sum" : "dsc_scatter_chain") + "_group" +
              to_string(fk.parts.size()) + "_g" + to_string(first);
    src << "extern \"C\" __global__ __launch_bounds__(" << g.block << ") void " << g.entry << "(" << em.kernel_params_decl() << ") {\n";
    src << "    __shared__ __attribute__((aligned(16))) char dsc_lds[" << lds << "];\n";
    src << body.str() << "}\n";
    g.source = src.str();
    g.grid = first;
    g.n_buffers = fk.n_buffers;
    g.note = to_string(fk.parts.size()) + " chains in one launch, the first: " + kinds;
    *out = g;
    return "";
}
}  // namespace

bool scatter_chain_in_lds(int64_t table_elements, int64_t total_values) {
    static const bool binned = !(std::getenv("DSC_SCATTER_BINNED") && std::getenv("DSC_SCATTER_BINNED")[0] == '0');
    // With the two-launch form available, accumulators above 8192 floats go there (the LDS copy is kept in double:
    // 64 KiB, so two workgroups still share a CU).  Measured on the hash grid's 2.1 M values per level with the
    // launches grouped: the LDS chain costs about 4 us per level, the two launches 12 us at any size; moving the
    // 13122-float level to LDS (105 KiB, one workgroup per CU for the whole group) gained 10 us there and lost 6 here.
    const int64_t limit = binned && total_values >= (1 << 18) ? 64 * 1024 : 144 * 1024;
    return table_elements * 8 <= limit && total_values >= 16 * table_elements && total_values >= 65536;
}

bool scatter_chain_binned(int64_t table_elements, int64_t total_values) {
    static const bool enabled = !(std::getenv("DSC_SCATTER_BINNED") && std::getenv("DSC_SCATTER_BINNED")[0] == '0');
    if (!enabled || scatter_chain_in_lds(table_elements, total_values)) return false;
    // enough values that two launches pay, several per accumulator line (the closing adds touch every line of every
    // segment that received something), and an accumulator the segment scan of stage 1 covers
    return total_values >= (1 << 18) && total_values * 4 >= table_elements && table_elements >= 16 * 256 && table_elements <= 256 * 16384;
}

bool scatter_rows_of_two(const dsc_kernel_desc& d) {
    return d.kind == DSC_KERNEL_SCATTER_ADD && d.axis == 0 && d.shape.rank == 2 && d.shape.dims[1] == 2 && d.n_inputs == 2 &&
           d.inputs[0].out_shape.rank == 2 && d.inputs[0].out_shape.dims[1] == 2;
}

BinnedScatterPlan binned_scatter_plan(int64_t table_elements, int64_t total_values, bool pairs) {
    // The accumulator's 64-byte lines are dealt to 256 segments in turn (line l belongs to segment l % 256): a hash
    // or a row-major grid index spreads evenly over the low bits of the line number even where its high bits are
    // skewed (measured on the reference's hash at 2^19 entries: contiguous segments received up to six times
    // their share), and a segment is still stored in whole lines.
    BinnedScatterPlan p;
    p.nseg = 256;
    const int64_t lines = (table_elements + 15) / 16;
    p.seg = (lines + p.nseg - 1) / p.nseg * 16;
    // a quarter more than an even spread needs; what does not fit goes to the accumulator directly
    const int64_t records = pairs ? total_values / 2 : total_values;
    p.cap = ((records / p.nseg) * 5 / 4 + 2048 + 63) / 64 * 64;
    p.record_bytes = pairs ? 12 : 8;
    p.slices = 1;
    return p;
}


namespace {
// One launch running several independent kernels: each part is generated as usual, its entry point turned into a
// device function taking the workgroup id, inside a namespace of its own (helper names repeat between parts).
string generate_multi(const FusedKernel& fk, Generated* out) {
    if (fk.parts.size() != fk.part_params.size() || fk.parts.empty()) return "multi: part tables differ";
    Generated g;
    std::ostringstream src, body;
    src << kPreludeSource << "\n";
    unsigned first = 0;
    string pool_terms;
    for (size_t i = 0; i < fk.parts.size(); ++i) {
        const FusedKernel& part = fk.parts[i];
        if (!can_be_part(part)) return "multi: kernel cannot be a part";
        Generated pg;
        FusedKernel as_part = part;
        as_part.as_part = true;
        string err = generate_one(as_part, &pg, false);
        if (!err.empty()) return err;
        if (pg.block != 256) return "multi: parts must use 256 threads";
        if ((int)fk.part_params[i].size() != part.n_buffers) return "multi: part parameter count";
        string text = pg.source;
        if (text.find("#define MM_AS_PART 1") == string::npos) {  // the MFMA template emits its part form itself
            const string head = "extern \"C\" __global__ __launch_bounds__(256) void " + pg.entry + "(";
            const size_t at = text.find(head);
            if (at == string::npos) return "multi: unexpected entry point form";
            text.replace(at, head.size(), "DSC_INLINE void part_entry(char* const dsc_pool, const uint dsc_block, ");
            for (size_t pos = text.find("blockIdx.x"); pos != string::npos; pos = text.find("blockIdx.x", pos)) text.replace(pos, 10, "dsc_block");
            if (text.find("gridDim") != string::npos) return "multi: part depends on the grid size";
            // The parts' LDS arrays overlie one another in the launch's one block (a kernel's distinct __shared__ arrays
            // are laid out side by side whether or not they are ever live together: three MatMul parts of 16-26 KB each
            // made a 62 KB launch of two workgroups per CU).  Every `__shared__ [aligned] T name[n]...;` becomes a
            // reference into the block.
            size_t used = 0;
            for (size_t pos = text.find("__shared__"); pos != string::npos; pos = text.find("__shared__", pos)) {
                size_t q = pos + 10;
                auto skip = [&]() { while (q < text.size() && (text[q] == ' ' || text[q] == '\t')) ++q; };
                auto word = [&]() { const size_t b = q; while (q < text.size() && (std::isalnum((unsigned char)text[q]) || text[q] == '_')) ++q; return text.substr(b, q - b); };
                skip();
                const string attr = "__attribute__((aligned(16)))";
                if (text.compare(q, attr.size(), attr) == 0) q += attr.size();
                skip();
                const string type = word();
                skip();
                const string name = word();
                const size_t size = type == "float" || type == "int" || type == "uint" ? 4 : type == "double" || type == "float2" ? 8 : type == "float4" ? 16 : 0;
                string dims;
                size_t count = 1;
                bool ok = size != 0 && !name.empty();
                while (ok && q < text.size() && text[q] == '[') {
                    const size_t b = ++q;
                    while (q < text.size() && std::isdigit((unsigned char)text[q])) ++q;
                    if (q == b || q >= text.size() || text[q] != ']') { ok = false; break; }
                    dims += "[" + text.substr(b, q - b) + "]";
                    count *= (size_t)std::stoll(text.substr(b, q - b));
                    ++q;
                }
                if (!ok || dims.empty() || q >= text.size() || text[q] != ';') return "multi: a part declares LDS in a form the launch's block cannot take";
                const string ref = type + " (&" + name + ")" + dims + " = *reinterpret_cast<" + type + " (*)" + dims + ">(dsc_pool + " + to_string(used) + ");";
                text.replace(pos, q + 1 - pos, ref);
                used = (used + count * size + 15) / 16 * 16;
                pos += ref.size();
            }
            text += "constexpr int dsc_part_lds_bytes = " + to_string(used) + ";\n";
        }
        pool_terms += (i ? ", " : "") + string("part") + to_string(i) + "::dsc_part_lds_bytes";
        src << "namespace part" << i << " {\n" << text << "}  // namespace part" << i << "\n\n";
        body << "    if (blockIdx.x < " << first + pg.grid << "u) { part" << i << "::part_entry(dsc_pool, blockIdx.x - " << first << "u";
        for (int j : fk.part_params[i]) body << ", b" << j;
        body << ", seed_cell, seed_value); return; }\n";
        first += pg.grid;
        g.algo_bytes += pg.algo_bytes;
        g.algo_flops += pg.algo_flops;
        g.note += (i ? " | " : "multi: ") + pg.note;
    }
    Emitter em(fk);
    g.entry = "dsc_multi_p" + to_string(fk.parts.size()) + "_g" + to_string(first);
    src << "constexpr int dsc_pool_sizes[] = {" << pool_terms << "};\n";
    src << "constexpr int dsc_pool_bytes() { int m = 16; for (int v : dsc_pool_sizes) m = v > m ? v : m; return m; }\n";
    src << "extern \"C\" __global__ __launch_bounds__(256) void " << g.entry << "(" << em.kernel_params_decl() << ") {\n";
    src << "    __shared__ __attribute__((aligned(16))) char dsc_pool[dsc_pool_bytes()];\n" << body.str() << "}\n";
    g.source = src.str();
    g.grid = first;
    g.block = 256;
    g.n_buffers = fk.n_buffers;
    *out = g;
    return "";
}
}  // namespace

const std::vector<std::string>& compile_options() {
    // packed fp32 instructions are kept off for every kernel; float atomicAdd maps to the hardware instruction;
    // a*b+c stays two rounded operations as written (the per-element semantics are "tmp = a * b; tmp2 = tmp + c")
    static const std::vector<std::string> opts = {"-O3", "-munsafe-fp-atomics", "-ffp-contract=off", "-Xclang", "-target-feature",
                                                  "-Xclang", "-packed-fp32-ops", "-std=c++17"};
    return opts;
}

}  // namespace dsc
