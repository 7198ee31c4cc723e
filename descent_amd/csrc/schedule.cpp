// Whole-graph schedules: cross-cluster fusion at creation, Environment::run semantics per step.
#include "schedule.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <set>
#include <sstream>

namespace dsc {

namespace {

// One launch being assembled: a fused kernel plus the op node bound to each pointer parameter.
struct Draft {
    bool alive = true;
    FusedKernel fk;
    std::vector<int> params;      // node id per pointer parameter
    std::vector<StepOutput> outs; // outputs, parallel to fk.outputs
    std::vector<int> covers;      // reference cluster indices folded into this launch
    bool keep_split = false;      // MatMul re-split over k on purpose: do not sum its chunks in one workgroup
    bool keep_output = false;     // first stage of a split reduction: its result must exist in memory
    std::vector<int> part_inputs; // multi-part launch: the distinct nodes its parts read
};

// The view walks its whole buffer in memory order (an identity view, or a reshape of one).
bool reads_in_order(const dsc_view& v) {
    int64_t base = 0, coef[DSC_MAX_DIM];
    if (!affine_form(v, &base, coef) || base != 0 || element_count(v.in_shape) != element_count(v.out_shape)) return false;
    int64_t st[DSC_MAX_DIM];
    strides_of(v.out_shape, st);
    for (int j = 0; j < v.out_shape.rank; ++j)
        if (v.out_shape.dims[j] > 1 && coef[j] != st[j]) return false;
    return true;
}

int param_index(Draft& d, int node, bool is_output) {
    for (size_t i = 0; i < d.params.size(); ++i)
        if (d.params[i] == node && d.fk.buffer_is_output[i] == is_output) return (int)i;
    d.params.push_back(node);
    d.fk.buffer_is_output.push_back(is_output);
    d.fk.n_buffers = (int)d.params.size();
    return (int)d.params.size() - 1;
}

// Copies p's virtual producers into q; returns the index offset applied to p's virtual ids.
int import_virtuals(Draft& q, const Draft& p) {
    const int offset = (int)q.fk.virtuals.size();
    for (const Virtual& v : p.fk.virtuals) {
        Virtual nv = v;
        for (Source& s : nv.inputs) {
            if (s.buffer >= 0) s.buffer = param_index(q, p.params[s.buffer], false);
            else s.virt += offset;
        }
        q.fk.virtuals.push_back(nv);
    }
    return offset;
}

Source import_source(Draft& q, const Draft& p, const Source& s, int virt_offset) {
    Source out;
    if (s.buffer >= 0) out.buffer = param_index(q, p.params[s.buffer], false);
    else out.virt = s.virt + virt_offset;
    return out;
}

template <class F>
void for_each_source(FusedKernel& fk, F f) {
    for (auto& s : fk.inputs) f(s);
    for (auto& st : fk.row_stages)
        for (auto& s : st.inputs)
            if (s.stage < 0) f(s);
    for (auto& v : fk.virtuals)
        for (auto& s : v.inputs) f(s);
    if (fk.has_epilogue)
        for (size_t i = 0; i < fk.epilogue_inputs.size(); ++i)
            if ((int)i != fk.epilogue_product_input) f(fk.epilogue_inputs[i]);
    if (fk.pool.on && fk.pool.has_epilogue)
        for (size_t i = 0; i < fk.pool.epilogue_inputs.size(); ++i)
            if ((int)i != fk.pool.epilogue_product_input) f(fk.pool.epilogue_inputs[i]);
    if (fk.dgrad.on && fk.dgrad.pm.on) f(fk.dgrad.pm.masks);
    if (fk.row_tail.on) {
        f(fk.row_tail.b);
        if (fk.row_tail.has_epilogue)
            for (size_t i = 0; i < fk.row_tail.epilogue_inputs.size(); ++i)
                if ((int)i != fk.row_tail.epilogue_product_input && (int)i != fk.row_tail.epilogue_a_input) f(fk.row_tail.epilogue_inputs[i]);
    }
}

// Drops pointer parameters nothing refers to and renumbers the rest.
void compact(Draft& d) {
    std::vector<bool> used(d.params.size(), false);
    for_each_source(d.fk, [&](Source& s) { if (s.buffer >= 0) used[s.buffer] = true; });
    for (int o : d.fk.outputs) used[o] = true;
    std::vector<int> remap(d.params.size(), -1);
    std::vector<int> params;
    std::vector<bool> is_out;
    for (size_t i = 0; i < d.params.size(); ++i) {
        if (!used[i]) continue;
        remap[i] = (int)params.size();
        params.push_back(d.params[i]);
        is_out.push_back(d.fk.buffer_is_output[i]);
    }
    for_each_source(d.fk, [&](Source& s) { if (s.buffer >= 0) s.buffer = remap[s.buffer]; });
    for (int& o : d.fk.outputs) o = remap[o];
    if (d.fk.colsum_out >= 0) d.fk.colsum_out = remap[d.fk.colsum_out];
    if (d.fk.sign_out >= 0) d.fk.sign_out = remap[d.fk.sign_out];
    d.params = params;
    d.fk.buffer_is_output = is_out;
    d.fk.n_buffers = (int)params.size();
}

std::vector<int> input_nodes(const Draft& d) {
    if (!d.fk.parts.empty()) return d.part_inputs;
    std::set<int> seen;
    std::vector<int> out;
    Draft& md = const_cast<Draft&>(d);
    for_each_source(md.fk, [&](Source& s) {
        if (s.buffer >= 0 && seen.insert(d.params[s.buffer]).second) out.push_back(d.params[s.buffer]);
    });
    return out;
}

bool is_cheap_producer(const dsc_kernel_desc& pe) {
    // a producer is re-evaluated by each read of its consumer: only inline copies and light arithmetic
    int work = 0;
    for (int i = 0; i < pe.n_ops; ++i) {
        const dsc_pe_op& op = pe.ops[i];
        if (op.kind == DSC_PE_UNARY && op.op != DSC_UN_MOV && op.op != DSC_UN_NEG) return false;
        if (op.kind == DSC_PE_BINARY && (op.op == DSC_BIN_DIV || op.op == DSC_BIN_POW || op.op == DSC_BIN_UREM)) return false;
        if (op.kind == DSC_PE_GATHER || op.kind == DSC_PE_RAND) return false;
        if (op.kind == DSC_PE_LOAD) work += 2;
        else if (op.kind == DSC_PE_UNARY || op.kind == DSC_PE_BINARY || op.kind == DSC_PE_SELECT) work += 1;
    }
    return work <= 12;
}

// Loads issued per evaluated element, following fused producers (a Reduce producer multiplies by its k).
double source_cost(const FusedKernel& fk, const Source& s);
// Elements of its input that one element of a kernel evaluated on demand reads: the reduced axis of a Reduce, the k of a
// MatMul, the windows that cover a pixel of a WindowsToImage (on average), the padded elements behind an element
// of an Unpad (one, away from the border).
double on_demand_reads(const dsc_kernel_desc& d) {
    switch (d.kind) {
    case DSC_KERNEL_REDUCE: return (double)d.inputs[0].out_shape.dims[d.axis];
    case DSC_KERNEL_MATMUL: return (double)matmul_dims(d).k;
    case DSC_KERNEL_UNPAD: return 1.0 + 2.0 * (double)d.pad / (double)d.shape.dims[d.axis];
    case DSC_KERNEL_WINDOWS_TO_IMAGE: {
        const dsc_view& v = d.inputs[0];
        const int r = v.out_shape.rank;
        return std::max(1.0, (double)(v.out_shape.dims[r - 3] * v.out_shape.dims[r - 2]) / (double)(d.stride_w * d.stride_h));
    }
    default: return 1.0;
    }
}
double virtual_cost(const FusedKernel& fk, const Virtual& v) {
    const dsc_kernel_desc& d = v.pe.raw();
    double c = 0;
    for (auto& s : v.inputs) c += source_cost(fk, s);
    if (d.kind != DSC_KERNEL_PER_ELEMENT) return c * on_demand_reads(d);
    return c + d.n_ops / 4.0;
}
double source_cost(const FusedKernel& fk, const Source& s) { return s.buffer >= 0 ? 1.0 : virtual_cost(fk, fk.virtuals[s.virt]); }
double draft_unit_cost(const Draft& d) {
    double c = 0;
    for (auto& s : d.fk.inputs) c += source_cost(d.fk, s);
    return c;
}
// How many times one evaluation of the main kernel's element reads `node`: the product of the loop lengths of
// the fused Reduce producers the read sits inside (1 when the main kernel reads the node directly).
double node_multiplicity(const Draft& d, int node) {
    const int nv = (int)d.fk.virtuals.size();
    std::vector<double> mult(nv, 0.0);
    auto visit = [&](const Source& s, double m, auto&& self) -> double {
        if (s.buffer >= 0) return d.params[s.buffer] == node ? m : 0.0;
        const Virtual& v = d.fk.virtuals[s.virt];
        const dsc_kernel_desc& vd = v.pe.raw();
        const double inner = m * (vd.kind != DSC_KERNEL_PER_ELEMENT ? on_demand_reads(vd) : 1.0);
        double best = 0.0;
        for (auto& in : v.inputs) best = std::max(best, self(in, inner, self));
        return best;
    };
    double best = 0.0;
    for (auto& s : d.fk.inputs) best = std::max(best, visit(s, 1.0, visit));
    if (d.fk.has_epilogue)
        for (size_t i = 0; i < d.fk.epilogue_inputs.size(); ++i)
            if ((int)i != d.fk.epilogue_product_input) best = std::max(best, visit(d.fk.epilogue_inputs[i], 1.0, visit));
    return std::max(best, 1.0);
}

int64_t draft_reads(const Draft& d) {  // how many elements the main kernel evaluates per input
    const dsc_kernel_desc& m = d.fk.main.raw();
    switch (m.kind) {
    case DSC_KERNEL_REDUCE: return element_count(m.inputs[0].out_shape);
    case DSC_KERNEL_MATMUL: {
        MatMulDims g = matmul_dims(m);
        return g.batch * std::max(g.m * g.k, g.k * g.n);
    }
    case DSC_KERNEL_WINDOWS_TO_IMAGE: return element_count(m.inputs[0].out_shape);
    case DSC_KERNEL_SCATTER_ADD: return element_count(m.inputs[0].out_shape);
    default: return element_count(m.shape);
    }
}

// Linear index into a view's input for integer output coordinates; the view must need no clamp.
int64_t view_index(const dsc_view& v, const int64_t* coord) {
    int64_t st[DSC_MAX_DIM], in[DSC_MAX_DIM];
    strides_of(v.in_shape, st);
    for (int i = 0; i < v.in_shape.rank; ++i) in[i] = v.in_offset[i];
    for (int j = 0; j < v.out_shape.rank; ++j)
        if (v.map_axis[j] >= 0) in[v.map_axis[j]] += v.map_step[j] * coord[j];
    int64_t idx = 0;
    for (int i = 0; i < v.in_shape.rank; ++i) idx += in[i] * st[i];
    return idx;
}

// The same with every input coordinate clamped into its axis: what a load through the view reads (padding by
// replication is a view whose coordinates leave the array and are clamped, src/shape.rs:374-379, 503-526).
int64_t view_index_clamped(const dsc_view& v, const int64_t* coord) {
    int64_t st[DSC_MAX_DIM], in[DSC_MAX_DIM];
    strides_of(v.in_shape, st);
    for (int i = 0; i < v.in_shape.rank; ++i) in[i] = v.in_offset[i];
    for (int j = 0; j < v.out_shape.rank; ++j)
        if (v.map_axis[j] >= 0) in[v.map_axis[j]] += v.map_step[j] * coord[j];
    int64_t idx = 0;
    for (int i = 0; i < v.in_shape.rank; ++i) idx += std::min(std::max<int64_t>(in[i], 0), v.in_shape.dims[i] - 1) * st[i];
    return idx;
}

dsc_pe_op pe_op(int kind, int op = 0, int a0 = 0, int a1 = 0, int a2 = 0, int a3 = 0) {
    dsc_pe_op o{};
    o.kind = kind;
    o.op = op;
    o.args[0] = a0; o.args[1] = a1; o.args[2] = a2; o.args[3] = a3;
    return o;
}
dsc_pe_op pe_literal(float value) {
    dsc_pe_op o = pe_op(DSC_PE_LITERAL_F32);
    std::memcpy(&o.bits, &value, 4);
    return o;
}
dsc_view identity_view(std::initializer_list<int64_t> dims) {
    dsc_view v{};
    v.in_shape.rank = v.out_shape.rank = (int)dims.size();
    int i = 0;
    for (int64_t d : dims) {
        v.in_shape.dims[i] = v.out_shape.dims[i] = d;
        v.map_axis[i] = d > 1 ? i : -1;
        v.map_step[i] = d > 1 ? 1 : 0;
        ++i;
    }
    return v;
}

// The fusion planner.  One draft per reference cluster goes in; each pass below merges, splits or re-targets
// drafts (and may add internal nodes).  Nothing is compiled here: a pass that is unsure whether a candidate can be
// expressed generates its source as a probe and drops the candidate when that fails.  `run` holds the order.
struct Planner {
    const uint32_t flags;
    int& n_nodes;
    std::vector<size_t>& node_bytes;
    std::vector<Draft>& drafts;
    std::vector<bool>& is_graph_output;
    std::vector<bool>& is_graph_input;

    // what pass 1d learns about each convolution, for pass 1e
    struct ConvSite {
        int copy_idx;    // draft that writes the im2col copy
        int a_node;      // the copy
        int image_node;  // the convolution's input [img, h, w, g*c]
        FusedKernel::ConvFwd geo;
        dsc_view a_view; // (group, row, k) -> element of the copy, as the forward MatMul reads it
    };
    std::vector<ConvSite> conv_sites;

    // One step of merging a chain of Reduces over neighbouring axes (pass 0a below says when): the Reduce in draft
    // `i` and the Reduce that alone consumes it become one Reduce over the merged axis, in draft `i`.
    bool merge_reduce_step(size_t i, bool small_only) {
            const dsc_kernel_desc r1 = drafts[i].fk.main.raw();
            if (r1.kind != DSC_KERNEL_REDUCE || !drafts[i].fk.virtuals.empty() || drafts[i].fk.has_epilogue) return false;
            if (small_only && element_count(r1.inputs[0].out_shape) > (1 << 18)) return false;
            {
                // a short Reduce along the rows of a matrix is left to the row fusion (pass 1b)
                const dsc_shape& os = r1.inputs[0].out_shape;
                bool innermost = true;
                for (int q = r1.axis + 1; q < os.rank; ++q)
                    if (os.dims[q] > 1) innermost = false;
                if (innermost && os.dims[r1.axis] <= 64) return false;
            }
            const int mid = drafts[i].outs[0].node;
            if (is_graph_output[mid] || drafts[i].outs[0].copy_from >= 0) return false;
            int j = -1, uses = 0;
            for (size_t q = 0; q < drafts.size(); ++q) {
                if (q == i) continue;
                for (int nd : input_nodes(drafts[q]))
                    if (nd == mid) { ++uses; j = (int)q; }
                for (auto& o : drafts[q].outs)
                    if (o.copy_from == mid) uses += 2;
            }
            if (uses != 1 || j < (int)i) return false;
            const dsc_kernel_desc r2 = drafts[j].fk.main.raw();
            if (r2.kind != DSC_KERNEL_REDUCE || r2.reduce_op != r1.reduce_op || !drafts[j].fk.virtuals.empty() ||
                drafts[j].fk.has_epilogue || !reads_in_order(r2.inputs[0]))
                return false;
            const dsc_view v = r1.inputs[0];
            const int a = r1.axis;
            // the second Reduce's axis, as an axis of the first one's output
            std::vector<int> kept1, kept2;
            for (int q = 0; q < v.out_shape.rank; ++q)
                if (q != a && v.out_shape.dims[q] > 1) kept1.push_back(q);
            for (int q = 0; q < r2.inputs[0].out_shape.rank; ++q)
                if (r2.inputs[0].out_shape.dims[q] > 1) kept2.push_back(q);
            if (kept1.size() != kept2.size()) return false;
            int b = -1;
            bool same = true;
            for (size_t q = 0; q < kept1.size(); ++q) {
                if (v.out_shape.dims[kept1[q]] != r2.inputs[0].out_shape.dims[kept2[q]]) same = false;
                if (kept2[q] == r2.axis) b = kept1[q];
            }
            if (!same || b < 0) return false;
            bool neighbours = true;
            for (int q = std::min(a, b) + 1; q < std::max(a, b); ++q)
                if (v.out_shape.dims[q] > 1) neighbours = false;
            const int ia = v.map_axis[a], ib = v.map_axis[b];
            if (!neighbours || ia < 0 || ib < 0 || ia == ib || (a < b) != (ia < ib)) return false;
            auto whole = [&](int out_axis, int in_axis) {
                return v.map_step[out_axis] == 1 && v.in_offset[in_axis] == 0 && v.out_shape.dims[out_axis] == v.in_shape.dims[in_axis];
            };
            if (!whole(a, ia) || !whole(b, ib)) return false;
            for (int q = std::min(ia, ib) + 1; q < std::max(ia, ib); ++q)
                if (v.in_shape.dims[q] > 1) neighbours = false;
            // no other output axis may walk the two input axes
            for (int q = 0; q < v.out_shape.rank; ++q)
                if (q != a && q != b && (v.map_axis[q] == ia || v.map_axis[q] == ib)) neighbours = false;
            if (!neighbours) return false;
            const int64_t merged = v.out_shape.dims[a] * v.out_shape.dims[b];
            const int lo_in = std::min(ia, ib), hi_in = std::max(ia, ib);
            const int lo_out = ia < ib ? a : b, hi_out = ia < ib ? b : a;
            dsc_view m = v;
            m.in_shape.dims[lo_in] = merged;
            m.in_shape.dims[hi_in] = 1;
            m.out_shape.dims[lo_out] = merged;
            m.out_shape.dims[hi_out] = 1;
            m.map_axis[hi_out] = -1;
            m.map_step[hi_out] = 0;
            dsc_kernel_desc d = r1;
            d.inputs = &m;
            d.axis = lo_out;
            d.shape = m.out_shape;
            d.shape.dims[lo_out] = 1;
            if (!validate(d).empty() || element_count(d.shape) != element_count(r2.shape)) return false;
            Draft mergedDraft;
            mergedDraft.fk = FusedKernel::plain(d);
            mergedDraft.params = {drafts[i].params[0], drafts[j].outs[0].node};
            mergedDraft.outs.push_back(drafts[j].outs[0]);
            mergedDraft.covers = drafts[i].covers;
            mergedDraft.covers.insert(mergedDraft.covers.end(), drafts[j].covers.begin(), drafts[j].covers.end());
            drafts[i] = mergedDraft;
            drafts.erase(drafts.begin() + j);
            return true;
    }

    std::vector<int> consumers_of(int node) const {
            std::vector<int> out;
            for (int i = 0; i < (int)drafts.size(); ++i) {
                if (!drafts[i].alive) continue;
                auto ins = input_nodes(drafts[i]);
                if (std::find(ins.begin(), ins.end(), node) != ins.end()) out.push_back(i);
            }
            return out;
    }

    // no launch between `from` and `to` may take one of `nodes` over in place (ScatterAdd accumulators)
    bool taken_in_place_between(int from, int to, const std::vector<int>& nodes) const {
            for (int i = from + 1; i < to; ++i) {
                if (!drafts[i].alive) continue;
                for (auto& o : drafts[i].outs)
                    if (o.copy_from >= 0 && std::find(nodes.begin(), nodes.end(), o.copy_from) != nodes.end()) return true;
            }
            for (auto& o : drafts[to].outs)
                if (o.copy_from >= 0 && std::find(nodes.begin(), nodes.end(), o.copy_from) != nodes.end()) return true;
            return false;
    }

    // A per-element cluster that can run as the epilogue of the launch producing `product_node` (`elements`
    // values): it is the node's only consumer, has one invocation per product element and reads the product
    // element-for-element through a plain load.
    // With `permuted` given, the view may also be any bijection of a small product's elements (a transposed or
    // re-split reading of it); *permuted then says whether it is one.
    // With `shared` given, the product may have further readers after the cluster (the kernel then stores the
    // product too); *shared says whether it has.
    void find_epilogue(int producer_idx, int product_node, int64_t elements, int* pe_idx, int* pe_input, bool* permuted = nullptr,
                       bool* shared = nullptr) const {
            *pe_idx = *pe_input = -1;
            if (permuted) *permuted = false;
            if (shared) *shared = false;
            if (is_graph_output[product_node]) return;
            auto cons = consumers_of(product_node);
            if (cons.empty() || cons[0] <= producer_idx) return;
            if (cons.size() != 1) {
                // the cluster must be the first reader, nobody may take the product over in place, and a large product
                // only (a small one costs less as a launch part than as a second store)
                if (!shared || elements < (1 << 16)) return;
                for (auto& dr : drafts)
                    if (dr.alive)
                        for (auto& o : dr.outs)
                            if (o.copy_from == product_node) return;
                *shared = true;
            }
            Draft& e = drafts[cons[0]];
            const dsc_kernel_desc& ed = e.fk.main.raw();
            if (ed.kind != DSC_KERNEL_PER_ELEMENT || e.fk.has_epilogue || ed.shape.dims[0] != elements) return;
            int hits = 0, input = -1;
            for (int k = 0; k < ed.n_inputs; ++k) {
                if (e.fk.inputs[k].buffer >= 0 && e.params[e.fk.inputs[k].buffer] == product_node) {
                    ++hits;
                    input = k;
                }
            }
            if (hits != 1) return;
            for (int k = 0; k < ed.n_ops; ++k)  // the product must be read element-for-element, not gathered
                if (ed.ops[k].kind == DSC_PE_GATHER && ed.ops[k].input_index == input) return;
            for (auto& v : e.fk.virtuals)  // and not through one of the consumer's own fused producers
                for (auto& src : v.inputs)
                    if (src.buffer >= 0 && e.params[src.buffer] == product_node) return;
            for (auto& o : e.outs)
                if (o.copy_from >= 0) return;
            if (!is_contiguous(ed.inputs[input])) {
                const dsc_view& v = ed.inputs[input];
                if (!permuted || elements > 65536 || element_count(v.in_shape) != elements || any_clamp(v)) return;
                // every element read exactly once, and recovered by the per-axis inverse the kernel will use
                std::vector<char> seen((size_t)elements, 0);
                int64_t ist[DSC_MAX_DIM], ost[DSC_MAX_DIM];
                strides_of(v.in_shape, ist);
                strides_of(v.out_shape, ost);
                for (int64_t e = 0; e < elements; ++e) {
                    int64_t cc[DSC_MAX_DIM], q = e;
                    for (int a = v.out_shape.rank - 1; a >= 0; --a) {
                        cc[a] = q % v.out_shape.dims[a];
                        q /= v.out_shape.dims[a];
                    }
                    const int64_t r = view_index(v, cc);
                    if (r < 0 || r >= elements || seen[(size_t)r]) return;
                    seen[(size_t)r] = 1;
                    int64_t back = 0;
                    for (int j = 0; j < v.out_shape.rank; ++j) {
                        if (v.out_shape.dims[j] <= 1 || v.map_axis[j] < 0) continue;
                        if (v.map_step[j] <= 0) return;
                        const int i = v.map_axis[j];
                        back += (((r / ist[i]) % v.in_shape.dims[i]) / v.map_step[j]) % v.out_shape.dims[j] * ost[j];
                    }
                    if (back != e) return;
                }
                if (shared && *shared) return;
                *permuted = true;
            }
            if (taken_in_place_between(producer_idx, cons[0], input_nodes(drafts[producer_idx]))) return;
            *pe_idx = cons[0];
            *pe_input = input;
    }

    // one load passed on unchanged
    static bool is_pure_copy(const dsc_kernel_desc& pe) {
            int loads = 0;
            for (int i = 0; i < pe.n_ops; ++i) {
                if (pe.ops[i].kind == DSC_PE_LOAD) ++loads;
                else if (!(pe.ops[i].kind == DSC_PE_UNARY && pe.ops[i].op == DSC_UN_MOV)) return false;
            }
            return loads == 1;
    }

    // Pass 00: the sign of a pre-activation read off the activation.  A cluster that stores both z and
    // a = (z > 0) ? z : z * c with a literal c >= 0, or : 0 (a leaky or plain ReLU beside its input, kept for the backward pass) and whose
    // z is read elsewhere only as the left side of "(z > 0) ? .. : .." selects: a > 0 exactly when z > 0 (z * c is
    // negative, a negative zero or a NaN whenever z is not positive), so those readers take a instead and z is not
    // stored.  One array less written by the forward kernel and one less read by the backward one, bit for bit the same
    // results.
    void sign_through_activation() {
        static const bool enabled = !(std::getenv("DSC_SIGN_THROUGH_ACTIVATION") && std::getenv("DSC_SIGN_THROUGH_ACTIVATION")[0] == '0');
        if (!enabled) return;
        auto is_zero = [](const dsc_pe_op& o) { return o.kind == DSC_PE_LITERAL_F32 && (o.bits & 0x7fffffffu) == 0; };
        auto plain_pe = [](const Draft& d) {
            return d.alive && d.fk.main.raw().kind == DSC_KERNEL_PER_ELEMENT && d.fk.virtuals.empty() && !d.fk.has_epilogue && d.fk.parts.empty() &&
                   d.fk.row_stages.empty() && (int)d.fk.inputs.size() == d.fk.main.raw().n_inputs;
        };
        for (int pi = 0; pi < (int)drafts.size(); ++pi) {
            if (!plain_pe(drafts[pi]) || drafts[pi].fk.main.raw().n_outputs < 2) continue;
            const dsc_kernel_desc& pd = drafts[pi].fk.main.raw();
            int oz = -1, oa = -1;  // which outputs are z and a
            for (int i = 0; i < pd.n_outputs && oz < 0; ++i)
                for (int j = 0; j < pd.n_outputs && oz < 0; ++j) {
                    if (i == j) continue;
                    const int z = pd.outputs[i];
                    const dsc_pe_op& sel = pd.ops[pd.outputs[j]];
                    if (sel.kind != DSC_PE_SELECT || sel.op != DSC_CMP_GT || sel.args[0] != z || sel.args[2] != z || !is_zero(pd.ops[sel.args[1]])) continue;
                    const dsc_pe_op& mul = pd.ops[sel.args[3]];
                    if (!is_zero(mul)) {  // a plain ReLU stores zero there; a leaky one z times a positive literal
                        if (mul.kind != DSC_PE_BINARY || mul.op != DSC_BIN_MUL) continue;
                        const int c = mul.args[0] == z ? mul.args[1] : mul.args[1] == z ? mul.args[0] : -1;
                        if (c < 0 || pd.ops[c].kind != DSC_PE_LITERAL_F32) continue;
                        float cv;
                        std::memcpy(&cv, &pd.ops[c].bits, 4);
                        if (!(cv >= 0.f) || !(cv < 3.0e38f)) continue;  // (z * 0 is a zero or a NaN: not positive either)
                    }
                    oz = i;
                    oa = j;
                }
            if (oz < 0) continue;
            const int z_node = drafts[pi].outs[oz].node, a_node = drafts[pi].outs[oa].node;
            if (is_graph_output[z_node] || drafts[pi].outs[oz].copy_from >= 0 || node_bytes[z_node] != node_bytes[a_node]) continue;
            // every reader of z: a plain per-element cluster that uses it only as the left side of (z > 0) selects
            bool ok = true;
            std::vector<std::pair<int, int>> uses;  // (draft, pointer parameter)
            for (int qi = 0; qi < (int)drafts.size() && ok; ++qi) {
                Draft& Q = drafts[qi];
                if (!Q.alive || qi == pi) continue;
                for (auto& o : Q.outs)
                    if (o.copy_from == z_node) ok = false;
                for (size_t b = 0; b < Q.params.size() && ok; ++b) {
                    if (Q.params[b] != z_node || Q.fk.buffer_is_output[b]) continue;
                    if (!plain_pe(Q) || qi < pi) { ok = false; break; }
                    const dsc_kernel_desc& qd = Q.fk.main.raw();
                    for (int in = 0; in < qd.n_inputs && ok; ++in) {
                        if (Q.fk.inputs[in].buffer != (int)b) continue;
                        for (int l = 0; l < qd.n_ops && ok; ++l) {
                            const dsc_pe_op& lo = qd.ops[l];
                            if (lo.kind == DSC_PE_GATHER && lo.input_index == in) ok = false;
                            if (lo.kind != DSC_PE_LOAD || lo.input_index != in) continue;
                            for (int o = 0; o < qd.n_outputs; ++o)
                                if (qd.outputs[o] == l) ok = false;
                            for (int u = 0; u < qd.n_ops && ok; ++u) {
                                const dsc_pe_op& uo = qd.ops[u];
                                const int nargs = uo.kind == DSC_PE_UNARY || uo.kind == DSC_PE_GATHER ? 1 : uo.kind == DSC_PE_BINARY ? 2 : uo.kind == DSC_PE_SELECT ? 4 : 0;
                                for (int a = 0; a < nargs; ++a) {
                                    if (uo.args[a] != l) continue;
                                    if (!(uo.kind == DSC_PE_SELECT && uo.op == DSC_CMP_GT && a == 0 && is_zero(qd.ops[uo.args[1]]))) ok = false;
                                }
                            }
                        }
                    }
                    uses.emplace_back(qi, (int)b);
                }
            }
            if (!ok || uses.empty()) continue;
            for (auto& u : uses) drafts[u.first].params[u.second] = a_node;
            // z is no output any more
            dsc_kernel_desc trimmed = pd;
            std::vector<int32_t> kept(pd.outputs, pd.outputs + pd.n_outputs);
            kept.erase(kept.begin() + oz);
            trimmed.outputs = kept.data();
            trimmed.n_outputs = (int32_t)kept.size();
            KernelDesc fixed(trimmed);
            if (!validate(fixed.raw()).empty()) {
                for (auto& u : uses) drafts[u.first].params[u.second] = z_node;
                continue;
            }
            Draft& P = drafts[pi];
            const int n_in = fixed.raw().n_inputs;
            P.params.erase(P.params.begin() + n_in + oz);
            P.outs.erase(P.outs.begin() + oz);
            P.fk = FusedKernel::plain(fixed.raw());
        }
    }

    // Pass 0: a MatMul whose output is small but whose k is long gets its k range split over many more
    // workgroups than the reference's ceil(K/1024) chunks; the partial products go to an internal buffer and
    // are summed by a Reduce (which pass 2 then inlines into the consumer when the split is small).
    void split_long_k() {
        for (size_t i = 0; i < drafts.size(); ++i) {
            if (drafts[i].fk.main.raw().kind != DSC_KERNEL_MATMUL) continue;
            const MatMulDims g = matmul_dims(drafts[i].fk.main.raw());
            if (g.k < 512) continue;
            if (((g.m + 63) / 64) * ((g.n + 63) / 64) * g.batch >= 128) continue;  // the tile grid is already wide
            if (ksplit_kernel_shape(drafts[i].fk)) continue;  // k is split inside the workgroups of one launch
            {
                // rows of k-contiguous memory times a few columns: the dot-product kernel spreads k over lanes itself
                const dsc_view& av = drafts[i].fk.main.raw().inputs[0];
                const int64_t c0[3] = {0, 0, 0}, c1[3] = {0, 0, 1};
                if (g.chunks == 1 && g.m >= 256 && dot_kernel_shape(g) && av.out_shape.rank == 3 && view_index(av, c1) - view_index(av, c0) == 1) continue;
            }
            const int64_t t64 = ((g.m + 63) / 64) * ((g.n + 63) / 64) * g.batch;
            const int64_t split_target = 4096;  // workgroup tiles a split product should reach
            int64_t S = std::min<int64_t>(split_target / t64, g.k / 64);
            {
                // a small output over a long k runs on the tall-k kernel, one workgroup of four waves per
                // (chunk, batch): a thousand workgroups with at least 256 k each.  With eight or more 16x16 tiles the
                // four waves' partial tiles take 32 KB or more of LDS and each workgroup ends with that much of a
                // reduction: half as many workgroups with twice the rows (64x64 over k = 262144: 35.1 -> 30.5 us,
                // 32x64 20.9 -> 19.0; 256 workgroups 39.7)
                MatMulDims t = g;
                const int64_t tk_target = ((g.m + 15) / 16) * ((g.n + 15) / 16) >= 8 ? 512 : 1024;
                t.chunks = std::min<int64_t>(std::max<int64_t>(tk_target / g.batch, 1), g.k / 256);
                if (t.chunks >= 2 && tallk_shape(t)) S = t.chunks;
            }
            if (S < 2) continue;
            const int64_t ktiles = (g.k + 15) / 16;
            const int64_t chunk_tiles = (ktiles + S - 1) / S;
            S = (ktiles + chunk_tiles - 1) / chunk_tiles;
            if (S < 2 || (g.chunks > 1 && S <= g.chunks)) continue;
            const int product = drafts[i].outs[0].node;
            const int64_t out_elems = g.batch * g.m * g.n;
            if (S * out_elems >= ((int64_t)1 << 28)) continue;
            if (g.chunks > 1) {
                // the reference already sums partials: retarget that Reduce
                if (is_graph_output[product]) continue;
                int ri = -1, uses = 0;
                for (size_t j = i + 1; j < drafts.size(); ++j)
                    for (int nd : input_nodes(drafts[j]))
                        if (nd == product) { ++uses; ri = (int)j; }
                if (uses != 1) continue;
                const dsc_kernel_desc& rd = drafts[ri].fk.main.raw();
                if (rd.kind != DSC_KERNEL_REDUCE || rd.reduce_op != DSC_REDUCE_SUM || rd.axis != 0 || !is_identity(rd.inputs[0]) ||
                    element_count(rd.inputs[0].in_shape) != g.chunks * out_elems)
                    continue;
                drafts[ri].fk.main.inputs[0].in_shape.dims[0] = S;
                drafts[ri].fk.main.inputs[0].out_shape.dims[0] = S;
            } else {
                // new internal node for the partials, and a Reduce writing the original node
                const int partials = n_nodes++;
                node_bytes.push_back(0);
                is_graph_output.push_back(false);
                is_graph_input.push_back(false);
                Draft r;
                dsc_kernel_desc rd{};
                rd.kind = DSC_KERNEL_REDUCE;
                rd.shape = drafts[i].fk.main.raw().shape;
                dsc_view v{};
                v.in_shape = rd.shape;
                v.in_shape.dims[0] = S;
                v.out_shape = v.in_shape;
                for (int a = 0; a < v.in_shape.rank; ++a) {
                    v.map_axis[a] = v.in_shape.dims[a] > 1 ? a : -1;
                    v.map_step[a] = v.in_shape.dims[a] > 1 ? 1 : 0;
                }
                rd.n_inputs = 1;
                rd.inputs = &v;
                rd.reduce_op = DSC_REDUCE_SUM;
                rd.axis = 0;
                r.fk = FusedKernel::plain(rd);
                r.params = {partials, product};
                r.outs.push_back(drafts[i].outs[0]);
                r.covers = drafts[i].covers;
                drafts[i].params[drafts[i].fk.outputs[0]] = partials;
                drafts[i].outs[0] = StepOutput{partials, -1, false, 0};
                drafts.insert(drafts.begin() + i + 1, r);
            }
            drafts[i].fk.main.d.shape.dims[0] = S;
            node_bytes[drafts[i].outs[0].node] = (size_t)(S * out_elems) * 4;
            drafts[i].keep_split = true;
        }
    }

    // Pass 0c: a bias gradient is the sum of dZ [K, N] over its rows, and the weight gradient A^T dZ of the same
    // layer reads dZ as its B operand, k chunk by k chunk.  The MFMA kernel then also writes the column sums of
    // the B tiles it loads, one row of partials per chunk, and the Reduce shrinks from K rows to `chunks` rows: one
    // pass over dZ instead of two.  Only large dZ (the Reduce is a launch of its own there).
    void bias_sums_ride_on_weight_gradients() {
        for (size_t ri = 0; ri < drafts.size(); ++ri) {
            if (drafts[ri].fk.main.raw().kind != DSC_KERNEL_REDUCE || drafts[ri].fk.main.raw().reduce_op != DSC_REDUCE_SUM ||
                !drafts[ri].fk.virtuals.empty())
                continue;
            // a sum taken axis by axis ([m, h, w, c] -> [h, w, c] -> [w, c] -> [c]) is looked at as one Reduce; the
            // chain stays as it was when no MatMul takes it
            const std::vector<Draft> before = drafts;
            const int nodes_before = n_nodes;
            bool merged_chain = false;
            while (merge_reduce_step(ri, false)) merged_chain = true;
            bool taken = false;
            struct Restore {
                std::vector<Draft>& drafts;
                const std::vector<Draft>& before;
                const bool& taken;
                const bool& merged;
                ~Restore() {
                    if (!taken && merged) drafts = before;
                }
            } restore{drafts, before, taken, merged_chain};
            (void)nodes_before;
            const dsc_kernel_desc rd = drafts[ri].fk.main.raw();
            const dsc_view rv = rd.inputs[0];
            if (!reads_in_order(rv)) continue;
            // [K, N] with the reduced axis first (size-1 axes aside)
            std::vector<int> big;
            for (int q = 0; q < rv.out_shape.rank; ++q)
                if (rv.out_shape.dims[q] > 1) big.push_back(q);
            if (big.size() != 2 || big[0] != rd.axis) continue;
            const int64_t K = rv.out_shape.dims[big[0]], N = rv.out_shape.dims[big[1]];
            if (K * N < (1 << 22) || N % 4 != 0) continue;
            const int x = drafts[ri].params[0];
            const int r_out = drafts[ri].outs[0].node;
            if (drafts[ri].outs[0].copy_from >= 0) continue;
            // the MatMul that reads x as B = [1, K, N] in order, after the Reduce in the list
            int mi = -1;
            for (size_t q = ri + 1; q < drafts.size() && mi < 0; ++q) {
                const Draft& md = drafts[q];
                const dsc_kernel_desc& m = md.fk.main.raw();
                if (m.kind != DSC_KERNEL_MATMUL || !md.fk.virtuals.empty() || md.fk.has_epilogue || md.fk.colsum_out >= 0) continue;
                if (md.fk.inputs[1].buffer < 0 || md.params[md.fk.inputs[1].buffer] != x) continue;
                const MatMulDims g = matmul_dims(m);
                // B[b][k][n] = x[k][b * n_per_batch + n]: with one batch x read in order, with several (the groups of
                // a convolution) each batch takes its own run of columns
                int64_t base = 0, coef[DSC_MAX_DIM];
                if (g.k != K || g.batch * g.n != N || g.n % 4 != 0 || !affine_form(m.inputs[1], &base, coef) || base != 0 ||
                    element_count(m.inputs[1].in_shape) != K * N || m.inputs[1].out_shape.rank != 3)
                    continue;
                if ((g.batch > 1 && coef[0] != g.n) || coef[1] != N || coef[2] != 1) continue;
                mi = (int)q;
            }
            if (mi < 0) continue;
            // everything between the two that hangs on the Reduce moves behind the MatMul with it
            std::set<int> produced{r_out};
            std::vector<int> moving{(int)ri};
            bool ok = true;
            for (int q = (int)ri + 1; q < mi; ++q) {
                bool dep = false;
                for (int nd : input_nodes(drafts[q]))
                    if (produced.count(nd)) dep = true;
                for (auto& o : drafts[q].outs)
                    if (o.copy_from >= 0 && produced.count(o.copy_from)) dep = true;
                if (!dep) continue;
                for (auto& o : drafts[q].outs) {
                    produced.insert(o.node);
                    if (o.copy_from >= 0) ok = false;
                }
                moving.push_back(q);
            }
            for (int nd : input_nodes(drafts[mi]))
                if (produced.count(nd)) ok = false;
            {
                // a launch that stays put must not take over, in place, a buffer that a delayed launch still reads
                std::set<int> read_by_moving;
                for (int q : moving)
                    for (int nd : input_nodes(drafts[q])) read_by_moving.insert(nd);
                for (int q = (int)ri + 1; q <= mi; ++q) {
                    if (std::find(moving.begin(), moving.end(), q) != moving.end()) continue;
                    for (auto& o : drafts[q].outs)
                        if (o.copy_from >= 0 && read_by_moving.count(o.copy_from)) ok = false;
                }
            }
            if (!ok) continue;
            // nothing that stays may write what a moving launch reads later than it does now... the moving launches
            // only read nodes produced before `ri` or by each other, and nodes are written once: safe to delay them
            const MatMulDims g = matmul_dims(drafts[mi].fk.main.raw());
            const int64_t chunks = drafts[mi].fk.sum_chunks ? 1 : g.chunks;
            Draft trial = drafts[mi];
            const int partials = n_nodes;
            trial.fk.colsum_out = param_index(trial, partials, true);
            trial.fk.outputs.push_back(trial.fk.colsum_out);
            trial.outs.push_back(StepOutput{partials, -1, false, 0});
            {
                Generated probe;
                if (!generate(trial.fk, &probe).empty()) continue;
            }
            // the Reduce over the partials [chunks, N]
            dsc_view pv{};
            pv.in_shape.rank = 2;
            pv.in_shape.dims[0] = chunks;
            pv.in_shape.dims[1] = N;
            pv.out_shape = rd.shape;
            int placed = 0;
            bool shaped = true;
            // the Reduce keeps its output shape; its input gets the same rank with `chunks` on the reduced axis
            if (rd.shape.rank != rv.out_shape.rank) shaped = false;
            for (int q = 0; q < pv.out_shape.rank && shaped; ++q) {
                if (q == rd.axis) {
                    pv.out_shape.dims[q] = chunks;
                    pv.map_axis[q] = chunks > 1 ? 0 : -1;
                    pv.map_step[q] = chunks > 1 ? 1 : 0;
                } else if (pv.out_shape.dims[q] > 1) {
                    if (pv.out_shape.dims[q] != N || placed++) shaped = false;
                    pv.map_axis[q] = 1;
                    pv.map_step[q] = 1;
                } else {
                    pv.map_axis[q] = -1;
                    pv.map_step[q] = 0;
                }
            }
            if (!shaped || placed != 1) continue;
            dsc_kernel_desc nd = rd;
            nd.inputs = &pv;
            if (!validate(nd).empty()) continue;
            taken = true;
            n_nodes++;
            node_bytes.push_back((size_t)(chunks * N) * 4);
            is_graph_output.push_back(false);
            is_graph_input.push_back(false);
            drafts[mi] = trial;
            Draft nr;
            nr.fk = FusedKernel::plain(nd);
            nr.params = {partials, r_out};
            nr.outs = drafts[ri].outs;
            nr.covers = drafts[ri].covers;
            drafts[ri] = nr;
            // move: stable order, right behind the MatMul
            std::vector<Draft> moved;
            for (int q : moving) moved.push_back(drafts[q]);
            for (int q = (int)moving.size() - 1; q >= 0; --q) drafts.erase(drafts.begin() + moving[q]);
            const int at = mi - (int)moving.size() + 1;
            drafts.insert(drafts.begin() + at, moved.begin(), moved.end());
            --ri;  // the slot now holds another draft
        }
    }

    // Pass 0a: chains of Reduces over neighbouring axes (the reference sums a bias gradient back to the bias' shape
    // one axis at a time: [m, h, w, c] -> [1, h, w, c] -> [1, w, c] -> [c], three clusters) become one Reduce over
    // the merged axis: fewer launches.  Only small inputs are merged (the tail of such a chain): a large first
    // Reduce streams its input with every lane on consecutive outputs, which a merged axis over short rows would
    // give up (measured on the ConvNet's conv bias gradients: merged 3666 steps/s, tail only 3950+).  Sums are
    // re-associated (as in every split reduction); max is order-free.
    void merge_reduce_chains() {
        for (size_t i = 0; i < drafts.size(); ++i)
            while (merge_reduce_step(i, true)) {
            }
    }

    // Pass 0b: a Reduce with few outputs and a long axis cannot fill the machine with one thread (or one
    // thread row) per output.  Split the axis k = s * (k/s): a first Reduce over k/s produces s partial rows
    // per output into an internal buffer, a second one combines the s partials (pass 2 inlines it into the
    // consumer when s is small).
    void split_long_reduces() {
        for (size_t i = 0; i < drafts.size(); ++i) {
            const dsc_kernel_desc rd = drafts[i].fk.main.raw();
            if (rd.kind != DSC_KERNEL_REDUCE || !drafts[i].fk.virtuals.empty() || rd.shape.rank >= DSC_MAX_DIM) continue;
            const dsc_view v = rd.inputs[0];
            const int axis = rd.axis;
            const int64_t k = v.out_shape.dims[axis], n_out = element_count(rd.shape);
            if (k < 512 || n_out > 16384 || (k * n_out < (1 << 20) && k < 8192) || v.map_axis[axis] < 0 || needs_clamp(v, v.map_axis[axis])) continue;
            {
                // rows that are contiguous along k are already read by whole wavefronts (one group of lanes per
                // output): with enough outputs that form is bandwidth bound on its own
                int64_t base, coef[DSC_MAX_DIM];
                if (n_out >= 1024 && affine_form(v, &base, coef) && coef[axis] == 1) continue;
            }
            const int64_t want = std::min<int64_t>(2048, std::max<int64_t>(2, (524288 + n_out - 1) / n_out));
            int64_t split = 0;
            for (int64_t c = want; c <= k / 8; ++c)
                if (k % c == 0) { split = c; break; }
            if (split == 0)
                for (int64_t c = std::min(want, k / 8); c >= 2; --c)
                    if (k % c == 0) { split = c; break; }
            if (split < 2) continue;
            // stage 1: view with the axis split in two; output [.., split, 1, ..]
            dsc_view v1 = v;
            v1.out_shape.rank = v.out_shape.rank + 1;
            for (int j = v.out_shape.rank; j > axis; --j) {
                v1.out_shape.dims[j] = v.out_shape.dims[j - 1];
                v1.map_axis[j] = v.map_axis[j - 1];
                v1.map_step[j] = v.map_step[j - 1];
            }
            v1.out_shape.dims[axis] = split;
            v1.map_step[axis] = v.map_step[axis] * (k / split);
            v1.out_shape.dims[axis + 1] = k / split;
            dsc_kernel_desc d1 = rd;
            d1.shape = v1.out_shape;
            d1.shape.dims[axis + 1] = 1;
            d1.inputs = &v1;
            d1.axis = axis + 1;
            // stage 2: reads the partials [.., split, 1, ..] as [.., split, ..] and reduces that axis
            dsc_view v2{};
            v2.in_shape = d1.shape;
            v2.out_shape = rd.shape;
            v2.out_shape.dims[axis] = split;
            for (int j = 0; j < v2.out_shape.rank; ++j) {
                const int in_axis = j <= axis ? j : j + 1;
                v2.map_axis[j] = v2.out_shape.dims[j] > 1 ? in_axis : -1;
                v2.map_step[j] = v2.out_shape.dims[j] > 1 ? 1 : 0;
            }
            dsc_kernel_desc d2 = rd;
            d2.inputs = &v2;
            if (!validate(d1).empty() || !validate(d2).empty()) continue;
            const int partials = n_nodes++;
            node_bytes.push_back((size_t)(split * n_out) * 4);
            is_graph_output.push_back(false);
            is_graph_input.push_back(false);
            Draft second;
            second.fk = FusedKernel::plain(d2);
            second.params = {partials, drafts[i].outs[0].node};
            second.outs.push_back(drafts[i].outs[0]);
            second.covers = drafts[i].covers;
            Draft first;
            first.fk = FusedKernel::plain(d1);
            first.params = {drafts[i].params[0], partials};
            first.outs.push_back(StepOutput{partials, -1, false, 0});
            first.covers = drafts[i].covers;
            first.keep_output = true;
            drafts[i] = first;
            drafts.insert(drafts.begin() + i + 1, second);
            ++i;
        }
    }

    // Pass 1: MatMul (+ Reduce over its split-K partials) (+ per-element consumer as epilogue).
    void matmul_with_reduce_and_epilogue() {
        for (int i = 0; i < (int)drafts.size(); ++i) {
            Draft& mm = drafts[i];
            if (!mm.alive || mm.fk.main.raw().kind != DSC_KERNEL_MATMUL || mm.fk.has_epilogue || mm.keep_split) continue;
            const MatMulDims g = matmul_dims(mm.fk.main.raw());
            int product_node = mm.outs[0].node;
            if (is_graph_output[product_node]) continue;
            int reduce_idx = -1;
            if (g.chunks > 1) {
                // summing all of K in one workgroup per tile serialises the k loop: only do it when the tile
                // grid alone fills the machine, or the partials are few
                const int64_t tile_groups = ((g.m + 127) / 128) * ((g.n + 127) / 128) * g.batch;
                if (tile_groups < 64 && g.chunks > 4) continue;
                auto cons = consumers_of(product_node);
                if (cons.size() != 1) continue;
                Draft& r = drafts[cons[0]];
                const dsc_kernel_desc& rd = r.fk.main.raw();
                if (rd.kind != DSC_KERNEL_REDUCE || rd.reduce_op != DSC_REDUCE_SUM || rd.axis != 0 || !r.fk.virtuals.empty()) continue;
                if (!is_identity(rd.inputs[0]) || element_count(rd.inputs[0].in_shape) != g.chunks * g.batch * g.m * g.n) continue;
                if (taken_in_place_between(i, cons[0], input_nodes(mm))) continue;
                reduce_idx = cons[0];
                product_node = r.outs[0].node;
            }
            // optional epilogue
            int pe_idx = -1, pe_input = -1;
            find_epilogue(i, product_node, g.batch * g.m * g.n, &pe_idx, &pe_input);
            if (reduce_idx < 0 && pe_idx < 0) continue;

            Draft fused;
            fused.fk.main = mm.fk.main;
            fused.fk.sum_chunks = true;
            const int voff = import_virtuals(fused, mm);
            for (auto& s : mm.fk.inputs) fused.fk.inputs.push_back(import_source(fused, mm, s, voff));
            fused.covers = mm.covers;
            if (reduce_idx >= 0) fused.covers.insert(fused.covers.end(), drafts[reduce_idx].covers.begin(), drafts[reduce_idx].covers.end());
            if (pe_idx >= 0) {
                Draft& e = drafts[pe_idx];
                fused.fk.has_epilogue = true;
                fused.fk.epilogue = e.fk.main;
                fused.fk.epilogue_product_input = pe_input;
                const int eoff = import_virtuals(fused, e);
                for (int k = 0; k < (int)e.fk.inputs.size(); ++k) {
                    if (k == pe_input) fused.fk.epilogue_inputs.push_back(Source{});
                    else fused.fk.epilogue_inputs.push_back(import_source(fused, e, e.fk.inputs[k], eoff));
                }
                for (auto& o : e.outs) {
                    fused.fk.outputs.push_back(param_index(fused, o.node, true));
                    fused.outs.push_back(o);
                }
                fused.covers.insert(fused.covers.end(), e.covers.begin(), e.covers.end());
                compact(fused);
                mm.alive = false;
                if (reduce_idx >= 0) drafts[reduce_idx].alive = false;
                drafts[pe_idx] = fused;  // runs where the per-element cluster ran: all of its inputs exist by then
            } else {
                Draft& r = drafts[reduce_idx];
                fused.fk.outputs.push_back(param_index(fused, r.outs[0].node, true));
                fused.outs.push_back(r.outs[0]);
                compact(fused);
                mm.alive = false;
                drafts[reduce_idx] = fused;
            }
        }
    }

    // Pass 1c: the data gradient of a stride-1 convolution arrives as MatMul (dC x filter^T, one row of
    // fh*fw*c window elements per output pixel) -> reshape copy -> WindowsToImage (sum of the windows that
    // cover each pixel of the padded image).  With few channels that is the product written out nine times
    // over and read back.  Run it as one MatMul over the padded image instead: row = padded pixel,
    // k = (fy, fx, oc), A'[pixel, k] = dC[pixel - tap, oc] where that output pixel exists (else 0),
    // B'[k, c] = filter[oc, fy, fx, c]; both operands are fused producers of the MatMul, nothing in between
    // is written.
    void conv_data_gradient() {
        for (int i = 0; i < (int)drafts.size(); ++i) {
            static const bool enabled = !(std::getenv("DSC_FUSE_DGRAD") && std::getenv("DSC_FUSE_DGRAD")[0] == '0');
            if (!enabled) break;
            Draft& mm = drafts[i];
            const dsc_kernel_desc& md = mm.fk.main.raw();
            if (!mm.alive || md.kind != DSC_KERNEL_MATMUL || !mm.fk.virtuals.empty() || mm.fk.has_epilogue || mm.keep_split ||
                md.output_mode != DSC_MATMUL_BATCHES)
                continue;
            const MatMulDims g = matmul_dims(md);
            if (g.chunks != 1 || is_graph_output[mm.outs[0].node] || mm.outs[0].copy_from >= 0) continue;
            auto cons = consumers_of(mm.outs[0].node);
            if (cons.size() != 1 || cons[0] <= i) continue;
            int copy_idx = -1, w_idx = cons[0];
            {
                const Draft& c = drafts[w_idx];
                const dsc_kernel_desc& cd = c.fk.main.raw();
                if (cd.kind == DSC_KERNEL_PER_ELEMENT) {
                    if (!c.fk.virtuals.empty() || c.fk.has_epilogue || cd.n_outputs != 1 || cd.n_inputs != 1 || cd.n_ops > 2 ||
                        cd.ops[0].kind != DSC_PE_LOAD || (cd.n_ops == 2 && !(cd.ops[1].kind == DSC_PE_UNARY && cd.ops[1].op == DSC_UN_MOV)) ||
                        any_clamp(cd.inputs[0]) || is_graph_output[c.outs[0].node] || c.outs[0].copy_from >= 0)
                        continue;
                    auto cons2 = consumers_of(c.outs[0].node);
                    if (cons2.size() != 1 || cons2[0] <= w_idx) continue;
                    copy_idx = w_idx;
                    w_idx = cons2[0];
                }
            }
            Draft& w = drafts[w_idx];
            const dsc_kernel_desc& wd = w.fk.main.raw();
            if (wd.kind != DSC_KERNEL_WINDOWS_TO_IMAGE || !w.fk.virtuals.empty() || w.fk.has_epilogue || wd.stride_w != 1 || wd.stride_h != 1 ||
                wd.shape.rank != 4 || w.outs[0].copy_from >= 0 || any_clamp(wd.inputs[0]))
                continue;
            const dsc_view& wv = wd.inputs[0];
            const int64_t IMG = wv.out_shape.dims[0], OH = wv.out_shape.dims[1], OW = wv.out_shape.dims[2], G = wv.out_shape.dims[3];
            const int64_t FH = wv.out_shape.dims[4], FW = wv.out_shape.dims[5], C = wv.out_shape.dims[6];
            const int64_t PH = OH + FH - 1, PW = OW + FW - 1, K = g.k;
            if (g.batch != G || g.m != IMG * OH * OW || g.n != FH * FW * C) continue;
            // worth it where the row-per-thread kernel runs: few channels on both sides
            if (C > 32 || FH * FW * K > 256 || FH * FW * K * C > 8192 || FH * FW < 2) continue;
            if (IMG * PH * PW * G * FH * FW * K >= ((int64_t)1 << 31)) continue;
            // the chain must hand element (img, oy, ox, g, fy, fx, c) of the windows exactly product element
            // [g][(img, oy, ox)][(fy, fx, c)]: checked on every window element of the first, middle and last image
            bool chain_ok = true;
            for (int64_t img : {(int64_t)0, IMG / 2, IMG - 1}) {
                for (int64_t rest = 0; rest < OH * OW * G * FH * FW * C && chain_ok; ++rest) {
                    int64_t c7[7], r = rest;
                    c7[6] = r % C; r /= C;
                    c7[5] = r % FW; r /= FW;
                    c7[4] = r % FH; r /= FH;
                    c7[3] = r % G; r /= G;
                    c7[2] = r % OW; r /= OW;
                    c7[1] = r;
                    c7[0] = img;
                    int64_t idx = view_index(wv, c7);
                    if (copy_idx >= 0) {
                        const dsc_view& cv = drafts[copy_idx].fk.main.raw().inputs[0];
                        int64_t cc[DSC_MAX_DIM], q = idx;
                        for (int a = cv.out_shape.rank - 1; a >= 0; --a) {
                            cc[a] = q % cv.out_shape.dims[a];
                            q /= cv.out_shape.dims[a];
                        }
                        idx = view_index(cv, cc);
                    }
                    const int64_t want = c7[3] * g.m * g.n + ((img * OH + c7[1]) * OW + c7[2]) * g.n + (c7[4] * FW + c7[5]) * C + c7[6];
                    if (idx != want) chain_ok = false;
                }
            }
            if (!chain_ok) continue;
            if (taken_in_place_between(i, w_idx, input_nodes(mm))) continue;

            // First choice: the dedicated kernel (image tile in LDS), which also takes the Unpads that fold the
            // padding border back (one along the image rows, one along the columns, in either order).
            {
                FusedKernel::ConvDgrad cv;
                cv.on = true;
                cv.img = IMG; cv.oh = OH; cv.ow = OW; cv.g = G; cv.fh = FH; cv.fw = FW; cv.c = C;
                std::vector<int> unpads;
                int last = w_idx;
                for (int step = 0; step < 2; ++step) {
                    if (is_graph_output[drafts[last].outs[0].node]) break;
                    auto uc = consumers_of(drafts[last].outs[0].node);
                    if (uc.size() != 1 || uc[0] <= last) break;
                    const Draft& u = drafts[uc[0]];
                    const dsc_kernel_desc& ud = u.fk.main.raw();
                    if (ud.kind != DSC_KERNEL_UNPAD || !u.fk.virtuals.empty() || u.fk.has_epilogue || u.outs[0].copy_from >= 0 ||
                        ud.shape.rank != 4 || !is_identity(ud.inputs[0]) || ud.pad < 1)
                        break;
                    if (ud.axis == 1 && cv.pad_h == 0) {
                        cv.pad_h = ud.pad;
                        if (step == 0) cv.rows_first = 1;
                    } else if (ud.axis == 2 && cv.pad_w == 0) {
                        cv.pad_w = ud.pad;
                        if (step == 0) cv.rows_first = 0;
                    } else {
                        break;
                    }
                    unpads.push_back(uc[0]);
                    last = uc[0];
                }
                const bool direct = !(flags & DSC_SCHEDULE_NO_CONV_KERNELS);
                if (direct && conv_dgrad_fits(cv, K) && !taken_in_place_between(i, last, input_nodes(mm))) {
                    Draft fused;
                    fused.fk.main = mm.fk.main;
                    fused.fk.dgrad = cv;
                    for (auto& src : mm.fk.inputs) fused.fk.inputs.push_back(import_source(fused, mm, src, 0));
                    fused.fk.outputs.push_back(param_index(fused, drafts[last].outs[0].node, true));
                    fused.outs.push_back(drafts[last].outs[0]);
                    fused.covers = mm.covers;
                    for (int j : std::vector<int>{copy_idx, w_idx})
                        if (j >= 0) fused.covers.insert(fused.covers.end(), drafts[j].covers.begin(), drafts[j].covers.end());
                    for (int j : unpads) fused.covers.insert(fused.covers.end(), drafts[j].covers.begin(), drafts[j].covers.end());
                    compact(fused);
                    mm.alive = false;
                    if (copy_idx >= 0) drafts[copy_idx].alive = false;
                    drafts[w_idx].alive = false;
                    for (int j : unpads) drafts[j].alive = false;
                    drafts[last] = fused;
                    continue;
                }
            }

            const dsc_view va = md.inputs[0], vb = md.inputs[1];
            const int64_t Mp = IMG * PH * PW, Kp = FH * FW * K;
            // A': out [G, IMG, PH, PW, FH, FW, K] onto dC
            dsc_view wa = va;
            wa.out_shape.rank = 7;
            const int64_t a_dims[7] = {G, IMG, PH, PW, FH, FW, K};
            const int a_from[7] = {0, 1, 1, 1, 1, 1, 2};
            const int64_t a_scale[7] = {1, OH * OW, OW, 1, -OW, -1, 1};
            for (int j = 0; j < 7; ++j) {
                wa.out_shape.dims[j] = a_dims[j];
                wa.map_axis[j] = va.map_axis[a_from[j]];
                wa.map_step[j] = va.map_axis[a_from[j]] >= 0 ? va.map_step[a_from[j]] * a_scale[j] : 0;
            }
            auto coord_view = [&](int pos_axis, int tap_axis, int64_t extent, int64_t taps) {
                dsc_view v{};
                v.in_shape.rank = 1;
                v.in_shape.dims[0] = extent + 2 * taps - 2;
                v.in_offset[0] = taps - 1;
                v.out_shape = wa.out_shape;
                for (int j = 0; j < 7; ++j) { v.map_axis[j] = -1; v.map_step[j] = 0; }
                v.map_axis[pos_axis] = 0; v.map_step[pos_axis] = 1;
                v.map_axis[tap_axis] = 0; v.map_step[tap_axis] = -1;
                return v;
            };
            const dsc_view builtin[2] = {coord_view(2, 4, OH, FH), coord_view(3, 5, OW, FW)};
            const dsc_pe_op a_ops[12] = {
                pe_op(DSC_PE_LOAD), pe_op(DSC_PE_COORD), pe_op(DSC_PE_COORD),
                pe_literal((float)(FH - 2)), pe_literal((float)(OH + FH - 1)), pe_literal((float)(FW - 2)), pe_literal((float)(OW + FW - 1)),
                pe_literal(0.f),
                pe_op(DSC_PE_SELECT, DSC_CMP_GT, 1, 3, 0, 7), pe_op(DSC_PE_SELECT, DSC_CMP_GT, 4, 1, 8, 7),
                pe_op(DSC_PE_SELECT, DSC_CMP_GT, 2, 5, 9, 7), pe_op(DSC_PE_SELECT, DSC_CMP_GT, 6, 2, 10, 7)};
            dsc_pe_op a_ops_m[12];
            std::memcpy(a_ops_m, a_ops, sizeof a_ops);
            a_ops_m[2].view_index = 1;
            const int32_t a_out = 11;
            dsc_kernel_desc ad{};
            ad.kind = DSC_KERNEL_PER_ELEMENT;
            ad.shape.rank = 1;
            ad.shape.dims[0] = G * Mp * Kp;
            ad.n_inputs = 1; ad.inputs = &wa;
            ad.n_ops = 12; ad.ops = a_ops_m;
            ad.n_outputs = 1; ad.outputs = &a_out;
            ad.n_builtin_views = 2; ad.builtin_views = builtin;
            // B': out [G, FH, FW, K, C] onto the filter operand
            dsc_view wb = vb;
            wb.out_shape.rank = 5;
            const int64_t b_dims[5] = {G, FH, FW, K, C};
            const int b_from[5] = {0, 2, 2, 1, 2};
            const int64_t b_scale[5] = {1, FW * C, C, 1, 1};
            for (int j = 0; j < 5; ++j) {
                wb.out_shape.dims[j] = b_dims[j];
                wb.map_axis[j] = vb.map_axis[b_from[j]];
                wb.map_step[j] = vb.map_axis[b_from[j]] >= 0 ? vb.map_step[b_from[j]] * b_scale[j] : 0;
            }
            for (int j = 5; j < DSC_MAX_DIM; ++j) { wb.out_shape.dims[j] = 0; wb.map_axis[j] = -1; wb.map_step[j] = 0; }
            const dsc_pe_op b_ops[1] = {pe_op(DSC_PE_LOAD)};
            const int32_t b_out = 0;
            dsc_kernel_desc bd{};
            bd.kind = DSC_KERNEL_PER_ELEMENT;
            bd.shape.rank = 1;
            bd.shape.dims[0] = G * Kp * C;
            bd.n_inputs = 1; bd.inputs = &wb;
            bd.n_ops = 1; bd.ops = b_ops;
            bd.n_outputs = 1; bd.outputs = &b_out;
            // the MatMul over the padded image, Rows mode: C[(img, py, px)][g][c]
            const dsc_view m_in[2] = {identity_view({G, Mp, Kp}), identity_view({G, Kp, C})};
            dsc_kernel_desc nd{};
            nd.kind = DSC_KERNEL_MATMUL;
            nd.shape.rank = 4;
            nd.shape.dims[0] = 1; nd.shape.dims[1] = Mp; nd.shape.dims[2] = G; nd.shape.dims[3] = C;
            nd.output_mode = DSC_MATMUL_ROWS;
            nd.n_inputs = 2; nd.inputs = m_in;
            if (!validate(ad).empty() || !validate(bd).empty() || !validate(nd).empty()) continue;

            Draft fused;
            fused.fk.main = KernelDesc(nd);
            Virtual va_v, vb_v;
            va_v.pe = KernelDesc(ad);
            va_v.out_op = a_out;
            va_v.inputs.push_back(Source{param_index(fused, mm.params[mm.fk.inputs[0].buffer], false), -1});
            vb_v.pe = KernelDesc(bd);
            vb_v.out_op = b_out;
            vb_v.inputs.push_back(Source{param_index(fused, mm.params[mm.fk.inputs[1].buffer], false), -1});
            fused.fk.virtuals.push_back(va_v);
            fused.fk.virtuals.push_back(vb_v);
            Source sa, sb;
            sa.virt = 0;
            sb.virt = 1;
            fused.fk.inputs = {sa, sb};
            fused.fk.outputs.push_back(param_index(fused, w.outs[0].node, true));
            fused.outs.push_back(w.outs[0]);
            fused.covers = mm.covers;
            if (copy_idx >= 0) fused.covers.insert(fused.covers.end(), drafts[copy_idx].covers.begin(), drafts[copy_idx].covers.end());
            fused.covers.insert(fused.covers.end(), w.covers.begin(), w.covers.end());
            compact(fused);
            mm.alive = false;
            if (copy_idx >= 0) drafts[copy_idx].alive = false;
            drafts[w_idx] = fused;
        }
    }

    // Pass 1d: the forward of a stride-1 convolution arrives as a copy cluster that writes the im2col of the
    // (replicate-padded) image, and a MatMul over it.  The dedicated kernel reads the image itself.  The geometry
    // is a hypothesis (filter height from the divisors of k / c, padding from the output size) that is then
    // checked on every (pixel, k) of three images against the addresses the copy's view really produces.
    void conv_forward() {
        for (int i = 0; i < (int)drafts.size(); ++i) {
            static const bool enabled = !(std::getenv("DSC_FUSE_CONV_FWD") && std::getenv("DSC_FUSE_CONV_FWD")[0] == '0');
            if (!enabled || (flags & DSC_SCHEDULE_NO_CONV_KERNELS)) break;
            Draft& mm = drafts[i];
            const dsc_kernel_desc& md = mm.fk.main.raw();
            if (!mm.alive || md.kind != DSC_KERNEL_MATMUL || !mm.fk.virtuals.empty() || mm.keep_split || mm.fk.colsum_out >= 0 ||
                mm.fk.dgrad.on || mm.fk.inputs[0].buffer < 0)
                continue;
            const MatMulDims g = matmul_dims(md);
            if (g.chunks != 1 || g.n > 16) continue;
            const int a_node = mm.params[mm.fk.inputs[0].buffer];
            int ci = -1;
            for (int q = 0; q < i; ++q)
                if (drafts[q].alive && !drafts[q].outs.empty() && drafts[q].outs[0].node == a_node) ci = q;
            if (ci < 0) continue;
            const Draft& cp = drafts[ci];
            const dsc_kernel_desc& cd = cp.fk.main.raw();
            if (cd.kind != DSC_KERNEL_PER_ELEMENT || !cp.fk.virtuals.empty() || cp.fk.has_epilogue || cd.n_outputs != 1 || cd.n_inputs != 1 ||
                cd.n_ops > 2 || cd.ops[0].kind != DSC_PE_LOAD || (cd.n_ops == 2 && !(cd.ops[1].kind == DSC_PE_UNARY && cd.ops[1].op == DSC_UN_MOV)) ||
                is_graph_output[a_node] || cp.outs[0].copy_from >= 0 || cp.fk.inputs[0].buffer < 0)
                continue;
            // (the filter gradient reads the same copy: it stays for that reader, which takes it as a fused producer)
            const bool only_reader = consumers_of(a_node).size() == 1;
            const dsc_view& cvw = cd.inputs[0];  // element of the copy -> element of the image
            const dsc_view& av = md.inputs[0];   // (batch, row, k) -> element of the copy
            if (cvw.in_shape.rank != 4 || any_clamp(av)) continue;
            const int64_t IMG = cvw.in_shape.dims[0], H = cvw.in_shape.dims[1], W = cvw.in_shape.dims[2], GC = cvw.in_shape.dims[3];
            const int64_t G = g.batch;
            if (GC % G != 0 || g.m % IMG != 0) continue;
            const int64_t C = GC / G, PIX = g.m / IMG;
            if (g.k % C != 0) continue;
            const int64_t taps = g.k / C;
            auto image_index = [&](int64_t cb, int64_t cm, int64_t ck) {
                const int64_t c3[3] = {cb, cm, ck};
                int64_t idx = view_index(av, c3);
                int64_t cc[DSC_MAX_DIM];
                for (int a = cvw.out_shape.rank - 1; a >= 0; --a) {
                    cc[a] = idx % cvw.out_shape.dims[a];
                    idx /= cvw.out_shape.dims[a];
                }
                return view_index_clamped(cvw, cc);
            };
            FusedKernel::ConvFwd found;
            for (int64_t FH = 1; FH <= taps && !found.on; ++FH) {
                if (taps % FH != 0) continue;
                const int64_t FW = taps / FH;
                for (int64_t ph = 0; ph <= FH && !found.on; ++ph) {
                    const int64_t OH = H + 2 * ph - FH + 1;
                    if (OH < 1 || PIX % OH != 0) continue;
                    const int64_t OW = PIX / OH;
                    if ((OW + FW - 1 - W) % 2 != 0) continue;
                    const int64_t pw = (OW + FW - 1 - W) / 2;
                    if (pw < 0 || pw > FW) continue;
                    auto clampv = [](int64_t v, int64_t hi) { return v < 0 ? 0 : (v > hi ? hi : v); };
                    bool ok = true;
                    for (int64_t img : {(int64_t)0, IMG / 2, IMG - 1}) {
                        for (int64_t p = 0; p < PIX && ok; ++p)
                            for (int64_t cb = 0; cb < G && ok; ++cb)
                                for (int64_t ck = 0; ck < g.k && ok; ++ck) {
                                    const int64_t tap = ck / C, ch = ck % C;
                                    const int64_t y = clampv(p / OW + tap / FW - ph, H - 1), x = clampv(p % OW + tap % FW - pw, W - 1);
                                    const int64_t want = ((img * H + y) * W + x) * GC + cb * C + ch;
                                    if (image_index(cb, img * PIX + p, ck) != want) ok = false;
                                }
                    }
                    if (!ok) continue;
                    found.on = true;
                    found.img = IMG; found.h = H; found.w = W; found.g = G; found.c = C;
                    found.fh = FH; found.fw = FW; found.oh = OH; found.ow = OW; found.pad_h = ph; found.pad_w = pw;
                }
            }
            if (!found.on) continue;
            const int image_node = cp.params[cp.fk.inputs[0].buffer];
            conv_sites.push_back(ConvSite{ci, a_node, image_node, found, av});
            if (!conv_fwd_fits(found, g.n)) continue;
            if (taken_in_place_between(ci, i, {image_node})) continue;
            Draft fused = mm;
            fused.fk.cfwd = found;
            fused.fk.inputs[0] = Source{};
            fused.fk.inputs[0].buffer = param_index(fused, image_node, false);
            {
                Generated probe;
                if (!generate(fused.fk, &probe).empty()) continue;
            }
            compact(fused);
            if (only_reader) {
                fused.covers.insert(fused.covers.end(), cp.covers.begin(), cp.covers.end());
                drafts[ci].alive = false;
            }
            drafts[i] = fused;
        }
    }

    // The filter gradient of a convolution whose input needs no gradient (a first layer): the tall-k MatMul
    // im2col^T x dC becomes the convolution backward kernel without its data-gradient phase.  dC may later become a
    // fused producer (pass 2): with no data gradient to compute from it, nothing else needs it in memory.
    void filter_gradient_alone(const ConvSite& site) {
        static const bool enabled = !(std::getenv("DSC_FUSE_CONV_WGRAD") && std::getenv("DSC_FUSE_CONV_WGRAD")[0] == '0');
        if (!enabled) return;
        const FusedKernel::ConvFwd& f = site.geo;
        int ti = -1;
        for (int q = 0; q < (int)drafts.size() && ti < 0; ++q) {
            const Draft& T = drafts[q];
            const dsc_kernel_desc& td = T.fk.main.raw();
            if (!T.alive || td.kind != DSC_KERNEL_MATMUL || !T.keep_split || !T.fk.virtuals.empty() || T.fk.has_epilogue ||
                td.output_mode != DSC_MATMUL_BATCHES || T.fk.dgrad.on || T.fk.cfwd.on || T.fk.inputs[0].buffer < 0 || T.fk.inputs[1].buffer < 0)
                continue;
            if (T.params[T.fk.inputs[0].buffer] != site.a_node) continue;
            const MatMulDims gt = matmul_dims(td);
            if (gt.batch != f.g || gt.m != f.fh * f.fw * f.c || gt.k != f.img * f.oh * f.ow || gt.n > 16 || gt.n % 4 != 0) continue;
            // its A is the forward's A transposed; its B is read as [g][(img, oy, ox)][oc] with nothing clamped
            int64_t bt, bf, ct[DSC_MAX_DIM], cf[DSC_MAX_DIM];
            if (!affine_form(td.inputs[0], &bt, ct) || !affine_form(site.a_view, &bf, cf) || bt != bf || ct[1] != cf[2] || ct[2] != cf[1] ||
                (gt.batch > 1 && ct[0] != cf[0]))
                continue;
            if (any_clamp(td.inputs[1])) continue;
            ti = q;
        }
        if (ti < 0) return;
        Draft& T = drafts[ti];
        const MatMulDims gt = matmul_dims(T.fk.main.raw());
        const bool bias = T.fk.colsum_out >= 0;
        if ((int)T.outs.size() != (bias ? 2 : 1) || T.outs[0].copy_from >= 0 || is_graph_output[T.outs[0].node]) return;
        auto only_reduce_of = [&](int node) {
            auto cons = consumers_of(node);
            if (cons.size() != 1 || cons[0] <= ti) return -1;
            const Draft& r = drafts[cons[0]];
            const dsc_kernel_desc& rd = r.fk.main.raw();
            if (rd.kind != DSC_KERNEL_REDUCE || rd.reduce_op != DSC_REDUCE_SUM || !r.fk.virtuals.empty() || r.fk.has_epilogue) return -1;
            return cons[0];
        };
        const int r1 = only_reduce_of(T.outs[0].node);
        if (r1 < 0) return;
        {
            const dsc_kernel_desc& rd = drafts[r1].fk.main.raw();
            if (rd.axis != 0 || !is_identity(rd.inputs[0]) || rd.inputs[0].in_shape.dims[0] != gt.chunks ||
                element_count(rd.inputs[0].in_shape) != gt.chunks * gt.batch * gt.m * gt.n)
                return;
        }
        int r2 = -1;
        if (bias) {
            if (is_graph_output[T.outs[1].node]) return;
            r2 = only_reduce_of(T.outs[1].node);
            if (r2 < 0) return;
            const dsc_kernel_desc& rd = drafts[r2].fk.main.raw();
            const dsc_view& pv = rd.inputs[0];
            if (pv.in_shape.rank != 2 || pv.in_shape.dims[0] != gt.chunks || pv.in_shape.dims[1] != gt.batch * gt.n ||
                pv.out_shape.dims[rd.axis] != gt.chunks || (gt.chunks > 1 && pv.map_axis[rd.axis] != 0))
                return;
        }
        // the image must still be what the forward convolution read
        {
            bool image_ok = true;
            for (int q = 0; q <= ti && image_ok; ++q) {
                if (!drafts[q].alive) continue;
                for (auto& o : drafts[q].outs)
                    if (o.copy_from == site.image_node) image_ok = false;
            }
            if (!image_ok) return;
        }
        // bands of at least four output rows: the tiles of a band are small enough for eight workgroups to share a CU,
        // which is what hides each workgroup's fill -> barrier -> products -> reduction chain
        const int64_t bands = (f.oh % 4 == 0 && f.oh >= 16) ? 4 : (f.oh % 2 == 0 && f.oh >= 8) ? 2 : 1;
        // image sets: about a thousand workgroups, a multiple of eight sets (measured on the ConvNet's first
        // convolution together with the Reduce over the partials that follows: 4096 workgroups 5354 steps/s, 2048
        // 5350, 1024 5379, 512 clearly slower)
        const int64_t per_group = std::max<int64_t>(8, 1024 / (f.g * bands));
        const int64_t images_per_set = (f.img + per_group - 1) / per_group;
        const int64_t sets = ((f.img + images_per_set - 1) / images_per_set + 7) / 8 * 8;
        Draft fused = T;
        fused.keep_split = false;
        FusedKernel::ConvDgrad& cv = fused.fk.dgrad;
        cv.on = true;
        cv.img = f.img; cv.oh = f.oh; cv.ow = f.ow; cv.g = f.g; cv.fh = f.fh; cv.fw = f.fw; cv.c = f.c;
        cv.pad_h = f.pad_h; cv.pad_w = f.pad_w;
        cv.wgrad = true;
        cv.wgrad_only = true;
        cv.bias = bias;
        cv.chunks = sets;
        cv.bands = bands;
        const int64_t partials = sets * cv.bands;
        fused.fk.colsum_out = -1;
        fused.fk.outputs.clear();
        for (auto& o : T.outs) fused.fk.outputs.push_back(param_index(fused, o.node, true));
        {
            Source xs;
            xs.buffer = param_index(fused, site.image_node, false);
            fused.fk.inputs[0] = xs;  // the im2col operand of the MatMul is read from the image itself
            fused.fk.inputs.push_back(xs);
        }
        compact(fused);
        if (!conv_bwd_fits(fused.fk.dgrad, gt.n)) return;
        {
            Generated probe;
            if (!generate(fused.fk, &probe).empty()) return;
        }
        node_bytes[T.outs[0].node] = (size_t)(partials * gt.batch * gt.m * gt.n) * 4;
        drafts[r1].fk.main.inputs[0].in_shape.dims[0] = partials;
        drafts[r1].fk.main.inputs[0].out_shape.dims[0] = partials;
        if (bias) {
            node_bytes[T.outs[1].node] = (size_t)(partials * gt.batch * gt.n) * 4;
            const int axis = drafts[r2].fk.main.raw().axis;
            dsc_view& pv = drafts[r2].fk.main.inputs[0];
            pv.in_shape.dims[0] = partials;
            pv.out_shape.dims[axis] = partials;
            pv.map_axis[axis] = 0;
            pv.map_step[axis] = 1;
        }
        drafts[ti] = fused;
        if (drafts[site.copy_idx].alive && consumers_of(site.a_node).empty()) {
            drafts[ti].covers.insert(drafts[ti].covers.end(), drafts[site.copy_idx].covers.begin(), drafts[site.copy_idx].covers.end());
            drafts[site.copy_idx].alive = false;
        }
    }

    // Pass 1e: both gradients of a convolution in one kernel.  The data-gradient kernel (pass 1c) holds dC of an
    // image in LDS; the filter gradient im2col^T x dC of the same convolution -- by now a MatMul whose k (images x
    // output pixels) pass 0 split into many chunks, summed by a Reduce, possibly with the bias gradient's column
    // sums riding on it (pass 0c) -- needs the same dC and the image's input tile.  The kernel takes both: its
    // workgroups each own a set of images, and the partial products (and column sums) come out once per set, in
    // the layout the MatMul's chunks had, so the Reduces stay and only learn the new number of partials.
    void conv_backward() {
        for (const ConvSite& site : conv_sites) {
            static const bool enabled = !(std::getenv("DSC_FUSE_CONV_BWD") && std::getenv("DSC_FUSE_CONV_BWD")[0] == '0');
            if (!enabled || (flags & DSC_SCHEDULE_SPLIT_CONV_GRADS)) break;
            const FusedKernel::ConvFwd& f = site.geo;
            int di = -1;
            for (int q = 0; q < (int)drafts.size() && di < 0; ++q) {
                const Draft& D = drafts[q];
                if (!D.alive || !D.fk.dgrad.on || D.fk.dgrad.wgrad || D.fk.inputs[0].buffer < 0) continue;
                const FusedKernel::ConvDgrad& cv = D.fk.dgrad;
                if (cv.img == f.img && cv.oh == f.oh && cv.ow == f.ow && cv.g == f.g && cv.fh == f.fh && cv.fw == f.fw && cv.c == f.c &&
                    cv.pad_h == f.pad_h && cv.pad_w == f.pad_w)
                    di = q;
            }
            if (di < 0) {
                filter_gradient_alone(site);
                continue;
            }
            const MatMulDims gd = matmul_dims(drafts[di].fk.main.raw());  // [g][(img, oy, ox)][oc] x [g][oc][(fy, fx, c)]
            const int dc_node = drafts[di].params[drafts[di].fk.inputs[0].buffer];
            int ti = -1;
            for (int q = 0; q < (int)drafts.size() && ti < 0; ++q) {
                const Draft& T = drafts[q];
                const dsc_kernel_desc& td = T.fk.main.raw();
                if (!T.alive || q == di || td.kind != DSC_KERNEL_MATMUL || !T.keep_split || !T.fk.virtuals.empty() || T.fk.has_epilogue ||
                    td.output_mode != DSC_MATMUL_BATCHES || T.fk.dgrad.on || T.fk.cfwd.on || T.fk.inputs[0].buffer < 0 || T.fk.inputs[1].buffer < 0)
                    continue;
                if (T.params[T.fk.inputs[0].buffer] != site.a_node || T.params[T.fk.inputs[1].buffer] != dc_node) continue;
                const MatMulDims gt = matmul_dims(td);
                if (gt.batch != f.g || gt.m != f.fh * f.fw * f.c || gt.n != gd.k || gt.k != gd.m) continue;
                // its A is the forward's A transposed, its B is the data gradient's A: same elements of the same nodes
                int64_t bt, bf, ct[DSC_MAX_DIM], cf[DSC_MAX_DIM];
                if (!affine_form(td.inputs[0], &bt, ct) || !affine_form(site.a_view, &bf, cf) || bt != bf || ct[1] != cf[2] || ct[2] != cf[1] ||
                    (gt.batch > 1 && ct[0] != cf[0]))
                    continue;
                if (!affine_form(td.inputs[1], &bt, ct) || !affine_form(drafts[di].fk.main.raw().inputs[0], &bf, cf) || bt != bf || ct[1] != cf[1] ||
                    ct[2] != cf[2] || (gt.batch > 1 && ct[0] != cf[0]))
                    continue;
                ti = q;
            }
            if (ti < 0) continue;
            Draft& T = drafts[ti];
            const MatMulDims gt = matmul_dims(T.fk.main.raw());
            const bool bias = T.fk.colsum_out >= 0;
            if ((int)T.outs.size() != (bias ? 2 : 1) || T.outs[0].copy_from >= 0 || is_graph_output[T.outs[0].node]) continue;
            // the Reduces over the partials and over the column sums
            auto only_reduce_of = [&](int node) {
                auto cons = consumers_of(node);
                if (cons.size() != 1 || cons[0] <= ti) return -1;
                const Draft& r = drafts[cons[0]];
                const dsc_kernel_desc& rd = r.fk.main.raw();
                if (rd.kind != DSC_KERNEL_REDUCE || rd.reduce_op != DSC_REDUCE_SUM || !r.fk.virtuals.empty() || r.fk.has_epilogue) return -1;
                return cons[0];
            };
            const int r1 = only_reduce_of(T.outs[0].node);
            if (r1 < 0) continue;
            {
                const dsc_kernel_desc& rd = drafts[r1].fk.main.raw();
                if (rd.axis != 0 || !is_identity(rd.inputs[0]) || rd.inputs[0].in_shape.dims[0] != gt.chunks ||
                    element_count(rd.inputs[0].in_shape) != gt.chunks * gt.batch * gt.m * gt.n)
                    continue;
            }
            int r2 = -1;
            if (bias) {
                if (is_graph_output[T.outs[1].node]) continue;
                r2 = only_reduce_of(T.outs[1].node);
                if (r2 < 0) continue;
                const dsc_kernel_desc& rd = drafts[r2].fk.main.raw();
                const dsc_view& pv = rd.inputs[0];
                if (pv.in_shape.rank != 2 || pv.in_shape.dims[0] != gt.chunks || pv.in_shape.dims[1] != gt.batch * gt.n ||
                    pv.out_shape.dims[rd.axis] != gt.chunks || (gt.chunks > 1 && pv.map_axis[rd.axis] != 0))
                    continue;
            }
            const int at = std::min(di, ti), other = std::max(di, ti);
            {
                std::vector<int> reads = input_nodes(drafts[di]);
                reads.push_back(site.image_node);
                if (taken_in_place_between(at, other, reads)) continue;
            }
            // image sets: about a thousand workgroups, a multiple of eight sets
            // (measured on the ConvNet's second convolution, 2000 image-groups: ~1000 workgroups 38.8 us, ~2000 43.9, ~500 43.1)
            Draft fused = drafts[di];
            fused.fk.dgrad.wgrad = true;
            fused.fk.dgrad.bias = bias;
            auto sets_for = [&](int64_t workgroups) {
                const int64_t per_group = std::max<int64_t>(8, workgroups / f.g);
                const int64_t images_per_set = (f.img + per_group - 1) / per_group;
                return ((f.img + images_per_set - 1) / images_per_set + 7) / 8 * 8;
            };
            // with loader waves two workgroups of eight waves share a CU: one round of 512 workgroups, whose sets are
            // long enough for the fills to run beside the matrix phases
            int64_t sets = sets_for(512);
            fused.fk.dgrad.chunks = sets;
            if (!conv_bwd_loader_waves(fused.fk)) sets = sets_for(1024);
            fused.fk.dgrad.chunks = sets;
            {
                Source xs;
                xs.buffer = param_index(fused, site.image_node, false);
                fused.fk.inputs.push_back(xs);
            }
            for (auto& o : T.outs) {
                fused.fk.outputs.push_back(param_index(fused, o.node, true));
                fused.outs.push_back(o);
            }
            if (!conv_bwd_fits(fused.fk.dgrad, gd.k)) continue;
            {
                Generated probe;
                if (!generate(fused.fk, &probe).empty()) continue;
            }
            fused.covers.insert(fused.covers.end(), T.covers.begin(), T.covers.end());
            // the Reduces sum `sets` partials now
            node_bytes[T.outs[0].node] = (size_t)(sets * gt.batch * gt.m * gt.n) * 4;
            drafts[r1].fk.main.inputs[0].in_shape.dims[0] = sets;
            drafts[r1].fk.main.inputs[0].out_shape.dims[0] = sets;
            if (bias) {
                node_bytes[T.outs[1].node] = (size_t)(sets * gt.batch * gt.n) * 4;
                const int axis = drafts[r2].fk.main.raw().axis;
                dsc_view& pv = drafts[r2].fk.main.inputs[0];
                pv.in_shape.dims[0] = sets;
                pv.out_shape.dims[axis] = sets;
                pv.map_axis[axis] = 0;
                pv.map_step[axis] = 1;
            }
            drafts[other].alive = false;
            drafts[at] = fused;
            // the im2col copy has lost a reader; with the last one it goes
            if (drafts[site.copy_idx].alive && consumers_of(site.a_node).empty()) {
                drafts[at].covers.insert(drafts[at].covers.end(), drafts[site.copy_idx].covers.begin(), drafts[site.copy_idx].covers.end());
                drafts[site.copy_idx].alive = false;
            }
        }
    }

    // Pass 1g: a WindowsToImage whose windows neither overlap nor leave gaps (the backward of a pooling: stride =
    // window size) adds nothing up -- every image element is one window element.  It becomes a per-element copy
    // through the window view with its axes reordered: [.., oy, ox, g, fy, fx, c] read as [.., oy, fy, ox, fx, g, c],
    // whose row-major order is the image's.  Pass 2 then evaluates the copy inside whoever reads the image.
    void disjoint_windows_to_copies() {
        static const bool enabled = !(std::getenv("DSC_WINDOW_COPIES") && std::getenv("DSC_WINDOW_COPIES")[0] == '0');
        if (!enabled) return;
        for (auto& D : drafts) {
            const dsc_kernel_desc& d = D.fk.main.raw();
            if (!D.alive || d.kind != DSC_KERNEL_WINDOWS_TO_IMAGE || !D.fk.virtuals.empty() || D.fk.has_epilogue || !D.fk.parts.empty() ||
                D.outs.size() != 1 || D.outs[0].copy_from >= 0 || D.fk.inputs.size() != 1)
                continue;
            const dsc_view& v = d.inputs[0];
            const int r = v.out_shape.rank, bd = d.shape.rank - 3;
            if (r < 6 || bd != r - 6) continue;
            const int64_t oh = v.out_shape.dims[r - 6], ow = v.out_shape.dims[r - 5], fh = v.out_shape.dims[r - 3], fw = v.out_shape.dims[r - 2];
            if (d.stride_h != fh || d.stride_w != fw || d.shape.dims[bd] != oh * fh || d.shape.dims[bd + 1] != ow * fw) continue;
            // output axis -> window-view axis
            int from[DSC_MAX_DIM];
            for (int i = 0; i < bd; ++i) from[i] = i;
            from[bd + 0] = bd + 0;  // oy
            from[bd + 1] = bd + 3;  // fy
            from[bd + 2] = bd + 1;  // ox
            from[bd + 3] = bd + 4;  // fx
            from[bd + 4] = bd + 2;  // g
            from[bd + 5] = bd + 5;  // c
            dsc_view nv = v;
            dsc_kernel_desc nd{};
            nd.kind = DSC_KERNEL_PER_ELEMENT;
            nd.shape.rank = 1;  // a per-element kernel is described over its linear element count
            nd.shape.dims[0] = element_count(d.shape);
            for (int j = 0; j < r; ++j) {
                nv.out_shape.dims[j] = v.out_shape.dims[from[j]];
                nv.map_axis[j] = v.map_axis[from[j]];
                nv.map_step[j] = v.map_step[from[j]];
            }
            dsc_pe_op ops[2] = {pe_op(DSC_PE_LOAD), pe_op(DSC_PE_UNARY, DSC_UN_MOV, 0)};
            ops[0].input_index = 0;
            int32_t outputs[1] = {1};
            nd.n_inputs = 1;
            nd.inputs = &nv;
            nd.n_ops = 2;
            nd.ops = ops;
            nd.n_outputs = 1;
            nd.outputs = outputs;
            if (!validate(nd).empty()) continue;
            FusedKernel fk = FusedKernel::plain(nd);
            if (fk.n_buffers != (int)D.params.size()) continue;
            D.fk = fk;
        }
    }

    // Pass 1b: clusters that all work on the rows of one [m, n] array with a short n -- Reduces along n and the
    // per-element clusters around them (softmax cross-entropy: row max, exp, row sum, log-probability, gradient,
    // per-row loss; the accuracy count: arg-max and comparison with the label) -- become one row-fused launch.
    // The launch runs where the first of them ran, so a member may only read what exists by then or what
    // another member computes.
    void row_kernels() {
        std::vector<int> producer_of(n_nodes, -1);  // draft index writing each node
        auto refresh_producers = [&]() {
            std::fill(producer_of.begin(), producer_of.end(), -1);
            for (int i = 0; i < (int)drafts.size(); ++i)
                if (drafts[i].alive)
                    for (auto& o : drafts[i].outs) producer_of[o.node] = i;
        };
        auto is_plain = [&](const Draft& d) {
            if (!d.alive || !d.fk.virtuals.empty() || d.fk.has_epilogue || !d.fk.row_stages.empty() || d.keep_output || d.keep_split) return false;
            for (auto& o : d.outs)
                if (o.copy_from >= 0) return false;
            return true;
        };
        auto shape_is = [](const dsc_shape& sh, int64_t a, int64_t b) { return sh.rank == 2 && sh.dims[0] == a && sh.dims[1] == b; };
        for (int seed = 0; seed < (int)drafts.size(); ++seed) {
            if (!is_plain(drafts[seed])) continue;
            const dsc_kernel_desc& sd = drafts[seed].fk.main.raw();
            if (sd.kind != DSC_KERNEL_REDUCE || sd.inputs[0].out_shape.rank != 2 || sd.axis != 1) continue;
            const int64_t m = sd.inputs[0].out_shape.dims[0], n = sd.inputs[0].out_shape.dims[1];
            if (n < 2 || n > 64 || m < 2 || !shape_is(sd.shape, m, 1)) continue;
            refresh_producers();
            std::vector<int> members;      // draft indices, in order
            std::vector<int> member_of(drafts.size(), -1);
            auto try_add = [&](int j) {
                const Draft& d = drafts[j];
                if (!is_plain(d)) return false;
                const dsc_kernel_desc& k = d.fk.main.raw();
                bool wide = false;
                if (k.kind == DSC_KERNEL_REDUCE) {
                    if (k.axis != 1 || !shape_is(k.inputs[0].out_shape, m, n) || !shape_is(k.shape, m, 1)) return false;
                } else if (k.kind == DSC_KERNEL_PER_ELEMENT) {
                    wide = k.shape.dims[0] == m * n;
                    if (!wide && k.shape.dims[0] != m) return false;
                    auto shape_ok = [&](const dsc_shape& sh) {
                        return wide ? shape_is(sh, m, n) : (shape_is(sh, m, 1) || (sh.rank == 1 && sh.dims[0] == m));
                    };
                    for (int i = 0; i < k.n_inputs; ++i)
                        if (!shape_ok(k.inputs[i].out_shape)) return false;
                    for (int i = 0; i < k.n_builtin_views; ++i)
                        if (!shape_ok(k.builtin_views[i].out_shape)) return false;
                    for (int i = 0; i < k.n_ops; ++i)
                        if (k.ops[i].kind == DSC_PE_GATHER) return false;
                } else {
                    return false;
                }
                for (int i = 0; i < k.n_inputs; ++i) {
                    const int node = d.params[d.fk.inputs[i].buffer];
                    const int p = producer_of[node];
                    if (p >= 0 && member_of[p] >= 0) {
                        // computed by a member: must be read element for element (or one value per row)
                        const dsc_kernel_desc& pk = drafts[p].fk.main.raw();
                        const bool p_wide = pk.kind == DSC_KERNEL_PER_ELEMENT && pk.shape.dims[0] == m * n;
                        const dsc_view& v = k.inputs[i];
                        if (element_count(v.in_shape) != (p_wide ? m * n : m)) return false;
                        int64_t base, coef[DSC_MAX_DIM];
                        if (!affine_form(v, &base, coef) || base != 0) return false;
                        if (p_wide) {
                            if (!(k.kind == DSC_KERNEL_REDUCE || wide) || coef[0] != n || coef[1] != 1) return false;
                        } else {
                            if (k.kind == DSC_KERNEL_REDUCE || coef[0] != 1) return false;
                            if (v.out_shape.rank == 2 && v.out_shape.dims[1] > 1 && coef[1] != 0) return false;
                        }
                    } else if (p >= seed) {
                        return false;  // does not exist yet where the fused launch runs
                    }
                }
                return true;
            };
            for (int j = seed; j < (int)drafts.size(); ++j) {
                if (!try_add(j)) {
                    if (j == seed) break;
                    continue;
                }
                member_of[j] = (int)members.size();
                members.push_back(j);
            }
            if (members.size() < 2 || members.size() > 24) continue;
            Draft fused;
            fused.fk.main = drafts[seed].fk.main;
            fused.fk.row_m = m;
            fused.fk.row_n = n;
            for (int j : members) {
                const Draft& d = drafts[j];
                const dsc_kernel_desc& k = d.fk.main.raw();
                RowStage st;
                st.k = d.fk.main;
                for (int i = 0; i < k.n_inputs; ++i) {
                    const int node = d.params[d.fk.inputs[i].buffer];
                    const int p = producer_of[node];
                    Source src;
                    if (p >= 0 && member_of[p] >= 0) {
                        src.stage = member_of[p];
                        for (size_t o = 0; o < drafts[p].outs.size(); ++o)
                            if (drafts[p].outs[o].node == node) src.stage_out = (int)o;
                    } else {
                        src.buffer = param_index(fused, node, false);
                    }
                    st.inputs.push_back(src);
                }
                for (auto& o : d.outs) {
                    bool needed = is_graph_output[o.node];
                    for (int c : consumers_of(o.node))
                        if (member_of[c] < 0) needed = true;
                    if (needed) {
                        st.outputs.push_back((int)fused.fk.outputs.size());
                        fused.fk.outputs.push_back(param_index(fused, o.node, true));
                        fused.outs.push_back(o);
                    } else {
                        st.outputs.push_back(-1);
                    }
                }
                fused.fk.row_stages.push_back(st);
                fused.covers.insert(fused.covers.end(), d.covers.begin(), d.covers.end());
            }
            if (fused.fk.outputs.empty()) continue;
            for (int j : members) drafts[j].alive = false;
            drafts[seed] = fused;
            absorb_matmul_into_rows(seed);
        }
    }

    // The [m, n] product a row-fused launch starts from (the logits of a classifier head) joins it as its first
    // stage when it is small enough for the dot-product kernel and has no other reader: one launch less, and the
    // product never leaves registers.  DSC_FUSE_ROWS_MATMUL=0 keeps the two launches.
    void absorb_matmul_into_rows(int ri) {
        if (const char* e = std::getenv("DSC_FUSE_ROWS_MATMUL"))
            if (e[0] == '0') return;
        Draft& r = drafts[ri];
        const int64_t m = r.fk.row_m, n = r.fk.row_n;
        // the producer of a buffer the stages read
        int pi = -1;
        for (auto& st : r.fk.row_stages)
            for (auto& src : st.inputs) {
                if (src.buffer < 0) continue;
                const int node = r.params[src.buffer];
                for (int j = 0; j < ri; ++j) {
                    if (!drafts[j].alive || drafts[j].fk.main.raw().kind != DSC_KERNEL_MATMUL) continue;
                    for (auto& o : drafts[j].outs)
                        if (o.node == node) pi = j;
                }
            }
        if (pi < 0) return;
        Draft& p = drafts[pi];
        if (!p.fk.parts.empty() || !p.fk.row_stages.empty() || !p.fk.virtuals.empty() || p.keep_split || p.keep_output || !matmul_fits_row_stage(p.fk)) return;
        const MatMulDims g = matmul_dims(p.fk.main.raw());
        if (g.m != m || g.n != n) return;
        for (auto& src : p.fk.inputs)
            if (src.buffer < 0) return;
        if (p.fk.has_epilogue)
            for (size_t i = 0; i < p.fk.epilogue_inputs.size(); ++i)
                if ((int)i != p.fk.epilogue_product_input && p.fk.epilogue_inputs[i].buffer < 0) return;
        for (auto& o : p.outs) {
            if (is_graph_output[o.node] || o.copy_from >= 0) return;
            for (int c : consumers_of(o.node))
                if (c != ri) return;
        }
        if (taken_in_place_between(pi, ri, input_nodes(p))) return;
        // every stage that reads one of the product's arrays reads it element for element
        for (auto& st : r.fk.row_stages) {
            const dsc_kernel_desc& k = st.k.raw();
            for (int i = 0; i < k.n_inputs; ++i) {
                if (st.inputs[i].buffer < 0) continue;
                const int node = r.params[st.inputs[i].buffer];
                bool from_p = false;
                for (auto& o : p.outs) from_p = from_p || o.node == node;
                if (!from_p) continue;
                const dsc_view& v = k.inputs[i];
                int64_t base, coef[DSC_MAX_DIM];
                const bool wide_reader = k.kind == DSC_KERNEL_REDUCE || (k.kind == DSC_KERNEL_PER_ELEMENT && k.shape.dims[0] == m * n);
                if (!wide_reader || element_count(v.in_shape) != m * n || v.out_shape.rank != 2 || !affine_form(v, &base, coef) || base != 0 || coef[0] != n || coef[1] != 1) return;
            }
        }
        Draft fused;
        fused.fk.main = r.fk.main;
        fused.fk.row_m = m;
        fused.fk.row_n = n;
        const int shift = p.fk.has_epilogue ? 2 : 1;
        {
            RowStage mm;
            mm.k = p.fk.main;
            for (auto& src : p.fk.inputs) mm.inputs.push_back(import_source(fused, p, src, 0));
            mm.outputs.push_back(-1);
            fused.fk.row_stages.push_back(mm);
        }
        if (p.fk.has_epilogue) {
            RowStage ep;
            ep.k = p.fk.epilogue;
            for (size_t i = 0; i < p.fk.epilogue_inputs.size(); ++i) {
                Source src;
                if ((int)i == p.fk.epilogue_product_input) src.stage = 0;
                else src = import_source(fused, p, p.fk.epilogue_inputs[i], 0);
                ep.inputs.push_back(src);
            }
            for (int o = 0; o < p.fk.epilogue.raw().n_outputs; ++o) ep.outputs.push_back(-1);
            fused.fk.row_stages.push_back(ep);
        }
        for (auto& st : r.fk.row_stages) {
            RowStage ns;
            ns.k = st.k;
            for (auto& src : st.inputs) {
                Source s2;
                if (src.stage >= 0) {
                    s2.stage = src.stage + shift;
                    s2.stage_out = src.stage_out;
                } else {
                    const int node = r.params[src.buffer];
                    int from = -1;
                    for (size_t o = 0; o < p.outs.size(); ++o)
                        if (p.outs[o].node == node) from = (int)o;
                    if (from >= 0) {
                        s2.stage = shift - 1;  // the epilogue's output `from`, or the product itself
                        s2.stage_out = from;
                    } else {
                        s2.buffer = param_index(fused, node, false);
                    }
                }
                ns.inputs.push_back(s2);
            }
            for (int oi : st.outputs) {
                if (oi < 0) { ns.outputs.push_back(-1); continue; }
                ns.outputs.push_back((int)fused.fk.outputs.size());
                fused.fk.outputs.push_back(param_index(fused, r.params[r.fk.outputs[oi]], true));
                fused.outs.push_back(r.outs[oi]);
            }
            fused.fk.row_stages.push_back(ns);
        }
        fused.covers = p.covers;
        fused.covers.insert(fused.covers.end(), r.covers.begin(), r.covers.end());
        p.alive = false;
        drafts[ri] = fused;
    }

    // The A operand [m, k] of the product a row-fused launch starts from is often a light per-element cluster's only
    // output -- the hidden layer's activation: bias and leaky_relu over the sum of the previous product's k chunks --
    // that later launches read as well (the backward pass).  The row-fused launch evaluates every element of A exactly
    // once, so it can run that cluster itself and store the result on the way: one launch less.
    // DSC_FUSE_ROWS_OPERAND=0 keeps the cluster a launch of its own.
    void rows_take_their_operands_producer(int ri) {
        if (const char* e = std::getenv("DSC_FUSE_ROWS_OPERAND"))
            if (e[0] == '0') return;
        Draft& r = drafts[ri];
        if (r.fk.row_stages.empty() || r.fk.row_stages[0].k.raw().kind != DSC_KERNEL_MATMUL) return;
        RowStage& mm = r.fk.row_stages[0];
        if (mm.inputs[0].buffer < 0 || mm.store_a >= 0) return;
        const int node = r.params[mm.inputs[0].buffer];
        const dsc_kernel_desc& md = mm.k.raw();
        const MatMulDims g = matmul_dims(md);
        int64_t base = 0, coef[DSC_MAX_DIM];
        if (md.inputs[0].out_shape.rank != 3 || !affine_form(md.inputs[0], &base, coef) || base != 0 || coef[1] != g.k || coef[2] != 1 ||
            element_count(md.inputs[0].in_shape) != g.m * g.k)
            return;
        int qi = -1;
        for (int j = 0; j < ri; ++j)
            if (drafts[j].alive)
                for (auto& o : drafts[j].outs)
                    if (o.node == node) qi = j;
        if (qi < 0) return;
        const Draft& q = drafts[qi];
        const dsc_kernel_desc& qd = q.fk.main.raw();
        if (qd.kind != DSC_KERNEL_PER_ELEMENT || qd.n_outputs != 1 || q.fk.has_epilogue || !q.fk.row_stages.empty() || !q.fk.parts.empty() || q.keep_output ||
            q.fk.row_width || q.outs.size() != 1 || q.outs[0].copy_from >= 0 || qd.shape.dims[0] != g.m * g.k || !is_cheap_producer(qd) ||
            q.fk.virtuals.size() + r.fk.virtuals.size() + 1 > 8)
            return;
        for (int c : consumers_of(node))
            if (c < ri) return;  // someone ahead of the row-fused launch needs the array in memory
        if (taken_in_place_between(qi, ri, input_nodes(q))) return;
        Draft fused = r;
        {
            const int new_virt = (int)fused.fk.virtuals.size();
            fused.fk.virtuals.emplace_back();
            const int voff = import_virtuals(fused, q);
            Virtual nv;
            nv.pe = q.fk.main;
            nv.out_op = qd.outputs[0];
            for (auto& s : q.fk.inputs) nv.inputs.push_back(import_source(fused, q, s, voff));
            fused.fk.virtuals[new_virt] = nv;
            RowStage& fm = fused.fk.row_stages[0];
            fm.inputs[0] = Source{};
            fm.inputs[0].virt = new_virt;
            fm.store_a = (int)fused.fk.outputs.size();
            fused.fk.outputs.push_back(param_index(fused, node, true));
            fused.outs.push_back(q.outs[0]);
        }
        compact(fused);
        {
            Generated probe;
            if (!generate(fused.fk, &probe).empty()) return;
        }
        fused.covers.insert(fused.covers.end(), q.covers.begin(), q.covers.end());
        drafts[qi].alive = false;
        drafts[ri] = fused;
    }

    // Pass 2c: the data gradient of the layer a row-fused launch starts from.  The launch begins with Z = A x W
    // ([m, k] x [k, n], n <= 64) and, in a training graph, produces dZ [m, n] among its outputs; the backward pass then
    // wants dA = dZ x W^T [m, k], usually masked by the stored activation A (a short-k MatMul with a per-element
    // consumer).  A lane of the row-fused kernel still owns the blocks of four k it multiplied in stage 0, dZ's row is
    // in the registers of its row's lanes and W is small: the product runs behind the last stage, and its launch --
    // on which the gradients of the layer below wait -- goes.  DSC_FUSE_ROWS_DGRAD=0 keeps it.
    void rows_take_the_data_gradient(int ri) {
        if (const char* e = std::getenv("DSC_FUSE_ROWS_DGRAD"))
            if (e[0] == '0') return;
        Draft& r = drafts[ri];
        if (r.fk.row_stages.empty() || r.fk.row_stages[0].k.raw().kind != DSC_KERNEL_MATMUL || r.fk.row_tail.on) return;
        const int64_t m = r.fk.row_m, n = r.fk.row_n;
        const MatMulDims g0 = matmul_dims(r.fk.row_stages[0].k.raw());
        if (g0.k % 4 != 0 || n * g0.k > 8192) return;
        for (int ti = ri + 1; ti < (int)drafts.size(); ++ti) {
            Draft& t = drafts[ti];
            if (!t.alive || t.fk.main.raw().kind != DSC_KERNEL_MATMUL || !t.fk.virtuals.empty() || !t.fk.parts.empty() || !t.fk.row_stages.empty() ||
                t.keep_split || t.keep_output || t.fk.dgrad.on || t.fk.cfwd.on || t.fk.pair.on || t.fk.colsum_out >= 0 || t.fk.out_slice_width)
                continue;
            const dsc_kernel_desc& td = t.fk.main.raw();
            const MatMulDims g = matmul_dims(td);
            if (g.batch != 1 || (g.chunks != 1 && !t.fk.sum_chunks) || g.m != m || g.k != n || g.n != g0.k || td.output_mode == DSC_MATMUL_ROWS) continue;
            if (t.fk.inputs[0].buffer < 0 || t.fk.inputs[1].buffer < 0) continue;
            // A = a wide value of the launch, read element for element
            const int x_node = t.params[t.fk.inputs[0].buffer];
            int xs = -1, xo = 0;
            for (int si = 0; si < (int)r.fk.row_stages.size(); ++si) {
                const RowStage& st = r.fk.row_stages[si];
                const dsc_kernel_desc& sd = st.k.raw();
                if (sd.kind != DSC_KERNEL_PER_ELEMENT || sd.shape.dims[0] != m * n) continue;
                for (size_t o = 0; o < st.outputs.size(); ++o)
                    if (st.outputs[o] >= 0 && r.params[r.fk.outputs[st.outputs[o]]] == x_node) { xs = si; xo = (int)o; }
            }
            if (xs < 0) continue;
            int64_t base = 0, coef[DSC_MAX_DIM];
            if (td.inputs[0].out_shape.rank != 3 || !affine_form(td.inputs[0], &base, coef) || base != 0 || coef[1] != n || coef[2] != 1) continue;
            // B must exist when the row-fused launch runs
            const int b_node = t.params[t.fk.inputs[1].buffer];
            bool early = true;
            for (int j = ri; j < ti; ++j)
                if (drafts[j].alive)
                    for (auto& o : drafts[j].outs)
                        if (o.node == b_node) early = false;
            if (!early) continue;
            // the consumer's other operands: the A operand the launch stores (element for element), or arrays that
            // exist before the launch
            const int a_node = r.fk.row_stages[0].store_a >= 0 ? r.params[r.fk.outputs[r.fk.row_stages[0].store_a]] : -1;
            int a_input = -1;
            bool ok = true;
            if (t.fk.has_epilogue) {
                const dsc_kernel_desc& ed = t.fk.epilogue.raw();
                if (ed.shape.dims[0] != m * g.n) continue;
                for (int i = 0; i < ed.n_inputs && ok; ++i) {
                    if (i == t.fk.epilogue_product_input) {
                        ok = is_identity(ed.inputs[i]) || reads_in_order(ed.inputs[i]);
                        continue;
                    }
                    const Source& src = t.fk.epilogue_inputs[i];
                    if (src.buffer < 0) { ok = false; break; }
                    const int nd = t.params[src.buffer];
                    if (nd == a_node) {
                        if (a_input >= 0 || !reads_in_order(ed.inputs[i])) ok = false;
                        a_input = i;
                        continue;
                    }
                    for (int j = ri; j < ti; ++j)
                        if (drafts[j].alive)
                            for (auto& o : drafts[j].outs)
                                if (o.node == nd) ok = false;
                }
                for (int i = 0; i < ed.n_ops && ok; ++i)
                    if (ed.ops[i].kind == DSC_PE_RAND || ed.ops[i].kind == DSC_PE_COORD || ed.ops[i].kind == DSC_PE_GATHER) ok = false;
            }
            if (!ok) continue;
            for (auto& o : t.outs)
                if (o.copy_from >= 0) ok = false;
            if (!ok) continue;
            {
                std::vector<int> reads = input_nodes(t);
                if (taken_in_place_between(ri, ti, reads)) continue;
            }
            Draft fused = r;
            FusedKernel::RowTail& rt = fused.fk.row_tail;
            rt.on = true;
            rt.mm = t.fk.main;
            rt.mm.d.shape.dims[0] = 1;  // one full sum over the n columns
            rt.x_stage = xs;
            rt.x_stage_out = xo;
            rt.b = import_source(fused, t, t.fk.inputs[1], 0);
            rt.has_epilogue = t.fk.has_epilogue;
            if (t.fk.has_epilogue) {
                rt.epilogue = t.fk.epilogue;
                rt.epilogue_product_input = t.fk.epilogue_product_input;
                rt.epilogue_a_input = a_input;
                for (size_t i = 0; i < t.fk.epilogue_inputs.size(); ++i) {
                    if ((int)i == t.fk.epilogue_product_input || (int)i == a_input) rt.epilogue_inputs.push_back(Source{});
                    else rt.epilogue_inputs.push_back(import_source(fused, t, t.fk.epilogue_inputs[i], 0));
                }
            }
            for (size_t o = 0; o < t.outs.size(); ++o) {
                rt.outputs.push_back((int)fused.fk.outputs.size());
                fused.fk.outputs.push_back(param_index(fused, t.outs[o].node, true));
                fused.outs.push_back(t.outs[o]);
            }
            compact(fused);
            {
                Generated probe;
                if (!generate(fused.fk, &probe).empty()) continue;
            }
            fused.covers.insert(fused.covers.end(), t.covers.begin(), t.covers.end());
            t.alive = false;
            drafts[ri] = fused;
            return;
        }
    }

    // Pass 1i: per-element clusters over [rows, w] that pick their value by comparing the column with literals (each
    // concat of the reference is one: select(column > n - 1, pad(b), pad(a))) are marked to run a thread per row,
    // the column a constant of each of the row's w evaluations.  A chain of concats inlined into the last one then
    // costs each column only the branch it takes, not one load per link.
    void column_partitions() {
        if (const char* e = std::getenv("DSC_ROW_PARTITIONS"))
            if (e[0] == '0') return;
        for (Draft& d : drafts) {
            if (!d.alive || !d.fk.parts.empty() || !d.fk.row_stages.empty() || d.fk.has_epilogue || !d.fk.virtuals.empty()) continue;
            const dsc_kernel_desc& pd = d.fk.main.raw();
            if (pd.kind != DSC_KERNEL_PER_ELEMENT) continue;
            const int64_t w = column_partition_width(pd);
            if (w && pd.shape.dims[0] / w >= 16384) d.fk.row_width = w;
        }
    }

    // Pass 1h: a per-element cluster that reads nothing but small arrays (all of its inputs together fit the L2 of
    // one XCD: the coordinates of a mini-batch) and writes large ones is evaluated again by each of its readers, and
    // its outputs are neither written nor read back.  The hashed corner indices and bilinear weights of a grid level
    // are such outputs: a megabyte each, four of each per level, read by the forward gather and again by the four
    // ScatterAdds of the backward pass, all of them integer and float arithmetic on two coordinates.
    void recompute_from_small_inputs() {
        if (const char* e = std::getenv("DSC_RECOMPUTE_SMALL"))
            if (e[0] == '0') return;
        const size_t kInputLimit = (size_t)4 << 20, kOutputFloor = (size_t)256 << 10;
        for (int i = 0; i < (int)drafts.size(); ++i) {
            Draft& p = drafts[i];
            if (!p.alive || !p.fk.parts.empty() || !p.fk.row_stages.empty() || p.fk.has_epilogue || p.keep_output) continue;
            if (p.fk.row_width) continue;  // a link of a concat chain: pass 2 inlines it into the chain's row kernel
            const dsc_kernel_desc& pd = p.fk.main.raw();
            if (pd.kind != DSC_KERNEL_PER_ELEMENT) continue;
            // the cluster and whatever was already inlined into it (an earlier cluster of this kind)
            // A reader evaluates only what the outputs it takes depend on (the compiler drops the rest), so the bound
            // on the work a reader repeats is on the ops behind one output: the cluster that turns the two coordinates of a
            // point into a cell and a fraction per level of a hash grid has 85 ops and 32 outputs of five ops each --
            // stored, it was 67 MB written per step and read back by the encoding and by every ScatterAdd.
            auto ops_behind = [](const dsc_kernel_desc& d, int out_op) {
                std::vector<char> seen(d.n_ops, 0);
                std::vector<int> todo{out_op};
                int count = 0;
                while (!todo.empty()) {
                    const int o = todo.back();
                    todo.pop_back();
                    if (o < 0 || o >= d.n_ops || seen[o]) continue;
                    seen[o] = 1;
                    ++count;
                    const dsc_pe_op& op = d.ops[o];
                    const int n_args = op.kind == DSC_PE_UNARY || op.kind == DSC_PE_GATHER ? 1 : op.kind == DSC_PE_BINARY ? 2 : op.kind == DSC_PE_SELECT ? 4 : 0;
                    for (int a = 0; a < n_args; ++a) todo.push_back(op.args[a]);
                }
                return count;
            };
            auto is_plain = [&](const dsc_kernel_desc& d, int only_output /* -1: every output */) {
                if (d.kind != DSC_KERNEL_PER_ELEMENT || d.n_ops > 256) return false;
                for (int o = 0; o < d.n_outputs; ++o)
                    if ((only_output < 0 || d.outputs[o] == only_output) && ops_behind(d, d.outputs[o]) > 40) return false;
                for (int o = 0; o < d.n_ops; ++o) {
                    const dsc_pe_op& op = d.ops[o];
                    if (op.kind == DSC_PE_GATHER || op.kind == DSC_PE_RAND) return false;
                    if (op.kind == DSC_PE_UNARY && (op.op == DSC_UN_SQRT || op.op == DSC_UN_EXP || op.op == DSC_UN_LOG || op.op == DSC_UN_SIN || op.op == DSC_UN_COS)) return false;
                    if (op.kind == DSC_PE_BINARY && (op.op == DSC_BIN_POW || op.op == DSC_BIN_DIV)) return false;
                }
                return true;
            };
            bool plain = is_plain(pd, -1) && p.fk.virtuals.size() <= 8;
            for (auto& v : p.fk.virtuals) plain = plain && is_plain(v.pe.raw(), v.out_op);
            if (!plain) continue;
            size_t in_bytes = 0;
            bool ok = true;
            const std::vector<int> p_inputs = input_nodes(p);
            for (int node : p_inputs) in_bytes += node_bytes[node];
            if (p_inputs.empty() || in_bytes > kInputLimit) continue;
            std::set<int> readers;
            for (auto& out : p.outs) {
                if (is_graph_output[out.node] || out.copy_from >= 0 || node_bytes[out.node] < kOutputFloor) { ok = false; break; }
                for (int ci : consumers_of(out.node)) readers.insert(ci);
            }
            if (!ok || readers.empty()) continue;
            for (int ci : readers) {
                Draft& q = drafts[ci];
                const int qk = q.fk.main.raw().kind;
                if (ci <= i || !q.fk.parts.empty() || !q.fk.row_stages.empty() || q.fk.dgrad.on || q.fk.cfwd.on || q.fk.pool.on) ok = false;
                if (qk != DSC_KERNEL_PER_ELEMENT && qk != DSC_KERNEL_REDUCE && qk != DSC_KERNEL_SCATTER_ADD) ok = false;
                {
                    // (a reader takes a producer per output it reads, not per output there is)
                    int taken = 0;
                    for (auto& out : p.outs) {
                        bool reads = false;
                        for_each_source(q.fk, [&](Source& src) {
                            if (src.buffer >= 0 && q.params[src.buffer] == out.node && !q.fk.buffer_is_output[src.buffer]) reads = true;
                        });
                        taken += reads;
                    }
                    if ((int)q.fk.virtuals.size() + (int)p.fk.virtuals.size() + taken > 24) ok = false;
                }
                for (auto& o : q.outs)
                    for (auto& out : p.outs)
                        if (o.copy_from == out.node) ok = false;  // updated in place by the reader
                if (ok && taken_in_place_between(i, ci, input_nodes(p))) ok = false;
                if (q.fk.has_epilogue && q.fk.epilogue_product_input >= 0) {
                    const Source& ps = q.fk.epilogue_inputs[q.fk.epilogue_product_input];
                    for (auto& out : p.outs)
                        if (ps.buffer >= 0 && q.params[ps.buffer] == out.node) ok = false;
                }
            }
            if (!ok) continue;
            for (int ci : readers) {
                Draft& q = drafts[ci];
                const int voff = import_virtuals(q, p);
                for (size_t o = 0; o < p.outs.size(); ++o) {
                    const int node = p.outs[o].node;
                    bool reads = false;
                    for_each_source(q.fk, [&](Source& src) {
                        if (src.buffer >= 0 && q.params[src.buffer] == node && !q.fk.buffer_is_output[src.buffer]) reads = true;
                    });
                    if (!reads) continue;
                    const int new_virt = (int)q.fk.virtuals.size();
                    Virtual nv;
                    nv.pe = p.fk.main;
                    nv.out_op = pd.outputs[o];
                    for (auto& src : p.fk.inputs) nv.inputs.push_back(import_source(q, p, src, voff));
                    q.fk.virtuals.push_back(nv);
                    for_each_source(q.fk, [&](Source& src) {
                        if (src.buffer >= 0 && q.params[src.buffer] == node && !q.fk.buffer_is_output[src.buffer]) {
                            src.buffer = -1;
                            src.virt = new_virt;
                        }
                    });
                }
                q.covers.insert(q.covers.end(), p.covers.begin(), p.covers.end());
                compact(q);
            }
            p.alive = false;
        }
    }

    // Pass 2: per-element producers whose result need not exist in memory are evaluated inside their
    // consumers: pure copies (materialised im2col / pooling windows) into every consumer, light arithmetic
    // into a single consumer.
    void inline_producers() {
        // tuning hook: DSC_FUSE_INTO_MATMUL=0 keeps producers of MatMul operands materialised
        const char* fim = std::getenv("DSC_FUSE_INTO_MATMUL");
        const bool fuse_into_matmul = !(fim && fim[0] == '0');
        // DSC_CONV_BWD_LOADERS=2: loader waves, but dC of the convolution backward kernel stays a buffer
        const char* lw = std::getenv("DSC_CONV_BWD_LOADERS");
        const bool no_dc_producer = lw && lw[0] == '2';
        // tuning hook: DSC_FUSE_GATHER_SUMS=0 keeps every Unpad, WindowsToImage and outer product a launch of its own
        const char* fgs = std::getenv("DSC_FUSE_GATHER_SUMS");
        const bool sum_on_demand = !(fgs && fgs[0] == '0');
        auto on_demand_sum_kind = [](const Draft& p) {
            const FusedKernel& f = p.fk;
            const dsc_kernel_desc& d = f.main.raw();
            if (f.has_epilogue || !f.parts.empty() || !f.row_stages.empty() || f.dgrad.on || f.cfwd.on || f.pool.on || f.pair.on || f.colsum_out >= 0 ||
                f.sign_out >= 0 || f.out_slice_width || p.keep_split || p.outs.size() != 1 || f.outputs.size() != 1)
                return false;
            if (d.kind == DSC_KERNEL_UNPAD || d.kind == DSC_KERNEL_WINDOWS_TO_IMAGE) return true;
            if (d.kind != DSC_KERNEL_MATMUL) return false;
            const MatMulDims g = matmul_dims(d);
            return g.chunks == 1 && g.k <= 2;
        };
        // tuning hook: DSC_CONV_TAKES_SUMS=0 keeps a WindowsToImage in front of a convolution backward kernel a launch
        // tuning hook: DSC_ROWS_TAKE_PRODUCERS=0 keeps a light producer in front of a row-fused launch a launch
        const char* rtp = std::getenv("DSC_ROWS_TAKE_PRODUCERS");
        const bool rows_take_producers = !(rtp && rtp[0] == '0');
        const char* cts = std::getenv("DSC_CONV_TAKES_SUMS");
        const bool conv_takes_sums = !(cts && cts[0] == '0');
        auto carries_on_demand_sum = [](const FusedKernel& f) {
            for (auto& v : f.virtuals) {
                const int k = v.pe.raw().kind;
                if (k == DSC_KERNEL_UNPAD || k == DSC_KERNEL_WINDOWS_TO_IMAGE || k == DSC_KERNEL_MATMUL) return true;
            }
            return false;
        };
        bool changed = true;
        while (changed) {
            changed = false;
            for (int i = 0; i < (int)drafts.size() && !changed; ++i) {
                Draft& p = drafts[i];
                if (!p.alive) continue;
                const dsc_kernel_desc& pd = p.fk.main.raw();
                if (!p.fk.row_stages.empty()) continue;
                const bool is_pe = pd.kind == DSC_KERNEL_PER_ELEMENT && pd.n_outputs == 1 && !p.fk.has_epilogue;
                const bool is_red = pd.kind == DSC_KERNEL_REDUCE;
                // An Unpad, a WindowsToImage or a product over a k of one or two (an outer product): each of their
                // elements is a short sum of gathered elements, which a single consumer can evaluate where it reads it.
                // (The backward pass of a strided convolution arrives as MatMul -> copy -> WindowsToImage -> Unpad ->
                // Unpad, src/array.rs:954-975,989-1031: five arrays through memory for one.)
                const bool is_sum = sum_on_demand && on_demand_sum_kind(p);
                if ((!is_pe && !is_red && !is_sum) || p.keep_output) continue;
                const int node = p.outs[0].node;
                if (is_graph_output[node] || p.outs[0].copy_from >= 0) continue;
                auto cons = consumers_of(node);
                if (cons.empty()) continue;
                // A reader that evaluates whole rows with the column a constant (see column_partitions) runs, per
                // column, only the producers that column selects: there a producer need not be light (a gather of
                // four table entries), and the chain of producers may be as long as the row is wide.
                const bool into_rows = is_pe && cons.size() == 1 && drafts[cons[0]].fk.row_width > 0 && drafts[cons[0]].fk.main.raw().kind == DSC_KERNEL_PER_ELEMENT;
                if (is_pe && !into_rows && (!is_cheap_producer(pd) || p.fk.virtuals.size() > 8)) continue;
                if (is_pe && cons.size() > 1 && !is_pure_copy(pd)) continue;
                bool ok = true;
                if (is_sum) {
                    if (cons.size() != 1) continue;
                    const Draft& q = drafts[cons[0]];
                    const dsc_kernel_desc& cd = q.fk.main.raw();
                    const bool plain = q.fk.parts.empty() && q.fk.row_stages.empty() && q.fk.row_width == 0 && !q.fk.has_epilogue;
                    // (the convolution backward kernels evaluate dC where they fill their tile: a WindowsToImage over
                    // overlapping windows -- the gradient of a stride-1 pooling -- in front of them is evaluated there too.
                    // Measured on the ConvBlurNet at batch 1000: the kernel with both gradients 34.3 -> 45.2 us for a
                    // launch of 18.7 us less, the filter gradient alone 20.9 -> 42.3 us for one of 34.5 us less)
                    const bool conv_dc = conv_takes_sums && cd.kind == DSC_KERNEL_MATMUL && q.fk.dgrad.on && (q.fk.dgrad.wgrad || q.fk.dgrad.wgrad_only) &&
                                         pd.kind == DSC_KERNEL_WINDOWS_TO_IMAGE && !q.fk.dgrad.pm.on;
                    if (!plain || (cd.kind != DSC_KERNEL_PER_ELEMENT && cd.kind != DSC_KERNEL_UNPAD && cd.kind != DSC_KERNEL_WINDOWS_TO_IMAGE && !conv_dc)) continue;
                    if (conv_dc) {
                        if (draft_unit_cost(p) * on_demand_reads(pd) * node_multiplicity(q, node) > 24.0) continue;
                    } else {
                    // a per-element consumer that reads each element several times over (a broadcast) leaves it in memory
                    if (cd.kind == DSC_KERNEL_PER_ELEMENT && 2 * element_count(cd.shape) > 3 * element_count(pd.shape)) continue;
                    // loads per element the consumer stores: what one evaluation costs, times the evaluations behind each of
                    // the consumer's own reads, times those reads (a WindowsToImage over overlapping windows evaluates each
                    // element once per window: measured on the gradient of a 2x2 stride-1 max pooling, 30 loads per stored
                    // element took as long as the four launches they replaced, and with the chain evaluated four channels at a
                    // time still 184 us against 35 + 20 for the two launches)
                    const double fan_in = cd.kind == DSC_KERNEL_PER_ELEMENT ? 1.0 : on_demand_reads(cd);
                    const double per_read = draft_unit_cost(p) * on_demand_reads(pd) * node_multiplicity(q, node);
                    if (per_read > 24.0 || per_read * fan_in > 16.0) continue;
                    }
                }
                if (is_pe && carries_on_demand_sum(p.fk))
                    for (int ci : cons)
                        if (drafts[ci].fk.main.raw().kind == DSC_KERNEL_MATMUL || cons.size() > 1) ok = false;
                if (is_pe && !fuse_into_matmul)
                    for (int ci : cons)
                        if (drafts[ci].fk.main.raw().kind == DSC_KERNEL_MATMUL) ok = false;
                if (is_red) {
                    // a reduction is re-run by every element that reads it: only short ones, and only where the
                    // consumers stay small
                    const int64_t k = pd.inputs[0].out_shape.dims[pd.axis];
                    const double unit = (double)k * draft_unit_cost(p);
                    if (k > 64 || unit > 512.0) ok = false;
                    for (int ci : cons) {
                        const dsc_kernel_desc& cd = drafts[ci].fk.main.raw();
                        const double per_read = unit * node_multiplicity(drafts[ci], node);  // loads per main-kernel read
                        if ((double)draft_reads(drafts[ci]) * per_read > (double)(1 << 22) || cd.kind == DSC_KERNEL_MATMUL) ok = false;
                        if (per_read > 512.0) ok = false;
                        // a reduction consumer with few outputs would run the inlined loops serially per output
                        if (cd.kind == DSC_KERNEL_REDUCE && element_count(cd.shape) < 4096 &&
                            (double)cd.inputs[0].out_shape.dims[cd.axis] * per_read > 512.0)
                            ok = false;
                    }
                }
                for (int ci : cons) {
                    Draft& q = drafts[ci];
                    if (ci <= i) ok = false;
                    for (auto& o : q.outs)
                        if (o.copy_from == node) ok = false;  // updated in place by the consumer
                    if (taken_in_place_between(i, ci, input_nodes(p))) ok = false;
                    if ((int)q.fk.virtuals.size() + (int)p.fk.virtuals.size() + 1 > (into_rows ? 512 : 8)) ok = false;
                    if (!q.fk.row_stages.empty()) {
                        // a row-fused launch takes a light producer that its stages read element for element (the sum of a
                        // product's k-chunks with the bias on it, in front of a softmax cross-entropy: the linear classifier's
                        // step 5 -> 4 launches, 47.9 -> 54.2 thousand steps per second)
                        bool in_order = rows_take_producers && is_pe && cons.size() == 1 && !q.fk.row_tail.on;
                        for (auto& st : q.fk.row_stages)
                            for (size_t si = 0; si < st.inputs.size(); ++si) {
                                const Source& src = st.inputs[si];
                                if (src.stage >= 0 || src.buffer < 0 || q.params[src.buffer] != node) continue;
                                if (st.k.raw().kind == DSC_KERNEL_MATMUL || !reads_in_order(st.k.raw().inputs[si])) in_order = false;
                            }
                        if (!in_order) ok = false;
                    }
                    // a MatMul that sums its B operand's columns on the side took over the operand's other reader: the
                    // operand stays a buffer, as it was when two launches read it
                    if (q.fk.colsum_out >= 0 && q.fk.inputs[1].buffer >= 0 && q.params[q.fk.inputs[1].buffer] == node) ok = false;
                    // the kernel that takes both gradients of a convolution requests dC of its next image while it
                    // works on the current one: plain loads, nothing evaluated in between
                    // (the filter gradient alone has one round trip per image anyway and takes dC as a producer; its
                    // image has to be a buffer)
                    // (with loader waves the fills run beside the matrix phases, on waves of their own: there dC is a
                    // producer again, and the pooling gradient it usually is never goes through memory)
                    if (q.fk.dgrad.on && q.fk.dgrad.wgrad && q.fk.inputs[0].buffer >= 0 && q.params[q.fk.inputs[0].buffer] == node &&
                        !(conv_bwd_loader_waves(q.fk) && !no_dc_producer))
                        ok = false;
                    // an epilogue reads its product from the accumulator, never through a producer
                    if (q.fk.has_epilogue && q.fk.epilogue_product_input >= 0) {
                        const Source& ps = q.fk.epilogue_inputs[q.fk.epilogue_product_input];
                        if (ps.buffer >= 0 && q.params[ps.buffer] == node) ok = false;
                    }
                }
                if (!ok) continue;
                for (int ci : cons) {
                    Draft& q = drafts[ci];
                    const int new_virt = (int)q.fk.virtuals.size();
                    q.fk.virtuals.emplace_back();
                    const int voff = import_virtuals(q, p);
                    {
                        Virtual nv;
                        nv.pe = p.fk.main;
                        nv.out_op = is_pe ? pd.outputs[0] : 0;  // (kinds evaluated on demand have one result)
                        for (auto& s : p.fk.inputs) nv.inputs.push_back(import_source(q, p, s, voff));
                        q.fk.virtuals[new_virt] = nv;
                    }
                    for_each_source(q.fk, [&](Source& s) {
                        if (s.buffer >= 0 && q.params[s.buffer] == node && !q.fk.buffer_is_output[s.buffer]) {
                            s.buffer = -1;
                            s.virt = new_virt;
                        }
                    });
                    q.covers.insert(q.covers.end(), p.covers.begin(), p.covers.end());
                    compact(q);
                }
                p.alive = false;
                changed = true;
            }
        }
    }

    // Pass 3: a Reduce, WindowsToImage or Unpad whose only consumer is a per-element cluster over its outputs (a
    // scalar accumulated into a running sum, the optimiser update of a bias gradient, the activation derivative
    // applied to a pooling gradient) applies that cluster to each result before the store.
    void attach_epilogues() {
        for (int i = 0; i < (int)drafts.size(); ++i) {
            Draft& r = drafts[i];
            const int rk = r.fk.main.raw().kind;
            if (!r.alive || (rk != DSC_KERNEL_REDUCE && rk != DSC_KERNEL_WINDOWS_TO_IMAGE && rk != DSC_KERNEL_UNPAD) || r.fk.has_epilogue ||
                r.keep_output || !r.fk.row_stages.empty())
                continue;
            int pe_idx = -1, pe_input = -1;
            bool permuted = false, shared = false;
            find_epilogue(i, r.outs[0].node, element_count(r.fk.main.raw().shape), &pe_idx, &pe_input, rk == DSC_KERNEL_REDUCE ? &permuted : nullptr, &shared);
            if (pe_idx < 0) continue;
            Draft& e = drafts[pe_idx];
            if ((int)r.fk.virtuals.size() + (int)e.fk.virtuals.size() > 8) continue;
            Draft fused;
            fused.fk.main = r.fk.main;
            fused.fk.epilogue_permuted = permuted;
            const int voff = import_virtuals(fused, r);
            for (auto& src : r.fk.inputs) fused.fk.inputs.push_back(import_source(fused, r, src, voff));
            fused.covers = r.covers;
            fused.fk.has_epilogue = true;
            fused.fk.epilogue = e.fk.main;
            fused.fk.epilogue_product_input = pe_input;
            const int eoff = import_virtuals(fused, e);
            for (int k = 0; k < (int)e.fk.inputs.size(); ++k) {
                if (k == pe_input) fused.fk.epilogue_inputs.push_back(Source{});
                else fused.fk.epilogue_inputs.push_back(import_source(fused, e, e.fk.inputs[k], eoff));
            }
            for (auto& o : e.outs) {
                fused.fk.outputs.push_back(param_index(fused, o.node, true));
                fused.outs.push_back(o);
            }
            if (shared) {
                fused.fk.epilogue_keeps_product = true;
                fused.fk.outputs.push_back(param_index(fused, r.outs[0].node, true));
                fused.outs.push_back(r.outs[0]);
            }
            fused.covers.insert(fused.covers.end(), e.covers.begin(), e.covers.end());
            compact(fused);
            r.alive = false;
            drafts[pe_idx] = fused;  // runs where the per-element cluster ran: all of its inputs exist by then
        }
    }

    // Pass 3d: a MatMul product [m, n] whose readers all take narrow column slices of it (the gradient of sixteen
    // concatenated two-feature encodings, read back two columns at a time by sixty-four ScatterAdd links) is stored
    // slice by slice instead of row by row: a reader of w columns then walks consecutive memory instead of w floats
    // out of every n, which cost the whole product's lines once per reader.  Only the row-per-thread kernel has
    // the store (a lane owns a row, so lanes write consecutive places of every slice), and every reader's view
    // must be one whose rows and columns can be told apart: [.., m, n] with whole-slice column ranges, unclamped.
    void slice_major_products() {
        static const bool enabled = !(std::getenv("DSC_SLICE_MAJOR") && std::getenv("DSC_SLICE_MAJOR")[0] == '0');
        if (!enabled) return;
        for (int pi = 0; pi < (int)drafts.size(); ++pi) {
            Draft& P = drafts[pi];
            if (!P.alive || P.fk.main.raw().kind != DSC_KERNEL_MATMUL || P.fk.has_epilogue || P.fk.dgrad.on || P.fk.cfwd.on || !P.fk.parts.empty() ||
                !P.fk.row_stages.empty() || P.fk.colsum_out >= 0 || P.outs.size() != 1 || P.outs[0].copy_from >= 0)
                continue;
            const MatMulDims g = matmul_dims(P.fk.main.raw());
            if (g.batch != 1 || (g.chunks != 1 && !P.fk.sum_chunks) || g.m < 16384 || P.fk.main.raw().output_mode == DSC_MATMUL_ROWS) continue;
            const int X = P.outs[0].node;
            if (is_graph_output[X] || node_bytes[X] != (size_t)(g.m * g.n) * 4) continue;
            // every view through which X is read
            std::vector<dsc_view*> views;
            bool ok = true;
            for (int di = 0; di < (int)drafts.size() && ok; ++di) {
                Draft& D = drafts[di];
                if (!D.alive || di == pi) continue;
                for (auto& o : D.outs)
                    if (o.copy_from == X) ok = false;
                bool reads = false;
                for (size_t b = 0; b < D.params.size(); ++b)
                    if (D.params[b] == X) reads = true;
                if (!reads) continue;
                FusedKernel& fk = D.fk;
                if (fk.dgrad.on || fk.cfwd.on || fk.pool.on || !fk.row_stages.empty() || !fk.parts.empty() || fk.binned_stage) { ok = false; break; }
                auto take = [&](KernelDesc& kd, std::vector<Source>& srcs, int skip) {
                    if (srcs.size() != kd.inputs.size()) { ok = false; return; }
                    for (size_t i = 0; i < srcs.size(); ++i) {
                        if ((int)i == skip || srcs[i].buffer < 0 || D.params[srcs[i].buffer] != X) continue;
                        for (auto& op : kd.ops)
                            if (op.kind == DSC_PE_GATHER && op.input_index == (int)i) ok = false;  // indexed by data, not through the view
                        if (kd.raw().kind != DSC_KERNEL_PER_ELEMENT && kd.raw().kind != DSC_KERNEL_SCATTER_ADD && kd.raw().kind != DSC_KERNEL_REDUCE) ok = false;
                        views.push_back(&kd.inputs[i]);
                    }
                };
                take(fk.main, fk.inputs, -1);
                for (auto& v : fk.virtuals) take(v.pe, v.inputs, -1);
                if (fk.has_epilogue) take(fk.epilogue, fk.epilogue_inputs, fk.epilogue_product_input);
            }
            if (!ok || views.size() < 2) continue;
            // the slice width: the widest column range any reader takes, which must divide n and hold every range whole
            int64_t W = 0;
            for (const dsc_view* v : views) {
                const int r = v->in_shape.rank;
                if (r < 2 || r + 1 > DSC_MAX_DIM || v->in_shape.dims[r - 1] != g.n || v->in_shape.dims[r - 2] != g.m || any_clamp(*v)) { ok = false; break; }
                for (int i = 0; i < r - 2; ++i)
                    if (v->in_shape.dims[i] != 1) ok = false;
                int64_t lo, hi;
                axis_span(*v, r - 1, &lo, &hi);
                W = std::max(W, hi - lo + 1);
            }
            if (!ok || W < 1 || W * 4 > 16 || W * 2 > g.n || g.n % W != 0) continue;
            for (const dsc_view* v : views) {
                int64_t lo, hi;
                axis_span(*v, v->in_shape.rank - 1, &lo, &hi);
                if (lo / W != hi / W) ok = false;
            }
            if (!ok) continue;
            FusedKernel trial = P.fk;
            trial.out_slice_width = W;
            Generated probe;
            if (!generate(trial, &probe).empty()) continue;
            P.fk.out_slice_width = W;
            for (dsc_view* v : views) {
                // [.., m, n] -> [.., n / W, m, W]: rows keep their axis' mapping one place down, the slice becomes an offset
                const int r = v->in_shape.rank;
                int64_t lo, hi;
                axis_span(*v, r - 1, &lo, &hi);
                const int64_t slice = lo / W;
                v->in_shape.rank = r + 1;
                v->in_shape.dims[r - 2] = g.n / W;
                v->in_shape.dims[r - 1] = g.m;
                v->in_shape.dims[r] = W;
                v->in_offset[r] = v->in_offset[r - 1] - slice * W;
                v->in_offset[r - 1] = v->in_offset[r - 2];
                v->in_offset[r - 2] = slice;
                for (int j = 0; j < v->out_shape.rank; ++j)
                    if (v->map_axis[j] >= r - 2) v->map_axis[j] += 1;
            }
        }
    }

    // Pass 3c: max-pooling joins the convolution that feeds it.  By now the pooling is a Reduce(max) over four
    // window elements whose input is a fused producer -- the window copy of the convolution kernel's (activated)
    // output -- possibly with a per-element consumer of its own (pass 3: a dropout select).  The convolution
    // kernel has those values in registers: it takes the maximum over each 2x2 window with two shuffles and runs the
    // consumer, and the convolution's output is not read back.  The geometry is checked element by element: every
    // pooled element of three images must read exactly the four window elements the kernel will combine.
    void pool_joins_conv_forward() {
        for (int ri = 0; ri < (int)drafts.size(); ++ri) {
            static const bool enabled = !(std::getenv("DSC_FUSE_CONV_POOL") && std::getenv("DSC_FUSE_CONV_POOL")[0] == '0');
            if (!enabled || (flags & DSC_SCHEDULE_NO_CONV_KERNELS)) break;
            Draft& R = drafts[ri];
            const dsc_kernel_desc& rd = R.fk.main.raw();
            if (!R.alive || rd.kind != DSC_KERNEL_REDUCE || rd.reduce_op != DSC_REDUCE_MAX || R.fk.virtuals.size() != 1 || R.fk.epilogue_permuted ||
                !R.fk.row_stages.empty() || R.fk.inputs[0].virt != 0 || R.keep_output || rd.inputs[0].out_shape.dims[rd.axis] != 4)
                continue;
            const Virtual& win = R.fk.virtuals[0];
            const dsc_kernel_desc& wd = win.pe.raw();
            if (wd.kind != DSC_KERNEL_PER_ELEMENT || wd.n_inputs != 1 || win.inputs[0].buffer < 0) continue;
            {
                int loads = 0;
                bool copy = true;
                for (int q = 0; q < wd.n_ops; ++q) {
                    if (wd.ops[q].kind == DSC_PE_LOAD) ++loads;
                    else if (!(wd.ops[q].kind == DSC_PE_UNARY && wd.ops[q].op == DSC_UN_MOV)) copy = false;
                }
                if (!copy || loads != 1) continue;
            }
            const int x_node = R.params[win.inputs[0].buffer];
            int fi = -1, source = -1;
            for (int q = 0; q < ri && fi < 0; ++q) {
                if (!drafts[q].alive || !drafts[q].fk.cfwd.on || drafts[q].fk.pool.on) continue;
                for (size_t o = 0; o < drafts[q].outs.size(); ++o)
                    if (drafts[q].outs[o].node == x_node) { fi = q; source = (int)o; }
            }
            if (fi < 0) continue;
            Draft& F = drafts[fi];
            const FusedKernel::ConvFwd& cv = F.fk.cfwd;
            const dsc_kernel_desc& fd = F.fk.main.raw();
            const MatMulDims g = matmul_dims(fd);
            const bool rows = fd.output_mode == DSC_MATMUL_ROWS;
            const int64_t batch_stride = rows ? g.n : g.m * g.n, row_stride = rows ? g.batch * g.n : g.n;
            if (cv.oh % 2 || cv.ow % 2 || g.n % 4 || batch_stride % 4 || row_stride % 4) continue;
            const int64_t OH2 = cv.oh / 2, OW2 = cv.ow / 2, pooled_elems = cv.img * OH2 * OW2 * g.batch * g.n;
            if (element_count(rd.shape) != pooled_elems || element_count(wd.inputs[0].in_shape) != cv.img * cv.oh * cv.ow * g.batch * g.n) continue;
            const int64_t pbs = rows ? g.n : cv.img * OH2 * OW2 * g.n, prs = rows ? g.batch * g.n : g.n;
            // pooled element -> the four elements of x it reads, through the Reduce's view and the window copy's view
            const dsc_view& rv = rd.inputs[0];
            const dsc_view& wv = wd.inputs[0];
            auto sources_of = [&](int64_t e, int64_t* out4) {
                int64_t oc[DSC_MAX_DIM], q = e;
                for (int a = rd.shape.rank - 1; a >= 0; --a) {
                    oc[a] = q % rd.shape.dims[a];
                    q /= rd.shape.dims[a];
                }
                for (int64_t w = 0; w < 4; ++w) {
                    int64_t rc[DSC_MAX_DIM];
                    for (int a = 0; a < rv.out_shape.rank; ++a) rc[a] = a == rd.axis ? w : oc[a];
                    int64_t idx = view_index_clamped(rv, rc), cc[DSC_MAX_DIM];
                    for (int a = wv.out_shape.rank - 1; a >= 0; --a) {
                        cc[a] = idx % wv.out_shape.dims[a];
                        idx /= wv.out_shape.dims[a];
                    }
                    out4[w] = view_index_clamped(wv, cc);
                }
                std::sort(out4, out4 + 4);
            };
            if (rv.out_shape.rank != rd.shape.rank || element_count(rv.in_shape) != element_count(wv.out_shape)) continue;
            bool ok = true;
            for (int64_t img : {(int64_t)0, cv.img / 2, cv.img - 1})
                for (int64_t yp = 0; yp < OH2 && ok; ++yp)
                    for (int64_t xp = 0; xp < OW2 && ok; ++xp)
                        for (int64_t cb = 0; cb < g.batch && ok; ++cb)
                            for (int64_t cn = 0; cn < g.n && ok; ++cn) {
                                const int64_t e = cb * pbs + (img * OH2 * OW2 + yp * OW2 + xp) * prs + cn;
                                int64_t got[4], want[4];
                                sources_of(e, got);
                                for (int64_t w = 0; w < 4; ++w)
                                    want[w] = cb * batch_stride + (img * cv.oh * cv.ow + (2 * yp + w / 2) * cv.ow + 2 * xp + w % 2) * row_stride + cn;
                                std::sort(want, want + 4);
                                for (int w = 0; w < 4; ++w)
                                    if (got[w] != want[w]) ok = false;
                            }
            if (!ok) continue;
            // the Reduce's consumer (if any) moves to where the convolution runs: what it reads must exist by then
            std::vector<int> produced_before(n_nodes, 0);
            for (int q = 0; q < fi; ++q)
                if (drafts[q].alive)
                    for (auto& o : drafts[q].outs) produced_before[o.node] = 1;
            for (int nd : input_nodes(R)) {
                if (nd == x_node) continue;
                if (!is_graph_input[nd] && !produced_before[nd]) ok = false;
            }
            for (auto& o : R.outs)
                if (o.copy_from >= 0) ok = false;
            if (!ok || taken_in_place_between(fi, ri, input_nodes(R)) || taken_in_place_between(fi, ri, input_nodes(F))) continue;
            Draft fused = F;
            fused.fk.pool.on = true;
            fused.fk.pool.source = source;
            fused.fk.pool.has_epilogue = R.fk.has_epilogue;
            fused.fk.pool.store_pooled = !R.fk.has_epilogue || R.fk.epilogue_keeps_product;
            if (R.fk.has_epilogue) {
                fused.fk.pool.epilogue = R.fk.epilogue;
                fused.fk.pool.epilogue_product_input = R.fk.epilogue_product_input;
                // (R's only fused producer is the window copy, which the Reduce's main input used: the consumer's own
                // inputs are buffers)
                bool plain = true;
                for (size_t q = 0; q < R.fk.epilogue_inputs.size(); ++q) {
                    if ((int)q == R.fk.epilogue_product_input) {
                        fused.fk.pool.epilogue_inputs.push_back(Source{});
                        continue;
                    }
                    if (R.fk.epilogue_inputs[q].buffer < 0) plain = false;
                    else fused.fk.pool.epilogue_inputs.push_back(import_source(fused, R, R.fk.epilogue_inputs[q], 0));
                }
                if (!plain) continue;
            }
            // outputs: the convolution's, then the consumer's, then the pooled array
            const int n_epi = R.fk.has_epilogue ? R.fk.epilogue.raw().n_outputs : 0;
            for (int o = 0; o < n_epi; ++o) {
                fused.fk.outputs.push_back(param_index(fused, R.outs[o].node, true));
                fused.outs.push_back(R.outs[o]);
            }
            if (fused.fk.pool.store_pooled) {
                const StepOutput& po = R.outs[n_epi];
                fused.fk.outputs.push_back(param_index(fused, po.node, true));
                fused.outs.push_back(po);
            }
            {
                Generated probe;
                if (!generate(fused.fk, &probe).empty()) continue;
            }
            fused.covers.insert(fused.covers.end(), R.covers.begin(), R.covers.end());
            R.alive = false;
            drafts[fi] = fused;
        }
    }

    // Pass 3g: the gradient of a 2x2 max-pooling read off two bits per element.  The backward pass of "convolution,
    // activation, 2x2 max-pool" reads the activation A twice -- (A == its window's maximum P) ? dP : 0, then
    // (A > 0) ? that : that x c -- and nothing else does once the pooling itself runs inside the convolution kernel
    // (pass 3c).  That kernel has A and P in registers: it writes the two comparisons' outcomes, one word per window
    // and four channels, and A is never stored; the convolution backward kernel that evaluated the four producers of
    // this chain where it fills dC (pass 2) reads a word and the window's dP instead (ConvPool::masks,
    // ConvDgrad::PoolMasks).  Bit for bit the same gradient: the comparisons are made on the same values.
    // The chain is matched op by op, and its index arithmetic is checked element by element on three images.
    void pooling_gradients_read_window_words() {
        const char* sw = std::getenv("DSC_POOL_WORDS");
        if ((sw && sw[0] == '0') || (flags & DSC_SCHEDULE_NO_CONV_KERNELS)) return;
        auto strip = [](const dsc_kernel_desc& pe, int op) {
            while (pe.ops[op].kind == DSC_PE_UNARY && pe.ops[op].op == DSC_UN_MOV) op = pe.ops[op].args[0];
            return op;
        };
        auto is_zero = [&](const dsc_kernel_desc& pe, int op) {
            op = strip(pe, op);
            return pe.ops[op].kind == DSC_PE_LITERAL_F32 && pe.ops[op].bits == 0u;
        };
        // element id of a per-element cluster -> the element its input `in` reads there
        auto through = [](const dsc_kernel_desc& pe, int in, int64_t gid) {
            const dsc_view& v = pe.inputs[in];
            int64_t c[DSC_MAX_DIM];
            for (int a = v.out_shape.rank - 1; a >= 0; --a) {
                c[a] = gid % v.out_shape.dims[a];
                gid /= v.out_shape.dims[a];
            }
            return view_index_clamped(v, c);
        };
        for (int fi = 0; fi < (int)drafts.size(); ++fi) {
            Draft& F = drafts[fi];
            if (!F.alive || !F.fk.cfwd.on || !F.fk.pool.on || F.fk.pool.masks || !F.fk.pool.store_pooled || !F.fk.parts.empty()) continue;
            const FusedKernel::ConvFwd& cv = F.fk.cfwd;
            const dsc_kernel_desc& fd = F.fk.main.raw();
            const MatMulDims g = matmul_dims(fd);
            const bool rows = fd.output_mode == DSC_MATMUL_ROWS;
            const int64_t batch_stride = rows ? g.n : g.m * g.n, row_stride = rows ? g.batch * g.n : g.n;
            const int64_t OH2 = cv.oh / 2, OW2 = cv.ow / 2, K = g.n, G = g.batch;
            const int64_t pbs = rows ? g.n : cv.img * OH2 * OW2 * g.n, prs = rows ? g.batch * g.n : g.n;
            const int n_out = F.fk.has_epilogue ? F.fk.epilogue.raw().n_outputs : 1;
            const int n_epi = F.fk.pool.has_epilogue ? F.fk.pool.epilogue.raw().n_outputs : 0;
            if (K % 4 != 0 || (int)F.outs.size() != n_out + n_epi + 1) continue;
            const int a_node = F.outs[F.fk.pool.source].node, p_node = F.outs[n_out + n_epi].node;
            if (is_graph_output[a_node] || F.outs[F.fk.pool.source].copy_from >= 0) continue;
            const auto cons = consumers_of(a_node);
            if (cons.size() != 1 || cons[0] <= fi) continue;
            const int qi = cons[0];
            Draft& Q = drafts[qi];
            const FusedKernel::ConvDgrad& dg = Q.fk.dgrad;
            if (!dg.on || !dg.wgrad || dg.pm.on || !Q.fk.parts.empty() || Q.fk.has_epilogue) continue;
            const int DC = dg.wgrad_only ? 1 : 0;
            const dsc_kernel_desc& qd = Q.fk.main.raw();
            const MatMulDims gq = matmul_dims(qd);
            if (dg.img != cv.img || dg.oh != cv.oh || dg.ow != cv.ow || dg.g != G || (dg.wgrad_only ? gq.n : gq.k) != K) continue;
            if (Q.fk.inputs[DC].virt < 0 || Q.fk.virtuals.size() != 4) continue;
            // every other operand of the kernel is a buffer that is not A
            bool clean = true;
            for (size_t in = 0; in < Q.fk.inputs.size(); ++in)
                if ((int)in != DC && (Q.fk.inputs[in].buffer < 0 || Q.params[Q.fk.inputs[in].buffer] == a_node)) clean = false;
            if (!clean) continue;
            // V0 = (A > 0) ? X : X x c
            const int v0 = Q.fk.inputs[DC].virt;
            const Virtual& V0 = Q.fk.virtuals[v0];
            const dsc_kernel_desc& d0 = V0.pe.raw();
            if (d0.kind != DSC_KERNEL_PER_ELEMENT || d0.n_inputs != 2) continue;
            const dsc_pe_op& sel0 = d0.ops[strip(d0, V0.out_op)];
            if (sel0.kind != DSC_PE_SELECT || sel0.op != DSC_CMP_GT || !is_zero(d0, sel0.args[1])) continue;
            const int a_op = strip(d0, sel0.args[0]), x_op = strip(d0, sel0.args[2]), y_op = strip(d0, sel0.args[3]);
            if (d0.ops[a_op].kind != DSC_PE_LOAD || d0.ops[x_op].kind != DSC_PE_LOAD || d0.ops[y_op].kind != DSC_PE_BINARY || d0.ops[y_op].op != DSC_BIN_MUL) continue;
            const int a_in0 = d0.ops[a_op].input_index, x_in0 = d0.ops[x_op].input_index;
            if (a_in0 == x_in0 || V0.inputs[a_in0].buffer < 0 || Q.params[V0.inputs[a_in0].buffer] != a_node || V0.inputs[x_in0].virt < 0) continue;
            uint32_t leak_bits = 0;
            {
                const int m0 = strip(d0, d0.ops[y_op].args[0]), m1 = strip(d0, d0.ops[y_op].args[1]);
                const bool x_first = d0.ops[m0].kind == DSC_PE_LOAD && d0.ops[m0].input_index == x_in0 && d0.ops[m1].kind == DSC_PE_LITERAL_F32;
                const bool x_second = d0.ops[m1].kind == DSC_PE_LOAD && d0.ops[m1].input_index == x_in0 && d0.ops[m0].kind == DSC_PE_LITERAL_F32;
                if (!x_first && !x_second) continue;
                leak_bits = d0.ops[x_first ? m1 : m0].bits;
            }
            // V1 = copy of V2
            const Virtual& V1 = Q.fk.virtuals[V0.inputs[x_in0].virt];
            const dsc_kernel_desc& d1 = V1.pe.raw();
            if (d1.kind != DSC_KERNEL_PER_ELEMENT || d1.n_inputs != 1 || !is_pure_copy(d1) || V1.inputs[0].virt < 0) continue;
            // V2 = (V3 == P) ? dP : 0
            const Virtual& V2 = Q.fk.virtuals[V1.inputs[0].virt];
            const dsc_kernel_desc& d2 = V2.pe.raw();
            if (d2.kind != DSC_KERNEL_PER_ELEMENT || d2.n_inputs != 3) continue;
            const dsc_pe_op& sel2 = d2.ops[strip(d2, V2.out_op)];
            if (sel2.kind != DSC_PE_SELECT || sel2.op != DSC_CMP_EQ || !is_zero(d2, sel2.args[3])) continue;
            const int w_op = strip(d2, sel2.args[0]), p_op = strip(d2, sel2.args[1]), dp_op = strip(d2, sel2.args[2]);
            if (d2.ops[w_op].kind != DSC_PE_LOAD || d2.ops[p_op].kind != DSC_PE_LOAD || d2.ops[dp_op].kind != DSC_PE_LOAD) continue;
            const int w_in = d2.ops[w_op].input_index, p_in = d2.ops[p_op].input_index, dp_in = d2.ops[dp_op].input_index;
            if (w_in == p_in || w_in == dp_in || p_in == dp_in) continue;
            if (V2.inputs[w_in].virt < 0 || V2.inputs[p_in].buffer < 0 || V2.inputs[dp_in].buffer < 0 || Q.params[V2.inputs[p_in].buffer] != p_node) continue;
            const int dp_node = Q.params[V2.inputs[dp_in].buffer];
            if (dp_node == a_node || dp_node == p_node) continue;
            // V3 = copy of A
            const Virtual& V3 = Q.fk.virtuals[V2.inputs[w_in].virt];
            const dsc_kernel_desc& d3 = V3.pe.raw();
            if (d3.kind != DSC_KERNEL_PER_ELEMENT || d3.n_inputs != 1 || !is_pure_copy(d3) || V3.inputs[0].buffer < 0 || Q.params[V3.inputs[0].buffer] != a_node) continue;
            if ((int64_t)node_bytes[dp_node] != cv.img * OH2 * OW2 * G * K * 4) continue;
            // the indices, element by element: A at the pixel itself (both reads), P and dP at the pixel's window
            const dsc_view& dcv = qd.inputs[DC];
            bool ok = dcv.out_shape.rank == 3;
            for (int64_t img : {(int64_t)0, cv.img / 2, cv.img - 1})
                for (int64_t y = 0; y < cv.oh && ok; ++y)
                    for (int64_t x = 0; x < cv.ow && ok; ++x)
                        for (int64_t cb = 0; cb < G && ok; ++cb)
                            for (int64_t oc = 0; oc < K && ok; ++oc) {
                                const int64_t pix = (img * cv.oh + y) * cv.ow + x;
                                const int64_t c3[3] = {cb, dg.wgrad_only ? pix : pix, oc};
                                const int64_t gid0 = view_index_clamped(dcv, c3);
                                const int64_t a_at = cb * batch_stride + pix * row_stride + oc;
                                const int64_t win = (img * OH2 + y / 2) * OW2 + x / 2;
                                if (through(d0, a_in0, gid0) != a_at) ok = false;
                                const int64_t gid1 = through(d0, x_in0, gid0), gid2 = through(d1, 0, gid1);
                                const int64_t gid3 = through(d2, w_in, gid2);
                                if (through(d3, 0, gid3) != a_at) ok = false;
                                if (through(d2, p_in, gid2) != cb * pbs + win * prs + oc) ok = false;
                                if (through(d2, dp_in, gid2) != win * (G * K) + cb * K + oc) ok = false;
                            }
            if (!ok) continue;
            // rewire: the forward kernel writes the words through the pointer that stood for A, the backward kernel reads
            // them and dP
            node_bytes.push_back((size_t)(G * cv.img * OH2 * OW2 * (K / 4)) * 4);
            is_graph_output.push_back(false);
            is_graph_input.push_back(false);
            const int words = n_nodes++;
            Draft f2 = F, q2 = Q;
            f2.fk.pool.masks = true;
            f2.params[f2.fk.outputs[f2.fk.pool.source]] = words;
            f2.outs[f2.fk.pool.source].node = words;
            q2.fk.virtuals.clear();
            q2.fk.inputs[DC] = Source{};
            q2.fk.inputs[DC].buffer = param_index(q2, dp_node, false);
            q2.fk.dgrad.pm.on = true;
            q2.fk.dgrad.pm.masks = Source{};
            q2.fk.dgrad.pm.masks.buffer = param_index(q2, words, false);
            q2.fk.dgrad.pm.leak_bits = leak_bits;
            compact(q2);
            // the pooled array itself, kept beside its consumer's output for this chain alone, is no longer written
            if (f2.fk.pool.has_epilogue && !is_graph_output[p_node] && F.outs[n_out + n_epi].copy_from < 0) {
                bool only_q = true;
                for (int c : consumers_of(p_node))
                    if (c != qi) only_q = false;
                if (only_q) {
                    f2.fk.pool.store_pooled = false;
                    f2.fk.outputs.pop_back();
                    f2.outs.pop_back();
                    compact(f2);
                }
            }
            Generated probe_f, probe_q;
            if (!generate(f2.fk, &probe_f).empty() || !generate(q2.fk, &probe_q).empty()) {
                node_bytes.pop_back();
                is_graph_output.pop_back();
                is_graph_input.pop_back();
                --n_nodes;
                continue;
            }
            drafts[fi] = f2;
            drafts[qi] = q2;
        }
    }

    // Pass 3b: ScatterAdds chained through one accumulator (each takes the previous one's result in place:
    // the four corner updates of one hash-grid level) commute, so the chain runs as one multi-part launch
    // whose parts all add into the same buffer.  It runs where the last one ran.
    void chain_scatter_adds() {
        for (int i = 0; i < (int)drafts.size(); ++i) {
            if (!drafts[i].alive || drafts[i].fk.main.raw().kind != DSC_KERNEL_SCATTER_ADD || !drafts[i].fk.parts.empty()) continue;
            std::vector<int> chain{i};
            for (;;) {
                const int node = drafts[chain.back()].outs[0].node;
                if (is_graph_output[node]) break;
                int next = -1, readers = 0;
                for (int j = chain.back() + 1; j < (int)drafts.size() && next < 0; ++j) {
                    if (!drafts[j].alive) continue;
                    for (auto& o : drafts[j].outs)
                        if (o.copy_from == node) next = j;
                }
                if (next < 0) break;
                const Draft& nx = drafts[next];
                if (nx.fk.main.raw().kind != DSC_KERNEL_SCATTER_ADD || !nx.fk.parts.empty() ||
                    !same_shape(nx.fk.main.raw().shape, drafts[i].fk.main.raw().shape))
                    break;
                for (int c : consumers_of(node)) (void)c, ++readers;  // nobody may read the intermediate sum
                if (readers != 0) break;
                chain.push_back(next);
                if (chain.size() >= 8) break;
            }
            if (chain.size() < 2) continue;
            const int last = chain.back();
            // every part's inputs must still be what they were when the merged launch runs
            bool ok = true;
            for (int j : chain)
                if (j != last && taken_in_place_between(j, last, input_nodes(drafts[j]))) ok = false;
            size_t bound = 0;
            for (int j : chain) bound += drafts[j].params.size();
            if (!ok || bound > 48) continue;
            const int final_node = drafts[last].outs[0].node;
            Draft multi;
            multi.fk.main = drafts[i].fk.main;
            std::set<int> seen;
            for (int j : chain) {
                const Draft& d = drafts[j];
                std::vector<int> map;
                for (size_t p = 0; p < d.params.size(); ++p) {
                    const bool is_out = d.fk.buffer_is_output[p];
                    map.push_back(param_index(multi, is_out ? final_node : d.params[p], is_out));
                }
                multi.fk.parts.push_back(d.fk);
                multi.fk.part_params.push_back(map);
                for (int nd : input_nodes(d))
                    if (seen.insert(nd).second) multi.part_inputs.push_back(nd);
                multi.covers.insert(multi.covers.end(), d.covers.begin(), d.covers.end());
            }
            {
                int64_t total_values = 0;
                for (int j : chain) total_values += element_count(drafts[j].fk.main.raw().inputs[0].out_shape);
                multi.fk.shared_scatter = scatter_chain_in_lds(element_count(drafts[i].fk.main.raw().shape), total_values);
            }
            StepOutput out = drafts[i].outs[0];  // the first link says where the accumulator comes from
            out.node = final_node;
            int64_t total_values = 0;
            for (int j : chain) total_values += element_count(drafts[j].fk.main.raw().inputs[0].out_shape);
            const int64_t table = element_count(drafts[i].fk.main.raw().shape);
            if (!multi.fk.shared_scatter && scatter_chain_binned(table, total_values) && (size_t)table * 4 == node_bytes[final_node]) {
                // two launches: the links' values go to bins by accumulator segment, then every segment is summed in LDS
                bool pairs = true;
                for (int j : chain) pairs = pairs && scatter_rows_of_two(drafts[j].fk.main.raw());
                const BinnedScatterPlan bp = binned_scatter_plan(table, total_values, pairs);
                auto new_node = [&](size_t bytes) {
                    node_bytes.push_back(bytes);
                    is_graph_output.push_back(false);
                    is_graph_input.push_back(false);
                    return n_nodes++;
                };
                const int records = new_node((size_t)(bp.nseg * bp.cap) * (size_t)bp.record_bytes);
                const int cursor = new_node((size_t)bp.nseg * 64);  // one counter per 64-byte line
                const int zero = new_node(0);                       // stands for the literal the counters start from
                const int mid = new_node(node_bytes[final_node]);   // the accumulator between the two launches
                for (size_t p = 0; p < multi.params.size(); ++p)
                    if (multi.params[p] == final_node && multi.fk.buffer_is_output[p]) multi.params[p] = mid;
                multi.fk.binned_stage = 1;
                multi.fk.binned_table = table;
                multi.fk.binned_total = total_values;
                multi.fk.binned_pairs = pairs;
                multi.fk.outputs = {param_index(multi, records, true), param_index(multi, cursor, true), param_index(multi, mid, true)};
                out.node = mid;
                multi.outs = {StepOutput{records, -1, false, 0}, StepOutput{cursor, zero, true, 0}, out};
                Draft sum;
                sum.fk.main = drafts[i].fk.main;
                sum.fk.binned_stage = 2;
                sum.fk.binned_table = table;
                sum.fk.binned_total = total_values;
                sum.fk.binned_pairs = pairs;
                sum.params = {records, cursor, final_node};
                sum.fk.buffer_is_output = {false, false, true};
                sum.fk.n_buffers = 3;
                Source from_records, from_cursor;
                from_records.buffer = 0;
                from_cursor.buffer = 1;
                sum.fk.inputs = {from_records, from_cursor};
                sum.fk.outputs = {2};
                sum.outs = {StepOutput{final_node, mid, false, 0}};
                for (int j : chain) drafts[j].alive = false;
                drafts[last] = multi;
                drafts.insert(drafts.begin() + last + 1, sum);
                continue;
            }
            multi.outs.push_back(out);
            multi.fk.outputs.push_back(param_index(multi, final_node, true));
            for (int j : chain) drafts[j].alive = false;
            drafts[last] = multi;
        }
    }

    // Pass 3e: the chain launches of a step (LDS chains, stage 1 and stage 2 kernels of binned chains) that stand
    // next to one another and do not depend on one another share launches: one for the LDS chains, one for all
    // first stages, one for all second stages.  Each of these kernels is a chain of memory round trips with
    // barriers in between that occupies a CU with one workgroup; sixteen hash-grid levels launched one by one
    // leave the machine waiting on those round trips sixteen (or thirty-two) times.
    void group_chain_launches() {
        static const bool enabled = !(std::getenv("DSC_CHAIN_GROUPS") && std::getenv("DSC_CHAIN_GROUPS")[0] == '0');
        if (!enabled) return;
        auto kind_of = [&](const Draft& d) {
            if (d.fk.chain_group) return 0;
            if (d.fk.binned_stage == 1) return 2;
            if (d.fk.binned_stage == 2) return 3;
            if (d.fk.shared_scatter && !d.fk.parts.empty()) return 1;
            return 0;
        };
        size_t lo = 0;
        while (lo < drafts.size()) {
            if (!drafts[lo].alive || kind_of(drafts[lo]) == 0) { ++lo; continue; }
            size_t hi = lo;
            std::vector<int> run;
            while (hi < drafts.size() && (!drafts[hi].alive || kind_of(drafts[hi]) != 0)) {
                if (drafts[hi].alive) run.push_back((int)hi);
                ++hi;
            }
            // nothing in the run may read or take over what another member writes, except a second stage its own first
            std::vector<int> writer(n_nodes, -1);
            for (int di : run)
                for (auto& o : drafts[di].outs) writer[o.node] = di;
            bool ok = run.size() >= 2;
            int prev_bin = -1;
            for (int di : run) {
                const Draft& d = drafts[di];
                const int kind = kind_of(d);
                std::vector<int> reads = input_nodes(d);
                for (auto& o : d.outs)
                    if (o.copy_from >= 0 && !o.from_literal) reads.push_back(o.copy_from);
                for (int nd : reads)
                    if (writer[nd] >= 0 && !(kind == 3 && writer[nd] == prev_bin)) ok = false;
                for (auto& o : d.outs) {
                    if (o.copy_from < 0 || o.from_literal) continue;
                    for (int dj : run) {
                        if (dj == di) continue;
                        auto ins = input_nodes(drafts[dj]);
                        if (std::find(ins.begin(), ins.end(), o.copy_from) != ins.end()) ok = false;
                    }
                }
                if (kind == 2) prev_bin = di;
                else if (kind == 3) prev_bin = -1;
            }
            if (!ok) { lo = hi; continue; }
            std::vector<Draft> grouped;
            for (int kind = 1; kind <= 3; ++kind) {
                std::vector<int> members;
                for (int di : run)
                    if (kind_of(drafts[di]) == kind) members.push_back(di);
                if (members.empty()) continue;
                size_t bound = 0;
                for (int di : members) bound += drafts[di].params.size();
                if (members.size() < 2 || bound > 240) {
                    for (int di : members) grouped.push_back(drafts[di]);
                    continue;
                }
                Draft G;
                G.fk.chain_group = true;
                G.fk.main = drafts[members[0]].fk.main;
                std::set<int> seen;
                for (int di : members) {
                    const Draft& d = drafts[di];
                    std::vector<int> map;
                    for (size_t p = 0; p < d.params.size(); ++p) map.push_back(param_index(G, d.params[p], d.fk.buffer_is_output[p]));
                    G.fk.parts.push_back(d.fk);
                    G.fk.part_params.push_back(map);
                    for (int nd : input_nodes(d))
                        if (seen.insert(nd).second) G.part_inputs.push_back(nd);
                    G.covers.insert(G.covers.end(), d.covers.begin(), d.covers.end());
                    for (size_t k = 0; k < d.outs.size(); ++k) {
                        G.outs.push_back(d.outs[k]);
                        G.fk.outputs.push_back(map[d.fk.outputs[k]]);
                    }
                }
                Generated probe;
                if (!generate(G.fk, &probe).empty()) {
                    for (int di : members) grouped.push_back(drafts[di]);
                    continue;
                }
                grouped.push_back(G);
            }
            // the launches take the last places of the run, in the order LDS chains, first stages, second stages
            for (int di : run) drafts[di].alive = false;
            for (size_t k = 0; k < grouped.size(); ++k) drafts[run[run.size() - grouped.size() + k]] = grouped[k];
            lo = hi;
        }
    }

    // Pass 3f: the two gradients of a layer with a few outputs (the last layer of a coordinate network, 256 -> 3) read
    // the same two arrays: the data gradient dY x W^T, a short-k MatMul whose consumer masks it with the stored
    // activation X, and the weight gradient X^T dY, a tall-k MatMul over the rows.  One kernel computes both from one
    // pass over X (FusedKernel::GradPair); the tall-k product's chunks become the row chunks of that kernel, so the
    // Reduce over its partials stays as it is.  The pair runs where the earlier of the two ran.
    void pair_output_layer_gradients() {
        static const bool enabled = !(std::getenv("DSC_FUSE_GRAD_PAIR") && std::getenv("DSC_FUSE_GRAD_PAIR")[0] == '0');
        if (!enabled) return;
        for (int si = 0; si < (int)drafts.size(); ++si) {
            if (!drafts[si].alive || drafts[si].fk.main.raw().kind != DSC_KERNEL_MATMUL || !drafts[si].fk.has_epilogue) continue;
            bool in_place = false;
            for (auto& o : drafts[si].outs)
                if (o.copy_from >= 0) in_place = true;
            if (in_place) continue;
            for (int ti = 0; ti < (int)drafts.size(); ++ti) {
                const Draft& S = drafts[si];
                const Draft& T = drafts[ti];
                if (ti == si || !T.alive || T.fk.main.raw().kind != DSC_KERNEL_MATMUL || T.outs.size() != 1 || T.outs[0].copy_from >= 0) continue;
                int64_t rows = 0, chunks = 0;
                if (!grad_pair_shapes(S.fk, T.fk, &rows, &chunks)) continue;
                const int dy = S.params[S.fk.inputs[0].buffer], x = T.params[T.fk.inputs[0].buffer];
                if (T.params[T.fk.inputs[1].buffer] != dy) continue;
                // X has to be something the data gradient's consumer reads anyway, element for element
                int x_param = -1;
                for (size_t p = 0; p < S.params.size(); ++p)
                    if (S.params[p] == x && !S.fk.buffer_is_output[p]) x_param = (int)p;
                const dsc_kernel_desc& pe = S.fk.epilogue.raw();
                bool reads_x = false;
                for (int i = 0; i < pe.n_inputs && x_param >= 0; ++i)
                    if (i != S.fk.epilogue_product_input && S.fk.epilogue_inputs[i].buffer == x_param && is_identity(pe.inputs[i])) reads_x = true;
                if (!reads_x) continue;
                // everything the later of the two reads must exist where the earlier one runs
                const int first = std::min(si, ti), last = std::max(si, ti);
                std::set<int> needed;
                for (int nd : input_nodes(drafts[last])) needed.insert(nd);
                bool ok = true;
                for (int q = first; q < last && ok; ++q) {
                    if (!drafts[q].alive) continue;
                    for (auto& o : drafts[q].outs)
                        if (needed.count(o.node)) ok = false;
                }
                if (!ok) continue;
                Draft F = S;
                F.fk.pair.on = true;
                F.fk.pair.x_buffer = x_param;
                F.fk.pair.chunk_rows = rows;
                F.fk.pair.chunks = chunks;
                F.fk.pair.out = param_index(F, T.outs[0].node, true);
                F.fk.outputs.push_back(F.fk.pair.out);
                F.outs.push_back(T.outs[0]);
                F.covers.insert(F.covers.end(), T.covers.begin(), T.covers.end());
                {
                    Generated probe;
                    if (!generate(F.fk, &probe).empty()) continue;
                }
                drafts[last].alive = false;
                drafts[first] = F;
                break;
            }
        }
    }

    // Pass 3h: what a dense layer's backward pass asks of the stored activation.  The data gradient of the layer
    // above, dX = (a > 0) ? g : g x c, is the epilogue of a MatMul and reads the activation a [m, n] element for element
    // -- as many bytes again as the product it masks -- to look at one bit of each.  The MatMul that wrote a has every
    // element in registers when it stores it: it writes a byte per four consecutive elements beside them (bit j set
    // where element 4i + j is positive), and the masked product reads those bytes, a sixteenth of the activation, all
    // of a unit's store rounds requested before the first (FusedKernel::sign_out / epilogue_sign_input).  a itself stays:
    // the next layer reads it.  Bit for bit the same results: "(a > 0)" is evaluated once, by the writer, on the same a.
    void activation_signs_as_bytes() {
        const char* sw = std::getenv("DSC_SIGN_BYTES");
        if (sw && sw[0] == '0') return;
        for (int di = 0; di < (int)drafts.size(); ++di) {
            Draft& D = drafts[di];
            const dsc_kernel_desc& dd = D.fk.main.raw();
            if (!D.alive || dd.kind != DSC_KERNEL_MATMUL || !D.fk.has_epilogue || D.fk.epilogue_sign_input >= 0 || !D.fk.parts.empty() || !D.fk.row_stages.empty() ||
                D.fk.dgrad.on || D.fk.cfwd.on || D.fk.pair.on || D.fk.out_slice_width || D.fk.colsum_out >= 0 || !D.fk.virtuals.empty())
                continue;
            const dsc_kernel_desc& pe = D.fk.epilogue.raw();
            const MatMulDims g = matmul_dims(dd);
            const int64_t count = g.batch * g.m * g.n;
            if (dd.output_mode != DSC_MATMUL_BATCHES || count % 4 != 0 || count < (1 << 20)) continue;
            for (int in = 0; in < pe.n_inputs; ++in) {
                if (in == D.fk.epilogue_product_input || D.fk.epilogue_inputs[in].buffer < 0) continue;
                if (!is_identity(pe.inputs[in]) || element_count(pe.inputs[in].out_shape) != count) continue;
                // every load of the input is the left side of a "> 0" select and nothing else
                bool only_signs = true, any = false;
                for (int q = 0; q < pe.n_ops && only_signs; ++q) {
                    if (pe.ops[q].kind != DSC_PE_LOAD || pe.ops[q].input_index != in) continue;
                    any = true;
                    for (int o = 0; o < pe.n_outputs; ++o)
                        if (pe.outputs[o] == q) only_signs = false;
                    for (int r = 0; r < pe.n_ops && only_signs; ++r) {
                        const dsc_pe_op& u = pe.ops[r];
                        const int nargs = u.kind == DSC_PE_UNARY || u.kind == DSC_PE_GATHER ? 1 : u.kind == DSC_PE_BINARY ? 2 : u.kind == DSC_PE_SELECT ? 4 : 0;
                        for (int a = 0; a < nargs; ++a) {
                            if (u.args[a] != q) continue;
                            const bool as_sign = u.kind == DSC_PE_SELECT && u.op == DSC_CMP_GT && a == 0 && pe.ops[u.args[1]].kind == DSC_PE_LITERAL_F32 &&
                                                 pe.ops[u.args[1]].bits == 0u && u.args[2] != q && u.args[3] != q;
                            if (!as_sign) only_signs = false;
                        }
                    }
                }
                if (!any || !only_signs) continue;
                const int a_node = D.params[D.fk.epilogue_inputs[in].buffer];
                // the MatMul that writes a, element for element in product order
                int fi = -1, src = -1;
                for (int q = 0; q < di && fi < 0; ++q) {
                    const Draft& F = drafts[q];
                    if (!F.alive || F.fk.main.raw().kind != DSC_KERNEL_MATMUL || !F.fk.has_epilogue || !F.fk.parts.empty() || !F.fk.row_stages.empty() || F.fk.dgrad.on ||
                        F.fk.cfwd.on || F.fk.pair.on || F.fk.out_slice_width || F.fk.main.raw().output_mode != DSC_MATMUL_BATCHES)
                        continue;
                    const MatMulDims gf = matmul_dims(F.fk.main.raw());
                    if (gf.batch != g.batch || gf.m != g.m || gf.n != g.n) continue;  // the same rows of the same width: one byte layout
                    const int n_epi = F.fk.epilogue.raw().n_outputs;
                    for (int o = 0; o < n_epi && o < (int)F.outs.size(); ++o)
                        if (F.outs[o].node == a_node && F.outs[o].copy_from < 0) { fi = q; src = o; }
                }
                if (fi < 0) continue;
                Draft f2 = drafts[fi], d2 = D;
                int bytes_node = -1;
                bool fresh = false;
                if (f2.fk.sign_out >= 0) {
                    if (f2.fk.sign_source != src) continue;
                    bytes_node = f2.params[f2.fk.sign_out];
                } else {
                    node_bytes.push_back((size_t)((count / 4 + 3) / 4 * 4));
                    is_graph_output.push_back(false);
                    is_graph_input.push_back(false);
                    bytes_node = n_nodes++;
                    fresh = true;
                    f2.fk.sign_out = param_index(f2, bytes_node, true);
                    f2.fk.sign_source = src;
                    f2.fk.outputs.push_back(f2.fk.sign_out);
                    f2.outs.push_back(StepOutput{bytes_node, -1, false, 0});
                }
                d2.fk.epilogue_inputs[in].buffer = param_index(d2, bytes_node, false);
                d2.fk.epilogue_sign_input = in;
                compact(d2);
                Generated probe_f, probe_d;
                if (!generate(f2.fk, &probe_f).empty() || !generate(d2.fk, &probe_d).empty()) {
                    if (fresh) {
                        node_bytes.pop_back();
                        is_graph_output.pop_back();
                        is_graph_input.pop_back();
                        --n_nodes;
                    }
                    continue;
                }
                drafts[fi] = f2;
                drafts[di] = d2;
                break;  // one such operand per product
            }
        }
    }

    // Pass 4: launches of a few workgroups each (optimiser updates of small tensors, short reductions, scalar
    // bookkeeping) cost a launch apiece while using a fraction of the machine.  Runs of them that do not
    // depend on one another become one multi-part launch; a later launch is hoisted into the run when nothing
    // it reads is produced in between.  One large kernel may ride along (its workgroups come last, so the
    // small parts start at once and finish in its shadow).
    void share_launches() {
        static const int64_t small_grid = std::getenv("DSC_MULTI_GRID") ? std::atoll(std::getenv("DSC_MULTI_GRID")) : 1024;
        // A kernel that moves this much is a launch's worth of work whatever its grid (a tall-k MatMul walks 268 MB with
        // 1024 workgroups): sharing a launch with another large kernel would only tie the two to the registers and
        // LDS of the hungrier one.
        static const double heavy_bytes = std::getenv("DSC_MULTI_BYTES") ? std::atof(std::getenv("DSC_MULTI_BYTES")) : 128e6;
        std::vector<int64_t> grid_of(drafts.size(), -1);
        std::vector<char> heavy(drafts.size(), 0);
        auto is_large = [&](int i) { return grid_of[i] > small_grid || heavy[i]; };
        auto partable = [&](int i) {
            const Draft& d = drafts[i];
            if (!d.alive || !can_be_part(d.fk)) return false;
            for (auto& o : d.outs)
                if (o.copy_from >= 0) return false;
            if (grid_of[i] < 0) {
                Generated g;
                FusedKernel probe = d.fk;
                probe.as_part = true;  // a kernel may pick another workgroup shape inside a shared launch
                if (!generate(probe, &g).empty() || g.block != 256) { grid_of[i] = (int64_t)1 << 40; return false; }
                grid_of[i] = g.grid;
                heavy[i] = g.algo_bytes > heavy_bytes;
            }
            return grid_of[i] < ((int64_t)1 << 30);
        };
        std::vector<bool> taken(drafts.size(), false);
        for (int i = 0; i < (int)drafts.size() && small_grid > 0; ++i) {
            if (taken[i] || !partable(i)) continue;
            std::vector<int> batch{i};
            int large = is_large(i) ? 1 : 0;
            int64_t total_grid = grid_of[i];
            std::set<int> blocked, bound;
            for (auto& o : drafts[i].outs) blocked.insert(o.node);
            for (int nd : drafts[i].params) bound.insert(nd);
            for (int j = i + 1; j < (int)drafts.size(); ++j) {
                if (!drafts[j].alive || taken[j]) continue;
                bool depends = false;
                for (int nd : input_nodes(drafts[j]))
                    if (blocked.count(nd)) depends = true;
                std::set<int> would = bound;
                for (int nd : drafts[j].params) would.insert(nd);
                if (!depends && batch.size() < 16 && would.size() <= 48 && partable(j) && (!is_large(j) || large == 0) &&
                    total_grid + grid_of[j] < ((int64_t)1 << 30)) {
                    batch.push_back(j);
                    bound = would;
                    large += is_large(j) ? 1 : 0;
                    total_grid += grid_of[j];
                }
                for (auto& o : drafts[j].outs) blocked.insert(o.node);
            }
            // a lone large kernel with nothing small to carry stays as it is
            if (batch.size() < 2) continue;
            std::stable_sort(batch.begin(), batch.end(), [&](int a, int b) { return grid_of[a] < grid_of[b]; });
            if (batch.size() < 2) continue;
            Draft multi;
            multi.fk.main = drafts[i].fk.main;
            std::set<int> seen;
            for (int j : batch) {
                const Draft& d = drafts[j];
                std::vector<int> map;
                for (size_t p = 0; p < d.params.size(); ++p) map.push_back(param_index(multi, d.params[p], d.fk.buffer_is_output[p]));
                multi.fk.parts.push_back(d.fk);
                multi.fk.part_params.push_back(map);
                for (int nd : input_nodes(d))
                    if (seen.insert(nd).second) multi.part_inputs.push_back(nd);
                for (size_t o = 0; o < d.outs.size(); ++o) {
                    multi.outs.push_back(d.outs[o]);
                    multi.fk.outputs.push_back(param_index(multi, d.outs[o].node, true));
                }
                multi.covers.insert(multi.covers.end(), d.covers.begin(), d.covers.end());
            }
            for (int j : batch) {
                taken[j] = true;
                drafts[j].alive = false;
            }
            drafts[i] = multi;
            taken[i] = true;
        }
    }

    // The order matters: each pass names the ones it relies on.
    void run() {
        sign_through_activation();              // pass 00
        split_long_k();                         // pass 0
        bias_sums_ride_on_weight_gradients();   // pass 0c
        merge_reduce_chains();                  // pass 0a
        split_long_reduces();                   // pass 0b
        matmul_with_reduce_and_epilogue();      // pass 1
        conv_data_gradient();                   // pass 1c
        conv_forward();                         // pass 1d
        conv_backward();                        // pass 1e
        disjoint_windows_to_copies();           // pass 1g
        row_kernels();                          // pass 1b
        column_partitions();                    // pass 1i
        recompute_from_small_inputs();          // pass 1h
        inline_producers();                     // pass 2
        for (int i = 0; i < (int)drafts.size(); ++i)
            if (drafts[i].alive) rows_take_their_operands_producer(i);  // pass 2b
        for (int i = 0; i < (int)drafts.size(); ++i)
            if (drafts[i].alive) rows_take_the_data_gradient(i);        // pass 2c
        attach_epilogues();                     // pass 3
        slice_major_products();                 // pass 3d
        pool_joins_conv_forward();              // pass 3c
        pooling_gradients_read_window_words();  // pass 3g
        chain_scatter_adds();                   // pass 3b
        group_chain_launches();                 // pass 3e
        pair_output_layer_gradients();          // pass 3f
        activation_signs_as_bytes();            // pass 3h
        share_launches();                       // pass 4
    }
};

}  // namespace

// ---------------------------------------------------------------------------------------------------------

int Schedule::build(Context* ctx, const dsc_schedule_desc& desc, uint32_t flags) {
    graph_replay = (flags & DSC_SCHEDULE_GRAPH_REPLAY) != 0;
    n_nodes = desc.n_nodes;
    n_params = desc.n_params;
    n_clusters = desc.n_clusters;
    node_bytes.assign(n_nodes, 0);
    for (int i = 0; i < n_nodes; ++i) node_bytes[i] = (size_t)desc.node_elements[i] * 4;
    inputs.assign(desc.inputs, desc.inputs + desc.n_inputs);
    outputs.assign(desc.outputs, desc.outputs + desc.n_outputs);
    for (auto& io : inputs)
        if (io.node < 0 || io.node >= n_nodes || io.param < 0 || io.param >= n_params) return fail(DSC_ERR_INVALID, "schedule: bad input entry");
    for (auto& io : outputs)
        if (io.node < 0 || io.node >= n_nodes || io.param < 0 || io.param >= n_params) return fail(DSC_ERR_INVALID, "schedule: bad output entry");

    std::vector<bool> is_graph_output(n_nodes, false), is_graph_input(n_nodes, false);
    for (auto& io : outputs) is_graph_output[io.node] = true;
    for (auto& io : inputs) is_graph_input[io.node] = true;

    // one draft per reference cluster
    std::vector<Draft> drafts(desc.n_clusters);
    for (int c = 0; c < desc.n_clusters; ++c) {
        const dsc_cluster& cl = desc.clusters[c];
        std::string err = validate(cl.kernel);
        if (!err.empty()) return fail(DSC_ERR_INVALID, "schedule: cluster " + std::to_string(c) + ": " + err);
        const int want_in = cl.kernel.kind == DSC_KERNEL_FILL ? 0 : cl.kernel.n_inputs;
        const int want_out = cl.kernel.kind == DSC_KERNEL_PER_ELEMENT ? cl.kernel.n_outputs : 1;
        if (cl.n_inputs != want_in || cl.n_outputs != want_out)
            return fail(DSC_ERR_INVALID, "schedule: cluster " + std::to_string(c) + " binds the wrong number of nodes");
        Draft& d = drafts[c];
        d.fk = FusedKernel::plain(cl.kernel);
        for (int i = 0; i < cl.n_inputs; ++i) {
            if (cl.inputs[i] < 0 || cl.inputs[i] >= n_nodes) return fail(DSC_ERR_INVALID, "schedule: bad node id");
            d.params.push_back(cl.inputs[i]);
        }
        for (int o = 0; o < cl.n_outputs; ++o) {
            const dsc_cluster_output& co = cl.outputs[o];
            if (co.node < 0 || co.node >= n_nodes || co.copy_from >= n_nodes) return fail(DSC_ERR_INVALID, "schedule: bad node id");
            d.params.push_back(co.node);
            d.outs.push_back(StepOutput{co.node, co.copy_from, co.copy_from_is_literal != 0, co.literal_bits});
        }
        d.covers.push_back(c);
    }

    if (!(flags & DSC_SCHEDULE_NO_FUSION)) {
        Planner planner{flags, n_nodes, node_bytes, drafts, is_graph_output, is_graph_input};
        planner.run();
    }

    // materialise the steps
    for (auto& d : drafts) {
        if (!d.alive) continue;
        Step st;
        int status = DSC_OK;
        st.kernel = get_kernel(ctx, d.fk, &status);
        if (!st.kernel) return status;
        st.params = d.params;
        st.inputs = input_nodes(d);
        st.outputs = d.outs;
        st.covers = d.covers;
        for (auto& o : st.outputs) {
            if (o.copy_from >= 0 && o.from_literal) {
                dsc_kernel_desc fd{};
                fd.kind = DSC_KERNEL_FILL;
                fd.shape.rank = 1;
                fd.shape.dims[0] = (int64_t)(node_bytes[o.node] / 4);
                fd.fill_bits = o.literal_bits;
                o.fill = get_kernel(ctx, FusedKernel::plain(fd), &status);
                if (!o.fill) return status;
            }
        }
        steps.push_back(st);
    }
    if (!(flags & DSC_SCHEDULE_NO_FUSION)) {
        std::vector<std::pair<int, uint32_t>> fills;  // (node, literal bits)
        for (auto& st : steps)
            for (auto& o : st.outputs)
                if (o.copy_from >= 0 && o.from_literal) fills.emplace_back(o.node, o.literal_bits);
        for (size_t first = 0; fills.size() >= 2 && first < fills.size(); first += 32) {
            const size_t last = std::min(fills.size(), first + 32);
            if (last - first < 2) break;
            FusedKernel multi;
            Prefill pf;
            for (size_t i = first; i < last; ++i) {
                dsc_kernel_desc fd{};
                fd.kind = DSC_KERNEL_FILL;
                fd.shape.rank = 1;
                fd.shape.dims[0] = (int64_t)(node_bytes[fills[i].first] / 4);
                fd.fill_bits = fills[i].second;
                multi.parts.push_back(FusedKernel::plain(fd));
                multi.part_params.push_back({(int)(i - first)});
                multi.outputs.push_back((int)(i - first));
                multi.buffer_is_output.push_back(true);
                pf.nodes.push_back(fills[i].first);
            }
            multi.main = multi.parts[0].main;
            multi.n_buffers = (int)pf.nodes.size();
            int status = DSC_OK;
            pf.kernel = get_kernel(ctx, multi, &status);
            if (!pf.kernel) return status;
            prefills.push_back(pf);
        }
    }
    return DSC_OK;
}

static bool graphs_by_env() {
    static const bool on = [] {
        const char* e = std::getenv("DSC_GRAPHS");
        return e && e[0] == '1';
    }();
    return on;
}

int Schedule::run(Context* ctx, dsc_buf* params, uint32_t rand_seed) {
    if ((graph_replay || graphs_by_env()) && replay_fixed && !ctx->profiling && launches_per_run() >= 4) {
        bool handled = false;
        const int rc = run_replayed(ctx, params, rand_seed, &handled);
        if (handled) return rc;
    }
    // environment.rs:326-516, over the fused steps.  Unlike the reference (which panics), a run that cannot be put
    // together leaves `params` and the caller's buffers as they were: until every launch's pointers are resolved
    // nothing the caller owns is released or handed on, and what the attempt allocated is given back.
    std::vector<int> usage(n_nodes, 0);
    std::vector<dsc_buf> buffer(n_nodes, 0);
    for (auto& st : steps)
        for (int n : st.inputs) usage[n] += 1;
    // A node that becomes a parameter's new value stays alive even when later clusters also read it (the
    // reference frees it after its last cluster use and then panics on the hand-off, environment.rs:491-515).
    for (auto& io : outputs) usage[io.node] += 1;

    std::vector<bool> param_is_output(n_params, false), param_is_input(n_params, false);
    for (auto& io : outputs) param_is_output[io.param] = true;
    for (auto& io : inputs) param_is_input[io.param] = true;

    std::set<dsc_buf> callers;  // buffers the caller handed in: released only once the run is certain to go ahead
    const std::vector<dsc_buf> handed_in(params, params + n_params);
    for (int i = 0; i < n_params; ++i)
        if (params[i]) callers.insert(params[i]);
    for (auto& io : inputs) {
        if (params[io.param] == 0) return fail(DSC_ERR_INVALID, "schedule run: an input parameter has no buffer");
        buffer[io.node] = params[io.param];
        if (!param_is_output[io.param]) usage[io.node] += 1;  // pinned: the parameter keeps its buffer
    }

    // Pass 1: buffer bookkeeping only -- resolve every launch's pointers (allocation and release are host-side
    // and stream-ordered, so a buffer freed here may be handed to a later launch of the same step).
    typedef PlannedLaunch Launch;
    std::vector<Launch> launches;
    std::vector<void*> pointers;
    launches.reserve(steps.size() + 4);
    std::vector<dsc_buf> prefilled(prefills.empty() ? 0 : n_nodes, 0);
    auto give_up = [&](int status, const std::string& msg) {
        for (dsc_buf h : buffer)
            if (h && !callers.count(h)) ctx->heap.free(h);
        for (dsc_buf h : prefilled)
            if (h) ctx->heap.free(h);
        return fail(status, msg);
    };
    auto release = [&](dsc_buf h) {
        if (!callers.count(h)) ctx->heap.free(h);
    };
    for (auto& pf : prefills) {
        launches.push_back(Launch{pf.kernel, pointers.size(), (int)pf.nodes.size()});
        for (int node : pf.nodes) {
            const dsc_buf h = ctx->heap.alloc(node_bytes[node]);
            if (!h) return give_up(DSC_ERR_OOM, "schedule run: out of device memory");
            void* p = nullptr;
            ctx->heap.info(h, &p, nullptr);
            pointers.push_back(p);
            prefilled[node] = h;
        }
    }
    for (auto& st : steps) {
        for (int n : st.inputs) usage[n] -= 1;
        for (auto& o : st.outputs) {
            dsc_buf h = 0;
            if (o.copy_from < 0) {
                h = ctx->heap.alloc(node_bytes[o.node]);
                if (!h) return give_up(DSC_ERR_OOM, "schedule run: out of device memory");
            } else {
                if (usage[o.copy_from] != 0) return give_up(DSC_ERR_UNSUPPORTED, "schedule run: accumulator source still in use (deep copy)");
                if (buffer[o.copy_from] != 0) {
                    h = buffer[o.copy_from];
                    buffer[o.copy_from] = 0;
                } else if (o.from_literal && !prefilled.empty() && prefilled[o.node] != 0) {
                    h = prefilled[o.node];  // allocated and filled at the start of the run
                    prefilled[o.node] = 0;
                } else if (o.from_literal) {
                    h = ctx->heap.alloc(node_bytes[o.node]);
                    if (!h) return give_up(DSC_ERR_OOM, "schedule run: out of device memory");
                    void* p = nullptr;
                    ctx->heap.info(h, &p, nullptr);
                    launches.push_back(Launch{o.fill, pointers.size(), 1});
                    pointers.push_back(p);
                } else {
                    return give_up(DSC_ERR_INVALID, "schedule run: cannot copy-on-write node");
                }
            }
            if (buffer[o.node] != 0) {
                if (!callers.count(h)) ctx->heap.free(h);
                return give_up(DSC_ERR_INVALID, "schedule run: node written twice");
            }
            buffer[o.node] = h;
        }
        const int n = (int)st.params.size();
        launches.push_back(Launch{st.kernel, pointers.size(), n});
        for (int i = 0; i < n; ++i) {
            void* p = nullptr;
            if (!ctx->heap.info(buffer[st.params[i]], &p, nullptr))
                return give_up(DSC_ERR_INVALID, "schedule run: node " + std::to_string(st.params[i]) + " has no buffer at '" + st.kernel->label + "'");
            pointers.push_back(p);
        }
        for (int nd : st.inputs) {
            if (usage[nd] == 0 && buffer[nd] != 0) {
                release(buffer[nd]);
                buffer[nd] = 0;
            }
        }
    }
    for (auto& io : outputs)
        if (buffer[io.node] == 0) return give_up(DSC_ERR_INVALID, "schedule run: output node has no buffer");
    // from here on the run goes ahead: parameters that are rewritten give their old buffers up, outputs move in
    for (auto& io : inputs)
        if (param_is_output[io.param]) params[io.param] = 0;
    for (auto& io : outputs) {
        if (!param_is_input[io.param]) params[io.param] = 0;
        params[io.param] = buffer[io.node];
        buffer[io.node] = 0;
    }
    // a rewritten parameter's old buffer goes back to the heap, unless it was taken over in place and is some
    // parameter's new value
    {
        const std::set<dsc_buf> kept(params, params + n_params);
        for (int i = 0; i < n_params; ++i)
            if (param_is_output[i] && handed_in[i] && !kept.count(handed_in[i])) ctx->heap.free(handed_in[i]);
    }

    // Pass 2: enqueue.  With per-launch timing on, or graphs off, launch one by one; otherwise replay the graph
    // captured for this exact pointer table, capturing it first if it is new.
    auto enqueue_all = [&]() -> int {
        for (auto& l : launches) {
            int rc = launch_kernel(ctx, l.kernel, pointers.data() + l.first, l.n, rand_seed);
            if (rc != DSC_OK) return rc;
        }
        return DSC_OK;
    };
    // opt-in (DSC_SCHEDULE_GRAPH_REPLAY, or DSC_GRAPHS=1 for every schedule); a graph that run_replayed could not lay
    // out at fixed addresses replays only when the heap happens to hand out the same buffers again
    if (ctx->profiling || !(graph_replay || graphs_by_env()) || launches.size() < 4) {
        ++direct_runs;
        return enqueue_all();
    }
    return replay_or_capture(ctx, launches, pointers, rand_seed);
}

int Schedule::replay_or_capture(Context* ctx, const std::vector<PlannedLaunch>& launches, const std::vector<void*>& pointers, uint32_t rand_seed) {
    auto enqueue_all = [&]() -> int {
        for (auto& l : launches) {
            int rc = launch_kernel(ctx, l.kernel, pointers.data() + l.first, l.n, rand_seed);
            if (rc != DSC_OK) return rc;
        }
        return DSC_OK;
    };
    // captured launches read the seed from the context's device cell
    int rc = set_seed(ctx, rand_seed);
    if (rc != DSC_OK) return rc;
    for (auto& c : captured) {
        if (c.pointers == pointers) {
            ++replays;
            hipError_t e = hipGraphLaunch(c.exec, ctx->stream);
            if (e != hipSuccess) return fail(DSC_ERR_HIP, std::string("hipGraphLaunch: ") + hipGetErrorString(e));
            return DSC_OK;
        }
    }
    if (captured.size() >= kMaxCaptured) {
        ++direct_runs;
        return enqueue_all();
    }
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return fail(DSC_ERR_HIP, std::string("hipStreamBeginCapture: ") + hipGetErrorString(e));
    ctx->seed_through_cell = true;
    rc = enqueue_all();
    ctx->seed_through_cell = false;
    hipGraph_t graph = nullptr;
    e = hipStreamEndCapture(ctx->stream, &graph);
    if (rc != DSC_OK) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc;
    }
    if (e != hipSuccess) return fail(DSC_ERR_HIP, std::string("hipStreamEndCapture: ") + hipGetErrorString(e));
    CapturedStep c;
    c.pointers = pointers;
    e = hipGraphInstantiate(&c.exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return fail(DSC_ERR_HIP, std::string("hipGraphInstantiate: ") + hipGetErrorString(e));
    captured.push_back(c);
    e = hipGraphLaunch(c.exec, ctx->stream);
    if (e != hipSuccess) return fail(DSC_ERR_HIP, std::string("hipGraphLaunch: ") + hipGetErrorString(e));
    return DSC_OK;
}

int Schedule::run_replayed(Context* ctx, dsc_buf* params, uint32_t rand_seed, bool* handled) {
    *handled = false;
    auto give_back = [&]() {
        if (replay_region) ctx->heap.free(replay_region);
        for (dsc_buf h : replay_spare)
            if (h) ctx->heap.free(h);
        replay_region = 0;
        replay_spare.clear();
        replay_fixed = false;
    };
    if (replay_spare.empty()) {
        // first run: a spare per written parameter, then the region, sized by a placement in an unbounded one
        replay_spare.assign(n_params, 0);
        for (auto& io : outputs) {
            if (replay_spare[io.param]) continue;
            replay_spare[io.param] = ctx->heap.alloc(std::max<size_t>(node_bytes[io.node], 4));
            if (!replay_spare[io.param]) { give_back(); return DSC_OK; }
        }
        FixedPlan probe;
        if (plan_fixed(ctx, params, replay_spare.data(), nullptr, (size_t)1 << 46, &probe) != DSC_OK) { give_back(); return DSC_OK; }
        replay_region_bytes = std::max<size_t>(probe.high, DeviceHeap::kAlign);
        replay_region = ctx->heap.alloc(replay_region_bytes);
        if (!replay_region) { give_back(); return DSC_OK; }
    }
    void* base = nullptr;
    if (!ctx->heap.info(replay_region, &base, nullptr)) { give_back(); return DSC_OK; }
    FixedPlan plan;
    if (plan_fixed(ctx, params, replay_spare.data(), static_cast<char*>(base), replay_region_bytes, &plan) != DSC_OK) {
        // e.g. a parameter that was handed in without a buffer: let run() say so in its own words
        return DSC_OK;
    }
    *handled = true;
    const int rc = replay_or_capture(ctx, plan.launches, plan.pointers, rand_seed);
    if (rc != DSC_OK) return rc;
    for (int slot : plan.swapped) std::swap(params[slot], replay_spare[slot]);
    // a written parameter that came in without a buffer (an output nobody wrote before the first run) leaves no old
    // buffer behind to be the next run's spare: give its slot a new one, or every later placement would fail
    for (auto& io : outputs) {
        if (replay_spare[io.param] || !params[io.param]) continue;
        replay_spare[io.param] = ctx->heap.alloc(std::max<size_t>(node_bytes[io.node], 4));
        if (!replay_spare[io.param]) {
            give_back();  // out of memory: the allocating run() serves this schedule from now on
            break;
        }
    }
    return DSC_OK;
}

namespace {

// Offsets inside a fixed region: first fit over the free ranges in address order, 256-byte granules, neighbours merged
// on release.  Host-side bookkeeping only.
class RegionPlanner {
  public:
    explicit RegionPlanner(size_t bytes) { free_[0] = bytes; }
    bool take(size_t bytes, size_t* offset) {
        const size_t need = std::max<size_t>(DeviceHeap::kAlign, (bytes + DeviceHeap::kAlign - 1) / DeviceHeap::kAlign * DeviceHeap::kAlign);
        for (auto it = free_.begin(); it != free_.end(); ++it) {
            if (it->second < need) continue;
            *offset = it->first;
            const size_t rest = it->second - need;
            free_.erase(it);
            if (rest) free_[*offset + need] = rest;
            in_use_ += need;
            high_ = std::max(high_, *offset + need);
            return true;
        }
        return false;
    }
    void give(size_t offset, size_t bytes) {
        size_t size = std::max<size_t>(DeviceHeap::kAlign, (bytes + DeviceHeap::kAlign - 1) / DeviceHeap::kAlign * DeviceHeap::kAlign);
        in_use_ -= size;
        auto next = free_.lower_bound(offset);
        if (next != free_.end() && offset + size == next->first) {
            size += next->second;
            next = free_.erase(next);
        }
        if (next != free_.begin()) {
            auto prev = std::prev(next);
            if (prev->first + prev->second == offset) {
                prev->second += size;
                return;
            }
        }
        free_[offset] = size;
    }
    size_t in_use() const { return in_use_; }
    size_t high_water() const { return high_; }

  private:
    std::map<size_t, size_t> free_;  // offset -> size
    size_t in_use_ = 0, high_ = 0;
};

}  // namespace

int Schedule::plan_fixed(Context* ctx, const dsc_buf* params, const dsc_buf* spare, char* scratch, size_t scratch_bytes, FixedPlan* plan) {
    // Environment::run's bookkeeping (environment.rs:326-516) with the allocator taken out: where run() asks the heap,
    // a node that ends up as a parameter's new value is placed in the caller's spare buffer of that slot, and every
    // other node at an offset of `scratch`.  A buffer that one node hands to the next (ScatterAdd accumulators) is
    // placed once, where the last node of that chain needs it.
    enum Where { kNone = 0, kParam, kSpare, kScratch };
    struct Place {
        Where where = kNone;
        void* ptr = nullptr;
        int slot = -1;      // kParam / kSpare
        size_t offset = 0;  // kScratch
        size_t bytes = 0;
    };
    std::vector<int> usage(n_nodes, 0), out_slot(n_nodes, -1), successor(n_nodes, -1);
    std::vector<Place> place(n_nodes);
    for (auto& st : steps) {
        for (int n : st.inputs) usage[n] += 1;
        for (auto& o : st.outputs)
            if (o.copy_from >= 0) successor[o.copy_from] = o.node;
    }
    for (auto& io : outputs) {
        usage[io.node] += 1;
        if (out_slot[io.node] >= 0) return fail(DSC_ERR_UNSUPPORTED, "static run: one node is the new value of two parameters");
        out_slot[io.node] = io.param;
    }
    std::vector<bool> param_is_output(n_params, false), spare_taken(n_params, false);
    for (auto& io : outputs) param_is_output[io.param] = true;
    for (auto& io : inputs) {
        void* p = nullptr;
        size_t have = 0;
        if (params[io.param] == 0 || !ctx->heap.info(params[io.param], &p, &have))
            return fail(DSC_ERR_INVALID, "static run: an input parameter has no buffer");
        if (have < node_bytes[io.node]) return fail(DSC_ERR_INVALID, "static run: an input parameter's buffer is smaller than the parameter");
        place[io.node] = Place{kParam, p, io.param, 0, have};
        if (!param_is_output[io.param]) usage[io.node] += 1;  // the parameter keeps its buffer
    }

    RegionPlanner region(scratch_bytes);
    size_t peak = 0;
    std::string error;
    // where a node that nothing hands a buffer to gets its memory
    auto settle_node = [&](int node) -> bool {
        int slot = -1;
        for (int n = node; n >= 0 && slot < 0; n = successor[n]) slot = out_slot[n];
        Place pl;
        pl.bytes = node_bytes[node];
        if (slot >= 0) {
            void* p = nullptr;
            size_t have = 0;
            if (spare[slot] == 0 || !ctx->heap.info(spare[slot], &p, &have)) {
                error = "static run: parameter slot " + std::to_string(slot) + " is written and has no spare buffer";
                return false;
            }
            if (spare[slot] == params[slot] || spare_taken[slot] || have < node_bytes[node]) {
                error = "static run: the spare buffer of parameter slot " + std::to_string(slot) +
                        (have < node_bytes[node] ? " is smaller than the parameter" : " is the parameter's own buffer or is used twice");
                return false;
            }
            spare_taken[slot] = true;
            pl.where = kSpare;
            pl.ptr = p;
            pl.slot = slot;
        } else {
            if (!region.take(pl.bytes, &pl.offset)) {
                error = "static run: an intermediate of " + std::to_string(pl.bytes) + " bytes does not fit beside the " +
                        std::to_string(region.in_use()) + " bytes of intermediates alive at that point; the static scratch array holds " +
                        std::to_string(scratch_bytes) + " bytes (dsc_schedule_run has no such limit)";
                return false;
            }
            peak = std::max(peak, region.in_use());
            pl.where = kScratch;
            pl.ptr = scratch + pl.offset;
        }
        place[node] = pl;
        return true;
    };
    auto settle = [&](int node) -> int {
        if (settle_node(node)) return DSC_OK;
        return fail(error.find("does not fit") != std::string::npos ? DSC_ERR_UNSUPPORTED : DSC_ERR_INVALID, error);
    };

    typedef PlannedLaunch Launch;
    std::vector<Launch>& launches = plan->launches;
    std::vector<void*>& pointers = plan->pointers;
    launches.clear();
    pointers.clear();
    plan->swapped.clear();
    launches.reserve(steps.size() + 4);
    std::vector<Place> prefilled(prefills.empty() ? 0 : n_nodes);
    for (auto& pf : prefills) {
        launches.push_back(Launch{pf.kernel, pointers.size(), (int)pf.nodes.size()});
        for (int node : pf.nodes) {
            if (int rc = settle(node)) return rc;
            prefilled[node] = place[node];
            place[node] = Place{};
            pointers.push_back(prefilled[node].ptr);
        }
    }
    for (auto& st : steps) {
        for (int n : st.inputs) usage[n] -= 1;
        for (auto& o : st.outputs) {
            if (place[o.node].where != kNone) return fail(DSC_ERR_INVALID, "static run: node written twice");
            if (o.copy_from < 0) {
                if (int rc = settle(o.node)) return rc;
                continue;
            }
            if (usage[o.copy_from] != 0) return fail(DSC_ERR_UNSUPPORTED, "static run: accumulator source still in use (deep copy)");
            if (place[o.copy_from].where != kNone) {
                place[o.node] = place[o.copy_from];
                place[o.copy_from] = Place{};
            } else if (o.from_literal && !prefilled.empty() && prefilled[o.node].where != kNone) {
                place[o.node] = prefilled[o.node];
                prefilled[o.node] = Place{};
            } else if (o.from_literal) {
                if (int rc = settle(o.node)) return rc;
                launches.push_back(Launch{o.fill, pointers.size(), 1});
                pointers.push_back(place[o.node].ptr);
            } else {
                return fail(DSC_ERR_INVALID, "static run: cannot copy-on-write node");
            }
        }
        const int n = (int)st.params.size();
        launches.push_back(Launch{st.kernel, pointers.size(), n});
        for (int i = 0; i < n; ++i) {
            const Place& pl = place[st.params[i]];
            if (pl.where == kNone)
                return fail(DSC_ERR_INVALID, "static run: node " + std::to_string(st.params[i]) + " has no buffer at '" + st.kernel->label + "'");
            pointers.push_back(pl.ptr);
        }
        for (int nd : st.inputs) {
            if (usage[nd] != 0 || place[nd].where == kNone) continue;
            if (place[nd].where == kScratch) region.give(place[nd].offset, place[nd].bytes);
            place[nd] = Place{};  // a parameter's old buffer stays with the caller
        }
    }
    // every written parameter must have landed in its own slot's spare, or still sit in its own buffer (updated in
    // place): anything else would hand a caller's buffer to another slot
    for (auto& io : outputs) {
        const Place& pl = place[io.node];
        const bool in_spare = pl.where == kSpare && pl.slot == io.param;
        const bool in_place = pl.where == kParam && pl.slot == io.param;
        if (!in_spare && !in_place)
            return fail(DSC_ERR_UNSUPPORTED, "static run: parameter slot " + std::to_string(io.param) +
                                                 " would receive another parameter's buffer; use dsc_schedule_run for this graph");
    }

    for (auto& io : outputs)
        if (place[io.node].where == kSpare) plan->swapped.push_back(io.param);
    plan->peak = peak;
    plan->high = region.high_water();
    return DSC_OK;
}

int Schedule::run_static(Context* ctx, dsc_buf* params, dsc_buf* spare, uint32_t rand_seed, char* scratch, size_t scratch_bytes) {
    FixedPlan plan;
    if (int rc = plan_fixed(ctx, params, spare, scratch, scratch_bytes, &plan)) return rc;
    for (auto& l : plan.launches) {
        int rc = launch_kernel(ctx, l.kernel, plan.pointers.data() + l.first, l.n, rand_seed);
        if (rc != DSC_OK) return rc;
    }
    for (int slot : plan.swapped) std::swap(params[slot], spare[slot]);
    static_peak_bytes = std::max(static_peak_bytes, plan.peak);
    return DSC_OK;
}

Schedule::~Schedule() {
    for (auto& c : captured)
        if (c.exec) (void)hipGraphExecDestroy(c.exec);
}

void Schedule::release_replay_buffers(Context* ctx) {
    if (replay_region) ctx->heap.free(replay_region);
    for (dsc_buf h : replay_spare)
        if (h) ctx->heap.free(h);
    replay_region = 0;
    replay_spare.clear();
}

int Schedule::launches_per_run() const {
    int n = (int)steps.size() + (int)prefills.size();
    if (prefills.empty())
        for (auto& st : steps)
            for (auto& o : st.outputs)
                if (o.copy_from >= 0 && o.from_literal) ++n;
    return n;
}

std::string Schedule::describe() const {
    std::ostringstream o;
    o << launches_per_run() << " launches for " << n_clusters << " clusters\n";
    if (replays + direct_runs + (int64_t)captured.size() > 0)
        o << "# graph replays " << replays << ", captured " << captured.size() << ", direct runs " << direct_runs << "\n";
    if (static_peak_bytes) o << "# static runs: at most " << static_peak_bytes << " bytes of the scratch array in use at once\n";
    for (auto& pf : prefills)
        o << "prefill: " << pf.kernel->label << "  grid " << pf.kernel->gen.grid << "x" << pf.kernel->gen.block << " (" << pf.nodes.size()
          << " literal-initialised accumulators)\n";
    double bytes = 0, flops = 0;
    for (size_t i = 0; i < steps.size(); ++i) {
        const Step& st = steps[i];
        char work[64];
        std::snprintf(work, sizeof work, " %.3f MB", st.kernel->gen.algo_bytes / 1e6);
        o << i << ": " << st.kernel->label << "  [" << st.kernel->gen.note << "] grid " << st.kernel->gen.grid << "x"
          << st.kernel->gen.block << work << " clusters";
        for (int c : st.covers) o << " " << c;
        o << "\n";
        bytes += st.kernel->gen.algo_bytes;
        flops += st.kernel->gen.algo_flops;
    }
    char total[160];
    std::snprintf(total, sizeof total, "# algorithmic work per run: %.3f MB moved, %.3f GFLOP in MatMuls\n", bytes / 1e6, flops / 1e9);
    o << total;
    return o.str();
}

std::string Schedule::dot() const {
    auto escaped = [](const std::string& t) {
        std::string r;
        for (char ch : t) {
            if (ch == '"' || ch == '\\') r += '\\';
            r += ch;
        }
        return r;
    };
    std::ostringstream o;
    o << "digraph schedule {\n  rankdir=TB;\n  node [fontname=\"monospace\",fontsize=10];\n";
    std::vector<int> producer(n_nodes, -1);    // step that writes the node
    std::vector<int> from_param(n_nodes, -1);  // parameter slot the node's buffer comes from
    for (auto& io : inputs) {
        from_param[io.node] = io.param;
        o << "  pin" << io.param << " [shape=ellipse,label=\"parameter " << io.param << "\\n" << node_bytes[io.node] << " B\"];\n";
    }
    for (size_t pi = 0; pi < prefills.size(); ++pi) {
        o << "  f" << pi << " [shape=box,style=dashed,label=\"prefill: " << escaped(prefills[pi].kernel->label) << "\"];\n";
    }
    for (size_t i = 0; i < steps.size(); ++i) {
        const Step& st = steps[i];
        char work[64];
        std::snprintf(work, sizeof work, "%.3f MB", st.kernel->gen.algo_bytes / 1e6);
        o << "  s" << i << " [shape=box,style=filled,fillcolor=\"" << (st.covers.size() > 1 ? "#cfe8ff" : "#eeeeee") << "\",label=\"" << i
          << ": " << escaped(st.kernel->label) << "\\n" << escaped(st.kernel->gen.note) << "\\ngrid " << st.kernel->gen.grid << "x"
          << st.kernel->gen.block << ", " << work << ", clusters";
        for (int c : st.covers) o << " " << c;
        o << "\"];\n";
        for (int nd : st.inputs) {
            if (producer[nd] >= 0)
                o << "  s" << producer[nd] << " -> s" << i << " [label=\"n" << nd << ": " << node_bytes[nd] << " B\"];\n";
            else if (from_param[nd] >= 0)
                o << "  pin" << from_param[nd] << " -> s" << i << ";\n";
        }
        for (auto& out : st.outputs) {
            // an accumulator taken over from another node (or from a literal) continues that node's buffer
            if (out.copy_from >= 0 && producer[out.copy_from] >= 0)
                o << "  s" << producer[out.copy_from] << " -> s" << i << " [style=dashed,label=\"n" << out.copy_from << " in place\"];\n";
            else if (out.copy_from >= 0 && from_param[out.copy_from] >= 0)
                o << "  pin" << from_param[out.copy_from] << " -> s" << i << " [style=dashed,label=\"in place\"];\n";
            producer[out.node] = (int)i;
        }
    }
    for (auto& io : outputs) {
        o << "  pout" << io.param << " [shape=ellipse,peripheries=2,label=\"parameter " << io.param << "\\n" << node_bytes[io.node] << " B\"];\n";
        if (producer[io.node] >= 0) o << "  s" << producer[io.node] << " -> pout" << io.param << ";\n";
    }
    o << "}\n";
    return o.str();
}

}  // namespace dsc
