#include "desc.hpp"

#include <cstdio>

namespace dsc {

namespace {
template <class T>
void put(std::string& s, const T& v) {
    s.append(reinterpret_cast<const char*>(&v), sizeof(T));
}
void put_shape(std::string& s, const dsc_shape& sh) {
    put(s, sh.rank);
    for (int i = 0; i < sh.rank; ++i) put(s, sh.dims[i]);
}
void put_view(std::string& s, const dsc_view& v) {
    put_shape(s, v.in_shape);
    for (int i = 0; i < v.in_shape.rank; ++i) put(s, v.in_offset[i]);
    put_shape(s, v.out_shape);
    for (int j = 0; j < v.out_shape.rank; ++j) {
        put(s, v.map_axis[j]);
        put(s, v.map_step[j]);
    }
}
std::string check_shape(const dsc_shape& s, const char* what) {
    if (s.rank < 1 || s.rank > DSC_MAX_DIM) return std::string(what) + ": rank out of range";
    for (int i = 0; i < s.rank; ++i)
        if (s.dims[i] <= 0) return std::string(what) + ": non-positive extent";
    return "";
}
std::string check_view(const dsc_view& v, const char* what) {
    std::string e = check_shape(v.in_shape, what);
    if (!e.empty()) return e;
    e = check_shape(v.out_shape, what);
    if (!e.empty()) return e;
    for (int j = 0; j < v.out_shape.rank; ++j)
        if (v.map_axis[j] >= v.in_shape.rank) return std::string(what) + ": mapping names a missing input axis";
    return "";
}
}  // namespace

std::string KernelDesc::key() const {
    std::string s;
    put(s, d.kind);
    put_shape(s, d.shape);
    put(s, (int32_t)inputs.size());
    for (auto& v : inputs) put_view(s, v);
    put(s, (int32_t)ops.size());
    for (auto& op : ops) {
        put(s, op.kind);
        put(s, op.op);
        for (int a = 0; a < 4; ++a) put(s, op.args[a]);
        put(s, op.bits);
        put(s, op.input_index);
        put(s, op.view_index);
        put(s, op.axis);
        if (op.kind == DSC_PE_GATHER) put_shape(s, op.gather_shape);
    }
    put(s, (int32_t)outputs.size());
    for (auto o : outputs) put(s, o);
    put(s, (int32_t)builtin_views.size());
    for (auto& v : builtin_views) put_view(s, v);
    switch (d.kind) {
    case DSC_KERNEL_FILL: put(s, d.fill_bits); break;
    case DSC_KERNEL_REDUCE: put(s, d.reduce_op); put(s, d.axis); break;
    case DSC_KERNEL_UNPAD: put(s, d.axis); put(s, d.pad); break;
    case DSC_KERNEL_WINDOWS_TO_IMAGE: put(s, d.stride_w); put(s, d.stride_h); break;
    case DSC_KERNEL_SCATTER_ADD: put(s, d.axis); break;
    case DSC_KERNEL_MATMUL: put(s, d.output_mode); break;
    default: break;
    }
    return s;
}

int buffer_count(const dsc_kernel_desc& d) {
    switch (d.kind) {
    case DSC_KERNEL_FILL: return 1;
    case DSC_KERNEL_PER_ELEMENT: return d.n_inputs + d.n_outputs;
    case DSC_KERNEL_REDUCE:
    case DSC_KERNEL_UNPAD:
    case DSC_KERNEL_WINDOWS_TO_IMAGE: return 2;
    case DSC_KERNEL_MATMUL:
    case DSC_KERNEL_SCATTER_ADD: return 3;
    default: return 0;
    }
}

MatMulDims matmul_dims(const dsc_kernel_desc& d) {
    MatMulDims r{};
    const dsc_view& a = d.inputs[0];
    const dsc_view& b = d.inputs[1];
    r.m = a.out_shape.dims[1];
    r.k = a.out_shape.dims[2];
    r.n = b.out_shape.dims[2];
    r.chunks = d.shape.dims[0];
    r.batch = d.shape.dims[d.output_mode == DSC_MATMUL_ROWS ? 2 : 1];
    return r;
}

int64_t reference_group_count(const dsc_kernel_desc& d) {
    auto up = [](int64_t a, int64_t b) { return (a + b - 1) / b; };
    switch (d.kind) {
    case DSC_KERNEL_MATMUL: {
        MatMulDims g = matmul_dims(d);
        return g.batch * g.chunks * up(g.m, 16) * up(g.n, 16);
    }
    case DSC_KERNEL_SCATTER_ADD: return up(element_count(d.inputs[0].out_shape), 64);
    default: return up(element_count(d.shape), 64);
    }
}

std::string label_name(const dsc_kernel_desc& d) {
    char buf[160];
    switch (d.kind) {
    case DSC_KERNEL_FILL:
        std::snprintf(buf, sizeof buf, "Fill(0x%08x) %lld", d.fill_bits, (long long)d.shape.dims[0]);
        return buf;
    case DSC_KERNEL_PER_ELEMENT:
        std::snprintf(buf, sizeof buf, "PerElement (%d ops) [%lld]", d.n_ops, (long long)d.shape.dims[0]);
        return buf;
    case DSC_KERNEL_REDUCE:
        std::snprintf(buf, sizeof buf, "Reduce (k=%lld) ", (long long)d.inputs[0].out_shape.dims[d.axis]);
        return buf + shape_str(d.shape);
    case DSC_KERNEL_MATMUL:
        std::snprintf(buf, sizeof buf, "MatMul (k=%lld) ", (long long)matmul_dims(d).k);
        return buf + shape_str(d.shape);
    case DSC_KERNEL_UNPAD: return "Unpad " + shape_str(d.shape);
    case DSC_KERNEL_WINDOWS_TO_IMAGE: return "WindowsToImage " + shape_str(d.shape);
    case DSC_KERNEL_SCATTER_ADD: return "ScatterAdd " + shape_str(d.inputs[0].out_shape);
    default: return "?";
    }
}

std::string validate(const dsc_kernel_desc& d) {
    std::string e = check_shape(d.shape, "shape");
    if (!e.empty()) return e;
    if (d.n_inputs < 0 || (d.n_inputs > 0 && !d.inputs)) return "inputs missing";
    for (int i = 0; i < d.n_inputs; ++i) {
        e = check_view(d.inputs[i], "input view");
        if (!e.empty()) return e;
    }
    auto need_inputs = [&](int n) { return d.n_inputs == n ? "" : "wrong number of input views"; };
    switch (d.kind) {
    case DSC_KERNEL_FILL:
        if (d.shape.rank != 1) return "fill: shape must be [element_count]";
        return need_inputs(0);
    case DSC_KERNEL_PER_ELEMENT: {
        if (d.shape.rank != 1) return "per-element: shape must be [element_count]";
        if (d.n_ops <= 0 || !d.ops) return "per-element: no ops";
        if (d.n_outputs <= 0 || !d.outputs) return "per-element: no outputs";
        const int64_t n = d.shape.dims[0];
        for (int i = 0; i < d.n_builtin_views; ++i) {
            e = check_view(d.builtin_views[i], "builtin view");
            if (!e.empty()) return e;
            if (element_count(d.builtin_views[i].out_shape) != n) return "per-element: builtin view element count differs";
        }
        for (int i = 0; i < d.n_ops; ++i) {
            const dsc_pe_op& op = d.ops[i];
            int nargs = 0;
            switch (op.kind) {
            case DSC_PE_LOAD:
                if (op.input_index < 0 || op.input_index >= d.n_inputs) return "per-element: load of a missing input";
                if (element_count(d.inputs[op.input_index].out_shape) != n) return "per-element: load view element count differs";
                break;
            case DSC_PE_LITERAL_F32:
            case DSC_PE_LITERAL_U32: break;
            case DSC_PE_COORD:
            case DSC_PE_RAND:
                if (op.view_index < 0 || op.view_index >= d.n_builtin_views) return "per-element: missing builtin view";
                break;
            case DSC_PE_UNARY:
                if (op.op < 0 || op.op > DSC_UN_UINT_TO_FLOAT) return "per-element: unknown unary op";
                nargs = 1;
                break;
            case DSC_PE_BINARY:
                if (op.op < 0 || op.op > DSC_BIN_UBITXOR) return "per-element: unknown binary op";
                nargs = 2;
                break;
            case DSC_PE_SELECT:
                if (op.op < 0 || op.op > DSC_CMP_GT) return "per-element: unknown compare mode";
                nargs = 4;
                break;
            case DSC_PE_GATHER:
                if (op.input_index < 0 || op.input_index >= d.n_inputs) return "per-element: gather from a missing input";
                e = check_shape(op.gather_shape, "gather shape");
                if (!e.empty()) return e;
                if (element_count(op.gather_shape) != n) return "per-element: gather shape element count differs";
                if (op.gather_shape.rank != d.inputs[op.input_index].out_shape.rank) return "per-element: gather rank differs from its table view";
                if (op.axis < 0 || op.axis >= op.gather_shape.rank) return "per-element: gather axis out of range";
                nargs = 1;
                break;
            default: return "per-element: unknown op kind";
            }
            for (int a = 0; a < nargs; ++a)
                if (op.args[a] < 0 || op.args[a] >= i) return "per-element: argument is not an earlier op";
        }
        for (int o = 0; o < d.n_outputs; ++o)
            if (d.outputs[o] < 0 || d.outputs[o] >= d.n_ops) return "per-element: output names a missing op";
        return "";
    }
    case DSC_KERNEL_REDUCE: {
        e = need_inputs(1);
        if (!e.empty()) return e;
        const dsc_view& v = d.inputs[0];
        if (v.out_shape.rank != d.shape.rank) return "reduce: rank differs from input view";
        if (d.axis < 0 || d.axis >= d.shape.rank) return "reduce: axis out of range";
        for (int i = 0; i < d.shape.rank; ++i)
            if (d.shape.dims[i] != (i == d.axis ? 1 : v.out_shape.dims[i])) return "reduce: shape is not the input with the axis collapsed";
        if (d.reduce_op != DSC_REDUCE_MAX && d.reduce_op != DSC_REDUCE_SUM) return "reduce: unknown op";
        return "";
    }
    case DSC_KERNEL_MATMUL: {
        e = need_inputs(2);
        if (!e.empty()) return e;
        const dsc_view& a = d.inputs[0];
        const dsc_view& b = d.inputs[1];
        if (a.out_shape.rank != 3 || b.out_shape.rank != 3 || d.shape.rank != 4) return "matmul: operands must be rank 3, output rank 4";
        if (d.output_mode != DSC_MATMUL_BATCHES && d.output_mode != DSC_MATMUL_ROWS) return "matmul: unknown output mode";
        MatMulDims g = matmul_dims(d);
        if (a.out_shape.dims[0] != g.batch || b.out_shape.dims[0] != g.batch) return "matmul: batch mismatch";
        if (b.out_shape.dims[1] != g.k) return "matmul: inner dimension mismatch";
        const bool rows = d.output_mode == DSC_MATMUL_ROWS;
        if (d.shape.dims[rows ? 1 : 2] != g.m || d.shape.dims[3] != g.n) return "matmul: output shape mismatch";
        if (g.chunks < 1) return "matmul: bad chunk count";
        return "";
    }
    case DSC_KERNEL_UNPAD: {
        e = need_inputs(1);
        if (!e.empty()) return e;
        const dsc_view& v = d.inputs[0];
        if (v.out_shape.rank != d.shape.rank) return "unpad: rank differs from input view";
        if (d.axis < 0 || d.axis >= d.shape.rank || d.pad < 0) return "unpad: bad axis or pad";
        for (int i = 0; i < d.shape.rank; ++i)
            if (v.out_shape.dims[i] != d.shape.dims[i] + (i == d.axis ? 2 * d.pad : 0)) return "unpad: shape mismatch";
        return "";
    }
    case DSC_KERNEL_WINDOWS_TO_IMAGE: {
        e = need_inputs(1);
        if (!e.empty()) return e;
        const dsc_view& v = d.inputs[0];
        const int r = v.out_shape.rank;
        if (r < 6 || d.shape.rank != r - 3) return "windows_to_image: rank mismatch";
        if (d.stride_w <= 0 || d.stride_h <= 0) return "windows_to_image: bad stride";
        const int64_t oh = v.out_shape.dims[r - 6], ow = v.out_shape.dims[r - 5], g = v.out_shape.dims[r - 4];
        const int64_t fh = v.out_shape.dims[r - 3], fw = v.out_shape.dims[r - 2], nc = v.out_shape.dims[r - 1];
        const int bd = d.shape.rank - 3;
        for (int i = 0; i < bd; ++i)
            if (d.shape.dims[i] != v.out_shape.dims[i]) return "windows_to_image: batch dims mismatch";
        if (d.shape.dims[bd] != (oh - 1) * d.stride_h + fh || d.shape.dims[bd + 1] != (ow - 1) * d.stride_w + fw ||
            d.shape.dims[bd + 2] != g * nc)
            return "windows_to_image: image shape mismatch";
        return "";
    }
    case DSC_KERNEL_SCATTER_ADD: {
        e = need_inputs(2);
        if (!e.empty()) return e;
        const dsc_view& v = d.inputs[0];
        const dsc_view& ix = d.inputs[1];
        if (v.out_shape.rank != d.shape.rank) return "scatter_add: rank mismatch";
        if (d.axis < 0 || d.axis >= d.shape.rank) return "scatter_add: axis out of range";
        if (ix.out_shape.rank != 1 || ix.out_shape.dims[0] != v.out_shape.dims[d.axis]) return "scatter_add: index count mismatch";
        for (int i = 0; i < d.shape.rank; ++i)
            if (i != d.axis && v.out_shape.dims[i] != d.shape.dims[i]) return "scatter_add: values shape mismatch";
        return "";
    }
    default: return "unknown kernel kind";
    }
}

}  // namespace dsc
