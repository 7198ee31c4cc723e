// Owned, hashable copies of the C-ABI descriptors plus the View arithmetic the code generator needs.
#pragma once

#include "../../include/descent_hip.h"

#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

namespace dsc {

inline int64_t element_count(const dsc_shape& s) {
    int64_t n = 1;
    for (int i = 0; i < s.rank; ++i) n *= s.dims[i];
    return n;
}

inline bool same_shape(const dsc_shape& a, const dsc_shape& b) {
    if (a.rank != b.rank) return false;
    for (int i = 0; i < a.rank; ++i)
        if (a.dims[i] != b.dims[i]) return false;
    return true;
}

inline void strides_of(const dsc_shape& s, int64_t* out) {
    int64_t st = 1;
    for (int i = s.rank - 1; i >= 0; --i) {
        out[i] = st;
        st *= s.dims[i];
    }
}

inline std::string shape_str(const dsc_shape& s) {
    std::string out = "[";
    for (int i = 0; i < s.rank; ++i) {
        if (i) out += ", ";
        out += std::to_string(s.dims[i]);
    }
    return out + "]";
}

// Range [lo, hi] of the coordinate a view can produce on one input axis (shape.rs:503-526).
inline void axis_span(const dsc_view& v, int axis, int64_t* lo, int64_t* hi) {
    *lo = *hi = v.in_offset[axis];
    for (int j = 0; j < v.out_shape.rank; ++j) {
        if (v.map_axis[j] == axis) {
            int64_t d = (v.out_shape.dims[j] - 1) * v.map_step[j];
            if (d < 0) *lo += d; else *hi += d;
        }
    }
}

inline bool needs_clamp(const dsc_view& v, int axis) {
    int64_t lo, hi;
    axis_span(v, axis, &lo, &hi);
    return lo < 0 || hi > v.in_shape.dims[axis] - 1;
}

inline bool any_clamp(const dsc_view& v) {
    for (int i = 0; i < v.in_shape.rank; ++i)
        if (needs_clamp(v, i)) return true;
    return false;
}

inline bool is_identity(const dsc_view& v) {
    if (!same_shape(v.in_shape, v.out_shape)) return false;
    for (int i = 0; i < v.in_shape.rank; ++i) {
        if (v.in_offset[i] != 0) return false;
        if (v.in_shape.dims[i] > 1 ? (v.map_axis[i] != i || v.map_step[i] != 1) : (v.map_axis[i] != -1)) return false;
    }
    return true;
}

// An un-clamped view is affine in the output coordinates: index = base + sum_j coef[j]*coord[j].
// Returns false when some axis needs a clamp.
inline bool affine_form(const dsc_view& v, int64_t* base, int64_t* coef /*[out_rank]*/) {
    if (any_clamp(v)) return false;
    int64_t st[DSC_MAX_DIM];
    strides_of(v.in_shape, st);
    *base = 0;
    for (int i = 0; i < v.in_shape.rank; ++i) *base += v.in_offset[i] * st[i];
    for (int j = 0; j < v.out_shape.rank; ++j) coef[j] = v.map_axis[j] >= 0 ? v.map_step[j] * st[v.map_axis[j]] : 0;
    return true;
}

// Same linear element order as the input (shape.rs:403-419).
inline bool is_contiguous(const dsc_view& v) {
    if (element_count(v.in_shape) != element_count(v.out_shape)) return false;
    int64_t base, coef[DSC_MAX_DIM], ost[DSC_MAX_DIM];
    if (!affine_form(v, &base, coef) || base != 0) return false;
    for (int i = 0; i < v.in_shape.rank; ++i)
        if (v.in_offset[i] != 0) return false;
    strides_of(v.out_shape, ost);
    for (int j = 0; j < v.out_shape.rank; ++j)
        if (v.map_axis[j] >= 0 && coef[j] != ost[j]) return false;
    return true;
}

// Deep copy of a dsc_kernel_desc; `raw()` re-exposes it with pointers into the owned vectors.
struct KernelDesc {
    dsc_kernel_desc d{};
    std::vector<dsc_view> inputs;
    std::vector<dsc_pe_op> ops;
    std::vector<int32_t> outputs;
    std::vector<dsc_view> builtin_views;

    KernelDesc() = default;
    explicit KernelDesc(const dsc_kernel_desc& src) { assign(src); }
    KernelDesc(const KernelDesc& o) { assign(o.raw()); }
    KernelDesc& operator=(const KernelDesc& o) {
        if (this != &o) assign(o.raw());
        return *this;
    }

    void assign(const dsc_kernel_desc& src) {
        d = src;
        inputs.assign(src.inputs, src.inputs + (src.inputs ? src.n_inputs : 0));
        ops.assign(src.ops, src.ops + (src.ops ? src.n_ops : 0));
        outputs.assign(src.outputs, src.outputs + (src.outputs ? src.n_outputs : 0));
        builtin_views.assign(src.builtin_views, src.builtin_views + (src.builtin_views ? src.n_builtin_views : 0));
        normalise();
        fix();
    }

    const dsc_kernel_desc& raw() const { return d; }

    // canonical bytes: the cache key (kernel.rs:1037-1056 keys on descriptor equality)
    std::string key() const;

  private:
    void fix() {
        d.n_inputs = (int32_t)inputs.size();
        d.inputs = inputs.data();
        d.n_ops = (int32_t)ops.size();
        d.ops = ops.data();
        d.n_outputs = (int32_t)outputs.size();
        d.outputs = outputs.data();
        d.n_builtin_views = (int32_t)builtin_views.size();
        d.builtin_views = builtin_views.data();
    }
    // zero everything past `rank` so that byte-wise comparison is content comparison
    static void norm_shape(dsc_shape& s) {
        for (int i = s.rank < 0 ? 0 : s.rank; i < DSC_MAX_DIM; ++i) s.dims[i] = 0;
    }
    static void norm_view(dsc_view& v) {
        norm_shape(v.in_shape);
        norm_shape(v.out_shape);
        for (int i = v.in_shape.rank < 0 ? 0 : v.in_shape.rank; i < DSC_MAX_DIM; ++i) v.in_offset[i] = 0;
        for (int j = 0; j < DSC_MAX_DIM; ++j) {
            if (j >= v.out_shape.rank) { v.map_axis[j] = -1; v.map_step[j] = 0; }
            else if (v.map_axis[j] < 0) { v.map_axis[j] = -1; v.map_step[j] = 0; }
        }
    }
    void normalise() {
        norm_shape(d.shape);
        for (auto& v : inputs) norm_view(v);
        for (auto& v : builtin_views) norm_view(v);
        for (auto& op : ops) {
            if (op.kind != DSC_PE_GATHER) { op.gather_shape = dsc_shape{}; op.axis = 0; }
            else norm_shape(op.gather_shape);
            int nargs = op.kind == DSC_PE_UNARY || op.kind == DSC_PE_GATHER ? 1 : op.kind == DSC_PE_BINARY ? 2 : op.kind == DSC_PE_SELECT ? 4 : 0;
            for (int a = nargs; a < 4; ++a) op.args[a] = 0;
            if (op.kind != DSC_PE_UNARY && op.kind != DSC_PE_BINARY && op.kind != DSC_PE_SELECT) op.op = 0;
            if (op.kind != DSC_PE_LOAD && op.kind != DSC_PE_GATHER) op.input_index = 0;
            if (op.kind != DSC_PE_COORD && op.kind != DSC_PE_RAND) op.view_index = 0;
            if (op.kind != DSC_PE_LITERAL_F32 && op.kind != DSC_PE_LITERAL_U32 && op.kind != DSC_PE_RAND) op.bits = 0;
        }
    }
};

// Validates ranks, axes, op argument indices and buffer counts.  Returns "" when the descriptor is well
// formed, else a message.
std::string validate(const dsc_kernel_desc& d);

// Kernel::buffer_count / group_count / label_name (kernel.rs:135-143).
int buffer_count(const dsc_kernel_desc& d);
int64_t reference_group_count(const dsc_kernel_desc& d);
std::string label_name(const dsc_kernel_desc& d);

// MatMul geometry helpers (kernel.rs:399-417).
struct MatMulDims {
    int64_t batch, m, n, k, chunks;
};
MatMulDims matmul_dims(const dsc_kernel_desc& d);

}  // namespace dsc
