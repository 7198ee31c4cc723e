// CPU oracle for the descent kernel set.  TEST INFRASTRUCTURE ONLY.
//
// A restatement, as plain loops, of what each of the reference's seven generated GLSL kernels computes for
// one descriptor (paths below are relative to the reference repository).  Only tests, the smoke check and the
// cpu_baseline leg of the benchmark may load this library; the product never calls it.
//
//   View addressing        src/kernel.rs:89-133, src/shape.rs:503-526          (load_index)
//   linear id -> coords    src/kernel_common.glsl:1-193                         (grid_coord)
//   pcg / rand_from_index  src/kernel_common.glsl:205-216                       (pcg, rand_from_index)
//   Fill                   src/kernel.rs:151-180
//   PerElement             src/kernel.rs:203-366
//   Reduce                 src/kernel.rs:573-629
//   MatMul                 src/kernel.rs:420-541 + src/kernel_matmul.glsl:43-97
//   Unpad                  src/kernel.rs:652-697
//   WindowsToImage         src/kernel.rs:719-797  (bounds-checked, see note below)
//   ScatterAdd             src/kernel.rs:820-857
//
// What pins each function (checked in tests/test_oracle_golden.py):
//   load_index/clamp: the reference's unpad_image test (edge 2, corner 4) and pad_image test, plus a
//     brute-force comparison with numpy edge padding / slicing / transposition;
//   matmul: array_api's [10,15,22], the conv2d test (8x8 nines), float64 numpy products, and the invariant
//     that split-K partials sum to the full product;
//   reduce: the reduce test (row sums of 0..99), numpy sum/max;
//   windows_to_image/unpad: adjoint identity <W x, y> == <x, W^T y> against the forward view, and the
//     max_pool2d test;
//   gather/scatter_add/concat: the reference tests of the same names, numpy fancy indexing / np.add.at;
//   pcg: the published PCG-RXS-M-XS-32 output function, cross-checked against an independent Python integer
//     implementation;
//   transcendental rounding (exp/log/sin/cos/pow/sqrt) and FMA contraction under a Vulkan driver: parity
//     unpinned (driver-dependent, a few ulp; inside the 1e-4 relative-L2 budget).
//
// Deviation from the reference, on purpose: WindowsToImage here checks 0 <= out_x < out_w and
// 0 <= out_y < out_h.  The reference declares out_w/out_h but never tests them (src/kernel.rs:750-751,
// 775-776), so for stride-1 3x3 windows its border pixels read aliased or out-of-buffer elements.  The
// oracle computes the true adjoint of image_to_windows.
//
// Summation order: every sum is accumulated in fp32 in the same element order as the GLSL loops, built with
// -ffp-contract=off.  For MatMul the shader accumulates, per output element and k-chunk, k ascending; tiles do
// not change that order, so the oracle uses plain loops over dense copies of the operands.

#include "../include/descent_hip.h"

#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

namespace {

inline float u2f(uint32_t x) { float f; std::memcpy(&f, &x, 4); return f; }
inline uint32_t f2u(float x) { uint32_t u; std::memcpy(&u, &x, 4); return u; }
inline int32_t f2i(float x) { int32_t i; std::memcpy(&i, &x, 4); return i; }

int64_t element_count(const dsc_shape& s) {
    int64_t n = 1;
    for (int i = 0; i < s.rank; ++i) n *= s.dims[i];
    return n;
}

// compute_grid_coord: row-major decomposition of a linear id
inline void grid_coord(int64_t id, const dsc_shape& s, int64_t* coord) {
    for (int i = s.rank - 1; i > 0; --i) {
        int64_t q = id / s.dims[i];
        coord[i] = id - q * s.dims[i];
        id = q;
    }
    coord[0] = id;
}

// A view with everything the per-element address computation needs precomputed.
struct ViewEval {
    int in_rank, out_rank;
    int64_t in_dim[DSC_MAX_DIM], in_off[DSC_MAX_DIM], in_stride[DSC_MAX_DIM];
    bool clamp[DSC_MAX_DIM];
    int map_axis[DSC_MAX_DIM];
    int64_t map_step[DSC_MAX_DIM];
    dsc_shape out_shape;

    explicit ViewEval(const dsc_view& v) {
        in_rank = v.in_shape.rank;
        out_rank = v.out_shape.rank;
        out_shape = v.out_shape;
        int64_t s = 1;
        for (int i = in_rank - 1; i >= 0; --i) {
            in_dim[i] = v.in_shape.dims[i];
            in_off[i] = v.in_offset[i];
            in_stride[i] = s;
            s *= in_dim[i];
        }
        for (int j = 0; j < out_rank; ++j) {
            map_axis[j] = v.map_axis[j];
            map_step[j] = v.map_step[j];
        }
        // input_needs_clamp: reachable range of the axis coordinate leaves [0, dim-1]
        for (int i = 0; i < in_rank; ++i) {
            int64_t lo = in_off[i], hi = in_off[i];
            for (int j = 0; j < out_rank; ++j) {
                if (map_axis[j] == i) {
                    int64_t d = (v.out_shape.dims[j] - 1) * map_step[j];
                    if (d < 0) lo += d; else hi += d;
                }
            }
            clamp[i] = lo < 0 || hi > in_dim[i] - 1;
        }
    }

    inline int64_t load_index(const int64_t* coord) const {
        int64_t c[DSC_MAX_DIM];
        for (int i = 0; i < in_rank; ++i) c[i] = in_off[i];
        for (int j = 0; j < out_rank; ++j)
            if (map_axis[j] >= 0) c[map_axis[j]] += map_step[j] * coord[j];
        int64_t idx = 0;
        for (int i = 0; i < in_rank; ++i) {
            int64_t x = c[i];
            if (clamp[i]) x = x < 0 ? 0 : (x > in_dim[i] - 1 ? in_dim[i] - 1 : x);
            idx += x * in_stride[i];
        }
        return idx;
    }

    bool is_identity() const {
        if (in_rank != out_rank) return false;
        for (int i = 0; i < in_rank; ++i) {
            if (in_off[i] != 0 || in_dim[i] != out_shape.dims[i]) return false;
            if (in_dim[i] > 1 ? (map_axis[i] != i || map_step[i] != 1) : (map_axis[i] != -1)) return false;
        }
        return true;
    }
};

inline uint32_t pcg(uint32_t v) {
    uint32_t state = v * 747796405u + 2891336453u;
    uint32_t word = ((state >> ((state >> 28u) + 4u)) ^ state) * 277803737u;
    return (word >> 22u) ^ word;
}

inline float rand_from_index(uint32_t uid, int32_t index, uint32_t seed) {
    uint32_t hash = pcg(pcg((uint32_t)index) + seed + uid);
    return (float)hash / (float)0xffffffffu;
}

// ---------------------------------------------------------------------------------------------------------

int run_fill(const dsc_kernel_desc& d, float* const* bufs) {
    int64_t n = d.shape.dims[0];
    float v = u2f(d.fill_bits);
    float* out = bufs[0];
    for (int64_t i = 0; i < n; ++i) out[i] = v;
    return 0;
}

int run_per_element(const dsc_kernel_desc& d, float* const* bufs, uint32_t seed) {
    const int64_t n = d.shape.dims[0];
    std::vector<ViewEval> in_views, bi_views;
    for (int i = 0; i < d.n_inputs; ++i) in_views.emplace_back(d.inputs[i]);
    for (int i = 0; i < d.n_builtin_views; ++i) bi_views.emplace_back(d.builtin_views[i]);
    std::vector<bool> in_identity(d.n_inputs), bi_identity(d.n_builtin_views);
    for (int i = 0; i < d.n_inputs; ++i) in_identity[i] = in_views[i].is_identity();
    for (int i = 0; i < d.n_builtin_views; ++i) bi_identity[i] = bi_views[i].is_identity();

    for (int oi = 0; oi < d.n_ops; ++oi) {  // reject malformed op lists before any work
        const dsc_pe_op& op = d.ops[oi];
        if (op.kind < DSC_PE_LOAD || op.kind > DSC_PE_GATHER) return 1;
        if (op.kind == DSC_PE_UNARY && (op.op < 0 || op.op > DSC_UN_UINT_TO_FLOAT)) return 1;
        if (op.kind == DSC_PE_BINARY && (op.op < 0 || op.op > DSC_BIN_UBITXOR)) return 1;
        if (op.kind == DSC_PE_SELECT && (op.op < 0 || op.op > DSC_CMP_GT)) return 1;
        const int nargs = op.kind == DSC_PE_UNARY || op.kind == DSC_PE_GATHER ? 1
                        : op.kind == DSC_PE_BINARY ? 2 : op.kind == DSC_PE_SELECT ? 4 : 0;
        for (int a = 0; a < nargs; ++a)
            if (op.args[a] < 0 || op.args[a] >= oi) return 1;
        if ((op.kind == DSC_PE_LOAD || op.kind == DSC_PE_GATHER) && (op.input_index < 0 || op.input_index >= d.n_inputs)) return 1;
        if ((op.kind == DSC_PE_COORD || op.kind == DSC_PE_RAND) && (op.view_index < 0 || op.view_index >= d.n_builtin_views)) return 1;
    }
    const int64_t CH = 1024;  // ops are evaluated chunk-wise so the inner loops vectorise
#pragma omp parallel
    {
        std::vector<float> tmp((size_t)d.n_ops * CH);
        int64_t coord[DSC_MAX_DIM];
#pragma omp for schedule(static)
        for (int64_t base = 0; base < n; base += CH) {
            const int64_t cnt = (n - base < CH) ? (n - base) : CH;
            for (int oi = 0; oi < d.n_ops; ++oi) {
                const dsc_pe_op& op = d.ops[oi];
                float* t = &tmp[(size_t)oi * CH];
                const float* a0 = &tmp[(size_t)op.args[0] * CH];
                const float* a1 = &tmp[(size_t)op.args[1] * CH];
                const float* a2 = &tmp[(size_t)op.args[2] * CH];
                const float* a3 = &tmp[(size_t)op.args[3] * CH];
                switch (op.kind) {
                case DSC_PE_LOAD: {
                    const ViewEval& v = in_views[op.input_index];
                    const float* src = bufs[op.input_index];
                    if (in_identity[op.input_index]) {
                        for (int64_t e = 0; e < cnt; ++e) t[e] = src[base + e];
                    } else {
                        for (int64_t e = 0; e < cnt; ++e) {
                            grid_coord(base + e, v.out_shape, coord);
                            t[e] = src[v.load_index(coord)];
                        }
                    }
                    break;
                }
                case DSC_PE_LITERAL_F32:
                case DSC_PE_LITERAL_U32: {
                    float v = u2f(op.bits);
                    for (int64_t e = 0; e < cnt; ++e) t[e] = v;
                    break;
                }
                case DSC_PE_COORD: {
                    const ViewEval& v = bi_views[op.view_index];
                    for (int64_t e = 0; e < cnt; ++e) {
                        grid_coord(base + e, v.out_shape, coord);
                        t[e] = (float)v.load_index(coord);
                    }
                    break;
                }
                case DSC_PE_RAND: {
                    const ViewEval& v = bi_views[op.view_index];
                    for (int64_t e = 0; e < cnt; ++e) {
                        int64_t idx = base + e;
                        if (!bi_identity[op.view_index]) {
                            grid_coord(base + e, v.out_shape, coord);
                            idx = v.load_index(coord);
                        }
                        t[e] = rand_from_index(op.bits, (int32_t)idx, seed);
                    }
                    break;
                }
                case DSC_PE_UNARY:
                    switch (op.op) {
                    case DSC_UN_MOV: for (int64_t e = 0; e < cnt; ++e) t[e] = a0[e]; break;
                    case DSC_UN_NEG: for (int64_t e = 0; e < cnt; ++e) t[e] = -a0[e]; break;
                    case DSC_UN_SQRT: for (int64_t e = 0; e < cnt; ++e) t[e] = std::sqrt(a0[e]); break;
                    case DSC_UN_EXP: for (int64_t e = 0; e < cnt; ++e) t[e] = std::exp(a0[e]); break;
                    case DSC_UN_LOG: for (int64_t e = 0; e < cnt; ++e) t[e] = std::log(a0[e]); break;
                    case DSC_UN_SIN: for (int64_t e = 0; e < cnt; ++e) t[e] = std::sin(a0[e]); break;
                    case DSC_UN_COS: for (int64_t e = 0; e < cnt; ++e) t[e] = std::cos(a0[e]); break;
                    case DSC_UN_FLOAT_TO_UINT:
                        for (int64_t e = 0; e < cnt; ++e) t[e] = u2f((uint32_t)a0[e]);
                        break;
                    case DSC_UN_UINT_TO_FLOAT:
                        for (int64_t e = 0; e < cnt; ++e) t[e] = (float)f2u(a0[e]);
                        break;
                    default: break;
                    }
                    break;
                case DSC_PE_BINARY:
                    switch (op.op) {
                    case DSC_BIN_ADD: for (int64_t e = 0; e < cnt; ++e) t[e] = a0[e] + a1[e]; break;
                    case DSC_BIN_SUB: for (int64_t e = 0; e < cnt; ++e) t[e] = a0[e] - a1[e]; break;
                    case DSC_BIN_MUL: for (int64_t e = 0; e < cnt; ++e) t[e] = a0[e] * a1[e]; break;
                    case DSC_BIN_DIV: for (int64_t e = 0; e < cnt; ++e) t[e] = a0[e] / a1[e]; break;
                    case DSC_BIN_POW: for (int64_t e = 0; e < cnt; ++e) t[e] = std::pow(a0[e], a1[e]); break;
                    case DSC_BIN_UADD: for (int64_t e = 0; e < cnt; ++e) t[e] = u2f(f2u(a0[e]) + f2u(a1[e])); break;
                    case DSC_BIN_UMUL: for (int64_t e = 0; e < cnt; ++e) t[e] = u2f(f2u(a0[e]) * f2u(a1[e])); break;
                    case DSC_BIN_UREM: for (int64_t e = 0; e < cnt; ++e) t[e] = u2f(f2u(a0[e]) % f2u(a1[e])); break;
                    case DSC_BIN_UBITXOR: for (int64_t e = 0; e < cnt; ++e) t[e] = u2f(f2u(a0[e]) ^ f2u(a1[e])); break;
                    default: break;
                    }
                    break;
                case DSC_PE_SELECT:
                    if (op.op == DSC_CMP_EQ)
                        for (int64_t e = 0; e < cnt; ++e) t[e] = (a0[e] == a1[e]) ? a2[e] : a3[e];
                    else
                        for (int64_t e = 0; e < cnt; ++e) t[e] = (a0[e] > a1[e]) ? a2[e] : a3[e];
                    break;
                case DSC_PE_GATHER: {
                    const ViewEval& v = in_views[op.input_index];
                    const float* src = bufs[op.input_index];
                    for (int64_t e = 0; e < cnt; ++e) {
                        grid_coord(base + e, op.gather_shape, coord);
                        coord[op.axis] = f2i(a0[e]);
                        t[e] = src[v.load_index(coord)];
                    }
                    break;
                }
                default: break;
                }
            }
            for (int o = 0; o < d.n_outputs; ++o) {
                float* out = bufs[d.n_inputs + o];
                const float* t = &tmp[(size_t)d.outputs[o] * CH];
                for (int64_t e = 0; e < cnt; ++e) out[base + e] = t[e];
            }
        }
    }
    return 0;
}

int run_reduce(const dsc_kernel_desc& d, float* const* bufs) {
    const ViewEval v(d.inputs[0]);
    const int64_t n = element_count(d.shape);
    const int64_t k = v.out_shape.dims[d.axis];
    const float* in = bufs[0];
    float* out = bufs[1];
#pragma omp parallel for schedule(static)
    for (int64_t id = 0; id < n; ++id) {
        int64_t coord[DSC_MAX_DIM];
        grid_coord(id, d.shape, coord);
        float result = d.reduce_op == DSC_REDUCE_MAX ? u2f(0xff800000u) : 0.f;
        for (int64_t kk = 0; kk < k; ++kk) {
            coord[d.axis] = kk;
            float t = in[v.load_index(coord)];
            if (d.reduce_op == DSC_REDUCE_MAX) result = (result < t) ? t : result;  // GLSL max(x, y)
            else result += t;
        }
        out[id] = result;
    }
    return 0;
}

int run_matmul(const dsc_kernel_desc& d, float* const* bufs) {
    const ViewEval va(d.inputs[0]), vb(d.inputs[1]);
    if (va.out_rank != 3 || vb.out_rank != 3) return 1;
    const int64_t M = va.out_shape.dims[1], K = va.out_shape.dims[2], N = vb.out_shape.dims[2];
    const int64_t chunks = d.shape.dims[0];
    const bool rows = d.output_mode == DSC_MATMUL_ROWS;
    const int64_t batch = d.shape.dims[rows ? 2 : 1];
    const int64_t k_tiles = (K + 15) / 16;
    const int64_t chunk_tiles = (k_tiles + chunks - 1) / chunks;  // K_CHUNK_SIZE_IN_TILES, kernel.rs:436
    const int64_t batch_stride = rows ? N : M * N, row_stride = rows ? batch * N : N;
    const float* A = bufs[0];
    const float* B = bufs[1];
    float* Cout = bufs[2];

    std::vector<float> a((size_t)M * K), b((size_t)K * N);
    for (int64_t bi = 0; bi < batch; ++bi) {
        // dense copies of this batch's operands, read through the views
#pragma omp parallel for schedule(static)
        for (int64_t m = 0; m < M; ++m) {
            int64_t coord[3] = {bi, m, 0};
            for (int64_t k = 0; k < K; ++k) { coord[2] = k; a[(size_t)m * K + k] = A[va.load_index(coord)]; }
        }
#pragma omp parallel for schedule(static)
        for (int64_t k = 0; k < K; ++k) {
            int64_t coord[3] = {bi, k, 0};
            for (int64_t n = 0; n < N; ++n) { coord[2] = n; b[(size_t)k * N + n] = B[vb.load_index(coord)]; }
        }
        for (int64_t kc = 0; kc < chunks; ++kc) {
            const int64_t k0 = kc * chunk_tiles * 16;
            int64_t k1 = (kc + 1) * chunk_tiles * 16;
            if (k1 > K) k1 = K;
#pragma omp parallel
            {
                std::vector<float> acc((size_t)N);
#pragma omp for schedule(static)
                for (int64_t m = 0; m < M; ++m) {
                    for (int64_t n = 0; n < N; ++n) acc[n] = 0.f;
                    for (int64_t k = k0; k < k1; ++k) {
                        const float av = a[(size_t)m * K + k];
                        const float* brow = &b[(size_t)k * N];
                        for (int64_t n = 0; n < N; ++n) acc[n] += av * brow[n];
                    }
                    float* crow = Cout + kc * (batch * M * N) + bi * batch_stride + m * row_stride;
                    for (int64_t n = 0; n < N; ++n) crow[n] = acc[n];
                }
            }
        }
    }
    return 0;
}

int run_unpad(const dsc_kernel_desc& d, float* const* bufs) {
    const ViewEval v(d.inputs[0]);
    const int64_t n = element_count(d.shape);
    const float* in = bufs[0];
    float* out = bufs[1];
    const int64_t last = d.shape.dims[d.axis] - 1;
#pragma omp parallel for schedule(static)
    for (int64_t id = 0; id < n; ++id) {
        int64_t coord[DSC_MAX_DIM];
        grid_coord(id, d.shape, coord);
        const int64_t oc = coord[d.axis];
        const int64_t ic = oc + d.pad;
        const int64_t k_min = ic - (oc == 0 ? d.pad : 0);
        const int64_t k_max = ic + (oc == last ? d.pad : 0);
        float sum = 0.f;
        for (int64_t k = k_min; k <= k_max; ++k) {
            coord[d.axis] = k;
            sum += in[v.load_index(coord)];
        }
        out[id] = sum;
    }
    return 0;
}

int run_windows_to_image(const dsc_kernel_desc& d, float* const* bufs) {
    const ViewEval v(d.inputs[0]);
    const int r = v.out_rank;
    if (r < 6 || d.shape.rank != r - 3) return 1;
    const int64_t out_h = v.out_shape.dims[r - 6], out_w = v.out_shape.dims[r - 5];
    const int64_t filter_h = v.out_shape.dims[r - 3], filter_w = v.out_shape.dims[r - 2];
    const int64_t group_nc = v.out_shape.dims[r - 1];
    const int64_t sw = d.stride_w, sh = d.stride_h;
    const int batch_dims = d.shape.rank - 3;
    const int64_t count_x = (filter_w + sw - 1) / sw, count_y = (filter_h + sh - 1) / sh;
    const int64_t n = element_count(d.shape);
    const float* in = bufs[0];
    float* out = bufs[1];
#pragma omp parallel for schedule(static)
    for (int64_t id = 0; id < n; ++id) {
        int64_t coord[DSC_MAX_DIM], ic[DSC_MAX_DIM];
        grid_coord(id, d.shape, coord);
        const int64_t in_y = coord[batch_dims], in_x = coord[batch_dims + 1], in_c = coord[batch_dims + 2];
        const int64_t group_index = in_c / group_nc, group_c = in_c - group_index * group_nc;
        const int64_t fbx = in_x % sw, fby = in_y % sh;
        const int64_t oxb = in_x / sw, oyb = in_y / sh;
        for (int i = 0; i < batch_dims; ++i) ic[i] = coord[i];
        float tmp = 0.f;
        for (int64_t iy = 0; iy < count_y; ++iy)
            for (int64_t ix = 0; ix < count_x; ++ix) {
                const int64_t fx = fbx + sw * ix, fy = fby + sh * iy;
                if (fx < filter_w && fy < filter_h) {
                    const int64_t ox = oxb - ix, oy = oyb - iy;
                    if (ox < 0 || ox >= out_w || oy < 0 || oy >= out_h) continue;  // see header note
                    ic[batch_dims] = oy;
                    ic[batch_dims + 1] = ox;
                    ic[batch_dims + 2] = group_index;
                    ic[batch_dims + 3] = fy;
                    ic[batch_dims + 4] = fx;
                    ic[batch_dims + 5] = group_c;
                    tmp += in[v.load_index(ic)];
                }
            }
        out[id] = tmp;
    }
    return 0;
}

int run_scatter_add(const dsc_kernel_desc& d, float* const* bufs) {
    const ViewEval vv(d.inputs[0]), vi(d.inputs[1]);
    const int64_t n = element_count(vv.out_shape);
    const float* values = bufs[0];
    const float* indices = bufs[1];
    float* out = bufs[2];
    int64_t stride[DSC_MAX_DIM];
    int64_t s = 1;
    for (int i = d.shape.rank - 1; i >= 0; --i) { stride[i] = s; s *= d.shape.dims[i]; }
    // serial: the reference's atomic order is unspecified; the oracle fixes element order
    for (int64_t id = 0; id < n; ++id) {
        int64_t coord[DSC_MAX_DIM];
        grid_coord(id, vv.out_shape, coord);
        const float value = values[vv.load_index(coord)];
        int64_t c1[1] = {coord[d.axis]};
        coord[d.axis] = f2i(indices[vi.load_index(c1)]);
        int64_t idx = 0;
        for (int i = 0; i < d.shape.rank; ++i) idx += coord[i] * stride[i];
        out[idx] += value;
    }
    return 0;
}

}  // namespace

extern "C" {

// Runs one kernel on host buffers bound in the reference's order (inputs, then outputs).
// Returns 0 on success, non-zero for a malformed descriptor.
int orc_run_kernel(const dsc_kernel_desc* d, float* const* bufs, int n_bufs, uint32_t rand_seed) {
    if (!d || !bufs) return 1;
    (void)n_bufs;
    switch (d->kind) {
    case DSC_KERNEL_FILL: return run_fill(*d, bufs);
    case DSC_KERNEL_PER_ELEMENT: return run_per_element(*d, bufs, rand_seed);
    case DSC_KERNEL_REDUCE: return run_reduce(*d, bufs);
    case DSC_KERNEL_MATMUL: return run_matmul(*d, bufs);
    case DSC_KERNEL_UNPAD: return run_unpad(*d, bufs);
    case DSC_KERNEL_WINDOWS_TO_IMAGE: return run_windows_to_image(*d, bufs);
    case DSC_KERNEL_SCATTER_ADD: return run_scatter_add(*d, bufs);
    default: return 1;
    }
}

uint32_t orc_pcg(uint32_t v) { return pcg(v); }
float orc_rand_from_index(uint32_t uid, int32_t index, uint32_t seed) { return rand_from_index(uid, index, seed); }
int64_t orc_load_index(const dsc_view* v, const int64_t* coord) { return ViewEval(*v).load_index(coord); }

}  // extern "C"
