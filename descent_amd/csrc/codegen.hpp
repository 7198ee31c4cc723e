// HIP C++ source generation for kernel descriptors.  Counterpart of the reference's `generate_source`
// implementations (src/kernel.rs:151-857): every shape, stride and offset is baked into the text as a
// literal, so each distinct kernel is its own translation unit compiled by hipRTC.
//
// Beyond the one-descriptor-one-kernel mapping of the reference, the generator accepts a `FusedKernel`:
// a main descriptor whose inputs may be *virtual* -- a per-element cluster evaluated on demand at the
// element the main kernel reads (this is how a materialised im2col / pooling-window copy, or any
// single-consumer elementwise producer, disappears into its consumer) -- and, for MatMul, an epilogue
// cluster applied to the accumulator before the store (split-K partials are then summed in registers).
#pragma once

#include "desc.hpp"

#include <string>
#include <vector>

namespace dsc {

// Where the elements of one kernel input come from.
struct Source {
    int buffer = -1;     // index of a pointer parameter of the generated kernel, or
    int virt = -1;       // index into FusedKernel::virtuals, or
    int stage = -1;      // (row-fused kernels) index of an earlier stage whose result stays in registers,
    int stage_out = 0;   // and which of that stage's outputs
};

// A per-element cluster evaluated lazily: value(gid) = ops[out_op] at linear element id `gid`.
struct Virtual {
    KernelDesc pe;
    int out_op = 0;
    std::vector<Source> inputs;  // one per pe input
};

// One cluster of a row-fused kernel (see FusedKernel::row_stages).
struct RowStage {
    KernelDesc k;                // PerElement over [m, n] or [m] elements, or Reduce of [m, n] along n, or (stage 0
                                 // only) the MatMul whose [m, n] product the other stages start from
    std::vector<Source> inputs;  // one per input view of k
    std::vector<int> outputs;    // per output of k: index into FusedKernel::outputs when stored, else -1
    // (stage 0 MatMul only) index into FusedKernel::outputs of the buffer that takes the A operand [m, k] as the stage
    // evaluates it -- each element exactly once, by the lane that multiplies it -- when A is a fused producer whose
    // result other launches read as well; -1 otherwise
    int store_a = -1;
};

struct FusedKernel {
    KernelDesc main;
    std::vector<Source> inputs;     // one per main input view
    std::vector<Virtual> virtuals;  // may reference one another (a virtual's inputs may be virtual), acyclic,
                                    // each referencing only virtuals with a larger index
    // MatMul only: per-element cluster applied to the product (all of K accumulated in-kernel)
    bool has_epilogue = false;
    KernelDesc epilogue;
    int epilogue_product_input = -1;       // which epilogue input is the product
    std::vector<Source> epilogue_inputs;   // one per epilogue input (the product's entry is ignored)
    // Reduce only: the epilogue reads the product through a view that is a bijection of the elements but not the
    // identity (a weight gradient summed as [k, n] and consumed as [n, k] by its optimiser update).  The kernel then
    // turns the index of each result into the epilogue element that reads it.
    bool epilogue_permuted = false;
    // Reduce, WindowsToImage, Unpad: the product has readers besides the epilogue, so the kernel stores it as well;
    // it is the last entry of `outputs`, after the epilogue's own.
    bool epilogue_keeps_product = false;
    // Row-fused kernel: clusters that all work on the rows of one [m, n] array with n <= 64 (a softmax
    // cross-entropy with its accuracy count: row max, exp, row sum, log, gradient, per-row loss) run as one
    // kernel.  A group of lanes owns a row, lane j holds column j of every [m, n] value, an [m]-shaped value is
    // the same in every lane of the group, a Reduce along n is a butterfly of shuffles.  Stages run in order;
    // `main` is the first stage's descriptor (for the label), only the outputs someone else needs are stored.
    std::vector<RowStage> row_stages;
    int64_t row_m = 0, row_n = 0;
    // Row-fused kernel whose first stage is a MatMul over k: after the last stage, the product of one of the stages'
    // [m, n] values X with a small matrix B2 [n, k] -- the data gradient of the layer the launch starts from, dZ x W^T
    // -- with its per-element consumer.  A lane owns the same blocks of four k it multiplied in stage 0: X's columns
    // come to it through shuffles, B2 sits in LDS, and where the consumer reads the A operand that stage 0 evaluated
    // and stored (the activation the gradient is masked with), it takes it from the lane's registers.
    struct RowTail {
        bool on = false;
        KernelDesc mm;                 // the MatMul [m, n] x [n, k]; inputs[1] is B2's view
        int x_stage = -1, x_stage_out = 0;
        Source b;                      // B2: a buffer
        bool has_epilogue = false;
        KernelDesc epilogue;
        int epilogue_product_input = -1;
        int epilogue_a_input = -1;     // epilogue input that reads stage 0's stored A operand element for element
        std::vector<Source> epilogue_inputs;
        std::vector<int> outputs;      // per output of the epilogue (or the product): index into FusedKernel::outputs
    } row_tail;
    // Several independent small kernels in one launch: workgroup ids [0, g0) run parts[0], [g0, g0 + g1) run
    // parts[1], ...  part_params[i][j] is the pointer parameter of this kernel that part i's parameter j binds.
    // `main` is parts[0].main (for the label); inputs/outputs of the launch are those of the parts.
    std::vector<FusedKernel> parts;
    std::vector<std::vector<int>> part_params;
    // Multi-part launch whose parts are ScatterAdds into one accumulator small enough for LDS: every workgroup keeps
    // ONE copy of the accumulator in LDS, folds its share of every part's values into it and adds the non-zero
    // totals to memory once.
    bool shared_scatter = false;
    // The same chain when the accumulator is too large for LDS, as two launches that replace one memory atomic per
    // value (a 64-byte read-modify-write at a random address each) by streamed records:
    // stage 1 ("bin", a multi-part kernel over the links): every workgroup sorts its share of (target, value)
    //   records by accumulator segment in LDS, reserves room in each segment's bin with one counter add and writes
    //   the records there in runs; records that find their bin full are added to the accumulator directly.
    //   outputs = {records, bin counters (start at 0), accumulator}.
    // stage 2 ("sum", inputs = {records, bin counters}, output = the accumulator taken over in place): workgroups
    //   own one segment (or a slice of one segment's records), sum the records in LDS and add the segment to the
    //   accumulator with consecutive addresses.
    // Several chain kernels (LDS chains, or stage 1 / stage 2 kernels of binned chains) in one launch of 1024-thread
    // workgroups: parts[] are those kernels, sharing one LDS block sized for the largest.  The chains of a step do
    // not depend on one another, and one launch of all of them keeps every CU's two workgroup slots busy while a
    // workgroup waits on its own chain of memory round trips.
    bool chain_group = false;
    int binned_stage = 0;
    int64_t binned_table = 0, binned_total = 0;  // accumulator elements, values of all links together
    // The accumulator is [entries, 2] and every link adds rows of two along axis 0: a record is then (target of the
    // row's first value, both values), twelve bytes for two values instead of sixteen, and one count per row.
    bool binned_pairs = false;
    // Data gradient of a stride-1 convolution with few channels, as one kernel: `main` is the MatMul dC x filter^T
    // ([g][(img, oy, ox)][oc] x [g][oc][(fy, fx, c)]); the kernel also does what the reference's WindowsToImage
    // (sum of the windows covering each pixel of the padded image) and the two Unpads after it (fold the
    // replicate-padding border back onto the edge pixels) would do.  One workgroup per image: dC of the image
    // sits in LDS inside a halo of zeros, the padded-image gradient goes back through LDS for the border folds.
    struct ConvDgrad {
        bool on = false;
        int64_t img = 0, oh = 0, ow = 0, g = 0, fh = 0, fw = 0, c = 0;  // windows [img, oh, ow, g, fh, fw, c]
        int64_t pad_h = 0, pad_w = 0;  // Unpads folded in (0: the output is the padded image)
        int32_t rows_first = 1;        // the Unpad along the image rows came first
        // The filter gradient of the same convolution rides along (`wgrad`): the workgroup that holds dC of an image
        // in LDS also takes the image's (replicate-padded) input tile and accumulates im2col^T x dC on the matrix
        // cores, over the `chunks` (a multiple of 8) sets the images are dealt into; with `bias` the column sums of
        // dC come out of the same products (one im2col row of ones).  Then inputs[2] is the image [img, h, w, g*c]
        // and the outputs are {data gradient, partials [chunks, g, fh*fw*c, k], (column sums [chunks, g*k])}.
        bool wgrad = false, bias = false;
        int64_t chunks = 0;
        // The filter gradient alone (a first layer, whose input needs no gradient): `main` is then the filter
        // gradient's own MatMul, im2col^T [g][(fy, fx, c)][(img, oy, ox)] x dC [g][(img, oy, ox)][oc]; inputs[1] is dC
        // (a buffer or a fused producer), inputs[0] and inputs[2] the image, outputs {partials, (column sums)}.
        bool wgrad_only = false;
        // (filter gradient alone) bands of output rows an image is cut into, one workgroup each: a band's tiles are a
        // fraction of the image's, so more workgroups share a CU; partials then number chunks x bands
        int64_t bands = 1;
        // dC is the gradient of a 2x2 max-pooling behind an activation with slope `leak` below zero, read off the words a
        // pooling convolution-forward kernel wrote (ConvPool::masks): dC[pixel][oc] = (equals its window's maximum ?
        // dP[window][oc] : 0) x (positive ? 1 : leak).  Then the dC operand of `main` is dP -- the pooled array's
        // gradient [img, oh/2, ow/2, g*k], a buffer -- and `masks` the words' buffer.
        struct PoolMasks {
            bool on = false;
            Source masks;
            uint32_t leak_bits = 0;
        } pm;
    } dgrad;
    // MatMul whose A operand is the im2col of a stride-1 convolution's (replicate-padded) input: the kernel reads the
    // image [img, h, w, g*c] itself, one workgroup per (image, group) with the group's channels of the image in LDS,
    // instead of the materialised or generated window copy (main.inputs[0] is the image; the descriptor keeps the
    // MatMul's shapes).  k = (fy * fw + fx) * c + ch, row = (img * oh + oy) * ow + ox.
    struct ConvFwd {
        bool on = false;
        int64_t img = 0, h = 0, w = 0, g = 0, c = 0, fh = 0, fw = 0, oh = 0, ow = 0, pad_h = 0, pad_w = 0;
    } cfwd;
    // Convolution-forward kernel that also max-pools what it computes (2x2 windows, stride 2): the Reduce(max) over
    // the window copy of one of the kernel's outputs, with that Reduce's own per-element consumer where it had one
    // (a dropout select), runs on the values while they are in registers.  The pooled array and the consumer's
    // outputs follow the kernel's own in `outputs`: {conv outputs..., consumer outputs..., pooled (when stored)}.
    struct ConvPool {
        bool on = false;
        int source = 0;                 // which of the convolution's outputs is pooled
        bool has_epilogue = false;      // the Reduce carried a per-element consumer
        bool store_pooled = true;       // the pooled array itself is written (no consumer, or a consumer that keeps it)
        // The pooled output's source is read by nothing but the backward pass of this pooling and of the activation in
        // front of it, which ask two things of each element: does it equal its window's maximum, and is it positive.
        // The kernel then writes those two bits per element in place of the element -- one word per pooling window and
        // four channels, [g][img * oh/2 * ow/2][n / 4], byte p of a word for the window's pixel p = (x & 1) + 2 (y & 1),
        // bits 2j and 2j + 1 of a byte for channel 4q + j -- through the pointer that stood for the source, which
        // is never stored (see ConvDgrad::masks for the reader).
        bool masks = false;
        KernelDesc epilogue;
        int epilogue_product_input = -1;
        std::vector<Source> epilogue_inputs;
    } pool;
    // MatMul [m, n] (one batch) whose readers all take narrow column slices [m, w] of the product: the product is
    // stored slice by slice, [n / w][m][w], so that a reader of one slice walks consecutive memory instead of w
    // floats out of every row.  The readers' views are rewritten to that layout by the planner.
    int64_t out_slice_width = 0;
    // A per-element kernel over [rows, w] whose value is chosen by comparing the column with literals (a chain of
    // concats): w > 0 makes a thread evaluate one whole row with the column a constant of each of its w evaluations,
    // so the compiler keeps, per column, only the branch that column takes.
    int64_t row_width = 0;
    // Short-k MatMul with a per-element consumer -- the data gradient dY x W^T of a layer with a few outputs, masked by
    // the stored activation X -- that also computes the layer's weight gradient X^T dY, the tall-k MatMul that reads
    // the same X [m, n] and the same dY [m, k]: a workgroup walks `chunk_rows` rows, a thread multiplies the 16 bytes
    // of X it holds anyway with the row's k values of dY, and the workgroup writes one partial [n, k] per chunk, the
    // layout the tall-k kernel's k chunks had (the Reduce over them stays as it is).  `x_buffer` is X's pointer
    // parameter, `out` the partials'.
    struct GradPair {
        bool on = false;
        int x_buffer = -1, out = -1;
        int64_t chunk_rows = 0, chunks = 0;
    } pair;
    bool sum_chunks = false;               // MatMul: ignore the descriptor's chunk count, write one full sum
    int colsum_out = -1;                   // MatMul (MFMA template): buffer that takes the column sums of B per k chunk
    // MatMul (MFMA template, 16-byte store path) with an epilogue: `sign_out` is a buffer that takes one byte per four
    // consecutive results of the epilogue's output `sign_source`, bit j set where result 4i + j is positive -- what the
    // backward pass asks of a stored activation when all it does with it is "(a > 0) ? x : y".  `epilogue_sign_input`
    // names an epilogue input that is read from such bytes instead of the activation itself (every use of that input
    // is the left side of a "> 0" select): one byte per lane and store round, requested for all of a unit's rounds
    // before the first, in place of a 16-byte load per round that the round then waited for.
    int sign_out = -1, sign_source = 0;
    int epilogue_sign_input = -1;
    bool as_part = false;                  // generated as one part of a multi-part launch (set while the launch is generated)
    std::vector<int> outputs;              // pointer parameter index of each output of main (or of the epilogue)
    int n_buffers = 0;                     // number of pointer parameters
    std::vector<bool> buffer_is_output;    // per pointer parameter

    // The reference binding: inputs then outputs, no fusion.
    static FusedKernel plain(const dsc_kernel_desc& d);
    std::string key() const;
};

struct Generated {
    std::string source;      // complete translation unit
    std::string entry;       // name of the __global__ function (dsc_<kind>)
    unsigned grid = 1;       // workgroups (1-D)
    unsigned block = 64;     // threads per workgroup
    int n_buffers = 0;       // pointer parameters, in order; followed by `const uint* seed_cell, uint seed_value`
    std::string note;        // strategy chosen (for schedule listings)
    size_t lds_bytes = 0;    // (chain kernels generated as parts) LDS the part needs from the launch's shared block
    // Work one launch stands for, counted the way a roofline wants it: bytes = 4 * (distinct elements of every
    // buffer read, a broadcast or windowed operand at its own size, + elements written; a scatter accumulator is
    // read and written where values land), flops = 2*b*M*N*K of a MatMul (0 otherwise).
    double algo_bytes = 0, algo_flops = 0;
    // MFMA MatMul with a short k: `grid` counts the (chunk, batch, tile) units, and the kernel accepts any smaller
    // grid (its workgroups then walk several units each, overlapping one unit's stores with the next one's first
    // loads).  The runtime shrinks the grid to what the device holds at once.
    bool persistent_ok = false;
};

// Returns "" on success or an error message.
std::string generate(const FusedKernel& k, Generated* out);

// Whether the convolution data-gradient kernel can take this geometry (k = output channels per group): the image
// tile must fit the workgroup's LDS.
bool conv_dgrad_fits(const FusedKernel::ConvDgrad& c, int64_t k);
// The same for the kernel that also takes the filter gradient (c.wgrad, c.bias and c.chunks set).
bool conv_bwd_fits(const FusedKernel::ConvDgrad& c, int64_t k);
// Whether that kernel runs with loader waves (512 threads: four waves fill the next image's tiles while four run the
// matrix phases of the current one); the planner deals the images into fewer, larger sets then.
bool conv_bwd_loader_waves(const FusedKernel& fk);
// Whether the convolution-forward kernel takes this geometry with n output channels per group.
bool conv_fwd_fits(const FusedKernel::ConvFwd& c, int64_t n);

// Whether a chain of ScatterAdds with this accumulator size and this many values in total runs as one kernel with
// the accumulator in LDS (shared_scatter).
bool scatter_chain_in_lds(int64_t table_elements, int64_t total_values);

// The two-launch form of a chain (FusedKernel::binned_stage): whether a chain of this size takes it, and its geometry.
struct BinnedScatterPlan {
    int64_t seg = 0;     // accumulator elements per segment (whole 64-byte lines; line l belongs to segment l % nseg)
    int64_t nseg = 0;    // segments = bins
    int64_t cap = 0;     // records a bin holds (a record is one value, or one row of two)
    int64_t record_bytes = 8;
    int64_t slices = 0;  // stage-2 workgroups per segment
};
bool scatter_chain_binned(int64_t table_elements, int64_t total_values);
BinnedScatterPlan binned_scatter_plan(int64_t table_elements, int64_t total_values, bool pairs = false);
// Whether a ScatterAdd adds rows of two values that share an index (accumulator [entries, 2], axis 0).
bool scatter_rows_of_two(const dsc_kernel_desc& d);
// A MatMul small enough to run as the first stage of a row-fused kernel over its [m, n] product: the shape the
// dot-product kernel takes (few columns, a moderate number of rows, B of a few KB), one batch, no k chunks.
bool matmul_fits_row_stage(const FusedKernel& fk);
// Width of the last axis if the per-element kernel selects by comparing that axis' coordinate with a literal, else 0.
int64_t column_partition_width(const dsc_kernel_desc& d);

// Whether a kernel can be one part of a multi-part launch (256 threads per workgroup, addressed by blockIdx.x only).
bool can_be_part(const FusedKernel& k);

// Whether a MatMul of these dimensions (already split into its chunks) runs on the tall-k kernel: a small output
// summed over a long k, one workgroup per (chunk, batch).  The schedule sizes its k re-split for that kernel.
bool tallk_shape(const MatMulDims& g);
// the kernel that splits k over the waves of a workgroup takes this product whole (no k re-split, no partials)
bool ksplit_kernel_shape(const FusedKernel& fk);
// the dot-product kernel takes this product (rows x few columns over a k of moderate length)
bool dot_kernel_shape(const MatMulDims& g);
// `s` is a short-k MatMul with a consumer and `t` a plain tall-k MatMul shaped like the data and weight gradient of
// one layer with a few outputs (see FusedKernel::GradPair; which buffers they read is the caller's to compare)
bool grad_pair_shapes(const FusedKernel& s, const FusedKernel& t, int64_t* chunk_rows, int64_t* chunks);

// hipRTC options every kernel is compiled with (after --offload-arch=<arch>).
const std::vector<std::string>& compile_options();

// The prelude and matmul template texts (embedded at build time from kernels/*.inc).
extern const char* const kPreludeSource;
extern const char* const kMatmulMfmaSource;

}  // namespace dsc
