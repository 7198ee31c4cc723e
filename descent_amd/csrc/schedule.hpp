// A whole graph's clusters, fused where profitable, executed with Environment::run's buffer discipline
// (src/environment.rs:326-516).
#pragma once

#include "runtime.hpp"

namespace dsc {

struct StepOutput {
    int node;
    int copy_from;      // -1: fresh allocation (InitialState::Undefined)
    bool from_literal;  // copy_from is a Literal node: Fill a fresh buffer when no buffer can be taken over
    uint32_t literal_bits;
    Kernel* fill = nullptr;
};

struct Step {
    Kernel* kernel = nullptr;
    std::vector<int> params;   // op node bound to each pointer parameter of the kernel
    std::vector<int> inputs;   // distinct nodes read (use counting)
    std::vector<StepOutput> outputs;
    std::vector<int> covers;   // reference cluster indices this launch stands for
};

// One launch of a planned run: `n` pointer arguments starting at `first` in the run's pointer table.
struct PlannedLaunch {
    Kernel* kernel = nullptr;
    size_t first = 0;
    int n = 0;
};

// A run whose buffers all sit at addresses known before anything is launched: intermediates at offsets of one
// region, written parameters in the spare buffer of their slot.
struct FixedPlan {
    std::vector<PlannedLaunch> launches;
    std::vector<void*> pointers;
    std::vector<int> swapped;  // parameter slots whose new value sits in the spare buffer
    size_t peak = 0;           // most bytes of the region in use at once
    size_t high = 0;           // end of the highest placement in the region
};

// One step's launches with their resolved device pointers, captured once as a HIP graph and replayed whenever a
// later step resolves to the same pointers.
struct CapturedStep {
    std::vector<void*> pointers;  // every pointer argument of every launch, in order
    hipGraphExec_t exec = nullptr;
};

struct Schedule {
    static constexpr size_t kMaxCaptured = 8;
    std::vector<CapturedStep> captured;
    int64_t replays = 0, direct_runs = 0;
    size_t static_peak_bytes = 0;  // most scratch a run_static of this schedule has had in use at once
    bool graph_replay = false;  // DSC_SCHEDULE_GRAPH_REPLAY
    // Graph replay needs a step's pointers to repeat, which buffers taken from the shared heap do not (measured on
    // the ConvNet: no repeat within eight captures).  A schedule that replays therefore owns one region for its
    // intermediates and one spare buffer per written parameter: a written parameter alternates between the
    // caller's buffer and the spare, so the pointer table has period two and two captured graphs serve every step.
    dsc_buf replay_region = 0;
    size_t replay_region_bytes = 0;
    std::vector<dsc_buf> replay_spare;  // per parameter slot, 0 where the slot is not written
    bool replay_fixed = true;           // cleared when this graph cannot be laid out that way
    void release_replay_buffers(Context* ctx);  // before the schedule goes, while its context is alive
    bool has_captured_graphs() const { return !captured.empty(); }
    ~Schedule();

    int n_nodes = 0, n_params = 0, n_clusters = 0;
    std::vector<size_t> node_bytes;
    std::vector<dsc_param_io> inputs, outputs;
    std::vector<Step> steps;
    // Accumulators that start as a literal (a ScatterAdd into zeros): with several of them in one graph, all are
    // allocated and filled by one multi-part launch at the start of a run instead of one Fill launch each.
    struct Prefill {
        Kernel* kernel = nullptr;
        std::vector<int> nodes;  // one per pointer parameter
    };
    std::vector<Prefill> prefills;

    int build(Context* ctx, const dsc_schedule_desc& desc, uint32_t flags);
    int run(Context* ctx, dsc_buf* params, uint32_t rand_seed);
    // The same launches with every intermediate inside `scratch` (a fixed device array of `scratch_bytes`) and every
    // written parameter in the caller's `spare` buffer of its slot: no device allocation, no heap traffic.
    int run_static(Context* ctx, dsc_buf* params, dsc_buf* spare, uint32_t rand_seed, char* scratch, size_t scratch_bytes);
    // The placement both of them use; launches nothing.
    int plan_fixed(Context* ctx, const dsc_buf* params, const dsc_buf* spare, char* scratch, size_t scratch_bytes, FixedPlan* plan);
    // run() for a schedule that replays graphs, over its own region and spares; *handled is false when the graph
    // cannot be laid out at fixed addresses (run() then goes on as usual).
    int run_replayed(Context* ctx, dsc_buf* params, uint32_t rand_seed, bool* handled);
    int replay_or_capture(Context* ctx, const std::vector<PlannedLaunch>& launches, const std::vector<void*>& pointers, uint32_t rand_seed);
    std::string describe() const;
    // The schedule after fusion as a graphviz digraph (the reference exports its graph before scheduling,
    // src/graph.rs:656-760): one box per launch, one ellipse per parameter slot, one edge per buffer.
    std::string dot() const;
    // kernels one run enqueues: the steps, the prefill launches, and a Fill per literal-initialised accumulator
    // that no prefill covers
    int launches_per_run() const;
};

}  // namespace dsc
