// A model: parts built from a ModelSpec, weights loaded into them, and the forward pass of one
// step.  It knows nothing of any architecture: embedding, the blocks in the order the spec gives,
// final norm and head on the wanted rows, as the reference's forward does for its one sequence
// (src/models/turbo_generic.rs:1950-1987).
#pragma once
#include "linear.h"
#include "parts.h"
#include "step.h"
#include "store.h"

namespace tq {

class Model {
public:
    Model(const ModelSpec& spec, int dtype, bool on_gpu);

    ModelSpec spec;
    Json config;                                // the typed configuration it was made from, if any
    int dtype;                                  // F32 or BF16: the run's activation and weight type
    bool on_gpu;                                // false: host memory and no kernels (configuration and weights can still be looked at)
    std::vector<int32_t> stop_token_ids;        // what the configuration names; a model folder may add more
    std::vector<CacheNeed> needs;               // per run of the order
    std::vector<int> cache_of;
    bool graph_safe = false;
    bool loaded = false;

    TensorSpecs tensor_specs() const;
    // Takes the tensors (full names); every part gets its own.  Checks nothing: the loader has.
    void load(Loaded& tensors, hipStream_t stream);
    OwnedPtr held(const std::string& name) const;
    bool head_is_embedding() const { return spec.head_name.empty(); }

    // Runs the step's tokens through every run of the order; logits [wanted rows, vocab] float32 for
    // the step's wanted rows, written to `out` (device memory) or to workspace memory.
    Tensor forward(StepContext& c, const CacheStore& cache, float* out = nullptr);
    Json describe() const;
    // Lets the library try its kernels once for every product of the model at `rows` rows (more than the own kernels
    // take: fewer never reach the library) and keep the fastest for later calls.
    void tune_library(int64_t rows, hipStream_t stream);

private:
    BuildEnv env_;
    std::vector<std::shared_ptr<Block>> blocks_;
    std::shared_ptr<Norm> final_norm_;
    std::shared_ptr<Position> stream_position_;
    OwnedPtr embedding_, head_bias_;
    Weight head_;
    Tensor head_logits(StepContext& c, Stream& stream, float* out);
};

}  // namespace tq
