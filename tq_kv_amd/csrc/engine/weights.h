// Weights: safetensors files read by tensor name, one error for everything that is wrong, the
// dtype policy, and random weights from a configuration and a seed.
#pragma once
#include "model.h"

namespace tq {

// ---- safetensors -----------------------------------------------------------------------------
// An 8-byte little-endian header length, a JSON header {name: {dtype, shape, data_offsets}}, then
// the tensors' bytes.  The reference loads every *.safetensors file of a folder into one map by
// name (src/models/turbo_generic.rs:2039-2053); so does open_folder, but lazily: a tensor's bytes
// are only touched (through a memory map) when it is asked for.
struct StoredTensor {
    std::string name, dtype;            // dtype as the file names it: F32, BF16, F16, F64, I32, I64, ...
    std::vector<int64_t> shape;
    const uint8_t* data = nullptr;
    size_t bytes = 0;
    bool is_float() const { return dtype == "F32" || dtype == "BF16" || dtype == "F16" || dtype == "F64"; }
    int64_t numel() const { int64_t n = 1; for (int64_t s : shape) n *= s; return n; }
};

class SafetensorsFile {
public:
    explicit SafetensorsFile(const std::string& path);
    ~SafetensorsFile();
    SafetensorsFile(const SafetensorsFile&) = delete;
    SafetensorsFile& operator=(const SafetensorsFile&) = delete;
    std::vector<StoredTensor> tensors;
private:
    void* map_ = nullptr;
    size_t size_ = 0;
};

struct Folder {
    std::vector<std::unique_ptr<SafetensorsFile>> files;
    std::map<std::string, StoredTensor> tensors;
};
std::unique_ptr<Folder> open_folder(const std::string& model_dir);

struct TensorToWrite {
    std::string name, dtype;
    std::vector<int64_t> shape;
    std::function<void(FILE*)> write;       // writes exactly the tensor's bytes
    size_t bytes;
};
void write_safetensors(const std::string& path, const std::vector<TensorToWrite>& tensors, const Json& metadata);

// ---- loading -----------------------------------------------------------------------------------
// The reference reads tensors by their HF names and fails at the first missing one ("Missing
// tensor: {name}", src/models/turbo_generic.rs:2056-2066), checks no shapes, and casts BF16 to F32
// (:2060-2065).  Here the wanted names and shapes come from the model's parts, all of them are
// checked before anything is copied, and the dtype policy is:
//   run in bfloat16: floating tensors become bfloat16, except those stored in 32 (or 64) bit,
//                    which stay float32; integer tables become int32
//   run in float32:  every floating tensor becomes float32 (exact for bf16 and f16)
int target_dtype(const std::string& stored, const std::string& kind, int run_dtype);
// Raises one error (TQE_ERR_WEIGHTS) that lists every missing tensor, unexpected tensor, wrong
// shape and wrong kind; its detail is the same as JSON.  strict off: tensors the model does not
// ask for are named in `warning` instead.
void check_weights(const std::map<std::string, StoredTensor>& stored, const TensorSpecs& wanted, bool strict, std::string* warning);
void load_folder(Model& model, const std::string& model_dir, bool strict, std::string* warning, hipStream_t stream);
// a stored tensor converted to `dtype` and placed in memory of the current device
OwnedPtr upload_tensor(const StoredTensor& st, int dtype, hipStream_t stream);

// ---- random weights --------------------------------------------------------------------------------
// Not in the reference.  Element i of a tensor is a function of (seed, tensor name, i) alone: a
// 64-bit key from the seed and the name, a counter-based 64-bit hash of key and index, and from its
// bits one standard normal value by Box and Muller's transform, built from operations that IEEE
// arithmetic fixes exactly, so that the host and the GPU give the same bits.
uint64_t tensor_key(uint64_t seed, const std::string& name);
void standard_normal_host(uint64_t key, int64_t begin, int64_t count, float* out);
// how a TensorSpec's init fills a tensor: "normal", "one_plus_normal", "zeros" are built in; others
// can be registered (fill: writes count float32 values of the elements begin.. on the host)
using InitFill = std::function<void(const std::string& name, const TensorSpec& spec, uint64_t seed, int64_t begin, int64_t count, float* out)>;
void register_init(const std::string& kind, InitFill fill);
void random_weights(Model& model, uint64_t seed, hipStream_t stream);
void write_random_folder(const std::string& folder, const std::string& config_text, const TensorSpecs& wanted, uint64_t seed, int store_dtype);

uint16_t float_to_bf16(float f);
float bf16_to_float(uint16_t b);

}  // namespace tq
