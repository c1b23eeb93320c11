// Configuration: architectures by name, their typed configurations, stop tokens of a model folder.
#pragma once
#include "spec.h"

namespace tq {

// An architecture: how a parsed config.json becomes its typed configuration (every key it reads,
// defaults filled in, combinations checked; returned as JSON with exactly those keys) and how that
// becomes a ModelSpec.
struct Architecture {
    std::string name;
    std::vector<std::string> model_types;
    Json (*typed_config)(const Json& raw, const std::string& where);
    ModelSpec (*build_spec)(const Json& typed);
};
void register_architecture(const Architecture& a);
std::vector<std::string> known_architectures();
// config.json's architectures[0], or model_type, picks the architecture; an unknown name is an
// error that lists the known ones (in the manner of src/hub.rs:317-330)
const Architecture& architecture_for(const Json& raw);

std::string read_text_file(const std::string& path, const char* what, int error_code);
Json read_config_json(const std::string& model_dir);        // error texts as the reference's (src/models/turbo_generic.rs:2008-2011)
// The union of config.json's eos_token_id, generation_config.json's, and the ids of the reference's
// stop strings in tokenizer.json (src/engine.rs:301-316), each once, in that order.
std::vector<int32_t> folder_stop_token_ids(const std::string& model_dir, const std::vector<int32_t>& config_ids);
std::vector<int32_t> generation_config_stop_ids(const std::string& model_dir);
std::vector<int32_t> tokenizer_stop_ids(const std::string& model_dir);

void register_qwen2();

}  // namespace tq
