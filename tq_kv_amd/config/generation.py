"""Stop tokens of a model folder.

The reference asks its tokenizer for the ids of every stop string it knows and stops on any of
them (src/engine.rs:301-316; the token is not emitted, :381).  A model folder says the same thing
in up to three places, and the engine library reads them all (csrc/engine/config.cpp):

  config.json              eos_token_id (an id or a list), already in the typed config
  generation_config.json   eos_token_id (an id or a list): instruct checkpoints keep
                           their second stop id only here
  tokenizer.json           the ids of the reference's stop strings, where the file is
                           there (read as JSON: added_tokens and model.vocab)

The result is their union in that order, each id once.  A folder with none of them (random
weights) has no stop token; the reference's fallback id 2 (:312-314) belongs to a tokenizer this
library does not ship and is not applied.
"""
from .. import native

# src/engine.rs:301-308
STOP_STRINGS = ("<|eot_id|>", "<|im_end|>", "<|endoftext|>", "<|end|>", "<end_of_turn>", "</s>")


def stop_token_ids(model_dir, config_ids=None):
    """The union described in the module text (an id beyond the vocabulary is kept: it is never
    drawn, so it never stops anything).  config_ids: ids to put first (default: config.json's own)."""
    ids = native.parsed(native.library().tqe_stop_token_ids(native.enc(str(model_dir))))
    out = []
    for i in list(config_ids or ()) + ids:
        if i not in out:
            out.append(int(i))
    return tuple(out)
