"""Stop tokens of a model folder.

The reference asks its tokenizer for the ids of every stop string it knows and stops
on any of them (src/engine.rs:301-316; the token is not emitted, :381).  A model
folder says the same thing in up to three places, and they are all read here:

  config.json              eos_token_id (an id or a list), already in the typed config
  generation_config.json   eos_token_id (an id or a list): instruct checkpoints keep
                           their second stop id only here
  tokenizer.json           the ids of the reference's stop strings, where the file is
                           there (read as JSON: added_tokens and model.vocab)

The result is their union in that order, each id once.  A folder with none of them
(random weights) has no stop token; the reference's fallback id 2 (:312-314) belongs
to a tokenizer this library does not ship and is not applied.
"""
import json
import os

from .base import ConfigError, KeyReader

# src/engine.rs:301-308
STOP_STRINGS = ("<|eot_id|>", "<|im_end|>", "<|endoftext|>", "<|end|>", "<end_of_turn>", "</s>")


def _read_json(path, what):
    try:
        with open(path, "r", encoding="utf-8") as f:
            return json.load(f)
    except OSError as e:
        raise ConfigError("Cannot read %s: %s" % (what, e))
    except ValueError as e:
        raise ConfigError("Invalid %s: %s" % (what, e))


def generation_config_stop_ids(model_dir):
    """eos_token_id of generation_config.json; [] if the folder has no such file."""
    path = os.path.join(model_dir, "generation_config.json")
    if not os.path.exists(path):
        return []
    raw = _read_json(path, "generation_config.json")
    if not isinstance(raw, dict):
        raise ConfigError("generation_config.json: expected a JSON object at the top level")
    return KeyReader(raw, "generation_config.json").token_ids("eos_token_id")


def tokenizer_stop_ids(model_dir):
    """Ids of the reference's stop strings in tokenizer.json, in the order of STOP_STRINGS;
    [] if the folder has no such file."""
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.exists(path):
        return []
    raw = _read_json(path, "tokenizer.json")
    ids = {}
    if isinstance(raw, dict):
        vocab = raw.get("model", {}).get("vocab") if isinstance(raw.get("model"), dict) else None
        if isinstance(vocab, dict):
            for s in STOP_STRINGS:
                if isinstance(vocab.get(s), int):
                    ids[s] = vocab[s]
        for tok in raw.get("added_tokens") or []:
            if isinstance(tok, dict) and tok.get("content") in STOP_STRINGS and isinstance(tok.get("id"), int):
                ids[tok["content"]] = tok["id"]
    return [ids[s] for s in STOP_STRINGS if s in ids]


def stop_token_ids(model_dir, config_ids=()):
    """The union described in the module text (an id beyond the vocabulary is kept: it is
    never drawn, so it never stops anything)."""
    out = []
    for i in list(config_ids) + generation_config_stop_ids(model_dir) + tokenizer_stop_ids(model_dir):
        if i not in out:
            out.append(int(i))
    return tuple(out)
