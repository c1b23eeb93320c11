"""How the engine library comes by the kernel library: beside itself, where it is told, or from the program that loaded
it (the Python package compiles the kernels at the first call that needs them).  Runs without a GPU: the engine asks the
kernel library for its limits when it checks a configuration."""
import ctypes
import json
import os
import shutil

from tq_kv_amd import kernels, native

CONFIG = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 64, "num_hidden_layers": 1, "num_attention_heads": 2,
          "num_key_value_heads": 1, "intermediate_size": 96, "vocab_size": 50, "max_position_embeddings": 64, "rms_norm_eps": 1e-6,
          "rope_theta": 10000.0, "tie_word_embeddings": True}


def lonely_engine(tmp_path):
    """A copy of the engine library in a folder that holds no kernel library, loaded as a library of its own."""
    copy = os.path.join(str(tmp_path), "libtqengine_copy.so")
    shutil.copy(native.library_path(), copy)
    lib = ctypes.CDLL(copy)
    lib.tqe_write_random_folder.restype = ctypes.c_int
    lib.tqe_write_random_folder.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_uint64, ctypes.c_int]
    lib.tqe_last_error.restype = ctypes.c_char_p
    lib.tqe_kernel_library.restype = ctypes.c_char_p
    return lib


def test_the_engine_asks_its_loader_for_the_kernels_when_it_finds_none(tmp_path, monkeypatch):
    monkeypatch.delenv("TQ_KERNEL_LIBRARY", raising=False)
    lib = lonely_engine(tmp_path)
    text = json.dumps(CONFIG).encode()

    def write(name):             # builds the model's parts, which ask the kernels what sizes they take
        return lib.tqe_write_random_folder(os.path.join(str(tmp_path), name).encode(), text, 1, native.BF16)
    assert write("a") == native.ERR_DEVICE
    assert b"kernel library is not built" in lib.tqe_last_error()
    # a builder that cannot: the same error
    kind = ctypes.CFUNCTYPE(ctypes.c_void_p)
    calls = []
    cannot = kind(lambda: calls.append("cannot"))
    lib.tqe_set_kernel_builder.argtypes = [kind]
    lib.tqe_set_kernel_builder.restype = None
    lib.tqe_set_kernel_builder(cannot)
    assert write("b") == native.ERR_DEVICE and calls == ["cannot"]
    # one that can is asked once, and the library it names is the one in use from then on
    path = ctypes.create_string_buffer(kernels.library_path().encode())

    def build():
        calls.append("can")
        return ctypes.addressof(path)
    can = kind(build)
    lib.tqe_set_kernel_builder(can)
    assert write("c") == 0, lib.tqe_last_error()
    assert sorted(os.listdir(os.path.join(str(tmp_path), "c"))) == ["config.json", "model.safetensors"]
    assert write("d") == 0 and calls == ["cannot", "can"]
    assert lib.tqe_kernel_library() == path.value
