"""ctypes mirror of the data-in / weights-out part of include/eisen_graph.h."""
import ctypes as C

import numpy as np

from .lib import EisenHipError, load_library

IGNORE_INDEX = -1
_sz, _f, _i, _vp = C.c_size_t, C.c_float, C.c_int, C.c_void_p


def _lib():
    lib = load_library()
    lib.eisen_io_last_error.restype = C.c_char_p
    return lib


class BinaryDataLoader:
    """`BinaryDataLoader::new(path, seq_len, batch_size)` (src/data/dataloader.rs:97-203), without FIM."""

    def __init__(self, path, seq_len, batch_size):
        self.lib = _lib()
        self.seq_len, self.batch_size = int(seq_len), int(batch_size)
        h = _vp()
        rc = self.lib.eisen_data_loader_open(str(path).encode(), _sz(seq_len), _sz(batch_size), C.byref(h))
        if rc:
            raise EisenHipError("eisen_data_loader_open", rc, self.lib.eisen_io_last_error().decode())
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            self.lib.eisen_data_loader_close(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def total_batches(self):
        n = _sz()
        self.lib.eisen_data_loader_total_batches(self.h, C.byref(n))
        return n.value

    def next_batch(self):
        """-> (x f32 [batch*seq], targets int64 [batch*seq]) or None when the stream is exhausted."""
        n = self.batch_size * self.seq_len
        x, t, got = np.empty(n, np.float32), np.empty(n, np.int64), _i(0)
        rc = self.lib.eisen_data_loader_next_batch(self.h, x.ctypes.data_as(C.POINTER(C.c_float)), t.ctypes.data_as(C.POINTER(C.c_int64)), C.byref(got))
        if rc:
            raise EisenHipError("eisen_data_loader_next_batch", rc, self.lib.eisen_io_last_error().decode())
        return (x, t) if got.value else None

    def reset(self):
        self.lib.eisen_data_loader_reset(self.h)


def save_weights(g, path):
    """examples/train_llm.rs:93-105."""
    g._call("eisen_graph_save_weights", str(path).encode())


def load_weights(g, params, path):
    """examples/chat_cli.rs:161-180; returns the number of floats loaded."""
    ids = (C.c_size_t * len(params))(*params)
    n = _sz()
    g._call("eisen_graph_load_weights", ids, _sz(len(params)), str(path).encode(), C.byref(n))
    return n.value


def write_safetensors(g, lm, path):
    """src/tools/huggingface.rs:88-146 over the model's named parameters."""
    g._call("eisen_lm_write_safetensors", lm.h, str(path).encode())


def write_llama_config(path, vocab, hidden, ffn, layers, heads, kv_heads, max_position_embeddings, rms_norm_eps=1e-5, rope_theta=10000.0,
                       tie_word_embeddings=False):
    """src/tools/huggingface.rs:38-84 (with the real KV head count)."""
    lib = _lib()
    rc = lib.eisen_write_llama_config(str(path).encode(), _sz(vocab), _sz(hidden), _sz(ffn), _sz(layers), _sz(heads), _sz(kv_heads),
                                      _sz(max_position_embeddings), _f(rms_norm_eps), _f(rope_theta), _i(int(tie_word_embeddings)))
    if rc:
        raise EisenHipError("eisen_write_llama_config", rc, lib.eisen_io_last_error().decode())
