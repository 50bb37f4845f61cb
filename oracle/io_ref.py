"""Test infrastructure only: CPU restatement of the reference's byte formats around the training step.

Nothing in the product imports this file.  Each function follows the cited reference code; what pins it
is stated next to it.
"""
import io
import struct

import numpy as np

READER_CAPACITY = 4 * 1024 * 1024  # BufReader::with_capacity, src/data/dataloader.rs:105


class _BufReader:
    """std::io::BufReader<File>::read as the loader uses it: a request that finds the internal buffer
    empty and is at least as large as the buffer bypasses it; otherwise the buffer is filled with one
    read and min(request, buffered) bytes are returned."""

    def __init__(self, data: bytes):
        self.f = io.BytesIO(data)
        self.buf = b""

    def read(self, want):
        if not self.buf and want >= READER_CAPACITY:
            return self.f.read(want)
        if not self.buf:
            self.buf = self.f.read(READER_CAPACITY)
        out, self.buf = self.buf[:want], self.buf[want:]
        return out


def binary_loader_batches(data: bytes, seq_len, batch_size):
    """All batches BinaryDataLoader::next_batch yields for a file with these bytes, FIM off
    (src/data/dataloader.rs:132-198): list of (x f32 [B*S], targets int64 [B*S]).

    Pinned by: for every batch handed out, x / targets are the consecutive windows of the token stream
    (the stated intent, dataloader.rs:133, :161-163), checked in the tests against plain numpy slicing.
    Parity unpinned: the exact batch at which iteration stops when a short BufReader read leaves less
    than one batch buffered (no reference test or fixture exercises it; it follows from reading
    std::io::BufReader's documented behaviour)."""
    need = batch_size * (seq_len + 1)
    rd, buf, out = _BufReader(data), [], []
    while True:
        if len(buf) < need:
            raw = rd.read(need * 100 * 2)
            if len(raw) == 0 and len(buf) < need:
                break
            n = len(raw) // 2
            buf.extend(struct.unpack("<%dH" % n, raw[:2 * n]))
        if len(buf) < need:
            break
        w = np.array(buf[:need], dtype=np.int64).reshape(batch_size, seq_len + 1)
        out.append((w[:, :-1].astype(np.float32).reshape(-1), w[:, 1:].reshape(-1).copy()))
        del buf[:need]
    return out


def total_batches(file_size, seq_len, batch_size):
    """src/data/dataloader.rs:99-104."""
    return (file_size // 2) // (batch_size * (seq_len + 1))


def save_weights_bytes(tensors):
    """examples/train_llm.rs:93-105: every parameter in id order as f32 LE."""
    return b"".join(np.asarray(t, dtype="<f4").tobytes() for t in tensors)


def safetensors_bytes(named):
    """src/tools/huggingface.rs:88-146.  named: ordered list of (name, float32 array).
    Pinned by: the `safetensors` library parses the result back to the transposed arrays (tests)."""
    entries, payload = {}, bytearray()
    for name, arr in named:
        arr = np.asarray(arr, dtype=np.float32)
        if arr.ndim == 2 and name != "model.embed_tokens.weight":
            arr = np.ascontiguousarray(arr.T)
        begin = len(payload)
        payload += arr.astype("<f4").tobytes()
        entries[name] = (list(arr.shape), begin, len(payload))
    header = "{" + ",".join(
        '"%s":{"dtype":"F32","shape":[%s],"data_offsets":[%d,%d]}' % (n, ",".join(str(d) for d in s), b, e)
        for n, (s, b, e) in sorted(entries.items(), key=lambda kv: kv[0].encode())) + "}"
    while len(header) % 8:
        header += " "
    return struct.pack("<Q", len(header)) + header.encode() + bytes(payload)
