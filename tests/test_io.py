"""Data-loader wire format and config writer: host-only code of the library, checked on the CPU against
the oracle restatement (oracle/io_ref.py) and against plain numpy slicing of the token stream."""
import json

import numpy as np
import pytest

from eisen_amd import io as IO
from eisen_amd.lib import EisenHipError
from oracle import io_ref as IR


def _stream(n_tokens, seed, extra_byte=False):
    rng = np.random.default_rng(seed)
    tok = rng.integers(0, 65536, n_tokens, dtype=np.uint16)
    data = tok.astype("<u2").tobytes() + (b"\x7f" if extra_byte else b"")
    return tok, data


def _drain(dl):
    out = []
    while True:
        b = dl.next_batch()
        if b is None:
            return out
        out.append(b)


# the 3,000,000-token stream is 6 MB: larger than the reference's 4 MiB reader, so refills come back short
@pytest.mark.parametrize("n_tokens,seq,batch,extra", [(0, 8, 2, False), (17, 8, 2, False), (18, 8, 2, False), (1000, 8, 2, True), (5000, 16, 3, False),
                                                      (40000, 31, 4, False), (3_000_000, 255, 8, False), (2_200_000, 1024, 4, True)])
def test_binary_loader_matches_oracle_and_windows(tmp_path, n_tokens, seq, batch, extra):
    tok, data = _stream(n_tokens, 7 + n_tokens % 13, extra)
    path = tmp_path / "tokens.bin"
    path.write_bytes(data)
    dl = IO.BinaryDataLoader(path, seq, batch)
    assert dl.total_batches() == IR.total_batches(len(data), seq, batch) == (len(data) // 2) // (batch * (seq + 1))
    got = _drain(dl)
    exp = IR.binary_loader_batches(data, seq, batch)
    assert len(got) == len(exp)
    need = batch * (seq + 1)
    assert len(got) <= dl.total_batches()
    for i, ((x, t), (ex, et)) in enumerate(zip(got, exp)):
        assert x.dtype == np.float32 and t.dtype == np.int64
        assert np.array_equal(x, ex) and np.array_equal(t, et)          # bit-exact against the oracle
        w = tok[i * need:(i + 1) * need].reshape(batch, seq + 1)         # and both against the plain definition
        assert np.array_equal(x, w[:, :-1].astype(np.float32).reshape(-1))
        assert np.array_equal(t, w[:, 1:].astype(np.int64).reshape(-1))
    # streams that fit one refill are served completely
    if len(data) <= need * 100 * 2:
        assert len(got) == dl.total_batches()
    # reset() rewinds to the first batch
    dl.reset()
    again = _drain(dl)
    assert len(again) == len(got) and all(np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]) for a, b in zip(again, got))
    dl.close()


def test_binary_loader_errors(tmp_path):
    with pytest.raises(EisenHipError, match="Binary file not found"):
        IO.BinaryDataLoader(tmp_path / "missing.bin", 8, 2)
    (tmp_path / "t.bin").write_bytes(b"\0" * 64)
    with pytest.raises(EisenHipError):
        IO.BinaryDataLoader(tmp_path / "t.bin", 0, 2)


def test_llama_config_text(tmp_path):
    p = tmp_path / "config.json"
    IO.write_llama_config(p, 32000, 2048, 5632, 16, 32, 8, 1024, 1e-5, 10000.0, False)
    text = p.read_text()
    cfg = json.loads(text)
    assert cfg == {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 32000, "hidden_size": 2048,
                   "intermediate_size": 5632, "num_hidden_layers": 16, "num_attention_heads": 32, "num_key_value_heads": 8,
                   "max_position_embeddings": 1024, "rms_norm_eps": 1e-5, "rope_theta": 10000, "bos_token_id": 1, "eos_token_id": 2,
                   "pad_token_id": 0, "hidden_act": "silu", "tie_word_embeddings": False, "initializer_range": 0.02, "torch_dtype": "float32"}
    # the reference's `{}` formatting of the two f32 fields (src/tools/huggingface.rs:56-57): no exponent, shortest digits
    assert '"rms_norm_eps": 0.00001,\n' in text and '"rope_theta": 10000,\n' in text
    assert text.startswith('{\n  "architectures": ["LlamaForCausalLM"],\n  "model_type": "llama",\n') and text.endswith('"torch_dtype": "float32"\n}\n')
    IO.write_llama_config(p, 8, 8, 8, 1, 2, 2, 16, 1e-6, 500000.0, True)
    text = p.read_text()
    assert '"rms_norm_eps": 0.000001,' in text and '"rope_theta": 500000,' in text and '"tie_word_embeddings": true,' in text
