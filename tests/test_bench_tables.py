"""bench.py's hand-carried tables against the sources they describe (CPU): every kernel symbol that MEASURED_TRAFFIC holds a
counter figure for must still be a profile entry the library can emit, and every summary file it cites must exist, so that a
renamed kernel or a deleted summary fails here instead of silently turning `roofline.traffic` into null."""
import os
import re

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "eisen_amd", "csrc")


def _sources():
    text = ""
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".cuh", ".h")):
            text += open(os.path.join(CSRC, name)).read()
    return text


def test_every_traffic_key_names_a_profile_entry_of_the_library():
    text = _sources()
    strings = re.findall(r'"([^"\n]*)"', text)          # every string literal, format strings included
    literals = set(strings)
    tiles = {t for lit in strings for t in re.findall(r"\d+x\d+x\d+", lit)}
    suffixes = {s for lit in strings for s in re.findall(r"_[a-z_]+$", lit) if lit.startswith("_")} | {""}
    for workload, table in bench.MEASURED_TRAFFIC.items():
        for key in table:
            if key == "attn_bwd":       # bench.py's own sum of the two backward entries
                assert "attn_bwd_dq_bf16" in literals and "attn_bwd_dkv_bf16" in literals
                continue
            if key in literals:
                continue
            # GEMM entries are composed as gemm_<order>_bf16_<out>_<tile><suffix> (gemm_common in gemm.hip)
            m = re.fullmatch(r"gemm_(nn|nt|tn|tt)_bf16_(bf16out|f32out)_(\d+x\d+x\d+)(_[a-z_]+)?", key)
            assert m, f"{workload}: {key!r} is neither a literal profile name nor a composed GEMM name"
            assert m.group(3) in tiles, f"{workload}: {key!r}: tile {m.group(3)} is not one the library names"
            assert (m.group(4) or "") in suffixes, f"{workload}: {key!r}: suffix {m.group(4)} is not one the library names"


def test_every_cited_summary_exists_and_mentions_its_figures():
    for workload, path in bench.TRAFFIC_SOURCE.items():
        full = os.path.join(ROOT, path)
        assert os.path.isfile(full), path
        assert bench.MEASURED_TRAFFIC.get(workload), f"{workload} cites {path} but carries no figure from it"
