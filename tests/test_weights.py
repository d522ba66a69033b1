"""Safetensors reading, the weight contract and its one error, random-weights folders (no GPU)."""

import json
import os
import struct

import pytest
import torch

import burn_transformers_amd as bt
from burn_transformers_amd.weights import contract as wc
from burn_transformers_amd.weights.loader import load_checkpoint, store_from_tensors
from burn_transformers_amd.weights.safetensors_io import (PayloadReader, SafetensorsError, discover,
                                                          read_header, write_safetensors)

CONFIG = {"architectures": ["GPT2LMHeadModel"], "n_layer": 2, "n_embd": 32, "n_head": 2, "n_inner": 48,
          "vocab_size": 61, "n_positions": 24}


def family_and_contract():
    family = bt.resolve_family(CONFIG)
    config = family.config_class.from_dict(CONFIG)
    return family, config, family.contract(config)


def test_round_trip_matches_the_safetensors_package(tmp_path):
    import safetensors.torch
    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16),
               "c": torch.arange(6, dtype=torch.int32).reshape(2, 3)}
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, tensors)
    theirs = safetensors.torch.load_file(path)
    header, reader = read_header(path), PayloadReader()
    for name, tensor in tensors.items():
        assert torch.equal(theirs[name], tensor)
        mine = reader.tensor(header[name])
        assert mine.dtype == tensor.dtype and torch.equal(mine, tensor)
    theirs_path = str(tmp_path / "y.safetensors")
    safetensors.torch.save_file(tensors, theirs_path)
    header = read_header(theirs_path)
    assert all(torch.equal(reader.tensor(header[n]), t) for n, t in tensors.items())


def test_malformed_files_are_refused_before_any_payload(tmp_path):
    path = str(tmp_path / "bad.safetensors")
    header = json.dumps({"w": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 12]}}).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(header)) + header + b"\0" * 12)
    with pytest.raises(SafetensorsError, match="needs 16 bytes"):
        read_header(path)
    header = json.dumps({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},
                         "b": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(header)) + header + b"\0" * 12)
    with pytest.raises(SafetensorsError, match="overlap"):
        read_header(path)
    # the ranges must tile the payload: no gap between tensors, none before the first, none after the last
    for offsets, size, message in (([[0, 8], [12, 20]], 20, "4 bytes between tensors 'a' and 'b' belong to no tensor"),
                                   ([[4, 12], [12, 20]], 20, r"cover bytes \[4, 20\) of a payload of 20"),
                                   ([[0, 8], [8, 16]], 24, r"cover bytes \[0, 16\) of a payload of 24")):
        header = json.dumps({"a": {"dtype": "F32", "shape": [2], "data_offsets": offsets[0]},
                             "b": {"dtype": "F32", "shape": [2], "data_offsets": offsets[1]}}).encode()
        with open(path, "wb") as f:
            f.write(struct.pack("<Q", len(header)) + header + b"\0" * size)
        with pytest.raises(SafetensorsError, match=message):
            read_header(path)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", 10 ** 12))
    with pytest.raises(SafetensorsError, match="does not fit"):
        read_header(path)


def test_random_model_folder_has_the_stated_distributions(tmp_path):
    """src/models/gpt2/model_tests.rs:1116-1177 (per-tensor std within 10 %)."""
    config = dict(CONFIG, n_embd=128, n_head=4, n_inner=512, vocab_size=1000, n_layer=4)
    stored = bt.write_random_model(str(tmp_path), config, seed=5)
    assert sorted(os.listdir(tmp_path)) == ["config.json", "model.safetensors"]
    assert json.load(open(tmp_path / "config.json"))["n_embd"] == 128
    again = bt.write_random_model(str(tmp_path / "again"), config, seed=5)
    assert all(torch.equal(stored[k], again[k]) for k in stored)
    other = bt.write_random_model(str(tmp_path / "other"), config, seed=6)
    assert not torch.equal(stored["wte.weight"], other["wte.weight"])
    assert abs(float(stored["wte.weight"].std()) / 0.02 - 1) < 0.1
    assert abs(float(stored["h.1.attn.c_attn.weight"].std()) / 0.02 - 1) < 0.1
    residual = 0.02 / (2 * 4) ** 0.5
    assert abs(float(stored["h.2.attn.c_proj.weight"].std()) / residual - 1) < 0.1
    assert abs(float(stored["h.3.mlp.c_proj.weight"].std()) / residual - 1) < 0.1
    assert abs(float(stored["h.0.ln_1.weight"].mean()) - 1) < 0.01 and float(stored["h.0.ln_1.weight"].std()) > 0.005
    assert float(stored["h.0.mlp.c_fc.bias"].std()) > 0.005
    header = read_header(str(tmp_path / "model.safetensors"))
    assert {e.dtype for e in header.values()} == {"BF16"}
    assert header["h.0.attn.c_attn.weight"].shape == (128, 384)       # Conv1D [in, out]


def write_checkpoint(folder, tensors, name="model.safetensors"):
    os.makedirs(folder, exist_ok=True)
    write_safetensors(os.path.join(folder, name), tensors)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    family, config, contract = family_and_contract()
    _, tensors = bt.random_tensors(CONFIG, 0)
    broken = dict(tensors)
    del broken["h.1.ln_2.bias"], broken["ln_f.weight"]
    broken["h.0.attn.rotary.inv_freq"] = torch.zeros(4)
    broken["extra.weight"] = torch.zeros(2, 2)
    broken["h.0.mlp.c_fc.weight"] = torch.zeros(48, 32)               # transposed
    broken["wpe.weight"] = torch.zeros(24, 32, dtype=torch.int32)     # not floating point
    write_checkpoint(str(tmp_path), broken)
    with pytest.raises(bt.WeightError) as info:
        load_checkpoint(str(tmp_path), contract, torch.float32, "cpu")
    error = info.value
    assert error.missing == ["h.1.ln_2.bias", "ln_f.weight"]
    assert error.unexpected == ["extra.weight", "h.0.attn.rotary.inv_freq"]
    assert len(error.mismatched) == 2
    text = str(error)
    assert "h.0.mlp.c_fc.weight: stored F32[48, 32], the model needs [32, 48]" in text
    assert "wpe.weight: parameters must be floating point, stored as I32" in text
    assert "missing tensors (2): h.1.ln_2.bias, ln_f.weight" in text


def test_namespaces_ignored_buffers_and_the_tied_head(tmp_path):
    """src/models/gpt2/checkpoint.rs:61-71, 169-174, 182-188; checkpoint_tests.rs:59-89."""
    family, config, contract = family_and_contract()
    _, tensors = bt.random_tensors(CONFIG, 0)
    prefixed = {"transformer." + k: v for k, v in tensors.items()}
    prefixed["transformer.h.0.attn.bias"] = torch.ones(1, 1, 24, 24)          # legacy mask buffers
    prefixed["transformer.h.1.attn.masked_bias"] = torch.tensor(-1e4)
    prefixed["lm_head.weight"] = tensors["wte.weight"].clone()                # stored copy of the tied head
    write_checkpoint(str(tmp_path / "lm"), prefixed)
    store = load_checkpoint(str(tmp_path / "lm"), contract, torch.float32, "cpu")
    assert set(store) == set(tensors)
    assert torch.equal(store["h.0.attn.c_attn.weight"], tensors["h.0.attn.c_attn.weight"].t())   # held [out, in]
    assert store["h.0.ln_1.weight"].dtype == torch.float32
    exported = store.export()
    assert all(torch.equal(exported[k], tensors[k]) for k in tensors)
    # what loading did is on record (src/checkpoint/report.rs:58-100)
    assert store.report["namespace"] == "transformer." and store.report["applied"] == len(tensors)
    assert store.report["aliased"] == ["lm_head.weight"] and store.report["converted"] == {}
    assert store.report["ignored"] == ["transformer.h.0.attn.bias", "transformer.h.1.attn.masked_bias"]
    # a stored head that differs from the token table is refused
    prefixed["lm_head.weight"] = tensors["wte.weight"] + 1
    write_checkpoint(str(tmp_path / "untied"), prefixed)
    with pytest.raises(bt.WeightError, match="must be tied"):
        load_checkpoint(str(tmp_path / "untied"), contract, torch.float32, "cpu")
    # both namespaces at once, or neither
    both = dict(prefixed, **{"wte.weight": tensors["wte.weight"]})
    write_checkpoint(str(tmp_path / "both"), both)
    with pytest.raises(bt.WeightError, match="exactly one of `wte.weight`, `transformer.wte.weight`, found 2"):
        load_checkpoint(str(tmp_path / "both"), contract, torch.float32, "cpu")
    write_checkpoint(str(tmp_path / "none"), {"x": torch.zeros(1)})
    with pytest.raises(bt.WeightError, match="found 0"):
        load_checkpoint(str(tmp_path / "none"), contract, torch.float32, "cpu")
    # another buffer than the two legacy ones is not ignored
    prefixed["lm_head.weight"] = tensors["wte.weight"].clone()
    prefixed["transformer.h.0.attn.other"] = torch.zeros(1)
    write_checkpoint(str(tmp_path / "other"), prefixed)
    with pytest.raises(bt.WeightError, match="unexpected tensors \\(1\\): transformer.h.0.attn.other"):
        load_checkpoint(str(tmp_path / "other"), contract, torch.float32, "cpu")


def test_dtype_policy_and_sharded_checkpoints(tmp_path):
    family, config, contract = family_and_contract()
    _, tensors = bt.random_tensors(CONFIG, 1)
    names = sorted(tensors)
    half = len(names) // 2
    folder = str(tmp_path)
    write_checkpoint(folder, {k: tensors[k] for k in names[:half]}, "model-00001-of-00002.safetensors")
    write_checkpoint(folder, {k: tensors[k].to(torch.bfloat16) for k in names[half:]}, "model-00002-of-00002.safetensors")
    weight_map = {k: "model-00001-of-00002.safetensors" for k in names[:half]}
    weight_map.update({k: "model-00002-of-00002.safetensors" for k in names[half:]})
    weight_map["lm_head.weight"] = "model-00001-of-00002.safetensors"           # index-only alias of the tied head
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": weight_map}, f)
    assert len(discover(folder)[0]) == 2
    store = load_checkpoint(folder, contract, torch.bfloat16, "cpu")
    assert store["wte.weight"].dtype == torch.bfloat16                  # matrices and tables in the compute dtype
    assert store["ln_f.bias"].dtype == torch.float32                    # vectors always in float32
    rounded = tensors["h.0.mlp.c_fc.weight"].to(torch.bfloat16)         # one rounding to nearest even
    assert torch.equal(store["h.0.mlp.c_fc.weight"], rounded.t())
    matrices = [k for k in names if tensors[k].dim() == 2]
    assert store.report["converted"] == {"float32->bfloat16": sum(k in names[:half] for k in matrices),
                                         "bfloat16->float32": sum(k in names[half:] for k in names if k not in matrices)}
    assert store.report["namespace"] == "" and store.report["aliased"] == [] and store.report["ignored"] == []
    wide = load_checkpoint(folder, contract, torch.float32, "cpu")
    assert wide["wte.weight"].dtype == torch.float32
    with pytest.raises(ValueError, match="bfloat16 or float32"):
        bt.weights.compute_dtype("float16")


def test_in_memory_tensors_go_through_the_same_check():
    family, config, contract = family_and_contract()
    _, tensors = bt.random_tensors(CONFIG, 2)
    del tensors["ln_f.bias"]
    with pytest.raises(bt.WeightError, match="missing tensors \\(1\\): ln_f.bias"):
        store_from_tensors(tensors, contract, torch.float32, "cpu")


def test_packed_layout_of_a_matrix():
    """pack_columns: group g, chunk c, column j, element e of the packed copy is W[g * columns + j,
    c * chunk + e], zero beyond the matrix (chunks of 32 bfloat16 or 16 float32 values of K)."""
    import torch
    from burn_transformers_amd.kernels.library import pack_columns, skinny_columns
    for dtype, chunk in ((torch.bfloat16, 32), (torch.float32, 16)):
        w = torch.arange(50 * 72, dtype=torch.float32).reshape(50, 72).to(dtype)
        packed = pack_columns(w, 12)
        assert packed.shape == (5, (72 + chunk - 1) // chunk, 12, chunk) and packed.is_contiguous()
        for g, c, j, e in ((0, 0, 0, 0), (1, 2, 3, 7), (4, 1, 1, 5), (3, 0, 11, chunk - 1)):
            row, col = g * 12 + j, c * chunk + e
            want = w[row, col] if row < 50 and col < 72 else 0
            assert packed[g, c, j, e] == want
        assert packed[4, 0, 2:].abs().sum() == 0           # rows 50..59 do not exist
        assert packed[0, -1, :, 72 % chunk:].abs().sum() == 0 or 72 % chunk == 0
    # the launcher's rule: the fewest rounds of work-groups over the compute units, then the fewest columns
    assert skinny_columns(8, 4800, 1600, 1, torch.bfloat16, 256) == 20
    assert skinny_columns(8, 6400, 1600, 1, torch.bfloat16, 256) == 28
    assert skinny_columns(8, 1600, 6400, 5, torch.bfloat16, 256) == 32
    assert skinny_columns(8, 1600, 1600, 1, torch.bfloat16, 256) == 8


def test_chunk_major_layout_of_activations():
    """Chunked: element (row, column) lies at ((column // chunk) * rows + row) * chunk + column % chunk
    with chunks of 64 bytes; ``to_rows`` undoes it; the policy takes steps of 17 to 64 rows."""
    import torch
    from burn_transformers_amd.kernels.library import Chunked

    class Workspace:
        def buffer(self, key, rows, cols, dtype):
            return torch.zeros(rows, cols, dtype=dtype)

    for dtype, chunk in ((torch.bfloat16, 32), (torch.float32, 16)):
        rows, columns = 5, 72
        held = Chunked.take(Workspace(), "test", rows, columns, dtype)
        assert held.shape == (rows, columns) and held.data.numel() == rows * ((columns + chunk - 1) // chunk * chunk)
        flat = held.data.view(-1)
        want = torch.arange(rows * columns, dtype=torch.float32).reshape(rows, columns).to(dtype)
        for r in range(rows):
            for c in range(columns):
                flat[((c // chunk) * rows + r) * chunk + c % chunk] = want[r, c]
        assert torch.equal(held.to_rows(), want)
        assert held.stride(0) == columns and held.stride(1) == 1 and held.dtype == dtype
    assert [Chunked.wanted(n) for n in (1, 8, 9, 64, 65)] == [False, False, True, True, False]
    Chunked.enabled = False
    try:
        assert not Chunked.wanted(32)
    finally:
        Chunked.enabled = True
