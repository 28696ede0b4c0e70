"""The engine's host logic (batch building, block tables, slot mapping, page reuse) on the
CPU: the HIP kernels are replaced by their plain torch references (tests/kernel_refs.py), the
rest is the product's own code.  The same traces run on the GPU in test_engine_gpu.py."""
import numpy as np
import pytest
import torch

import kernel_refs
import test_engine_gpu as G
import tiny
import traces


@pytest.fixture(autouse=True)
def _emulated_kernels(monkeypatch):
    kernel_refs.install(monkeypatch)
    monkeypatch.setattr(G, "DEVICE", ["cpu"])


@pytest.mark.parametrize("mode", list(G.MODES))
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_replay_modes_host_logic(name, mode, tmp_path_factory):
    path, cfg, requests, ref = G._setup(name, "float32", tmp_path_factory, twice=mode == "mixed")
    steps = G.MODES[mode](requests)
    outputs, eng = G._replay(path, "float32", steps, tiny.PAGE_SIZE[name],
                             G._pool_tokens(name, mode, steps))
    G._compare(steps, outputs, ref, cfg["vocab_size"], 1e-5)
    if mode == "mixed":
        G._assert_pages_were_used_again(eng, steps)


def test_mixed_reuse_host_logic(tmp_path_factory):
    G.test_mixed_many_requests_reuse_pages("float32", tmp_path_factory)


def test_130_sequences_host_logic(tmp_path_factory):
    G.test_a_decode_step_of_130_sequences("B", "float32", tmp_path_factory)


def test_step_errors_host_logic(tmp_path_factory):
    G.test_step_errors_leave_cache_untouched(tmp_path_factory)


def test_cache_dtype_host_logic(tmp_path_factory):
    G.test_a_cache_of_another_dtype_is_refused(tmp_path_factory)


def test_bfloat16_storage_host_logic(tmp_path_factory):
    """bfloat16 weights and cache through the same host code."""
    path, cfg, requests, ref = G._setup("B", "bfloat16", tmp_path_factory)
    steps = traces.mixed(requests)
    outputs, _ = G._replay(path, "bfloat16", steps, 8)
    G._compare(steps, outputs, ref, cfg["vocab_size"], G.LOGITS_TOL_BF16)
