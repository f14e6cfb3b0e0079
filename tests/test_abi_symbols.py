"""CPU checks of the C-ABI library: it loads, exports every symbol include/nats_hip.h declares, and its
argument validation rejects bad calls before anything touches a GPU."""
import ctypes
import os
import re

import pytest

from neuralattentionsearch_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "nats_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nats_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in declared_symbols():
        assert hasattr(lib, name), name
    assert lib.nats_abi_version() == _lib.ABI_VERSION


def test_struct_sizes_match_header():
    assert ctypes.sizeof(_lib.EvictParams) == 15 * 8
    assert ctypes.sizeof(_lib.PastState) == 7 * 8
    assert ctypes.sizeof(_lib.EvictResult) == 64


def test_null_pointer_is_rejected_without_a_gpu():
    lib = _lib.load()
    rc = lib.nats_role_scan(None, 1, 1, 4, 4, 2, None, None, None)
    assert rc == -1
    assert b"NULL" in lib.nats_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc)


def test_window_not_multiple_of_chunk_is_rejected():
    lib = _lib.load()
    fake = ctypes.c_void_p(16)  # never dereferenced: validation fails first
    rc = lib.nats_role_scan(fake, 1, 1, 4, 6, 4, None, None, None)
    assert rc == -2
    rc = lib.nats_role_scan(fake, 1, 1, 4, 6, 0, None, None, None)
    assert rc == -2  # (any positive chunk size that divides the window is taken, as nats_chunk_layer_cache.py:47 asks)
    with pytest.raises(ValueError):
        _lib.check(rc)


def test_prefill_rejects_bad_head_dim_and_small_workspace():
    lib = _lib.load()
    fake = ctypes.c_void_p(256)
    st = _lib.i64_array([8, 8, 8])
    rc = lib.nats_prefill_fwd(fake, fake, fake, fake, fake, 1, 4, 2, 128, 96, 64, 128, st, st, st, st, 1.0, 0, fake, 1 << 20,
                              None)
    assert rc == -4
    rc = lib.nats_prefill_fwd(fake, fake, fake, fake, fake, 1, 4, 2, 128, 128, 64, 128, st, st, st, st, 1.0, 0, fake, 8, None)
    assert rc == -5
    rc = lib.nats_prefill_fwd(fake, fake, fake, fake, fake, 1, 5, 2, 128, 128, 64, 128, st, st, st, st, 1.0, 0, fake, 1 << 20,
                              None)
    assert rc == -2


def test_past_state_is_validated():
    lib = _lib.load()
    fake = ctypes.c_void_p(256)
    st = _lib.i64_array([8, 8, 8])
    args = lambda ps, ws=1 << 24: (fake, fake, fake, fake, fake, fake, fake, fake, 1, 4, 2, 100, 128, 16, 32,
                                   ctypes.byref(ps), st, st, st, st, st, 1.0, 0, fake, ws, None)
    ok = _lib.PastState(320, 5, 64, 16, 400, 5, 0)
    assert lib.nats_prefill_past_fwd(*args(ok, 8)) == -5  # everything valid but the workspace
    assert lib.nats_prefill_past_fwd(*args(_lib.PastState(320, 16, 64, 16, 400, 5, 0))) == -2  # old_fill >= C
    assert lib.nats_prefill_past_fwd(*args(_lib.PastState(320, 5, 16, 16, 400, 5, 0))) == -2  # gmin < W
    assert lib.nats_prefill_past_fwd(*args(_lib.PastState(320, 5, 64, 32, 400, 5, 0))) == -2  # tail >= W
    assert lib.nats_prefill_past_fwd(*args(_lib.PastState(20, 5, 64, 16, 400, 5))) == -2  # n_ctx_data < W + old_fill
    assert b"n_ctx_data" in lib.nats_last_error()
    need = lib.nats_prefill_past_workspace_bytes(1, 2, 420, 7)
    assert need >= 2 * (7 * 4 + 4 + 420 * 4 + 7 * 8)


def test_evict_params_are_validated():
    lib = _lib.load()
    fake = ctypes.c_void_p(256)
    p = _lib.EvictParams(1, 2, 128, 64, 96, 1, 64, 64, 96, 96, 0, 1, 256)  # W % C != 0
    rc = lib.nats_evict_plan(fake, fake, fake, ctypes.byref(p), fake, 1 << 20, fake, None, None)
    assert rc == -2
    p = _lib.EvictParams(1, 2, 128, 64, 128, 3, 64, 64, 128, 128, 0, 1, 256)  # S inconsistent with fill
    rc = lib.nats_evict_plan(fake, fake, fake, ctypes.byref(p), fake, 1 << 20, fake, None, None)
    assert rc == -2


def test_missing_library_raises_instead_of_falling_back(monkeypatch, tmp_path):
    """Without the built shared object every operator raises: there is no CPU or PyTorch path behind them."""
    import torch
    from neuralattentionsearch_amd import ops
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libnats_hip.so"))
    with pytest.raises(ImportError, match="no CPU or PyTorch fallback"):
        _lib.load()
    with pytest.raises(ImportError):
        ops.matvec_ok(torch.zeros(1, 8), torch.zeros(8, 8)) or ops.MatvecPlan(torch.zeros(8, 8))


def test_ops_reject_cpu_tensors():
    import torch
    from neuralattentionsearch_amd import ops
    with pytest.raises(ValueError):
        ops.role_scan(torch.zeros(1, 1, 4, dtype=torch.uint8), 4, 2)


def test_matvec_arguments_are_validated():
    lib = _lib.load()
    fake = ctypes.c_void_p(256)  # never dereferenced: validation fails first
    assert lib.nats_matvec(None, fake, fake, 1, 8, 64, 64, 64, 8, 0, 0, None) == -1
    assert lib.nats_matvec(fake, fake, fake, 5, 8, 64, 64, 64, 8, 0, 0, None) == -4  # at most four rows of x
    assert b"rows" in lib.nats_last_error()
    assert lib.nats_matvec(fake, fake, fake, 1, 8, 60, 64, 64, 8, 0, 0, None) == -2  # k not in 16-byte pieces (bf16)
    assert lib.nats_matvec(fake, fake, fake, 1, 8, 64, 60, 64, 8, 0, 0, None) == -2  # weight rows not 16-byte aligned
    assert lib.nats_matvec(fake, fake, fake, 1, 8, 64, 64, 64, 4, 0, 0, None) == -2  # y rows shorter than n_out
    assert lib.nats_matvec(fake, ctypes.c_void_p(264), fake, 1, 8, 64, 64, 64, 8, 0, 0, None) == -2  # x not 16-byte aligned
    assert lib.nats_matvec(fake, fake, fake, 1, 8, 64, 64, 64, 8, 0, 7, None) == -3  # dtype code


def test_rope_qk_arguments_are_validated():
    lib = _lib.load()
    fake = ctypes.c_void_p(256)
    st3, st2 = _lib.i64_array([4096, 128, 512]), _lib.i64_array([4096, 128])
    assert lib.nats_rope_qk(None, fake, fake, fake, fake, fake, 1, 4, 2, 8, 128, st3, st3, st2, 0, None) == -1
    assert lib.nats_rope_qk(fake, fake, fake, fake, fake, fake, 1, 4, 2, 8, 24, st3, st3, st2, 0, None) == -4  # D % 16
    assert lib.nats_rope_qk(fake, fake, fake, fake, fake, fake, 1, 4, 2, 0, 128, st3, st3, st2, 0, None) == -2  # no tokens
    odd = _lib.i64_array([4096, 124, 512])
    assert lib.nats_rope_qk(fake, fake, fake, fake, fake, fake, 1, 4, 2, 8, 128, odd, st3, st2, 0, None) == -2  # 16-byte rows
    assert lib.nats_rope_qk(fake, fake, fake, fake, fake, fake, 1, 4, 2, 8, 128, st3, st3, st2, 9, None) == -3  # dtype


def test_container_is_a_transformers_cache():
    """The reference's NAtSCache subclasses DynamicCache (components/cache/dyn_cache.py:66) and is handed to HF models
    as past_key_values; its constructor and the calls made before any update work without a GPU."""
    cache_utils = pytest.importorskip("transformers.cache_utils")
    from neuralattentionsearch_amd.cache import NAtSCache
    cache = NAtSCache(256, 64)
    assert isinstance(cache, cache_utils.Cache) and isinstance(cache, cache_utils.DynamicCache)
    assert cache.get_seq_length() == 0 and cache.get_seq_length(3) == 0 and len(cache) == 0
    assert cache.get_nats_chunk_fill_size(0) == 0 and cache.get_nats_cached_x_in_chunk(0) is None
    assert cache.sliding_window_size == 256 and cache.chunk_size == 64
    cache.reset_cache()
    assert cache.cache_model == []


def test_a_transformers_llama_model_takes_the_container_as_past_key_values():
    """The reference's callers hand NAtSCache to a Hugging Face model (experiments/long_bench/hf_pred.py:173-184,
    experiments/efficiency/eval_efficiency.py:297-340) whose attention layers they have patched
    (models/transformer/hf/llama_nats_chunk.py).  Everything the unpatched parts of such a model ask of the cache
    while they prepare a forward pass (sequence length, mask sizes, the sliding flags) must work on the container;
    here the attention layers are stand-ins that return zeros, so no GPU is needed."""
    pytest.importorskip("transformers")
    import torch
    from transformers import LlamaConfig, LlamaModel
    from transformers.models.llama import modeling_llama
    from neuralattentionsearch_amd.cache import NAtSCache

    seen = []

    def attention_stand_in(self, hidden_states, *args, **kwargs):
        cache = kwargs.get("past_key_values", kwargs.get("past_key_value"))
        seen.append(cache)
        return torch.zeros_like(hidden_states), None

    cfg = LlamaConfig(vocab_size=100, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, max_position_embeddings=512)
    model = LlamaModel(cfg).eval()
    original = modeling_llama.LlamaAttention.forward
    modeling_llama.LlamaAttention.forward = attention_stand_in
    try:
        cache = NAtSCache(16, 4)
        with torch.no_grad():
            out = model(input_ids=torch.randint(0, 100, (1, 12)), past_key_values=cache, use_cache=True)
            out1 = model(input_ids=torch.randint(0, 100, (1, 1)), past_key_values=cache, use_cache=True)
    finally:
        modeling_llama.LlamaAttention.forward = original
    assert out.last_hidden_state.shape == (1, 12, 64) and out1.last_hidden_state.shape == (1, 1, 64)
    assert out.past_key_values is cache and out1.past_key_values is cache  # (the callers go on with output.past_key_values)
    assert len(seen) == 4 and all(c is cache for c in seen)
    assert cache.get_mask_sizes(5, 0) == (5, 0) and cache.is_sliding == [] and not cache.is_compileable
