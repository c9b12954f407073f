"""The runtime's rules about the GPU it drives, checked without one (``torch.cuda`` stands in), and the
check of a model's sizes against the kernels, which needs no GPU either."""

import types

import pytest
import torch

from nnis_amd.errors import InvalidInput, KernelError, Unsupported


@pytest.fixture
def one_gpu(monkeypatch):
    """A process that sees two GPUs, of which cuda:0 is current; the kernels' library is not loaded."""
    from nnis_amd.kernels import ops

    state = {"current": 0}
    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(torch.cuda, "device_count", lambda: 2)
    monkeypatch.setattr(torch.cuda, "current_device", lambda: state["current"])
    monkeypatch.setattr(torch.cuda, "set_device", lambda index: state.update(current=int(index)))
    monkeypatch.setattr(ops, "core", lambda: None)
    monkeypatch.setattr(ops, "_device_index", None)
    return state


def test_a_runtime_makes_its_device_current_and_a_process_drives_one(one_gpu):
    from nnis_amd.engine.runtime import Runtime
    from nnis_amd.kernels import ops

    with pytest.raises(InvalidInput, match="ordinal 5 names no GPU"):
        Runtime("cuda:5")
    assert ops.bound_device() is None  # a refused runtime binds nothing
    rt = Runtime("cuda:1", "float32")
    assert one_gpu["current"] == 1 and ops.bound_device() == 1 and rt.device == torch.device("cuda", 1)
    Runtime("cuda:1")  # the same GPU again: fine
    with pytest.raises(KernelError, match="already runs its kernels on cuda:1"):
        Runtime("cuda:0")
    assert one_gpu["current"] == 1  # the refusal changed nothing
    rt.check_current()
    one_gpu["current"] = 0  # somebody made another GPU current
    with pytest.raises(InvalidInput, match="current device is cuda:0"):
        rt.check_current()
    with pytest.raises(KernelError, match="GPU only"):
        Runtime("cpu")


def test_an_unnamed_ordinal_is_the_current_device(one_gpu):
    from nnis_amd.engine.runtime import Runtime

    one_gpu["current"] = 1
    assert Runtime("cuda").device == torch.device("cuda", 1)


def test_sizes_are_checked_against_the_kernels_before_anything_is_loaded():
    from configs import TINY_B, llama
    from nnis_amd.config.registry import spec_from_config
    from nnis_amd.kernels import ops
    from nnis_amd.models.decoder import DecoderModel

    rt = types.SimpleNamespace(ops=ops, dtype=torch.bfloat16)
    DecoderModel(spec_from_config(TINY_B)[1]).check(rt)  # sizes that run
    for head_dim in (258, 1024):
        config = llama(num_hidden_layers=1, hidden_size=64, num_attention_heads=2, num_key_value_heads=1, head_dim=head_dim,
                       intermediate_size=96, vocab_size=100, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=True,
                       max_position_embeddings=128, torch_dtype="bfloat16")
        model = DecoderModel(spec_from_config(config)[1])  # the configuration itself allows it
        with pytest.raises(Unsupported, match=f"head_dim up to 256, got {head_dim}"):
            model.check(rt)
