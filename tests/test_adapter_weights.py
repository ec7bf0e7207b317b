"""Host-side packing of an adapter checkpoint into the pool's row format (no GPU): the key scheme and
the slicing of the reference's loader (valora/models/peft/layer_weights/lora_layer_weight.py:434-516)
against oracle/pool_oracle.py::w_combined, which restates the reference's own chain of transposes."""
import pytest
import torch

from oracle import pool_oracle as P
from valora_amd.infer_adapter import LoraAdapterWeights

NET = {"num_hidden_layers": 3, "hidden_size": 16, "num_attention_heads": 4}


def checkpoint(names, r, rows_b, seed=0, skip=()):
    g = torch.Generator().manual_seed(seed)
    H, sd = NET["hidden_size"], {}
    for l in range(NET["num_hidden_layers"]):
        for m in names:
            if (l, m) in skip:
                continue
            key = f"base_model.model.transformer.layers.{l}.self_attn.{m}"
            sd[f"{key}.lora_A.weight"] = torch.randn(r, H, generator=g)
            sd[f"{key}.lora_B.weight"] = torch.randn(rows_b.get(m, H), r, generator=g)
    return sd


def test_qwen_names_wide_b_is_cut_to_hidden_and_missing_module_is_zero():
    names, r, H = ("c_attn", "w1", "w2", "c_proj"), 4, NET["hidden_size"]
    sd = checkpoint(names, r, {"c_attn": 3 * H, "w1": 44, "w2": 44}, skip={(1, "c_proj")})
    ad = LoraAdapterWeights.from_hf_weights("dir", sd, {"r": r, "lora_alpha": 8}, NET, pin=False)
    assert ad.scaling == 2.0 and ad.n_slots == 4 and ad.r == r
    for l in range(NET["num_hidden_layers"]):
        A, B = [], []
        for m in names:
            key = f"base_model.model.transformer.layers.{l}.self_attn.{m}"
            a, b = sd.get(f"{key}.lora_A.weight"), sd.get(f"{key}.lora_B.weight")
            A.append(None if a is None else a[:, :H])     # tp_idx = (0, hidden) at world size 1
            B.append(None if b is None else b[:H, :])
        want = P.w_combined(A, B, r, NET["num_attention_heads"], H)
        assert torch.equal(ad.packed_home[l].reshape(want.shape), want), f"layer {l}"
    assert not ad.packed_home[1, :, 3 * r:].any()        # the module that is not in the checkpoint
    # the math view: delta = x @ A @ B * scaling with A = lora_A.weight.T, B = lora_B.weight[:H].T
    A0, B0 = ad.dense(2, 0)
    key = "base_model.model.transformer.layers.2.self_attn.c_attn"
    assert torch.equal(A0, sd[f"{key}.lora_A.weight"].T.half())
    assert torch.equal(B0, sd[f"{key}.lora_B.weight"][:H].T.half())


def test_llama_names_and_bf16():
    names = ("q_proj", "k_proj", "v_proj", "o_proj")
    sd = checkpoint(names, 2, {}, seed=1)
    ad = LoraAdapterWeights.from_hf_weights("d", sd, {"r": 2, "lora_alpha": 2}, NET, module_names=names,
                                            dtype=torch.bfloat16, pin=False)
    assert ad.packed_home.dtype == torch.bfloat16
    k = "base_model.model.transformer.layers.0.self_attn.v_proj"
    assert torch.equal(ad.packed_home[0, 0, 4:6], sd[f"{k}.lora_A.weight"].bfloat16())
    assert torch.equal(ad.packed_home[0, 1, 4:6].reshape(-1), sd[f"{k}.lora_B.weight"].bfloat16().reshape(-1))
    # the reference's default names find nothing in this checkpoint: all zeros, like its safe_reshape
    none = LoraAdapterWeights.from_hf_weights("d", sd, {"r": 2, "lora_alpha": 2}, NET, pin=False)
    assert not none.packed_home.any()


def test_checkpoint_errors():
    with pytest.raises(RuntimeError, match="empty"):
        LoraAdapterWeights.from_hf_weights("d", {}, {"r": 2, "lora_alpha": 2}, NET)
    with pytest.raises(RuntimeError, match="layers"):
        LoraAdapterWeights.from_hf_weights("d", {"foo.weight": torch.zeros(1)}, {"r": 2, "lora_alpha": 2}, NET)
    sd = checkpoint(("c_attn",), 2, {})
    with pytest.raises(RuntimeError, match="lora_A.weight has shape"):
        LoraAdapterWeights.from_hf_weights("d", sd, {"r": 4, "lora_alpha": 2}, NET, pin=False)
    sd = checkpoint(("c_attn",), 2, {"c_attn": 8})
    with pytest.raises(RuntimeError, match="lora_B.weight has shape"):
        LoraAdapterWeights.from_hf_weights("d", sd, {"r": 2, "lora_alpha": 2}, NET, pin=False)
