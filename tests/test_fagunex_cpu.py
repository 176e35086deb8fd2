"""Host-side parts of the Fagunex design (no GPU): configuration reader (layer list, loop, optional parts),
tensor table, registry and checkpoint loading, and the plain restatement's own consistency (a recurrence or
a token shift continued from its state equals the whole run; attention over a latent equals attention over the
keys and values it stands for)."""
import json
import os

import pytest
import torch

from oracle import ref_fagunex as ref
from fagunex_util import config_a, config_b, random_config


def test_config_reader_loop_and_tensor_table(mv):
    from micro_vllm_amd.models.fagunex import FagunexConfig, tensor_shapes
    cfg = config_a()
    again = FagunexConfig.from_json(json.loads(json.dumps(cfg.to_json())))
    assert again.vocab_size == 331 and again.width == 192 and again.side_dim == 20 and again.eps == 1e-5
    assert again.runs == [0, 1, 2, 3, 1, 2, 3, 1, 2, 3, 4] and again.num_hidden_layers == 11
    assert [i for i, _ in again.layer_runs()] == again.runs == ref.layer_runs(cfg.to_json())
    shapes = tensor_shapes(again)
    assert shapes["side.embed"] == (331, 5 * 20) and shapes["l0.norm1.alpha"] == () and shapes["l3.side.proj"] == (192, 20)
    assert shapes["l0.mix.dq"] == (56, 192) and shapes["l0.mix.uq"] == (3 * (24 + 16), 56) and shapes["l0.mix.sink"] == (3,)
    assert shapes["l0.mix.dkv"] == (72 + 16, 192) and shapes["l0.mix.uk"] == (3 * 24, 72) and shapes["l0.mix.g"] == (3 * 40, 192)
    assert shapes["l2.mix.q"] == (5 * (16 + 8), 192) and "l2.mix.sink" not in shapes and "l2.mix.g" not in shapes
    assert "l2.norm2" not in shapes and "l2.mlp.router" not in shapes                 # no feed-forward there
    assert shapes["l1.mix.f.b"] == (3 * 40,) and shapes["l1.mix.norm"] == (24,) and shapes["l1.mlp.e6.down"] == (192, 40)
    assert "l1.mlp.shared.sg" not in shapes and shapes["l4.mlp.shared.sg"] == (1, 192)
    plain = FagunexConfig.from_json(config_b().to_json())
    assert plain.loop is None and plain.side_dim == 0 and plain.runs == [0, 1, 2]
    assert "side.embed" not in tensor_shapes(plain) and "l0.side.gate" not in tensor_shapes(plain)
    for spoil in (lambda d: d["layers"][0].update(type="conv"), lambda d: d["layers"][0]["mlp"].update(kind="dense"),
                  lambda d: d["loop"].update(stop=9), lambda d: d["layers"][0]["mixer"]["rot"].update(dims=18)):
        bad = json.loads(json.dumps(cfg.to_json()))
        spoil(bad)
        with pytest.raises(ValueError):
            FagunexConfig.from_json(bad)
    for seed in range(20):
        c = random_config(seed)
        assert FagunexConfig.from_json(c.to_json()).runs == ref.layer_runs(c.to_json())


def test_registry_loads_a_checkpoint_directory(mv, tmp_path):
    from safetensors.torch import save_file
    from micro_vllm_amd.core.model_loader import load_model
    from micro_vllm_amd.models.fagunex import random_weights
    cfg = config_a()
    w = random_weights(cfg, 1)
    save_file(w, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_json()))
    model, tok = load_model(str(tmp_path))
    assert model.family == "ragged" and model.config.architecture == "Fagunex" and model.config.width == 192
    assert torch.equal(model.get("l1.mix.lower"), w["l1.mix.lower"]) and model.get("embed").dtype == torch.bfloat16
    assert tok.encode("3 17 330") == [3, 17, 330]
    os.remove(tmp_path / "model.safetensors")
    del w["l0.mix.sink"]
    save_file(w, str(tmp_path / "model.safetensors"))
    with pytest.raises(KeyError):
        load_model(str(tmp_path))


def test_cache_layout_follows_the_layer_runs(mv):
    """Every run of a looped layer has pages or state of its own; attention runs keep one latent per token and
    no separate values."""
    from micro_vllm_amd.core.layer.ragged_runner import RaggedRunner
    cfg = config_a()
    runner = RaggedRunner.__new__(RaggedRunner)
    runner.cfg, runner.width, runner.runs = cfg, cfg.width, cfg.layer_runs()
    kv, state = runner.cache_layout()
    assert sorted(kv) == [0, 2, 3, 5, 6, 8, 9] and sorted(state) == list(range(11))
    assert kv[0] == (1, 72 + 16, 0) and kv[2] == kv[5] == kv[8] == (1, 136 + 8, 0)
    assert state[1] == state[4] == {"shift": (192,), "gated": (3, 40, 24)} and state[2] == {"shift": (192,)}


def test_restatement_recurrence_and_shift_continue_from_their_state():
    g = torch.Generator().manual_seed(0)
    T, H, n, p = 30, 2, 5, 7
    q, v = torch.randn(T, H, n, generator=g, dtype=torch.float64), torch.randn(T, H, p, generator=g, dtype=torch.float64)
    f = torch.rand(T, H, n, generator=g, dtype=torch.float64)
    whole, S = ref.gated_write_recurrence(q, f, v)
    a, Sa = ref.gated_write_recurrence(q[:11], f[:11], v[:11])
    b, Sb = ref.gated_write_recurrence(q[11:], f[11:], v[11:], Sa)
    assert torch.allclose(torch.cat([a, b]), whole) and torch.allclose(Sb, S)
    # a gate of one keeps the state, a gate of zero replaces every row by the value
    o, S1 = ref.gated_write_recurrence(q[:1], torch.zeros(1, H, n, dtype=torch.float64), v[:1])
    assert torch.allclose(S1, v[0][:, None, :].expand(H, n, p))
    h, mix = torch.randn(9, 6, generator=g, dtype=torch.float64), torch.rand(6, generator=g, dtype=torch.float64)
    whole = ref.token_shift(h, mix)
    assert torch.allclose(torch.cat([ref.token_shift(h[:4], mix), ref.token_shift(h[4:], mix, h[3])]), whole)
    assert torch.allclose(whole[0], h[0] * (1 - mix))


def test_restatement_rotations_and_sink():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 3, 12, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 7, 100, 1000])
    for rotate in (ref.rotate_interleaved, ref.rotate_halves):
        y = rotate(x, pos, 8, 1e4)
        assert torch.allclose(y[0], x[0]) and torch.allclose(y[..., 8:], x[..., 8:])
        assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1))
        # a rotation: scores depend on the distance only
        a, b = rotate(x[:1].expand(5, 3, 12), pos, 8, 1e4), rotate(x[1:2].expand(5, 3, 12), pos + 3, 8, 1e4)
        d = (a * b).sum(-1)
        assert torch.allclose(d, d[:1].expand_as(d))
    # interleaved and halved layouts are a permutation of each other
    perm = [0, 2, 4, 6, 1, 3, 5, 7]
    assert torch.allclose(ref.rotate_interleaved(x, pos, 8, 1e4)[..., perm], ref.rotate_halves(x[..., perm + [8, 9, 10, 11]], pos, 8, 1e4)[..., :8])
    q, k, v = (torch.randn(6, 2, 4, generator=g, dtype=torch.float64) for _ in range(3))
    plain = ref.masked_softmax_attention(q, k, v, 0.5, 3)
    sunk = ref.masked_softmax_attention(q, k, v, 0.5, 3, torch.tensor([-1e9, 0.0], dtype=torch.float64))
    assert torch.allclose(sunk[:, 0], plain[:, 0]) and bool((sunk[:, 1].abs() < plain[:, 1].abs() + 1e-12).all())
    assert torch.allclose(plain[0], v[0])                       # the first token sees itself only
    one = ref.masked_softmax_attention(q, k, v, 0.5, 1)
    assert torch.allclose(one, v)                               # a window of one token
