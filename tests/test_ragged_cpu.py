"""Host-side parts of the ragged family (no GPU): configuration reader, tensor table, registry and
checkpoint loading, page / slot bookkeeping and step layout, the scheduler's mixed steps, and the plain
restatement's own consistency (a recurrence continued from its state equals the whole run)."""
import json
import os

import pytest
import torch

from oracle import ref_hybrid as ref
from ragged_util import config_a, config_b


def test_config_reader_and_tensor_table(mv):
    from micro_vllm_amd.models.pagazen import PagazenConfig, mamba2_sizes, tensor_shapes
    cfg = config_a()
    again = PagazenConfig.from_json(json.loads(json.dumps(cfg.to_json())))
    assert again.vocab_size == 331 and again.width == 192 and again.embed_scale == 3.5 and again.logit_softcap == 12.0
    assert [again.weights_layer(i) for i in range(4)] == [0, 1, 1, 0]
    shapes = tensor_shapes(again)
    s = mamba2_sizes(cfg.layers[1]["mixer"])
    assert shapes["l1.mix.in"] == (2 * s["inner"] + 2 * s["groups"] * s["n"] + s["heads"], 192)
    assert shapes["l1.mix.conv"] == (s["inner"] + 2 * s["groups"] * s["n"], 4)
    assert "l1.norm2" not in shapes and "l2.norm1" not in shapes and "l3.mix.left.q" not in shapes
    assert shapes["l0.mix.left.k"] == (2 * 40, 192) and shapes["l0.mix.right.g"] == (3 * 20, 192)
    no_cap = PagazenConfig.from_json({k: v for k, v in config_b().to_json().items()})
    assert no_cap.logit_softcap is None
    bad = cfg.to_json()
    bad["layers"] = [dict(bad["layers"][0], type="conv")]
    with pytest.raises(ValueError):
        PagazenConfig.from_json(bad)
    bad = cfg.to_json()
    bad["layers"] = [dict(l) for l in bad["layers"]]
    bad["layers"][3]["weights_of"] = 2          # layer 2 borrows its own
    with pytest.raises(ValueError):
        PagazenConfig.from_json(bad)


def test_registry_loads_a_checkpoint_directory(mv, tmp_path):
    from safetensors.torch import save_file
    from micro_vllm_amd.core.model_loader import load_model
    from micro_vllm_amd.models.pagazen import random_weights
    cfg = config_a()
    w = random_weights(cfg, 1)
    save_file(w, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_json()))
    model, tok = load_model(str(tmp_path))
    assert model.family == "ragged" and model.config.width == 192
    assert torch.equal(model.get("l1.mix.A_log"), w["l1.mix.A_log"]) and model.get("embed").dtype == torch.bfloat16
    assert tok.encode("3 17 330") == [3, 17, 330] and tok.decode([5, 6]) == "5 6"
    with pytest.raises(ValueError):
        tok.encode("331")
    os.remove(tmp_path / "model.safetensors")
    del w["l0.mix.right.g"]
    save_file(w, str(tmp_path / "model.safetensors"))
    with pytest.raises(KeyError):
        load_model(str(tmp_path))


def test_pages_slots_and_step_layout(mv):
    from micro_vllm_amd.core.state_cache import HybridCacheManager, PoolExhausted
    c = HybridCacheManager(5, 64, 2, {0: (2, 8, 4)}, {1: {"s": (3, 4, 2)}}, dtype=torch.float32, device="cpu",
                           max_tokens=256, max_rows=3, max_step_tokens=300)
    assert c.k_caches[0].shape == (5, 64, 2, 8) and c.v_caches[0].shape == (5, 64, 2, 4) and c.states[1]["s"].shape == (2, 3, 4, 2)
    c.reserve([("a", 70), ("b", 1)])
    st = c.plan([("a", list(range(70))), ("b", [9])])
    c.advance([("a", 70), ("b", 1)])
    assert st.tokens == 71 and st.rows == 2
    assert st.tok_row.tolist() == [0] * 70 + [1] and st.tok_pos.tolist() == list(range(70)) + [0]
    assert st.row_start.tolist() == [0, 70] and st.row_len.tolist() == [70, 1] and st.row_ctx.tolist() == [0, 0]
    assert sorted(st.row_slot.tolist()) == [0, 1]
    assert st.block_table[0, :2].tolist() == c.get_blocks("a") and st.block_table[0, 2].item() == -1
    assert c.stats["free"] == 2
    # the long row is cut into chunks of 64 for the chunked recurrence, the short one is not
    assert st.n_chunks == 2 and st.ch_start.tolist() == [0, 64] and st.ch_len.tolist() == [64, 6]
    assert st.row_ch0.tolist() == [0, 2] and st.row_nch.tolist() == [2, 0]
    c.reserve([("a", 58)])                       # fills its second page exactly: no new page
    assert c.stats["free"] == 2
    st = c.plan([("a", [1] * 58)])
    c.advance([("a", 58)])
    assert st.tok_pos.tolist() == list(range(70, 128)) and st.row_ctx.tolist() == [70]
    c.reserve([("a", 1)])                        # position 128 opens the third
    assert c.stats["free"] == 1
    with pytest.raises(PoolExhausted):
        c.reserve([("c", 1)])                    # no slot
    with pytest.raises(PoolExhausted):
        c.reserve([("b", 64 * 2)])               # b would need two more pages, one is free: nothing is taken
    assert c.stats["free"] == 1 and c.length("b") == 1
    first = c.get_blocks("a")[0]
    c.free("a")
    assert c.stats["free"] == 4 and c.stats["slots_free"] == 1
    c.reserve([("c", 200)])
    assert first in c.get_blocks("c") and c.slot_of("c") is not None    # used again
    c.advance([("c", 200)])
    with pytest.raises(ValueError):
        c.reserve([("c", 100)])                  # past what a block-table row describes
    c.reset()
    assert c.stats == {"total": 5, "free": 5, "used": 0, "slots_free": 2}


class _Tok:
    eos_token_id = None

    def encode(self, text, add_special_tokens=True):
        return [int(t) for t in text.split()]


def test_scheduler_mixed_steps(mv):
    from micro_vllm_amd.core.scheduler import Scheduler
    from micro_vllm_amd.core.sequence import Sequence
    refused = set()
    sch = Scheduler(max_batch_size=3, max_prefill_tokens=10, tokenizer=_Tok(), ragged=True,
                    reserve=lambda seq, n: seq.seq_id not in refused)
    seqs = [Sequence(i, " ".join(["1"] * n), _Tok(), max_tokens=3) for i, n in enumerate((4, 13, 2, 5))]
    for s in seqs:
        sch.add_request(s)

    def run(batch):
        for s in batch:
            s.num_computed += s._portion
            if s.num_computed == len(s.full_ids):
                s.update_state(7)

    batch, kind = sch.get_next_batch()
    assert kind == "mixed" and [(s.seq_id, s._portion) for s in batch] == [(0, 4), (1, 6)]     # budget 10, nothing padded
    run(batch)
    refused.add(2)
    batch, _ = sch.get_next_batch()
    # decode first, then the prompt under way; 2 has to wait and 3 does not overtake it
    assert [(s.seq_id, s._portion) for s in batch] == [(0, 1), (1, 7)]
    run(batch)
    refused.clear()
    batch, _ = sch.get_next_batch()
    assert [(s.seq_id, s._portion) for s in batch] == [(0, 1), (1, 1), (2, 2)]      # three rows at most
    run(batch)
    assert seqs[0].is_finished()
    batch, _ = sch.get_next_batch()
    assert [(s.seq_id, s._portion) for s in batch] == [(1, 1), (2, 1), (3, 5)]
    assert all(len(s.input_ids) == n for s, n in zip(seqs, (4, 13, 2, 5)))


def test_restatement_continues_from_its_state():
    g = torch.Generator().manual_seed(0)
    T, H, n, p = 12, 2, 5, 3
    q, k, v = (torch.randn(T, H, d, generator=g, dtype=torch.float64) for d in (n, n, p))
    decay, gain = torch.rand(T, H, generator=g, dtype=torch.float64), torch.rand(T, H, generator=g, dtype=torch.float64)
    whole, S = ref.decayed_outer_product_scan(q, k, v, decay, gain)
    a, Sa = ref.decayed_outer_product_scan(q[:5], k[:5], v[:5], decay[:5], gain[:5])
    b, Sb = ref.decayed_outer_product_scan(q[5:], k[5:], v[5:], decay[5:], gain[5:], state=Sa)
    assert torch.allclose(torch.cat([a, b]), whole) and torch.allclose(Sb, S)
    # closed form of one output: o_t = sum_s (prod_{s<r<=t} decay_r) gain_s (q_t . k_s) v_s
    t, h = 7, 1
    acc = torch.zeros(p, dtype=torch.float64)
    for s in range(t + 1):
        acc += decay[s + 1:t + 1, h].prod() * gain[s, h] * (q[t, h] @ k[s, h]) * v[s, h]
    assert torch.allclose(whole[t, h], acc)


def test_part_library_holds_every_entry_point_the_family_calls(mv):
    """The library of a part of the sources (what a first start in a fresh checkout builds) exports every
    C entry point that the ragged family's wrappers, projections, sampler and graph capture name."""
    import ctypes
    import importlib.util
    import inspect
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("mvllm_build", os.path.join(root, "micro-vllm_amd", "build.py"))
    b = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(b)
    lib = b.build(verbose=False, only="ragged")
    handle = ctypes.CDLL(lib)
    from micro_vllm_amd.core.layer import model_graph, ragged_runner, sampler
    from micro_vllm_amd.kernel import linear, ragged_ops
    text = inspect.getsource(ragged_ops) + inspect.getsource(ragged_runner)
    for fn in (linear.StreamedWeight.from_linear, linear.wgemm, linear.gemm_prefill, linear.gemm_workspace,
               sampler.greedy, sampler.sample, model_graph.HipGraph):
        text += inspect.getsource(fn)
    names = {n for n in re.findall(r"\bmv_[a-z0-9_]+", text) if not n.endswith("_")} | {"mv_status_string", "mv_last_hip_error", "mv_version"}
    assert {"mv_shuffle_weight", "mv_scan_chunked", "mv_graph_launch", "mv_wgemm"} <= names
    missing = sorted(n for n in names if not hasattr(handle, n))
    assert not missing, missing
