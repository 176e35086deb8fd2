"""Small Fagunex configurations for the tests (none with the proportions of a real checkpoint) and an engine
builder; the helpers that feed a request in portions are those of ragged_util."""
import torch

from micro_vllm_amd.models.fagunex import FagunexConfig, build_random_model


def hgrn2(heads=3, dim=40, vdim=24):
    return {"heads": heads, "dim": dim, "vdim": vdim}


def latent(kind, heads=3, dim=24, rot_dim=16, vdim=40, kv_rank=72, rot=16, base=5000.0, scale=0.2, window=37, q_rank=56):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "rot": {"base": base, "dims": rot}, "scale": scale}
    if kind == 1:
        m.update({"mask": {"size": window}, "q_rank": q_rank})
    return m


def moe(experts=5, top=2, ff=48, shared=72):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
            "shared": {"ff": shared} if shared else None}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config_a():
    """Odd sizes everywhere: attention first, a looped span of three layers run three times, a layer without
    feed-forward, one without shared expert, rotation over a part of the rotated dimensions."""
    return FagunexConfig(vocab_size=331, width=192, eps=1e-5, side_dim=20, loop={"start": 1, "stop": 4, "times": 3}, layers=[
        layer("latent_attention", latent(1), moe()),
        layer("hgrn2", hgrn2(), moe(experts=7, top=3, ff=40, shared=None)),
        layer("latent_attention_2", latent(2, heads=5, dim=16, rot_dim=8, vdim=16, kv_rank=136, rot=4, base=300.0, scale=0.3), None),
        layer("latent_attention", latent(1, heads=2, dim=40, rot_dim=24, vdim=24, kv_rank=40, rot=24, window=5, q_rank=30), moe()),
        layer("hgrn2", hgrn2(heads=1, dim=100, vdim=60), moe(experts=3, top=3, ff=64, shared=16)),
    ])


def config_b():
    """Values that other configurations keep apart made equal or one: one head, one expert of which one is
    used, a window of exactly one page, no loop, no token side input, no rotated part in one layer; widths the
    wave-tile projections take (so the bf16 run uses the relaid-out weights)."""
    return FagunexConfig(vocab_size=256, width=128, eps=1e-6, side_dim=0, loop=None, layers=[
        layer("hgrn2", hgrn2(heads=2, dim=64, vdim=64), moe(experts=1, top=1, ff=64, shared=64)),
        layer("latent_attention", latent(1, heads=1, dim=64, rot_dim=64, vdim=64, kv_rank=64, rot=64, base=100.0,
                                         scale=0.125, window=64, q_rank=64), moe(experts=4, top=1, ff=128, shared=None)),
        layer("latent_attention_2", latent(2, heads=2, dim=64, rot_dim=0, vdim=64, kv_rank=128, rot=0, scale=0.125), None),
    ])


def random_config(seed):
    """A configuration drawn at random: layer order, loop, head counts and widths, windows from 1 to beyond the
    prompt, rotation over none / part / all of the rotated dimensions, experts and how many are used, with and
    without shared expert, feed-forward and token side input."""
    import random
    rng = random.Random(seed)
    layers = []
    for _ in range(rng.randint(2, 5)):
        mlp = None
        if rng.random() < 0.8:
            E = rng.choice([1, 2, 4, 9, 20])
            mlp = moe(E, rng.randint(1, min(E, 4)), rng.choice([16, 40, 64, 96]), rng.choice([None, 24, 64]))
        kind = rng.choice(["hgrn2", "latent_attention", "latent_attention_2"])
        if kind == "hgrn2":
            layers.append(layer(kind, hgrn2(rng.randint(1, 4), rng.choice([8, 24, 32, 64, 80]), rng.choice([8, 20, 32, 64])), mlp))
        else:
            r = rng.choice([0, 8, 16, 32])
            layers.append(layer(kind, latent(
                1 if kind == "latent_attention" else 2, heads=rng.randint(1, 6), dim=rng.choice([8, 24, 32, 64]), rot_dim=r,
                vdim=rng.choice([8, 24, 32, 64]), kv_rank=rng.choice([16, 40, 64, 136, 264]),
                rot=rng.choice([x for x in (0, 4, 8, r) if x <= r]), base=rng.choice([100.0, 1e4, 1e6]),
                scale=rng.choice([0.1, 0.2, 0.5]), window=rng.choice([1, 2, 17, 64, 65, 100, 300]),
                q_rank=rng.choice([8, 30, 64])), mlp))
    n = len(layers)
    loop = None
    if rng.random() < 0.6:
        a = rng.randint(0, n - 1)
        loop = {"start": a, "stop": rng.randint(a, n), "times": rng.randint(1, 3)}
    return FagunexConfig(vocab_size=rng.choice([97, 256, 331, 1000]), width=rng.choice([48, 100, 192, 256]), layers=layers,
                         eps=rng.choice([1e-5, 1e-6]), loop=loop, side_dim=rng.choice([0, 8, 20]))


def make_engine(cfg, dtype=torch.float32, seed=0, pages=24, slots=4, rows=4, step_tokens=512, max_tokens=512):
    from micro_vllm_amd.core.engine import InferenceEngine
    return InferenceEngine(model=build_random_model(cfg, seed), max_batch_size=rows, max_prefill_tokens=step_tokens,
                           n_blocks=pages, max_tokens=max_tokens, state_slots=slots, dtype=dtype)
