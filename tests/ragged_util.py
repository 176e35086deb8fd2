"""Small Pagazen configurations for the tests (none with the proportions of a real checkpoint) and
helpers that run a request through the engine in given portions."""
import torch

from micro_vllm_amd.models.pagazen import PagazenConfig, build_random_model


def mamba(heads=4, vdim=24, state=40, groups=2, conv=4, norm_groups=2):
    return {"conv": conv, "groups": groups, "heads": heads, "norm_groups": norm_groups, "state": state, "vdim": vdim}


def parallel(heads=6, kv_heads=2, dim=40, vdim=56, window=37, scale=0.2, r_heads=3, r_dim=48, r_vdim=20, rot=32,
             base=5000.0, decay=(0.9, 0.97, 0.995), left_scale=0.7, right_scale=1.3):
    return {"left": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": window}, "scale": scale,
                     "vdim": vdim},
            "left_scale": left_scale,
            "right": {"decay": list(decay), "dim": r_dim, "heads": r_heads, "rot": {"base": base, "dims": rot},
                      "vdim": r_vdim},
            "right_scale": right_scale}


def layer(kind, mixer, ff=160, weights_of=None):
    d = {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def config_a():
    """Odd sizes everywhere: parallel first, a feed-forward-less layer, two layers on borrowed weights."""
    return PagazenConfig(vocab_size=331, width=192, eps=1e-5, embed_scale=3.5, logit_softcap=12.0, layers=[
        layer("parallel", parallel()),
        layer("mamba2", mamba(), ff=None),
        layer("mamba2", mamba(), ff=None, weights_of=1),
        layer("parallel", parallel(), weights_of=0),
    ])


def config_b():
    """Values that other configurations make equal or one: a single retention head, kv_heads == heads,
    groups == heads, norm_groups == heads, two taps, rotation over the whole head, no softcap,
    wave-tile friendly widths (so the bf16 run takes the relaid-out projections)."""
    return PagazenConfig(vocab_size=256, width=128, eps=1e-6, embed_scale=1.0, logit_softcap=None, layers=[
        layer("mamba2", mamba(heads=2, vdim=64, state=16, groups=2, conv=2, norm_groups=2), ff=128),
        layer("parallel", parallel(heads=2, kv_heads=2, dim=64, vdim=64, window=5, scale=0.125, r_heads=1, r_dim=64,
                                   r_vdim=64, rot=64, base=100.0, decay=(0.5,), left_scale=1.0, right_scale=1.0), ff=128),
        layer("mamba2", mamba(heads=1, vdim=128, state=8, groups=1, conv=1, norm_groups=1), ff=None),
    ])


def random_config(seed):
    """A configuration drawn at random: layer order, borrowed weights, head counts and widths (among them the
    shapes the matrix-core attention takes and ones it does not), windows from 1 to beyond the prompt, taps
    from 1 to 5, groups, norm groups, rotation over none / part / all of a head, with and without soft cap."""
    import random
    rng = random.Random(seed)
    layers = []
    for i in range(rng.randint(2, 5)):
        own = [k for k in range(i) if "weights_of" not in layers[k]]
        if own and rng.random() < 0.3:
            j = rng.choice(own)
            layers.append(dict(layers[j], weights_of=j))
            continue
        ff = rng.choice([None, 64, 150, 256])
        if rng.random() < 0.5:
            groups = rng.choice([1, 2, 3])
            heads = groups * rng.choice([1, 2, 4])
            vdim = rng.choice([8, 20, 32, 48, 64])
            ng = rng.choice([g for g in (1, 2, heads, groups) if (heads * vdim) % g == 0])
            layers.append(layer("mamba2", mamba(heads, vdim, rng.choice([4, 6, 16, 48, 128]), groups, rng.randint(1, 5), ng), ff))
        else:
            kv = rng.choice([1, 2, 3])
            dim, vdim = rng.choice([(8, 8), (24, 40), (32, 32), (64, 64), (96, 96), (128, 64), (64, 128), (40, 56), (128, 128)])
            rh, rdim = rng.randint(1, 3), rng.choice([8, 16, 48, 64])
            layers.append(layer("parallel", parallel(
                heads=kv * rng.choice([1, 2, 4]), kv_heads=kv, dim=dim, vdim=vdim, window=rng.choice([1, 2, 17, 64, 65, 100, 300]),
                scale=rng.choice([0.1, dim ** -0.5, 0.5]), r_heads=rh, r_dim=rdim, r_vdim=rng.choice([8, 20, 32, 64]),
                rot=rng.choice([r for r in (0, 2, 8, 16, rdim) if r <= rdim]), base=rng.choice([100.0, 1e4, 1e6]),
                decay=[rng.choice([0.5, 0.9, 0.99, 0.9995]) for _ in range(rh)], left_scale=rng.choice([0.5, 1.0, 1.7]),
                right_scale=rng.choice([0.3, 1.0, 2.0])), ff))
    return PagazenConfig(vocab_size=rng.choice([97, 256, 331, 1000]), width=rng.choice([48, 100, 192, 256]), layers=layers,
                         embed_scale=rng.choice([1.0, 4.0, 16.0]), eps=rng.choice([1e-5, 1e-6]),
                         logit_softcap=rng.choice([None, 15.0, 30.0]))


def make_engine(cfg, dtype=torch.float32, seed=0, pages=24, slots=4, rows=4, step_tokens=512, max_tokens=512):
    from micro_vllm_amd.core.engine import InferenceEngine
    return InferenceEngine(model=build_random_model(cfg, seed), max_batch_size=rows, max_prefill_tokens=step_tokens,
                           n_blocks=pages, max_tokens=max_tokens, state_slots=slots, dtype=dtype)


def run_in_portions(eng, sid, tokens, portions, release=True):
    """All logits [len(tokens), vocab] of one request fed in `portions` (their sum covers the tokens)."""
    out, pos = [], 0
    for n in portions:
        n = min(n, len(tokens) - pos)
        if n <= 0:
            break
        out.append(eng.run_ragged([(sid, tokens[pos:pos + n], list(range(n)))]).double().cpu())
        pos += n
    assert pos == len(tokens)
    if release:
        eng.release(sid)
    return torch.cat(out)


def rel_err(got, want):
    return ((got.double() - want.double()).norm() / want.double().norm()).item()
