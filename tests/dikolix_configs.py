"""Small Dikolix configurations for the tests, and model folders made from them with random weights."""
import functools
import json
import os
import tempfile

import plain_dikolix as P

YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale=None, base=10000.0, scaling=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale if scale is not None else 0.9 * (dim + rot_dim) ** -0.5, "rot": {"dims": rot_dim, "base": base}}
    if scaling is not None:
        m["rot"]["scaling"] = dict(scaling)
    return ("latent_attention", m)


def ssm(inner, state, conv, dt_rank):
    return ("mamba1", {"inner": inner, "state": state, "conv": conv, "dt_rank": dt_rank})


def retention(heads, dim, vdim, decay, rot_dims=None, base=10000.0):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
    return ("retention", m)


def moe(experts, top, ff, shared=None):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        f["shared"] = {"ff": shared}
    return f


def config(vocab, width, layers, eps=1e-5, mult=None, bigram=None, loop=None):
    c = {"architecture": "Dikolix", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "layers": [{"type": t, "mixer": m, "mlp": f} for (t, m), f in layers]}
    if mult is not None:
        c["residual_mult"] = mult
    if bigram is not None:
        c["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))}
    if loop is not None:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


CONFIGS = {
    # sizes that are no multiples of 16 (the plain kernels in both precisions): an odd width's neighbour, three heads,
    # a latent that differs from the queries' latent, scaled frequencies, a state of 12 elements with 3 taps, a loop of
    # the last two layers run three times, a layer without feed-forward, every expert chosen in one layer
    "a": config(97, 72, [
        (latent(3, 24, 8, 20, 40, 56, scaling=YARN), moe(5, 2, 32, shared=48)),
        (ssm(100, 12, 3, 5), None),
        (retention(2, 24, 40, [0.9, 0.996], rot_dims=16), moe(3, 3, 24))], mult=0.6, bigram=(53, 7, 3), loop=(1, 3, 3)),
    # sizes the matrix-core kernels take: the loop in the middle run twice, a recurrent layer first, retention without
    # rotation on part of the head, a shared expert, pages of 8
    "b": config(256, 128, [
        (retention(4, 64, 64, [0.97, 0.99, 0.999, 1.0], rot_dims=32, base=500000.0), moe(6, 3, 64, shared=64)),
        (latent(4, 32, 32, 32, 64, 96, base=250000.0, scaling={"factor": 8.0, "original": 32, "fast": 4.0, "slow": 0.5}), moe(8, 2, 32)),
        (ssm(256, 16, 4, 8), moe(4, 1, 64, shared=32)),
        (latent(8, 16, 16, 48, 96, 48, scale=0.2), moe(6, 3, 64, shared=64))], eps=1e-6, mult=0.8, bigram=(251, 29, 13), loop=(1, 3, 2)),
    # no pair table, no loop, no multiplier, one head, a state wider than a wave (two elements a lane), two taps,
    # retention without rotation, one expert a token
    "c": config(130, 96, [
        (ssm(160, 80, 2, 7), moe(3, 1, 40)),
        (latent(1, 64, 32, 16, 24, 64, scale=0.11, base=100.0), moe(8, 4, 24, shared=16)),
        (retention(3, 16, 8, [0.5, 0.9375, 0.99]), moe(2, 1, 16, shared=8))]),
    # a loop that starts at the first layer and covers all layers, run twice; one bucket; a width that is no multiple of 8;
    # one tap (no history); the rotated part larger than the unrotated one
    "d": config(51, 44, [
        (latent(2, 6, 10, 12, 20, 28, scale=0.3, base=200.0, scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}), moe(2, 1, 20, shared=12)),
        (ssm(36, 5, 1, 3), moe(4, 2, 12))], eps=1e-6, mult=1.3, bigram=(1, 5, 9), loop=(0, 2, 2)),
}


@functools.lru_cache(maxsize=None)
def tensors_of(name, seed=0):
    return P.random_model(CONFIGS[name], seed)


_dirs = {}


def write_model(cfg, tensors, prefix="dikolix_"):
    from pico_vllm_amd.weights.safetensors_io import write_safetensors
    d = tempfile.mkdtemp(prefix=prefix)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(d, "model.safetensors"), [(n, tuple(v.shape), v.dtype) for n, v in tensors.items()],
                      lambda n: tensors[n])
    return d


def model_dir(name, seed=0):
    """A folder with config.json and model.safetensors of configuration ``name``; made once a process."""
    key = (name, seed)
    if key not in _dirs:
        _dirs[key] = write_model(CONFIGS[name], tensors_of(name, seed), f"dikolix_{name}_")
    return _dirs[key]
