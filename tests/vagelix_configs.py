"""Small Vagelix configurations for the tests, and model folders made from them with random weights."""
import copy
import functools
import json
import os
import tempfile

import plain_vagelix as P


def attention(heads, kv_heads, dim, vdim, diff=0.5, scale=None, q_temp=(0.2, 16)):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
         "scale": scale if scale is not None else 2.0 * dim ** -0.5}
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return ("attention", m)


def parallel(left, right):
    heads, kv_heads, dim, chunk, rot_dims, base, scale = left
    a = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else 2.0 * dim ** -0.5}
    if chunk:
        a["mask"] = {"size": chunk}
    if rot_dims:
        a["rot"] = {"dims": rot_dims, "base": base}
    heads, kv_heads, dim, vdim, conv = right
    return ("parallel", {"left": a, "right": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}})


def mamba2(heads, vdim, state, groups, norm_groups, conv):
    return ("mamba2", {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv})


def config(vocab, width, layers, eps=1e-5):
    """layers: ((type, mixer), ff or None) or an int j for a layer that runs layer j's tensors."""
    out = []
    for l in layers:
        if isinstance(l, int):
            out.append(dict(copy.deepcopy(out[l]), weights_of=l))
        else:
            (t, m), ff = l
            out.append({"type": t, "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None})
    return {"architecture": "Vagelix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": out}


CONFIGS = {
    # sizes that are no multiples of 16 (the plain kernels in both precisions): three heads over one kv head, values
    # larger than keys, a chunk shorter than a page, rotation on part of the head, two taps, a layer without
    # feed-forward, the pair's tensors run a second time at the end
    "a": config(97, 72, [
        (attention(3, 1, 24, 40, diff=0.3), 48),
        (parallel((4, 2, 20, 11, 8, 500.0, None), (3, 1, 12, 20, 2)), None),
        (mamba2(3, 20, 12, 1, 3, 3), 56),
        1]),
    # sizes the matrix-core kernels take; a recurrent layer first; a chunk that spans pages of 8; rotation over the whole
    # head; the attention's tensors run three times
    "b": config(256, 128, [
        (mamba2(4, 32, 32, 2, 2, 4), 96),
        (attention(4, 2, 32, 32, diff=0.7, q_temp=(0.4, 8)), 64),
        (parallel((4, 2, 64, 40, 64, 100000.0, None), (4, 2, 32, 64, 4)), 128),
        1, 1]),
    # no mask (every earlier position is seen), no rotation, no temperature, one tap (no convolution history), one
    # norm part, as many kv heads as heads, one head
    "c": config(130, 96, [
        (parallel((2, 2, 32, 0, 0, 1.0, 0.3), (2, 2, 16, 16, 1)), 40),
        (attention(1, 1, 64, 16, diff=0.1, q_temp=None), None),
        (mamba2(1, 48, 80, 1, 1, 1), 64)]),
    # a chunk of one position (every query sees itself and the sink only), a width that is no multiple of 8, many key
    # channels in the walk, five taps
    "d": config(51, 44, [
        (parallel((2, 1, 6, 1, 2, 10.0, None), (2, 1, 136, 5, 5)), 20),
        (attention(2, 2, 6, 10, diff=0.5, q_temp=(1.0, 1)), 12),
        0]),
}


@functools.lru_cache(maxsize=None)
def tensors_of(name, seed=0):
    return P.random_model(CONFIGS[name], seed)


_dirs = {}


def write_model(cfg, tensors, prefix="vagelix_"):
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
        _dirs[key] = write_model(CONFIGS[name], tensors_of(name, seed), f"vagelix_{name}_")
    return _dirs[key]
