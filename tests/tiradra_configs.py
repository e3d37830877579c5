"""Small Tiradra configurations that differ from each other in every size, constant and option."""
import torch


def _rot(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def _attn(heads, kv_heads, dim, vdim, scale, conv, rot, ff=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if conv:
        m["conv"] = conv
    return {"type": "attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _latent(heads, dim, rot_dim, vdim, kv_rank, scale, rot, ff=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale, "rot": rot}
    return {"type": "latent_attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


TIRADRA = {
    # values smaller and larger than queries and keys; as many kv heads as heads; rotations over part of a head, with
    # and without stretched frequencies; 2 and 3 taps; a layer without a feed-forward; a loop of three passes in the
    # middle; a hash whose products pass 32 bits
    "TA": {
        "seed": 3, "architecture": "Tiradra", "vocab": 300, "width": 64, "norm": {"eps": 1e-5},
        "embedding": {"bigram": {"buckets": 97, "mul_prev": 200000003, "mul_cur": 129970921}},
        "loop": {"start": 1, "stop": 3, "times": 3}, "logit_softcap": 6.0,
        "layers": [
            _attn(4, 2, 16, 8, 0.3, 3, _rot(1000.0, 8, (4.0, 64, 8.0, 2.0)), ff=96),
            _latent(3, 16, 8, 12, 32, 0.25, _rot(100.0, 8, (3.0, 40, 4.0, 1.0)), ff=40),
            _attn(2, 2, 8, 24, 0.5, 2, _rot(50.0, 8)),
            _latent(1, 8, 4, 24, 16, 0.4, _rot(10000.0, 4), ff=64),
        ],
    },
    # sizes that fit no fast path (a width that is no multiple of 4, heads of 6 and 10 elements, a latent of 18, a
    # prime vocabulary) and things that are absent: no pair table, no loop, no cap, a layer without convolution, one
    # tap; one kv head; five taps (longer than the shortest portions)
    "TB": {
        "seed": 5, "architecture": "Tiradra", "vocab": 257, "width": 54, "norm": {"eps": 1e-3},
        "layers": [
            _attn(3, 1, 6, 6, 0.6, 5, _rot(30.0, 6, (2.5, 32, 6.0, 0.5)), ff=28),
            _latent(5, 4, 2, 6, 18, 0.6, _rot(50.0, 2), ff=30),
            _attn(2, 1, 10, 4, 0.4, 0, _rot(70.0, 4, (8.0, 16, 2.0, 1.0)), ff=54),
            _attn(1, 1, 8, 8, 0.35, 1, _rot(20.0, 8), ff=20),
        ],
    },
    # the loop from the first layer to the last, twice; one pass only would be "times": 1 (TD)
    "TC": {
        "seed": 7, "architecture": "Tiradra", "vocab": 128, "width": 32, "norm": {"eps": 1e-6},
        "embedding": {"bigram": {"buckets": 1, "mul_prev": 1, "mul_cur": 1}},
        "loop": {"start": 0, "stop": 2, "times": 2}, "logit_softcap": 30.0,
        "layers": [
            _latent(2, 8, 8, 8, 16, 0.3, _rot(1000.0, 8, (2.0, 48, 16.0, 1.0)), ff=48),
            _attn(2, 1, 8, 8, 0.4, 4, _rot(1000.0, 8, (2.0, 48, 16.0, 1.0)), ff=48),
        ],
    },
    # a loop of one pass that ends with the model's last layer
    "TD": {
        "seed": 11, "architecture": "Tiradra", "vocab": 90, "width": 40, "norm": {"eps": 1e-4},
        "embedding": {"bigram": {"buckets": 50, "mul_prev": 3, "mul_cur": 5}},
        "loop": {"start": 1, "stop": 2, "times": 1},
        "layers": [
            _attn(2, 2, 12, 12, 0.3, 2, _rot(500.0, 12), ff=32),
            _latent(2, 8, 6, 10, 12, 0.3, _rot(500.0, 6, (5.0, 20, 3.0, 1.0)), ff=32),
        ],
    },
    # sharp scores: a key just where a page ends, or hundreds of tokens back, carries most of a query's weight
    "TS": {
        "seed": 13, "architecture": "Tiradra", "vocab": 128, "width": 32, "norm": {"eps": 1e-5},
        "embedding": {"bigram": {"buckets": 31, "mul_prev": 5, "mul_cur": 3}},
        "layers": [
            _attn(2, 1, 16, 16, 1.5, 2, _rot(10000.0, 16, (2.0, 64, 8.0, 1.0)), ff=48),
            _latent(2, 8, 8, 8, 16, 1.5, _rot(10000.0, 8), ff=48),
        ],
    },
}

# with the sizes the vector and matrix-core paths need (GPU tests)
TIRADRA_FAST = {
    "TF": {
        "seed": 9, "architecture": "Tiradra", "vocab": 1000, "width": 256, "norm": {"eps": 1e-5},
        "embedding": {"bigram": {"buckets": 509, "mul_prev": 11, "mul_cur": 7}},
        "loop": {"start": 1, "stop": 3, "times": 2}, "logit_softcap": 25.0,
        "layers": [
            _latent(8, 32, 16, 32, 128, 0.15, _rot(500000.0, 16, (4.0, 128, 32.0, 1.0)), ff=512),
            _attn(8, 2, 64, 64, 0.125, 4, _rot(10000.0, 64, (2.0, 256, 32.0, 1.0)), ff=384),
            _attn(4, 4, 128, 128, 0.1, 3, _rot(10000.0, 32), ff=512),
            _latent(4, 64, 32, 64, 64, 0.1, _rot(10000.0, 32), ff=512),
        ],
    },
    # values half and twice the size of the keys at matrix-core head sizes (pages of 128 and 64), a latent that fills
    # no whole chunk (96 wide, 24 rotated), 20 heads (a tile of 16 rows runs over two tokens), 5 heads
    "TG": {
        "seed": 15, "architecture": "Tiradra", "vocab": 777, "width": 160, "norm": {"eps": 1e-6},
        "embedding": {"bigram": {"buckets": 1019, "mul_prev": 29, "mul_cur": 19}},
        "loop": {"start": 0, "stop": 2, "times": 2}, "logit_softcap": 12.0,
        "layers": [
            _attn(6, 3, 128, 64, 0.09, 4, _rot(30000.0, 64, (3.0, 100, 16.0, 1.0)), ff=288),
            _latent(20, 16, 24, 8, 96, 0.2, _rot(30000.0, 24, (2.0, 100, 16.0, 1.0)), ff=200),
            _attn(4, 1, 32, 64, 0.17, 2, _rot(777.0, 32), ff=64),
            _latent(5, 40, 24, 24, 96, 0.18, _rot(777.0, 24)),
        ],
    },
}


def tiradra_config_json(name: str) -> dict:
    return {k: v for k, v in {**TIRADRA, **TIRADRA_FAST}[name].items() if k != "seed"}


def write_tiradra(name: str, out_dir: str, dtype=torch.float32) -> str:
    from jax_llm_examples_amd.config import get_architecture
    from jax_llm_examples_amd.weights import write_random_model

    top = tiradra_config_json(name)
    arch = get_architecture(top["architecture"])
    return write_random_model(arch, arch.parse_config(top), out_dir, {**TIRADRA, **TIRADRA_FAST}[name]["seed"], dtype)
