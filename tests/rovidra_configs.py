"""Small Rovidra configurations that differ from each other in every size, constant and option."""
import torch


def _mixer(heads, dim, rot_dim, vdim, kv_rank, scale, base, dims=None, mask=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if mask is not None:
        m["mask"] = {"size": mask}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _layer(mixer, ff=None):
    return {"type": "latent_attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


ROVIDRA = {
    # readers of another layer's latent with other head counts and sizes; a reader whose window is shorter than its
    # writer's and one whose window is longer; a layer without a window (and a reader of it with one); fewer turning
    # elements than the rotated part has; layers without a feed-forward
    "RA": {
        "seed": 3, "architecture": "Rovidra", "vocab": 300, "width": 64, "embedding": {"scale": 3.5},
        "norm": {"eps": 1e-4},
        "layers": [
            _layer(_mixer(3, 16, 8, 12, 32, 0.3, 10000.0, mask=20), ff=96),
            _layer(_mixer(2, 24, 8, 16, 32, 0.25, 10000.0, mask=9, kv_from=0)),
            _layer(_mixer(4, 8, 8, 8, 16, 0.4, 100.0, dims=4), ff=40),
            _layer(_mixer(1, 8, 8, 24, 16, 0.5, 100.0, dims=4, mask=37, kv_from=2), ff=64),
            _layer(_mixer(2, 16, 16, 16, 24, 0.2, 5000.0, dims=8, mask=33)),
            _layer(_mixer(5, 8, 16, 4, 24, 0.35, 5000.0, dims=8, mask=50, kv_from=4), ff=48),
        ],
    },
    # sizes that fit no fast path: a width that is no multiple of 4, a latent that is no multiple of 4 or 8, a prime
    # vocabulary; values that happen to be 1 or equal: one head, equal sizes, a window of one token (a token sees only
    # itself), a window of exactly a page, and of a page and one
    "RB": {
        "seed": 5, "architecture": "Rovidra", "vocab": 257, "width": 54, "embedding": {"scale": 1.0},
        "norm": {"eps": 1e-3},
        "layers": [
            _layer(_mixer(1, 8, 8, 8, 18, 0.5, 50.0, mask=1), ff=28),
            _layer(_mixer(5, 4, 2, 6, 18, 0.6, 50.0, mask=16), ff=30),
            _layer(_mixer(2, 6, 2, 10, 18, 0.7, 50.0, mask=17, kv_from=1), ff=54),
        ],
    },
    # one layer with sharp scores (a large scale): a key just inside or just outside the window shows
    "RS": {
        "seed": 7, "architecture": "Rovidra", "vocab": 128, "width": 32, "embedding": {"scale": 5.0},
        "norm": {"eps": 1e-5},
        "layers": [_layer(_mixer(2, 8, 4, 8, 16, 2.5, 1000.0, mask=24), ff=48)],
    },
}

# with the sizes the vector paths need (GPU tests): widths that are multiples of 8, a latent of 128
ROVIDRA_FAST = {
    "RF": {
        "seed": 9, "architecture": "Rovidra", "vocab": 1000, "width": 256, "embedding": {"scale": 16.0},
        "norm": {"eps": 1e-5},
        "layers": [
            _layer(_mixer(8, 32, 16, 32, 128, 0.15, 500000.0, mask=100), ff=512),
            _layer(_mixer(8, 32, 16, 32, 128, 0.15, 500000.0, mask=70, kv_from=0), ff=384),
            _layer(_mixer(4, 64, 32, 64, 64, 0.1, 10000.0, mask=300), ff=512),
        ],
    },
    # latents and rotated parts that fill no whole chunk of the matrix-core kernels (96 and 160 wide, 24 and 40
    # rotated elements), 20 heads (a tile of 16 rows runs over two tokens), 6 heads, a window of one token
    "RG": {
        "seed": 13, "architecture": "Rovidra", "vocab": 777, "width": 192, "embedding": {"scale": 9.0},
        "norm": {"eps": 1e-6},
        "layers": [
            _layer(_mixer(20, 16, 24, 8, 96, 0.2, 30000.0, dims=16, mask=45), ff=320),
            _layer(_mixer(6, 40, 24, 24, 96, 0.18, 30000.0, dims=16, mask=1, kv_from=0)),
            _layer(_mixer(3, 8, 40, 16, 160, 0.15, 777.0, mask=130), ff=200),
            _layer(_mixer(17, 24, 40, 8, 160, 0.15, 777.0, kv_from=2), ff=64),
        ],
    },
}


def rovidra_config_json(name: str) -> dict:
    return {k: v for k, v in {**ROVIDRA, **ROVIDRA_FAST}[name].items() if k != "seed"}


def write_rovidra(name: str, out_dir: str, dtype=torch.float32) -> str:
    from jax_llm_examples_amd.config import get_architecture
    from jax_llm_examples_amd.weights import write_random_model

    top = rovidra_config_json(name)
    arch = get_architecture(top["architecture"])
    return write_random_model(arch, arch.parse_config(top), out_dir, {**ROVIDRA, **ROVIDRA_FAST}[name]["seed"], dtype)
