"""Driver-side tiling / normalisation (infer.py:16-173): pure host logic, checked on the CPU
against what the definitions fix (grid enumeration, tie rule, tile geometry, affine normalisation)."""
import numpy as np
import pytest
import torch

PIL = pytest.importorskip("PIL")
from PIL import Image  # noqa: E402

from calibquant_amd import preprocess as P  # noqa: E402


def test_target_grids_enumeration():
    grids = P.target_grids(1, 12)
    assert len(grids) == len(set(grids)) == sum(1 for i in range(1, 13) for j in range(1, 13) if i * j <= 12)
    counts = [c * r for c, r in grids]
    assert counts == sorted(counts) and grids[0] == (1, 1) and max(counts) == 12
    assert all(1 <= c * r <= 6 for c, r in P.target_grids(1, 6))


def test_closest_aspect_ratio_and_tie_rule():
    grids = P.target_grids(1, 12)
    assert P.find_closest_aspect_ratio(1.0, grids, 448, 448, 448) == (1, 1)        # small square: stays one tile
    # a large square image: (1,1), (2,2), (3,3) tie on the ratio; the area rule walks up to (3,3)
    assert P.find_closest_aspect_ratio(1.0, grids, 2000, 2000, 448) == (3, 3)
    assert P.find_closest_aspect_ratio(1.0, grids, 700, 700, 448) == (2, 2)        # 490k px > half of 4 tiles, < half of 9
    assert P.find_closest_aspect_ratio(4.0, grids, 1792, 448, 448) == (4, 1)
    assert P.find_closest_aspect_ratio(1 / 3, grids, 448, 1344, 448) == (1, 3)
    assert P.image_token_count(1792, 448) == 5 * 256 and P.image_token_count(448, 448) == 256
    assert P.image_token_count(4000, 3000) == 13 * 256                              # 4:3 at 12 tiles -> (4,3) + thumbnail


def test_tiles_cover_the_resized_image_row_by_row():
    rng = np.random.default_rng(0)
    arr = rng.integers(0, 256, size=(300, 650, 3), dtype=np.uint8)    # h=300, w=650: ratio 2.17 -> (2,1)
    img = Image.fromarray(arr, "RGB")
    tiles = P.dynamic_preprocess(img, image_size=64, max_num=6, use_thumbnail=True)
    cols, rows = P.find_closest_aspect_ratio(650 / 300, P.target_grids(1, 6), 650, 300, 64)
    assert len(tiles) == cols * rows + 1 and all(t.size == (64, 64) for t in tiles)
    resized = np.asarray(img.resize((64 * cols, 64 * rows)))
    for i in range(cols * rows):
        r, c = divmod(i, cols)
        assert np.array_equal(np.asarray(tiles[i]), resized[r * 64:(r + 1) * 64, c * 64:(c + 1) * 64])
    assert np.array_equal(np.asarray(tiles[-1]), np.asarray(img.resize((64, 64))))
    one = P.dynamic_preprocess(Image.fromarray(arr[:64, :64], "RGB"), image_size=64, max_num=6, use_thumbnail=True)
    assert len(one) == 1                                                # a single tile gets no thumbnail


def test_transform_is_resize_scale_and_affine_normalisation():
    rng = np.random.default_rng(1)
    arr = rng.integers(0, 256, size=(32, 32, 3), dtype=np.uint8)
    x = P.build_transform(32)(Image.fromarray(arr, "RGB"))             # same size: the resize is the identity
    want = (arr.astype(np.float32).transpose(2, 0, 1) / 255.0 - np.array(P.IMAGENET_MEAN, np.float32)[:, None, None]) \
        / np.array(P.IMAGENET_STD, np.float32)[:, None, None]
    assert x.shape == (3, 32, 32) and x.dtype == torch.float32
    assert np.allclose(x.numpy(), want, atol=1e-6)
    grey = Image.fromarray(arr[..., 0], "L")
    xg = P.build_transform(32)(grey)                                    # non-RGB input is converted first
    assert xg.shape == (3, 32, 32)
    px = P.load_image(Image.fromarray(rng.integers(0, 256, size=(100, 400, 3), dtype=np.uint8), "RGB"), input_size=32, max_num=6)
    assert px.shape == (4 + 1, 3, 32, 32)


def test_internvit_shaped_tower_shapes_and_pixel_shuffle():
    """The InternViT-shaped tower turns 448 x 448 tiles into 256 tokens of the language model's width;
    the pixel shuffle gathers every 2 x 2 block of patches into one token, block row first."""
    import torch
    from calibquant_amd.internvit import InternViTConfig, InternViTTower, pixel_shuffle
    x = torch.arange(2 * 4 * 6 * 3, dtype=torch.float32).reshape(2, 4, 6, 3)
    y = pixel_shuffle(x, 0.5)
    assert y.shape == (2, 2, 3, 12)
    for n in range(2):
        for w in range(2):
            for h in range(3):
                want = torch.cat([x[n, 2 * w + a, 2 * h + b] for a in range(2) for b in range(2)])
                assert torch.equal(y[n, w, h], want)
    torch.manual_seed(0)
    tower = InternViTTower(InternViTConfig.tiny(), llm_hidden=96).eval()
    with torch.no_grad():
        out = tower(torch.rand(3, 3, 448, 448))
    assert out.shape == (3, 256, 96) and tower.num_image_token == 256 and torch.isfinite(out).all()
    # the 300M preset has the published size (about 0.3 billion parameters); built without storage
    with torch.device("meta"):
        big = InternViTTower(InternViTConfig.internvit_300m(), llm_hidden=4096)
    enc = sum(p.numel() for n_, p in big.named_parameters() if not n_.startswith("mlp1"))
    assert 0.29e9 < enc < 0.32e9, enc
