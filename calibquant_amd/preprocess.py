"""Image side of the reference's driver: aspect-ratio tiling, resize and normalisation
(infer.py:16-45 `build_transform`, :48-84 `find_closest_aspect_ratio`, :87-144
`dynamic_preprocess`, :146-173 `load_image`).

Host-side only: it decides how many 448x448 tiles an image becomes, and therefore how many
image tokens (256 per tile) the prefill quantises.  torchvision is not needed: its
`Resize` / `ToTensor` / `Normalize` on PIL images are a PIL bicubic resize, a scale by 1/255 and
a per-channel affine map, which is what is done here.
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np
import torch

IMAGENET_MEAN = (0.485, 0.456, 0.406)   # infer.py:13
IMAGENET_STD = (0.229, 0.224, 0.225)    # infer.py:14


def _pil():
    from PIL import Image
    return Image


def build_transform(input_size: int):
    """PIL image -> (3, input_size, input_size) float32 tensor: RGB, bicubic resize,
    [0, 1] scaling, ImageNet normalisation (infer.py:38-44)."""
    mean = torch.tensor(IMAGENET_MEAN, dtype=torch.float32)[:, None, None]
    std = torch.tensor(IMAGENET_STD, dtype=torch.float32)[:, None, None]

    def transform(img):
        Image = _pil()
        if img.mode != "RGB":
            img = img.convert("RGB")
        img = img.resize((input_size, input_size), Image.BICUBIC)
        x = torch.from_numpy(np.asarray(img, dtype=np.uint8).copy()).permute(2, 0, 1).to(torch.float32).div(255.0)
        return (x - mean) / std

    return transform


def find_closest_aspect_ratio(aspect_ratio: float, target_ratios: Sequence[Tuple[int, int]], width: int, height: int,
                              image_size: int) -> Tuple[int, int]:
    """The (columns, rows) grid whose aspect ratio is closest to the image's; on a tie the later
    (larger) grid wins if the image has more than half of that grid's pixels (infer.py:71-84)."""
    best_diff, best = float("inf"), (1, 1)
    area = width * height
    for ratio in target_ratios:
        diff = abs(aspect_ratio - ratio[0] / ratio[1])
        if diff < best_diff:
            best_diff, best = diff, ratio
        elif diff == best_diff and area > 0.5 * image_size * image_size * ratio[0] * ratio[1]:
            best = ratio
    return best


def target_grids(min_num: int = 1, max_num: int = 12) -> List[Tuple[int, int]]:
    """All (columns, rows) grids with min_num <= columns*rows <= max_num, by tile count (infer.py:112-116)."""
    grids = {(i, j) for n in range(min_num, max_num + 1) for i in range(1, n + 1) for j in range(1, n + 1)
             if min_num <= i * j <= max_num}
    return sorted(grids, key=lambda g: g[0] * g[1])


def dynamic_preprocess(image, min_num: int = 1, max_num: int = 12, image_size: int = 448, use_thumbnail: bool = False):
    """Resize the image to the closest tile grid and cut it into image_size tiles, row by row;
    optionally append a thumbnail of the whole image (infer.py:108-144).  Returns PIL images."""
    w, h = image.size
    cols, rows = find_closest_aspect_ratio(w / h, target_grids(min_num, max_num), w, h, image_size)
    resized = image.resize((image_size * cols, image_size * rows))
    tiles = []
    for i in range(cols * rows):
        x0, y0 = (i % cols) * image_size, (i // cols) * image_size
        tiles.append(resized.crop((x0, y0, x0 + image_size, y0 + image_size)))
    if use_thumbnail and len(tiles) != 1:
        tiles.append(image.resize((image_size, image_size)))
    return tiles


def load_image(image, input_size: int = 448, max_num: int = 12) -> torch.Tensor:
    """Path or PIL image -> (tiles, 3, input_size, input_size) float32 pixel values, thumbnail
    included (infer.py:167-173)."""
    Image = _pil()
    if not hasattr(image, "size"):
        image = Image.open(image)
    image = image.convert("RGB")
    transform = build_transform(input_size)
    tiles = dynamic_preprocess(image, image_size=input_size, use_thumbnail=True, max_num=max_num)
    return torch.stack([transform(t) for t in tiles])


def image_token_count(width: int, height: int, max_num: int = 12, image_size: int = 448, tokens_per_tile: int = 256) -> int:
    """Image tokens the prefill will quantise for an image of this size: tiles (+ thumbnail) x 256."""
    cols, rows = find_closest_aspect_ratio(width / height, target_grids(1, max_num), width, height, image_size)
    tiles = cols * rows
    return (tiles + (1 if tiles != 1 else 0)) * tokens_per_tile
