"""Gradient sets the operators are measured on: tensor shapes only, plus seeded
synthetic values generated on the device (there are no datasets or checkpoints)."""
import math

import torch

from . import datagen

# VGG19 parameter-gradient sizes in the order of the reference's planner input
# (/root/reference/src/SeCoPa/input.txt:1-38): 16 conv weight+bias pairs, 3 dense.
VGG19 = [
    1728, 64, 36864, 64, 73728, 128, 147456, 128, 294912, 256, 589824, 256, 589824, 256, 589824, 256,
    1179648, 512, 2359296, 512, 2359296, 512, 2359296, 512, 2359296, 512, 2359296, 512, 2359296, 512,
    2359296, 512, 102760448, 4096, 16777216, 4096, 4096000, 1000,
]


def vgg19_sizes():
    return list(VGG19)


def resnet50_sizes():
    """53 conv weights (7x7 stem, bottleneck stages [3,4,6,3] at widths 64..512,
    four 1x1 downsample convs), a BN gamma/beta pair per conv, fc 2048x1000 + bias."""
    sizes = [7 * 7 * 3 * 64, 64, 64]
    cin = 64
    for width, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
        for b in range(blocks):
            sizes += [cin * width, width, width]            # 1x1 reduce + BN
            sizes += [3 * 3 * width * width, width, width]  # 3x3 + BN
            sizes += [width * 4 * width, 4 * width, 4 * width]  # 1x1 expand + BN
            if b == 0:
                sizes += [cin * 4 * width, 4 * width, 4 * width]  # downsample + BN
            cin = 4 * width
    sizes += [2048 * 1000, 1000]
    return sizes


def bert_large_sizes():
    """Embeddings (30522 / 512 / 2 x 1024 + LayerNorm), 24 encoder layers of
    Q, K, V, O (1024x1024 + bias), LayerNorm, FFN 1024x4096 and 4096x1024 (+ biases),
    LayerNorm, and the pooler."""
    h, ff = 1024, 4096
    sizes = [30522 * h, 512 * h, 2 * h, h, h]
    for _ in range(24):
        sizes += [h * h, h] * 4 + [h, h] + [h * ff, ff, ff * h, h] + [h, h]
    sizes += [h * h, h]
    return sizes


def chunk_sizes(sizes, chunk=1 << 20):
    """Per-tensor partition into chunks of at most `chunk` elements (4 MB of fp32)."""
    out = []
    for n in sizes:
        full, rest = divmod(n, chunk)
        out += [chunk] * full + ([rest] if rest else [])
    return out


assert sum(VGG19) == 143_667_240
assert sum(resnet50_sizes()) == 25_557_032 and len(resnet50_sizes()) == 53 * 3 + 2
assert sum(bert_large_sizes()) == 335_141_888
assert len(chunk_sizes(VGG19)) == 168


# Values come from the counter-based generator of datagen.py: element i of tensor t with seed s
# is a function of (s, t, i) alone.  Streams of one seed are kept apart by an offset in the
# tensor number.
_GRAD, _PICK, _LAPLACE, _UNIFORM = 0, 1 << 20, 2 << 20, 3 << 20


def normal_set(sizes, device, seed, sigma=None, log_sigma_range=None):
    """One N(0, sigma) tensor per size; with log_sigma_range=(a, b) each tensor
    draws its own sigma = 10**U(a, b)."""
    out = []
    for t, n in enumerate(sizes):
        s = sigma
        if log_sigma_range is not None:
            a, b = log_sigma_range
            s = 10.0 ** (a + (b - a) * datagen.scalar_uniform(seed, _GRAD + t))
        out.append(datagen.normal(n, device, seed, _GRAD + t, s))
    return out


def heavy_tailed_set(sizes, device, seed, sigma=1e-3, outlier_prob=0.01, laplace_scale=1e-2):
    """N(0, sigma) with each element replaced, with probability outlier_prob, by a
    Laplace(0, laplace_scale) draw."""
    out = []
    for t, n in enumerate(sizes):
        g = datagen.normal(n, device, seed, _GRAD + t, sigma)
        pick = datagen.bernoulli(n, device, seed, _PICK + t, outlier_prob)
        u = datagen.uniform(n, device, seed, _LAPLACE + t) - 0.5
        lap = -laplace_scale * torch.sign(u) * torch.log1p(-2 * u.abs())
        out.append(torch.where(pick, lap, g))
    return out


def uniform_set(sizes, device, seed):
    """U[0,1) float32 built from 24 random bits, so 1.0 is never produced."""
    return [datagen.uniform(n, device, seed, _UNIFORM + t) for t, n in enumerate(sizes)]


def total_bytes(sizes):
    return 4 * sum(sizes)


def describe(name, sizes):
    return f"{name}: {len(sizes)} tensors, {sum(sizes):,} fp32 elements ({total_bytes(sizes) / 2**20:.0f} MiB)"


if __name__ == "__main__":
    for nm, fn in (("vgg19", vgg19_sizes), ("resnet50", resnet50_sizes), ("bert_large", bert_large_sizes)):
        print(describe(nm, fn()), "largest", max(fn()), "log2", round(math.log2(max(fn())), 1))
