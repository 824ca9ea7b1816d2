"""Parameter-shape lists of the two EMA benchmark workloads (synthetic, no model
code): what bench.py and the parity tests build their parameter lists from."""


def resnet18_shapes():
    """torchvision ResNet-18 parameters() order: 62 tensors, 11,689,512 elements."""
    shapes = [(64, 3, 7, 7), (64,), (64,)]
    for _ in range(2):
        shapes += [(64, 64, 3, 3), (64,), (64,), (64, 64, 3, 3), (64,), (64,)]
    for c in (128, 256, 512):
        cin = c // 2
        shapes += [(c, cin, 3, 3), (c,), (c,), (c, c, 3, 3), (c,), (c,), (c, cin, 1, 1), (c,), (c,)]
        shapes += [(c, c, 3, 3), (c,), (c,), (c, c, 3, 3), (c,), (c,)]
    shapes += [(1000, 512), (1000,)]
    return shapes


def vit_base_shapes():
    """timm ViT-B/16 parameters() order: 152 tensors, 86,567,656 elements."""
    d = 768
    shapes = [(1, 1, d), (1, 197, d), (d, 3, 16, 16), (d,)]
    for _ in range(12):
        shapes += [(d,), (d,), (3 * d, d), (3 * d,), (d, d), (d,), (d,), (d,), (4 * d, d), (4 * d,), (d, 4 * d), (d,)]
    shapes += [(d,), (d,), (1000, d), (1000,)]
    return shapes


def numel(shape):
    n = 1
    for s in shape:
        n *= s
    return n
