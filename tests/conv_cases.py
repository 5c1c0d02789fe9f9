"""Convolution geometries shared by the CPU (oracle) and GPU (parity) tests.

REFERENCE_MATRIX mirrors the geometry matrix of the reference's own fixture
generator (tests/make_test_cases_from_pt.py:923-947: kernel, pad, stride, dilate,
channels in/out, bias, groups, relu) and its input-shape list (:996-997); the
generated JSON files themselves are not part of the reference checkout.
"""


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def case(kernel, pad, stride, dilate, cin, cout, bias, groups, relu, batch_limit=64):
    return dict(kernel=_pair(kernel), pad=_pair(pad), stride=_pair(stride), dilate=_pair(dilate),
                cin=cin, cout=cout, bias=bias, groups=groups,
                activation="relu" if relu else "identity", batch_limit=batch_limit)


REFERENCE_MATRIX = [
    case(5, 2, 1, 1, 98, 128, True, 1, True, 1),
    case(3, 1, 1, 1, 1, 1, False, 1, False),
    case(3, 1, 1, 1, 2, 1, False, 1, False),
    case(3, 1, 1, 1, 1, 2, False, 1, False),
    case(3, 1, 1, 1, 3, 8, False, 1, False),
    case(3, 1, 1, 1, 128, 64, False, 1, False),
    case(3, 1, 1, 1, 3, 8, True, 1, True),
    case(1, 0, 1, 1, 3, 5, False, 1, False),
    case(1, 0, 1, 1, 48, 1152, False, 1, False),
    case(1, 0, 1, 1, 48, 1152, False, 2, False),
    case((1, 2), 0, 1, 1, 48, 1152, False, 1, False),
    case((1, 2), 0, 1, 1, 48, 1152, False, 2, False),
    case(1, 0, 2, 1, 3, 5, False, 1, False),
    case(3, 1, 1, 1, 4, 8, True, 2, False),
    case(3, 1, 2, 1, 6, 8, True, 2, False),
    case(3, 1, 1, 1, 8, 8, True, 8, False),
    case((1, 7), (0, 3), 1, 1, 192, 160, True, 1, False),
    case((7, 1), (3, 0), 1, 1, 128, 192, True, 1, False),
    case((3, 5), (1, 2), (2, 3), (3, 2), 3, 8, False, 1, False),
    case(5, 2, 1, 1, 16, 32, True, 1, False),
    case(11, 2, 4, 1, 16, 32, True, 1, False),
]

# (batch, H, W) list of the reference generator, :996-997
REFERENCE_SHAPES = [(1, 2, 2), (1, 7, 7), (1, 8, 8), (1, 4, 4), (3, 4, 4), (2, 7, 7), (2, 10, 5), (2, 10, 10),
                    (2, 19, 19), (2, 20, 20), (2, 32, 32), (64, 64, 64), (53, 100, 100)]


def shape_ok(c, b, h, w):
    """Same admission rule as the generator (:999-1004)."""
    if b > c["batch_limit"]:
        return False
    lkh, lkw = c["kernel"][0] * c["dilate"][0], c["kernel"][1] * c["dilate"][1]
    if h + c["pad"][0] < lkh or w + c["pad"][1] < lkw:
        return False
    max_dim = 256 if c["cin"] * c["cout"] < 50000 else 10
    return h <= max_dim and w <= max_dim


def small_cases(max_macs=3e7):
    """(case, (B,H,W)) pairs cheap enough for the scalar CPU oracle."""
    out = []
    for c in REFERENCE_MATRIX:
        for (b, h, w) in REFERENCE_SHAPES:
            if not shape_ok(c, b, h, w):
                continue
            macs = b * h * w * c["cout"] * (c["cin"] // c["groups"]) * c["kernel"][0] * c["kernel"][1]
            if macs <= max_macs:
                out.append((c, (b, h, w)))
    return out


def case_id(v):
    if isinstance(v, dict):
        k, p, s, d = v["kernel"], v["pad"], v["stride"], v["dilate"]
        return "k%dx%d_p%d%d_s%d%d_d%d%d_c%d_o%d_g%d%s%s" % (k[0], k[1], p[0], p[1], s[0], s[1], d[0], d[1], v["cin"], v["cout"],
                                                            v["groups"], "_b" if v["bias"] else "", "_" + v["activation"])
    if isinstance(v, tuple):
        return "x".join(str(i) for i in v)
    return str(v)


def make_tensors(c, bhw, seed):
    """Seeded inputs owned by this build (numpy PCG64): x ~ U[-1,1], w ~ Kaiming-normal, bias ~ U[-0.1,0.1]."""
    import numpy as np

    rng = np.random.default_rng(seed)
    b, h, w = bhw
    cin_g = c["cin"] // c["groups"]
    x = rng.uniform(-1, 1, size=(b, c["cin"], h, w)).astype(np.float32)
    fan_in = cin_g * c["kernel"][0] * c["kernel"][1]
    wt = (rng.standard_normal(size=(c["cout"], cin_g, c["kernel"][0], c["kernel"][1])) * np.sqrt(2.0 / fan_in)).astype(np.float32)
    bias = rng.uniform(-0.1, 0.1, size=(c["cout"],)).astype(np.float32) if c["bias"] else None
    return x, wt, bias
