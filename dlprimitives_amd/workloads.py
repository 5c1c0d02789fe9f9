"""Layer lists of the benchmark / parity configurations (shapes only, no arithmetic).

RESNET18_CONVS is the ordered list of the 20 convolutions of ResNet-18 as the
reference ships it in docs/nets_for_benchmark/resnet18-b16.js, with batch norm
folded into weights + bias and ReLU fused (the `activation` column says what the
real graph applies; the benchmark configuration applies ReLU to every conv).
"""


def conv(name, kernel, stride, pad, cin, cout, hw, groups=1, activation="relu"):
    oh = (hw + 2 * pad - (kernel - 1) - 1) // stride + 1
    return dict(name=name, kernel=kernel, stride=stride, pad=pad, cin=cin, cout=cout, hw=hw, ohw=oh, groups=groups,
                activation=activation)


def _resnet18():
    layers = [conv("conv1_7x7s2_3to64_at224", 7, 2, 3, 3, 64, 224)]
    for i in range(4):
        layers.append(conv("l1_%d_3x3_64to64_at56" % i, 3, 1, 1, 64, 64, 56))
    cin, hw = 64, 56
    for stage, cout in ((2, 128), (3, 256), (4, 512)):
        layers.append(conv("l%d_0_3x3s2_%dto%d_at%d" % (stage, cin, cout, hw), 3, 2, 1, cin, cout, hw))
        layers.append(conv("l%d_ds_1x1s2_%dto%d_at%d" % (stage, cin, cout, hw), 1, 2, 0, cin, cout, hw))
        hw //= 2
        for i in range(3):
            layers.append(conv("l%d_%d_3x3_%dto%d_at%d" % (stage, i + 1, cout, cout, hw), 3, 1, 1, cout, cout, hw))
        cin = cout
    return layers


RESNET18_CONVS = _resnet18()



def _resnet50():
    """The 53 convolutions of ResNet-50 (torchvision v1.5 layout: stride on the 3x3), in graph order."""
    layers = [conv("conv1_7x7s2_3to64_at224", 7, 2, 3, 3, 64, 224)]
    cin, hw = 64, 56
    for stage, (mid, blocks) in enumerate(((64, 3), (128, 4), (256, 6), (512, 3)), start=1):
        for b in range(blocks):
            s = 2 if (b == 0 and stage > 1) else 1
            pre = "l%d_%d" % (stage, b)
            layers.append(conv("%s_1x1_%dto%d_at%d" % (pre, cin, mid, hw), 1, 1, 0, cin, mid, hw))
            layers.append(conv("%s_3x3%s_%dto%d_at%d" % (pre, "s2" if s == 2 else "", mid, mid, hw), 3, s, 1, mid, mid, hw))
            layers.append(conv("%s_1x1_%dto%d_at%d" % (pre, mid, 4 * mid, hw // s), 1, 1, 0, mid, 4 * mid, hw // s, activation="identity"))
            if b == 0:
                layers.append(conv("%s_ds_1x1%s_%dto%d_at%d" % (pre, "s2" if s == 2 else "", cin, 4 * mid, hw), 1, s, 0, cin, 4 * mid, hw,
                                   activation="identity"))
            cin, hw = 4 * mid, hw // s
    return layers


RESNET50_CONVS = _resnet50()

# MobileNet-v2 style depthwise 3x3 shapes (C, HW), each at stride 1 and 2, and 1x1 followers
MOBILENET_DEPTHWISE = [(144, 56), (192, 28), (384, 14), (960, 7)]
MOBILENET_POINTWISE = [(144, 24, 56), (144, 32, 28), (192, 32, 28), (192, 64, 14), (384, 64, 14), (384, 96, 14), (960, 160, 7),
                       (960, 320, 7)]

# Winograd configuration: (B, Cin, Cout, HW)
WINOGRAD_SHAPES = [(64, 128, 128, 28), (64, 256, 256, 14)]


def conv_flops(layer, batch):
    """2 * B*Cout*OH*OW * (Cin/groups * KH*KW) -- the reference's own accounting (tools/flops.cpp:660)."""
    return 2.0 * batch * layer["cout"] * layer["ohw"] ** 2 * (layer["cin"] // layer["groups"]) * layer["kernel"] ** 2


def conv_bytes(layer, batch, elem=4):
    """sizeof(T) * (|X| + |W| + |Y|), tools/flops.cpp:661."""
    x = batch * layer["cin"] * layer["hw"] ** 2
    w = layer["cout"] * (layer["cin"] // layer["groups"]) * layer["kernel"] ** 2
    y = batch * layer["cout"] * layer["ohw"] ** 2
    return elem * (x + w + y)
