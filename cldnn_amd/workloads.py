"""Convolution stacks of the benchmark networks as plain shape lists (synthetic data only).

Each entry is a dict: name, ifm, ofm, k (square filter), stride, pad, in_hw (input height = width),
groups, act ("relu" / "none" / "relu6"), closes_block (the 1x1 that takes the residual add),
follows_prev (in the network this layer reads the tensor the entry before it in the list writes, with nothing
but a fused residual sum in between: such neighbours may run as one convolution chain), shares_input (in the network
this layer reads the SAME tensor as the entry before it, with the same filter size, stride and padding: the two may run
as one launch).
"""


def _layer(name, ifm, ofm, k, stride, pad, in_hw, groups=1, act="relu", closes_block=False, follows_prev=False,
           shares_input=False):
    out_hw = (in_hw + 2 * pad - k) // stride + 1
    return dict(name=name, ifm=ifm, ofm=ofm, k=k, stride=stride, pad=pad, in_hw=in_hw, out_hw=out_hw, groups=groups,
                act=act, closes_block=closes_block, follows_prev=follows_prev, shares_input=shares_input)


def resnet50(stride_on_3x3=False):
    """53 convolutions of ResNet-50 at 224x224.  Default is the Caffe form (stride on the first 1x1
    of a down-sampling block); stride_on_3x3=True gives the "v1.5" form."""
    L = [_layer("conv1", 3, 64, 7, 2, 3, 224)]
    hw = 56  # after the 3x3/s2 max-pool, which is not a convolution
    cin = 64
    for stage, (blocks, width) in enumerate(((3, 64), (4, 128), (6, 256), (3, 512)), start=2):
        for b in range(blocks):
            s = 2 if (b == 0 and stage > 2) else 1
            n = "res%d%s" % (stage, chr(ord("a") + b))
            s1, s3 = (1, s) if stride_on_3x3 else (s, 1)
            mid_hw = hw // s1
            out_hw = hw // s
            if b == 0:
                L.append(_layer(n + "_branch1", cin, width * 4, 1, s, 0, hw, act="none"))
            # a block's first 1x1 reads the sum the block before it closes with (not in a block with a projection, whose
            # list neighbour is that projection)
            # ... and in such a block it reads what the projection reads
            L.append(_layer(n + "_branch2a", cin, width, 1, s1, 0, hw, follows_prev=b > 0, shares_input=b == 0 and s1 == s))
            L.append(_layer(n + "_branch2b", width, width, 3, s3, 1, mid_hw, follows_prev=True))
            L.append(_layer(n + "_branch2c", width, width * 4, 1, 1, 0, out_hw, closes_block=True, follows_prev=True))
            cin = width * 4
            hw = out_hw
    assert len(L) == 53
    return L


def vgg16():
    """13 3x3/s1/p1 convolutions of VGG-16 at 224x224."""
    cfg = [(3, 64, 224), (64, 64, 224), (64, 128, 112), (128, 128, 112), (128, 256, 56), (256, 256, 56), (256, 256, 56),
           (256, 512, 28), (512, 512, 28), (512, 512, 28), (512, 512, 14), (512, 512, 14), (512, 512, 14)]
    return [_layer("conv%d" % (i + 1), a, b, 3, 1, 1, hw) for i, (a, b, hw) in enumerate(cfg)]


def mobilenet_v2():
    """52 convolutions of MobileNet-v2 (width 1.0) at 224x224: 3x3 depthwise + 1x1 expand/project."""
    L = [_layer("conv1", 3, 32, 3, 2, 1, 224, act="relu6")]
    hw, cin = 112, 32
    idx = 0
    for t, c, n, s in ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2),
                       (6, 320, 1, 1)):
        for i in range(n):
            stride = s if i == 0 else 1
            idx += 1
            mid = cin * t
            # the stack has no residual sums, so every layer reads what the one before it writes
            if t != 1:
                L.append(_layer("b%d_expand" % idx, cin, mid, 1, 1, 0, hw, act="relu6", follows_prev=True))
            L.append(_layer("b%d_dw" % idx, mid, mid, 3, stride, 1, hw, groups=mid, act="relu6", follows_prev=True))
            hw = (hw + 2 - 3) // stride + 1
            L.append(_layer("b%d_project" % idx, mid, c, 1, 1, 0, hw, act="none", follows_prev=True))
            cin = c
    L.append(_layer("conv_last", cin, 1280, 1, 1, 0, hw, act="relu6", follows_prev=True))
    assert len(L) == 52, len(L)
    return L


def macs(layers):
    return sum(l["out_hw"] ** 2 * l["ofm"] * (l["ifm"] // l["groups"]) * l["k"] ** 2 for l in layers)
