"""The benchmark networks as operator-chain descriptions.

Each network is (input_dims, layers, num_categories); dims are (width, height, channels) and the
layer tuples repeat the arguments of the SequentialOperatorConfig builder calls:
    ("conv2d", in_dims, conv_size, conv_stride, conv_pad, out_channels, act_func)
    ("pool2d", in_dims, pool_size, pool_stride, pool_pad, pool_op, ceil_mode)
    ("affine", in_channels, out_channels, act_func)
    ("dropout", channels, drop_ratio)
    ("local_res_norm", in_dims, cross_size, scale, power, min_div)
    ("bnorm_conv2d", in_dims, conv_size, conv_stride, conv_pad, out_channels, act_func)
    ("stack_res_conv2d", in_dims, act_func)
    ("proj_stack_res_conv2d", in_dims, out_dims, act_func)
Geometry the benchmark text leaves open follows the reference's own tools:
LeNet from tools/train-mnist.rs:79-133 (conv pad 2, conv activations Identity, FC1 in 2450),
the CIFAR-10 net from tools/train-cifar10.rs:58-162 (3x3 stride-2 pools with pad 1),
NIN from examples/imagenet_nin.model (ceil pooling 54 -> 27 -> 13 -> 6, global average pool),
ResNet-18 from src/templates/resnet.rs:367-520 (build_resnet18_224x224).
"""
from .operator import SequentialOperatorConfig


def _chain(input_dims, spec):
    """spec entries: ("conv", size, stride, pad, out, act) | ("pool", size, stride, pad, op[, ceil]) | ("fc", out, act)
    | ("dropout", ratio) | ("lrn", cross_size, scale, power, min_div) | ("bnconv", size, stride, pad, out, act)
    | ("res", act) | ("projres", out_channels, stride, act)."""
    w, h, c = input_dims
    layers = []
    for s in spec:
        if s[0] == "conv":
            _, k, st, pad, out, act = s
            layers.append(("conv2d", (w, h, c), k, st, pad, out, act))
            w = max(0, w + 2 * pad - k + st) // st
            h = max(0, h + 2 * pad - k + st) // st
            c = out
        elif s[0] == "pool":
            k, st, pad, op = s[1:5]
            ceil = len(s) > 5 and s[5]
            layers.append(("pool2d", (w, h, c), k, st, pad, op, ceil))
            if ceil:
                w = max(0, w + 2 * pad - k + st - 1) // st + 1
                h = max(0, h + 2 * pad - k + st - 1) // st + 1
            else:
                w = max(0, w + 2 * pad - k + st) // st
                h = max(0, h + 2 * pad - k + st) // st
        elif s[0] == "fc":
            _, out, act = s
            layers.append(("affine", w * h * c, out, act))
            w, h, c = 1, 1, out
        elif s[0] == "dropout":
            layers.append(("dropout", w * h * c, s[1]))
        elif s[0] == "lrn":
            layers.append(("local_res_norm", (w, h, c), s[1], s[2], s[3], s[4]))
        elif s[0] == "bnconv":
            _, k, st, pad, out, act = s
            layers.append(("bnorm_conv2d", (w, h, c), k, st, pad, out, act))
            w = max(0, w + 2 * pad - k + st) // st
            h = max(0, h + 2 * pad - k + st) // st
            c = out
        elif s[0] == "res":
            layers.append(("stack_res_conv2d", (w, h, c), s[1]))
        elif s[0] == "projres":
            _, out, st, act = s
            assert w % st == 0 and h % st == 0
            layers.append(("proj_stack_res_conv2d", (w, h, c), (w // st, h // st, out), act))
            w, h, c = w // st, h // st, out
        else:
            raise ValueError(s[0])
    return layers, w * h * c


def lenet():
    dims = (28, 28, 1)
    layers, out = _chain(dims, [("conv", 5, 1, 2, 20, "Identity"), ("pool", 2, 2, 0, "Max"),
                                ("conv", 5, 1, 2, 50, "Identity"), ("pool", 2, 2, 0, "Max"),
                                ("fc", 500, "Rect"), ("fc", 10, "Identity")])
    return dims, layers, out


def cifar10():
    dims = (32, 32, 3)
    layers, out = _chain(dims, [("conv", 5, 1, 2, 32, "Rect"), ("pool", 3, 2, 1, "Max"),
                                ("conv", 5, 1, 2, 32, "Rect"), ("pool", 3, 2, 1, "Average"),
                                ("conv", 5, 1, 2, 64, "Rect"), ("pool", 3, 2, 1, "Average"),
                                ("fc", 64, "Rect"), ("fc", 10, "Identity")])
    return dims, layers, out


def alexnet():
    dims = (227, 227, 3)
    layers, out = _chain(dims, [("conv", 11, 4, 0, 96, "Rect"), ("pool", 3, 2, 0, "Max"),
                                ("conv", 5, 1, 2, 256, "Rect"), ("pool", 3, 2, 0, "Max"),
                                ("conv", 3, 1, 1, 384, "Rect"), ("conv", 3, 1, 1, 384, "Rect"),
                                ("conv", 3, 1, 1, 256, "Rect"), ("pool", 3, 2, 0, "Max"),
                                ("fc", 4096, "Rect"), ("fc", 4096, "Rect"), ("fc", 1000, "Identity")])
    return dims, layers, out


def nin():
    dims = (224, 224, 3)
    layers, out = _chain(dims, [("conv", 11, 4, 0, 96, "Rect"), ("conv", 1, 1, 0, 96, "Rect"), ("conv", 1, 1, 0, 96, "Rect"),
                                ("pool", 3, 2, 0, "Max", True),
                                ("conv", 5, 1, 2, 256, "Rect"), ("conv", 1, 1, 0, 256, "Rect"), ("conv", 1, 1, 0, 256, "Rect"),
                                ("pool", 3, 2, 0, "Max", True),
                                ("conv", 3, 1, 1, 384, "Rect"), ("conv", 1, 1, 0, 384, "Rect"), ("conv", 1, 1, 0, 384, "Rect"),
                                ("pool", 3, 2, 0, "Max", True),
                                ("conv", 3, 1, 1, 1024, "Rect"), ("conv", 1, 1, 0, 1024, "Rect"), ("conv", 1, 1, 0, 1000, "Rect"),
                                ("pool", 6, 1, 0, "Average", True)])
    return dims, layers, out


def resnet18():
    dims = (224, 224, 3)
    layers, out = _chain(dims, [("bnconv", 7, 2, 3, 64, "Rect"), ("pool", 3, 2, 1, "Max"),
                                ("res", "Rect"), ("res", "Rect"),
                                ("projres", 128, 2, "Rect"), ("res", "Rect"),
                                ("projres", 256, 2, "Rect"), ("res", "Rect"),
                                ("projres", 512, 2, "Rect"), ("res", "Rect"),
                                ("pool", 7, 1, 0, "Average"), ("fc", 1000, "Identity")])
    return dims, layers, out


NETWORKS = {"lenet": lenet, "cifar10": cifar10, "alexnet": alexnet, "nin": nin, "resnet18": resnet18}


def build_config(net, init_std=0.01, bnorm_mov_avg=("Exponential", 0.1), bnorm_epsilon=1e-5):
    """SequentialOperatorConfig for one of the networks above; weights N(0, init_std^2), bias 0; the filters of the
    batch-normalised operators N(0, 2/fan_in) (KaimingFwd, as the reference's templates set them)."""
    dims, layers, num_categories = net
    cfg = SequentialOperatorConfig().data3d(dims, normalize=False)
    for l in layers:
        if l[0] == "conv2d":
            cfg.conv2d(l[1], l[2], l[3], l[4], l[5], l[6], ("Normal", init_std))
        elif l[0] == "pool2d":
            cfg.pool2d(l[1], l[2], l[3], l[4], l[5], l[6])
        elif l[0] == "dropout":
            cfg.dropout(l[1], l[2])
        elif l[0] == "local_res_norm":
            cfg.local_res_norm(l[1], l[2], l[3], l[4], l[5])
        elif l[0] == "bnorm_conv2d":
            cfg.bnorm_conv2d(l[1], l[2], l[3], l[4], l[5], bnorm_mov_avg, bnorm_epsilon, l[6], "KaimingFwd")
        elif l[0] == "stack_res_conv2d":
            cfg.stack_res_conv2d(l[1], bnorm_mov_avg, bnorm_epsilon, l[2], "KaimingFwd")
        elif l[0] == "proj_stack_res_conv2d":
            cfg.proj_stack_res_conv2d(l[1], l[2], bnorm_mov_avg, bnorm_epsilon, l[3], "KaimingFwd")
        else:
            cfg.affine(l[1], l[2], l[3], ("Normal", init_std))
    return cfg.softmax_kl_loss(num_categories)


def train_flops(net, batch, forward_only=False):
    """GEMM-equivalent FLOPs of one train step: 2*N*K*C*R*S*P*Q per conv pass (no backward-data
    for the first layer), 2*B*in*out per affine GEMM; of the forward pass alone with forward_only."""
    _, layers, _ = net
    total = 0
    first = True
    passes = (lambda first: 1) if forward_only else (lambda first: 2 if first else 3)
    for l in layers:
        if l[0] in ("conv2d", "bnorm_conv2d"):
            (w, h, c), k, st, pad, out = l[1], l[2], l[3], l[4], l[5]
            P = max(0, h + 2 * pad - k + st) // st
            Q = max(0, w + 2 * pad - k + st) // st
            f = 2 * batch * out * c * k * k * P * Q
            total += f * passes(first)
        elif l[0] == "stack_res_conv2d":
            (w, h, c) = l[1]
            total += 2 * passes(False) * (2 * batch * c * c * 9 * w * h)
        elif l[0] == "proj_stack_res_conv2d":
            (w, h, c), (ow, oh, oc) = l[1], l[2]
            total += passes(False) * (2 * batch * ow * oh * oc * (9 * c + 9 * oc + c))
        elif l[0] == "affine":
            f = 2 * batch * l[1] * l[2]
            total += f * passes(first)
        else:
            continue
        first = False
    return total
