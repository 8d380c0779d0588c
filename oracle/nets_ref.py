"""TEST INFRASTRUCTURE — CPU restatement of the reference's Tucker ResNet-18 forward with plain torch
functional calls and UNFOLDED inference-mode BatchNorm, layer for layer as the reference model runs it
(inference/resnet_inet_tt.py:102-117 ``TTBasicBlock.forward``, :380-394 ``TTResNet.forward``; every 3x3
convolution is ``TKConv2dC.forward``, inference/TKConv.py:90-95).  Parameter keys are the reference's.
"""
import torch
import torch.nn.functional as F

BN_EPS = 1e-5
STAGES = ((64, 1), (128, 2), (256, 2), (512, 2))


def _bn(x, p, prefix):
    return F.batch_norm(x, p[prefix + ".running_mean"], p[prefix + ".running_var"], p[prefix + ".weight"],
                        p[prefix + ".bias"], False, 0.0, BN_EPS)


def _tk(x, p, prefix, stride):
    out = F.conv2d(x, p[prefix + ".first_kernel"])
    out = F.conv2d(out, p[prefix + ".core_kernel"], None, stride, 1, 1, 1)
    return F.conv2d(out, p[prefix + ".last_kernel"], None)


@torch.no_grad()
def tucker_resnet18_forward(p, x, return_features=False):
    feats = {}
    x = F.relu(_bn(F.conv2d(x, p["conv1.weight"], None, 2, 3), p, "bn1"))
    feats["stem"] = x
    x = F.max_pool2d(x, 3, 2, 1)
    feats["maxpool"] = x
    for s, (planes, stride) in enumerate(STAGES, start=1):
        for b in range(2):
            pre = f"layer{s}.{b}"
            st = stride if b == 0 else 1
            identity = x
            out = F.relu(_bn(_tk(x, p, pre + ".conv1", st), p, pre + ".bn1"))
            out = _bn(_tk(out, p, pre + ".conv2", 1), p, pre + ".bn2")
            if pre + ".downsample.0.weight" in p:
                identity = _bn(F.conv2d(x, p[pre + ".downsample.0.weight"], None, st), p, pre + ".downsample.1")
            x = F.relu(out + identity)
            feats[pre] = x
    x = F.adaptive_avg_pool2d(x, (1, 1))
    x = torch.flatten(x, 1)
    x = F.linear(x, p["fc.weight"], p["fc.bias"])
    return (x, feats) if return_features else x


DENSENET121_BLOCKS = (6, 12, 24, 16)


@torch.no_grad()
def tucker_densenet121_forward(p, x, return_features=False):
    """inference/densenet_inet_tt.py: TenDenseLayer.forward (:96-112, norm1 -> conv1 -> norm2 -> conv2 on the
    concatenation of all earlier features), TenDenseBlock.forward (:132-137), TenDenseTransition (:140-158),
    features -> norm5 -> global pool -> classifier.  The norm layers are BatchNorm + ReLU."""
    def bnrelu(t, prefix):
        return F.relu(_bn(t, p, prefix))

    out_feats = {}
    x = bnrelu(F.conv2d(x, p["features.conv0.weight"], None, 2, 3), "features.norm0")
    out_feats["stem"] = x
    x = F.max_pool2d(x, 3, 2, 1)
    for b, nl in enumerate(DENSENET121_BLOCKS, start=1):
        feats = [x]
        for l in range(1, nl + 1):
            pre = f"features.denseblock{b}.denselayer{l}"
            y = F.conv2d(bnrelu(torch.cat(feats, 1), pre + ".norm1"), p[pre + ".conv1.weight"])
            y = bnrelu(y, pre + ".norm2")
            y = F.conv2d(y, p[pre + ".conv2.first_kernel"])
            y = F.conv2d(y, p[pre + ".conv2.core_kernel"], None, 1, 1, 1, 1)
            y = F.conv2d(y, p[pre + ".conv2.last_kernel"], None)
            feats.append(y)
        x = torch.cat(feats, 1)
        out_feats[f"denseblock{b}"] = x
        if b < len(DENSENET121_BLOCKS):
            pre = f"features.transition{b}"
            x = F.avg_pool2d(F.conv2d(bnrelu(x, pre + ".norm"), p[pre + ".conv.weight"]), 2, 2)
    x = bnrelu(x, "features.norm5")
    x = torch.flatten(F.adaptive_avg_pool2d(x, (1, 1)), 1)
    x = F.linear(x, p["classifier.weight"], p["classifier.bias"])
    return (x, out_feats) if return_features else x
