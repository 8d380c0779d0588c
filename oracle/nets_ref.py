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
