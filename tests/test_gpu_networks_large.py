"""The benchmark configurations at sizes where the fp16 comparison with the CPU oracle means something: every
batch norm of the network normalises over hundreds to thousands of values per channel, as at full size, so the
noise that fp16 storage alone puts on the gradients (the yardstick of tests/test_gpu_networks.py, measured on
the oracle itself in the same test) stays small and the bounds derived from it are tight.  The oracle takes
1 - 2 minutes per test on the host cores."""
import numpy as np
import pytest

from saga_amd import networks as N
from tests.test_gpu_networks import run_training

pytestmark = pytest.mark.gpu


def test_resnet20_training_fp16_at_batch_128():
    """Config 3 as stated: batch 128, 32x32, mixed-precision Adam at lr 1e-3, loss scale starting at 2^15."""
    run_training(N.resnet20(128), 3, steps=1, lr=1e-3, loss_scale=32768.0,
                 check_params=["s1-conv-w", "s2_1-conv-2-w", "s3_0-conv-p-w", "s4_2-conv-2-w", "fc-w", "s2_0-bn-1-s",
                               "s4_2-bn-2-b"])


def test_resnet50_training_fp16_at_224_batch_32():
    """Config 4 at its real image size with batch 32 (the last stage still normalises over 32 x 7 x 7 = 1568
    values per channel): one training step, logits, loss, gradients from the stem to the classifier and the
    weights after the Adam step against the oracle network."""
    run_training(N.resnet50(32), 5, steps=1, lr=1e-4, loss_scale=1024.0,
                 check_params=["s1-conv-w", "s2_1-conv-p-w", "s2_3-conv-2-w", "s3_1-conv-2-w", "s4_2-conv-1-w",
                               "s5_3-conv-3-w", "fc3-w", "s4_2-bn-2-s", "s2_1-bn-1-b"])


def test_unet_training_fp16_at_real_widths():
    """Config 5 at its real widths (64 .. 1024 channels) and resolution (256 x 256), batch 2: forward, backward
    through the transposed convolutions and the strided concat outputs, Adam.  The per-pixel class scores are
    pooled into a classifier head so that the network has a scalar loss (the reference's softmax node has no
    backward pass).  The pooled head divides the gradient by the 65536 pixels, so the loss scale is the size a
    dynamic scale settles at for such a network (4096): at 256 most gradients of the network sit in the
    subnormal range of fp16, where the oracle's own fp16 run differs from its fp32 run by 20 - 30 %."""
    net = N.unet(2, image=256)
    b = N.Builder(net, 99)
    b.shape[net.output] = (8, 256, 256)
    net.output = b.fc(b.pool("avgpool", net.output, global_=True), "cls", 8)
    run_training(net, 6, steps=1, lr=1e-3, loss_scale=4096.0,
                 check_params=["down0a-w", "down3b-w", "mida-w", "up3-t-w", "up0-t-w", "up0a-w", "head-w", "up2-t-b",
                               "up1b-bn-s"])
