"""Device time of every distinct convolution of a ResNet-50 (u8 activations with zero point 128, i8 weights, ReLU,
u8 output; the three image channels of the first layer padded to 16) through vpx_nce_task, one layer after the other.

    python vpux_plugin_amd/examples/resnet50_layers.py [batch]

Each layer is captured in a HIP graph of 30 launches and the graph replayed once between two events, so the figure is
device time per launch without the host's launch cost.  Random data; nothing is checked here (the parity tests do that).
"""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))  # the repository root
from vpux_plugin_amd import runtime as rt  # noqa: E402

# name, input height = width, input channels, output channels, kernel, stride
LAYERS = [
    ("conv1 7x7", 224, 16, 64, 7, 2),
    ("conv2 1x1 64-64", 56, 64, 64, 1, 1), ("conv2 3x3 64", 56, 64, 64, 3, 1), ("conv2 1x1 64-256", 56, 64, 256, 1, 1),
    ("conv2 1x1 256-64", 56, 256, 64, 1, 1),
    ("conv3 1x1 256-128", 56, 256, 128, 1, 1), ("conv3 3x3 128 /2", 56, 128, 128, 3, 2), ("conv3 1x1 128-512", 28, 128, 512, 1, 1),
    ("conv3 1x1 512-128", 28, 512, 128, 1, 1), ("conv3 3x3 128", 28, 128, 128, 3, 1), ("conv3 shortcut 256-512 /2", 56, 256, 512, 1, 2),
    ("conv4 1x1 512-256", 28, 512, 256, 1, 1), ("conv4 3x3 256 /2", 28, 256, 256, 3, 2), ("conv4 1x1 256-1024", 14, 256, 1024, 1, 1),
    ("conv4 1x1 1024-256", 14, 1024, 256, 1, 1), ("conv4 3x3 256", 14, 256, 256, 3, 1), ("conv4 shortcut 512-1024 /2", 28, 512, 1024, 1, 2),
    ("conv5 1x1 1024-512", 14, 1024, 512, 1, 1), ("conv5 3x3 512 /2", 14, 512, 512, 3, 2), ("conv5 1x1 512-2048", 7, 512, 2048, 1, 1),
    ("conv5 1x1 2048-512", 7, 2048, 512, 1, 1), ("conv5 3x3 512", 7, 512, 512, 3, 1), ("conv5 shortcut 1024-2048 /2", 14, 1024, 2048, 1, 2),
]


def time_layer(name, N, H, IC, OC, K, stride, launches=30):
    dev = torch.device("cuda")
    inp = torch.randint(0, 256, (N, H, H, IC), dtype=torch.uint8, device=dev)
    w = torch.randint(-127, 128, (OC, K, K, IC), dtype=torch.int8, device=dev)
    wt = torch.from_numpy(rt.make_weights_table(np.full(OC, 20000), np.full(OC, 22), np.zeros(OC, np.int32), K * K * IC)).to(dev)
    pad = K // 2
    OH = (H + 2 * pad - K) // stride + 1
    out = torch.empty((N, OH, OH, OC), dtype=torch.uint8, device=dev)
    ppe = rt.PpeInt(rt.PPE_LRELU, 0, 255, 1, 0)

    def run(s=None):
        rt.nce_task(inp, w, wt, out, ppe, zp_in=128, strides=(stride, stride), pads=(pad, pad, pad, pad), stream=s)
    for _ in range(3):
        run()
    torch.cuda.synchronize()
    graph, s = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(s):
        run(s)  # (the first use of a stream may size the library's scratch buffer: not while capturing)
        s.synchronize()
        with torch.cuda.graph(graph, stream=s):
            for _ in range(launches):
                run(s)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    graph.replay()
    torch.cuda.synchronize()
    e0.record()
    graph.replay()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1000 / launches
    gop = 2.0 * N * OH * OH * OC * K * K * IC / 1e9
    print("%-28s [%d,%d,%d,%d] -> %d, %dx%d, stride %d: %-16s %6.1f us  %6.2f GOP  %5.2f POP/s" % (
        name, N, H, H, IC, OC, K, K, stride, rt.nce_last_kernel(), us, gop, gop / us), flush=True)
    return us, gop


def main():
    batch = int(sys.argv[1]) if len(sys.argv) > 1 else 32
    rt.lib()
    total_us = total_gop = 0.0
    for name, hw, ic, oc, k, s in LAYERS:
        us, gop = time_layer(name, batch, hw, ic, oc, k, s)
        total_us += us
        total_gop += gop
    print("one of each: %.0f us, %.1f GOP, %.2f POP/s" % (total_us, total_gop, total_gop / total_us))


if __name__ == "__main__":
    main()
