"""Launch semantics of the boundary on the GPU: the kernel runs on the stream it is given (torch's
current stream in the Python mirror, Utils.py:266-275 of the reference), asynchronously, and ordered
with the other work of that stream."""
import numpy as np
import pytest

from codegendemo_amd.kcg import SeededInputs as SI
from codegendemo_amd.kcg.ConfigGenerator import make_config
from tests.gemm_helpers import build_kernel, to_device

pytestmark = pytest.mark.gpu

M = N = K = 512
CONFIG = make_config(M, N, K, BM=64, BN=64, BK=16, TM=4, TN=4, is_atrans=0)   # precompiled by the build step


def test_launch_is_ordered_on_a_side_stream(oracle):
    import torch
    kpm, ui, kernel, info = build_kernel(CONFIG)
    a = SI.small_ints((M, K), SI.STREAM_A)
    b = SI.small_ints((K, N), SI.STREAM_B)
    want = oracle.matmul(a, b, a_trans=False)
    side = torch.cuda.Stream()           # default priority
    a_host = torch.from_numpy(a).pin_memory()
    b_dev = to_device(b, torch.float32)
    a_dev = torch.empty((M, K), dtype=torch.float32, device="cuda:0")
    c_dev = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda:0")
    torch.cuda.synchronize()
    print("[case] side-stream launch 512^3", flush=True)
    with torch.cuda.stream(side):
        # upload -> GEMM -> scale, all queued on the side stream without host synchronisation:
        # the GEMM must see the uploaded A and the scaling must see the finished C
        a_dev.copy_(a_host, non_blocking=True)
        kernel.run(a_dev, b_dev, c_dev)
        c_dev.mul_(2.0)
    side.synchronize()
    got = c_dev.cpu().numpy()
    kernel.unload()
    assert np.array_equal(got, 2.0 * want)
