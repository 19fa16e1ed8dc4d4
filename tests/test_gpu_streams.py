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
# the direct-staging kernel (static LDS stages, bare barriers and hand-counted waits in its K loop)
CONFIG_DIRECT = make_config(M, N, K, BM=128, BN=128, BK=32, TM=8, TN=8, is_atrans=0, shared_prefetch=1, reg_prefetch=1)
CONFIGS = {"register-staged": CONFIG, "direct-staging": CONFIG_DIRECT}


@pytest.mark.parametrize("which", list(CONFIGS))
def test_launch_is_ordered_on_a_side_stream(oracle, which):
    import torch
    kpm, ui, kernel, info = build_kernel(CONFIGS[which])
    assert (info["lds_bytes"] == 0) == (which == "direct-staging")
    a = SI.small_ints((M, K), SI.STREAM_A)
    b = SI.small_ints((K, N), SI.STREAM_B)
    want = oracle.matmul(a, b, a_trans=False)
    side = torch.cuda.Stream()           # default priority
    a_host = torch.from_numpy(a).pin_memory()
    b_dev = to_device(b, torch.float32)
    a_dev = torch.empty((M, K), dtype=torch.float32, device="cuda:0")
    c_dev = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda:0")
    torch.cuda.synchronize()
    print(f"[case] side-stream launch 512^3 {which}", flush=True)
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


@pytest.mark.parametrize("which", list(CONFIGS))
def test_launch_can_be_captured_in_a_hip_graph(oracle, which):
    """A launch through the boundary allocates nothing and synchronises nothing, so a caller may capture it
    into a HIP graph (once the module is loaded: the first run of a kernel loads it, which is not capturable).
    The graph is replayed four times on different operands with eager work and synchronisations in between;
    every replay must equal the eager result and the oracle bit for bit (small integers)."""
    import torch
    kpm, ui, kernel, info = build_kernel(CONFIGS[which])
    b = SI.small_ints((K, N), SI.STREAM_B)
    b_dev = to_device(b, torch.float32)
    a_dev = torch.zeros((M, K), dtype=torch.float32, device="cuda:0")
    c_dev = torch.zeros((M, N), dtype=torch.float32, device="cuda:0")
    c_eager = torch.zeros((M, N), dtype=torch.float32, device="cuda:0")
    print(f"[case] graph capture 512^3 {which}", flush=True)
    kernel.run(a_dev, b_dev, c_dev)      # loads the module
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()           # default priority
    with torch.cuda.graph(graph, stream=side):
        kernel.run(a_dev, b_dev, c_dev)
        c_dev.mul_(2.0)
    torch.cuda.synchronize()
    for rep in range(4):
        a = SI.small_ints((M, K), SI.STREAM_A, seed=SI.SEED + rep)
        a_dev.copy_(to_device(a, torch.float32))
        c_dev.fill_(float("nan"))        # a fill kernel, eager, outside the graph
        torch.cuda.synchronize()
        print(f"        replay {rep}", flush=True)
        graph.replay()
        torch.cuda.synchronize()
        kernel.run(a_dev, b_dev, c_eager)
        c_eager.mul_(2.0)
        torch.cuda.synchronize()
        got = c_dev.cpu().numpy()
        assert np.array_equal(got, c_eager.cpu().numpy()), f"replay {rep} differs from the eager result"
        assert np.array_equal(got, 2.0 * oracle.matmul(a, b, a_trans=False)), f"replay {rep} differs from the oracle"
    del graph
    kernel.unload()
