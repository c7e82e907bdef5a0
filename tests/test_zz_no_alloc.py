"""plh_lsr_forward_reduced_static (the entry point that allocates nothing; its partials live in a
device array inside the library) against plh_lsr_forward_reduced (caller's workspace), both called
straight through the C ABI: two calls in a row, the second on a smaller input, results bit-identical
(same kernels, same fixed-order reduction), and against the CPU oracle to the usual loss bar."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from oracle import synth

pytestmark = pytest.mark.gpu


def _run(lib, entry, x, y, ignore, smooth, mean, with_losses, workspace=None):
    n, c = x.shape[0], x.shape[1]
    m = x.numel() // (n * c)
    loss = torch.full((1,), -7.0, device=x.device)
    cnt = torch.full((1,), -7, dtype=torch.int64, device=x.device)
    per = torch.full((n, m), -7.0, device=x.device) if with_losses else None
    p = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if workspace is None:
        rc = getattr(lib, entry)(p(x), 0, p(y), p(per), p(loss), p(cnt), mean, n, c, m, ignore, smooth, st)
    else:
        rc = getattr(lib, entry)(p(x), 0, p(y), p(per), p(loss), p(cnt), mean, p(workspace), workspace.numel(),
                                 n, c, m, ignore, smooth, st)
    assert rc == 0, (entry, rc, lib.plh_error_string(rc))
    torch.cuda.synchronize()
    return loss.cpu().numpy()[0], int(cnt.item()), (per.cpu().numpy() if per is not None else None)


def test_static_scratch_entry_point_matches_workspace_entry_point():
    from pytorch_loss import _native
    lib = _native.load()
    dev = torch.device("cuda:0")
    # second call smaller than the first; the third shape takes another kernel form (rows in a wavefront)
    shapes = [((4, 19, 256, 256), 255), ((2, 19, 7, 9), 255), ((300, 100), -100), ((2, 19, 64, 64), 255)]
    for i, (shape, ignore) in enumerate(shapes):
        x_np = synth.normal(40 + i, 1, shape, 0.0, 2.0)
        y_np = synth.seg_labels(40 + i, shape[:1] + shape[2:], shape[1], ignore, 0.1)
        x = torch.from_numpy(x_np).to(dev)
        y = torch.from_numpy(y_np).to(dev)
        n_pix = y.numel()
        ws = torch.empty(lib.plh_reduce_workspace_bytes(n_pix), dtype=torch.uint8, device=dev)
        for mean in (1, 0):
            for with_losses in (False, True):
                want = _run(lib, "plh_lsr_forward_reduced", x, y, ignore, 0.1, mean, with_losses, ws)
                got = _run(lib, "plh_lsr_forward_reduced_static", x, y, ignore, 0.1, mean, with_losses)
                assert np.float32(got[0]).tobytes() == np.float32(want[0]).tobytes(), (shape, mean, got[0], want[0])
                assert got[1] == want[1] == int((y_np != ignore).sum())
                if with_losses:
                    assert np.array_equal(got[2], want[2])
                per = oracle.lsr_forward(x_np.astype(np.float64), y_np, ignore, 0.1)
                ref = per.sum() / (got[1] if mean else 1)
                assert abs(got[0] - ref) <= 1e-5 * abs(ref), (shape, mean, got[0], ref)


def test_static_scratch_entry_point_rejects_oversize_and_bad_arguments():
    from pytorch_loss import _native
    lib = _native.load()
    dev = torch.device("cuda:0")
    x = torch.zeros(8, device=dev)
    y = torch.zeros(8, dtype=torch.int64, device=dev)
    out = torch.zeros(1, device=dev)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    # more pixels than the built-in buffer serves: refused before anything is launched
    assert lib.plh_lsr_forward_reduced_static(p(x), 0, p(y), None, p(out), None, 1, (1 << 24) + 1, 2, 1, 255, 0.1, None) == -2
    assert lib.plh_lsr_forward_reduced_static(p(x), 0, p(y), None, p(out), None, 1, 1 << 13, 2, 1 << 12, 255, 0.1, None) == -2
    assert lib.plh_lsr_forward_reduced_static(p(x), 0, p(y), None, p(out), None, 1, -1, 2, 1, 255, 0.1, None) == -2
    assert lib.plh_lsr_forward_reduced_static(p(x), 7, p(y), None, p(out), None, 1, 1, 2, 1, 255, 0.1, None) == -7
    assert lib.plh_lsr_forward_reduced_static(p(x), 0, p(y), None, None, None, 1, 2, 2, 2, 255, 0.1, None) == -1
    torch.cuda.synchronize()


def test_static_scratch_entry_point_allocates_nothing_and_replays_from_a_graph():
    """What the entry point is for: the device's free memory is the same before and after its calls (the first call
    on a device, which looks the scratch array's address up, has happened by then), and a call captured in a HIP
    graph replays to the bits of the eager call, with eager work between the replays."""
    from pytorch_loss import _native
    lib = _native.load()
    dev = torch.device("cuda:0")
    shape, ignore = (3, 19, 96, 80), 255
    x_np = synth.normal(47, 1, shape, 0.0, 2.0)
    y_np = synth.seg_labels(47, shape[:1] + shape[2:], shape[1], ignore, 0.1)
    x, y = torch.from_numpy(x_np).to(dev), torch.from_numpy(y_np).to(dev)
    n, c, m = shape[0], shape[1], shape[2] * shape[3]
    loss = torch.zeros(1, device=dev)
    cnt = torch.zeros(1, dtype=torch.int64, device=dev)
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    def call(stream):
        rc = lib.plh_lsr_forward_reduced_static(p(x), 0, p(y), None, p(loss), p(cnt), 1, n, c, m, ignore, 0.1,
                                                ctypes.c_void_p(stream))
        assert rc == 0, rc

    call(torch.cuda.current_stream().cuda_stream)            # first call on the device: outside any capture
    torch.cuda.synchronize()
    want = (loss.clone(), cnt.clone())
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(5):
        call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(loss, want[0]) and torch.equal(cnt, want[1])

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(torch.cuda.current_stream().cuda_stream)
    for i in range(3):
        loss.fill_(-1.0)
        cnt.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(loss, want[0]) and torch.equal(cnt, want[1]), i
        # eager work between the replays, on the same scratch array (a smaller input)
        small = _run(lib, "plh_lsr_forward_reduced_static", x[:1].contiguous(), y[:1].contiguous(), ignore, 0.1, 1, False)
        assert small[1] == int((y_np[:1] != ignore).sum())
    per = oracle.lsr_forward(x_np.astype(np.float64), y_np, ignore, 0.1)
    ref = per.sum() / int((y_np != ignore).sum())
    assert abs(float(want[0].item()) - ref) <= 1e-5 * abs(ref)
