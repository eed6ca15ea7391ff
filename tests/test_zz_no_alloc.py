"""The pick that allocates nothing (xr_sample_static) against xr_sample, called through ctypes:
two calls in a row on one GPU, the second with fewer and shorter rows, so that what the first
call left in the library's own work area lies beside what the second one writes."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

P, I, F = C.c_void_p, C.c_int, C.c_float
COMMON = [P, P, I, I, I, P, P, P, P, P, P, P, P, I, P, I]      # out, logits, W, V, ld, temp .. n_exempt


def _picks(dll, static, logits, temp, draw):
    """Token ids of one call; ``logits [W, V]`` float32, ``temp`` and ``draw`` ``[W]`` on the GPU."""
    import torch
    W, V = logits.shape
    out = torch.full((W,), -7, dtype=torch.int32, device=logits.device)
    stream = torch.cuda.current_stream().cuda_stream
    args = [out.data_ptr(), logits.data_ptr(), W, V, logits.stride(0), temp.data_ptr(), None, None, None, None,
            draw.data_ptr(), None, None, 0, None, 0]
    if static:
        rc = dll.xr_sample_static(*args, stream)
    else:
        ws = torch.empty((W, 32, 2), dtype=torch.float32, device=logits.device)
        rc = dll.xr_sample(*args, ws.data_ptr(), stream)
    assert rc == 0, dll.xr_last_error().decode()
    return out.cpu().tolist()


def test_sample_static_matches_sample_on_two_calls_in_a_row():
    import torch
    from xyntetik_runner_amd.csrc.ops import load_ops
    dll = C.CDLL(load_ops().lib.path)
    dll.xr_last_error.restype = C.c_char_p
    dll.xr_sample.argtypes = COMMON + [P, P]
    dll.xr_sample_static.argtypes = COMMON + [P]
    dll.xr_sample.restype = dll.xr_sample_static.restype = dll.xr_sample_static_init.restype = I
    assert dll.xr_sample_static_init() == 0, dll.xr_last_error().decode()
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(11)
    for W, V in ((37, 50021), (5, 1003)):               # the second call is smaller in both sizes
        lg = rng.standard_normal((W, V)).astype(np.float32)
        lg[0, V - 1] = lg[0, 17] = 9.0                   # a tie: the first index wins
        lg[W - 1, :] = -3.0                              # all equal: index 0
        temp_h = np.zeros(W, dtype=np.float32)
        temp_h[1::4] = 0.7                               # sampled rows between the greedy ones
        logits = torch.tensor(lg, device=dev)
        temp = torch.tensor(temp_h, device=dev)
        draw = torch.tensor(rng.random(W).astype(np.float32), device=dev)
        want = _picks(dll, False, logits, temp, draw)
        got = _picks(dll, True, logits, temp, draw)
        assert got == want
        greedy = [r for r in range(W) if temp_h[r] == 0]
        assert [got[r] for r in greedy] == [int(np.argmax(lg[r])) for r in greedy]
        assert got[0] == 17 and got[W - 1] == 0
        # the sampled rows against the plain sampler (not only against the sibling entry point)
        import plain_llama as Plain
        for r in range(1, W, 4):
            assert got[r] == Plain.sample_pick(lg[r], 0.7, float(draw[r].item())), r
        assert torch.equal(logits.cpu(), torch.tensor(lg))          # logits untouched


def test_sample_static_refuses_more_rows_than_its_work_area_holds():
    import torch
    from xyntetik_runner_amd.csrc.ops import load_ops
    dll = C.CDLL(load_ops().lib.path)
    dll.xr_last_error.restype = C.c_char_p
    dll.xr_sample_static.argtypes = COMMON + [P]
    dll.xr_sample_static.restype = I
    dev = torch.device("cuda:0")
    W = 1025
    logits = torch.zeros((W, 8), device=dev)
    z = torch.zeros((W,), device=dev)
    out = torch.zeros((W,), dtype=torch.int32, device=dev)
    rc = dll.xr_sample_static(out.data_ptr(), logits.data_ptr(), W, 8, 8, z.data_ptr(), None, None, None, None,
                              z.data_ptr(), None, None, 0, None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc != 0 and b"1024" in dll.xr_last_error()
