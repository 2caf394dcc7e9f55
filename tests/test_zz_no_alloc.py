"""hipress_onebit_encode_static: the onebit encoder for callers that cannot allocate.

Called through the C ABI and compared bit for bit with hipress_onebit_encode (which takes
its workspace from the caller) on the same inputs, twice in a row on one GPU, the second
time with a smaller tensor, so that what the first call left in the library's static
scratch array lies behind the part the second call uses."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

STATIC_MAX_N = 1 << 28


def _run_pair(L, torch, n, seed, steps=2):
    """Runs `steps` consecutive steps of both entry points on identical inputs; returns
    the two (payload, residual) histories."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    nbytes = int(L.hipress_onebit_payload_bytes(n))
    ws = torch.empty(int(L.hipress_onebit_workspace_bytes(n)), dtype=torch.uint8, device="cuda")
    r_ref, r_new = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    p_ref = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    p_new = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    out = []
    for _ in range(steps):
        g = torch.randn(n, generator=gen, device="cuda") * 0.01
        rc = L.hipress_onebit_encode(g.data_ptr(), r_ref.data_ptr(), n, p_ref.data_ptr(), nbytes, ws.data_ptr(),
                                     ws.numel(), stream)
        assert rc == 0
        rc = L.hipress_onebit_encode_static(g.data_ptr(), r_new.data_ptr(), n, p_new.data_ptr(), nbytes, stream)
        assert rc == 0
        torch.cuda.synchronize()
        out.append((p_ref.cpu().numpy().copy(), r_ref.cpu().numpy().copy(), p_new.cpu().numpy().copy(),
                    r_new.cpu().numpy().copy()))
    return out


def test_static_scratch_encode_equals_the_workspace_encode_on_two_calls_in_a_row():
    import torch

    from hipress_amd import _lib

    L = _lib.lib()
    # first a tensor of 2,359,296 + 37 elements (577 tiles, the last one partial), then a
    # smaller one (24 tiles + a partial one): the second call reuses the front of the array
    for n, seed in ((2359296 + 37, 1), (100003, 2)):
        for step, (p_ref, r_ref, p_new, r_new) in enumerate(_run_pair(L, torch, n, seed)):
            assert np.array_equal(p_ref, p_new), f"payload differs, n={n}, step {step}"
            assert np.array_equal(r_ref.view(np.uint32), r_new.view(np.uint32)), f"residual differs, n={n}, step {step}"
            assert float(p_new[:4].view(np.float32)[0]) > 0.0
            assert int(p_new[4:8].view(np.uint32)[0]) == n


def test_static_scratch_encode_matches_the_oracle():
    import torch

    import oracle
    from hipress_amd import _lib

    L = _lib.lib()
    n = 70001
    g = np.random.default_rng(5).normal(0, 0.02, n).astype(np.float32)
    gd = torch.from_numpy(g).cuda()
    r = torch.zeros(n, device="cuda")
    pay = torch.zeros(int(L.hipress_onebit_payload_bytes(n)), dtype=torch.uint8, device="cuda")
    assert L.hipress_onebit_encode_static(gd.data_ptr(), r.data_ptr(), n, pay.data_ptr(), pay.numel(), None) == 0
    torch.cuda.synchronize()
    got = pay.cpu().numpy()
    s = got[:4].view(np.float32)[0]
    s_ref = oracle.onebit_scale(g, np.zeros(n, np.float32))
    assert abs(float(s) - float(s_ref)) <= 1e-5 * float(s_ref)
    want_pay, want_r = oracle.onebit_encode(g, np.zeros(n, np.float32), scale=s)
    assert np.array_equal(got, want_pay)
    assert np.array_equal(r.cpu().numpy(), want_r)


def test_static_scratch_encode_rejects_what_its_array_cannot_hold():
    from hipress_amd import _lib

    L = _lib.lib()
    # validated on the host before any launch: the pointers are never touched
    fake = ctypes.c_void_p(1 << 20)
    big = STATIC_MAX_N + 1
    assert L.hipress_onebit_encode_static(fake, fake, big, fake, 16 + 4 * ((big + 31) // 32), None) == -2
    assert _lib.strerror(-2).startswith("element count")
    assert L.hipress_onebit_encode_static(None, None, 16, None, 100, None) == -1


def test_static_scratch_encode_under_stream_capture():
    """What the entry point is for: the first call is made eagerly (it looks up the device's
    array), then the same call is captured into a HIP graph and replayed several times with the
    program's own eager work between the replays; every replay must leave what the eager
    workspace encoder leaves for the same gradient and residual."""
    import torch

    from hipress_amd import _lib

    L = _lib.lib()
    n = 300007
    nbytes = int(L.hipress_onebit_payload_bytes(n))
    gen = torch.Generator(device="cuda").manual_seed(9)
    g = torch.randn(n, generator=gen, device="cuda") * 0.01
    r = torch.zeros(n, device="cuda")
    pay = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    assert L.hipress_onebit_encode_static(g.data_ptr(), r.data_ptr(), n, pay.data_ptr(), nbytes,
                                          torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    r.zero_()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = L.hipress_onebit_encode_static(g.data_ptr(), r.data_ptr(), n, pay.data_ptr(), nbytes, side.cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    r.zero_()  # whatever the capture did or did not run, the replays start from a zero residual
    ws = torch.empty(int(L.hipress_onebit_workspace_bytes(n)), dtype=torch.uint8, device="cuda")
    r_ref = torch.zeros(n, device="cuda")
    p_ref = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    for replay in range(4):
        g.copy_(torch.randn(n, generator=gen, device="cuda") * 0.01)  # new gradient in the captured buffer
        pay.fill_(0xAB)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert L.hipress_onebit_encode(g.data_ptr(), r_ref.data_ptr(), n, p_ref.data_ptr(), nbytes, ws.data_ptr(), ws.numel(),
                                       torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(pay, p_ref), f"payload differs in replay {replay}"
        assert torch.equal(r.view(torch.int32), r_ref.view(torch.int32)), f"residual differs in replay {replay}"


def test_static_scratch_array_holds_exactly_the_largest_tensor():
    """Host arithmetic only: the largest n the entry point takes is 65,536 tiles of 4096, the
    size of its array (a static_assert in the library says the same), and one more element is
    one tile too many."""
    from hipress_amd import _lib

    L = _lib.lib()
    assert STATIC_MAX_N % 4096 == 0 and STATIC_MAX_N // 4096 == 65536
    # the workspace encoder asks for one float per tile: the array is that size at the limit
    assert int(L.hipress_onebit_workspace_bytes(STATIC_MAX_N)) >= 65536 * 4
    fake = ctypes.c_void_p(1 << 20)
    assert L.hipress_onebit_encode_static(fake, fake, STATIC_MAX_N + 1, fake, 16 + 4 * ((STATIC_MAX_N + 32) // 32), None) == -2


def test_static_scratch_encode_at_the_largest_size_its_array_holds():
    """n = 2^28: all 65,536 words of the array are in use (the last tile's sum is its last
    word).  Payload and residual equal the workspace encoder's; one more element is refused."""
    import torch

    from hipress_amd import _lib

    L = _lib.lib()
    n = STATIC_MAX_N
    nbytes = int(L.hipress_onebit_payload_bytes(n))
    gen = torch.Generator(device="cuda").manual_seed(3)
    g = torch.randn(n, generator=gen, device="cuda") * 0.01
    g[-4096:] *= 50.0  # the last tile carries weight in the scale: leaving its word out would show
    r_ref, r_new = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    p_ref = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    p_new = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    ws = torch.empty(int(L.hipress_onebit_workspace_bytes(n)), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert L.hipress_onebit_encode(g.data_ptr(), r_ref.data_ptr(), n, p_ref.data_ptr(), nbytes, ws.data_ptr(), ws.numel(), stream) == 0
    assert L.hipress_onebit_encode_static(g.data_ptr(), r_new.data_ptr(), n, p_new.data_ptr(), nbytes, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(p_ref, p_new)
    assert torch.equal(r_ref.view(torch.int32), r_new.view(torch.int32))
    scale = float(p_new[:4].view(torch.float32).item())
    want = float(g.abs().double().mean().item())
    assert abs(scale - want) <= 1e-5 * want
    assert L.hipress_onebit_encode_static(g.data_ptr(), r_new.data_ptr(), n + 1, p_new.data_ptr(), nbytes + 4, stream) == -2
