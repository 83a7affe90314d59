"""The allocation-free forward entry point (mlstm_hip_chunkwise_fw_noalloc) against the regular one
(mlstm_hip_chunkwise_fw with a caller-provided workspace), both called through the C ABI: identical kernels on
identical inputs, so H and the last states must agree bit for bit.  Two calls in a row share the library's static
scratch, the second with a smaller input (stale contents of the first call must not leak into it); a shape beyond the
scratch is rejected with a message."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call_both(B, NH, S, DHQK, DHHV, seed, gate, init):
    from mlstm_kernels_amd import _lib
    from mlstm_kernels_amd.torch.utils import current_stream_ptr, ptr

    lib = _lib.get_lib()
    dev = torch.device("cuda")
    g = torch.Generator(device=dev).manual_seed(seed)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    q, k, v = rn(B, NH, S, DHQK).bfloat16(), rn(B, NH, S, DHQK).bfloat16(), rn(B, NH, S, DHHV).bfloat16()
    i, f = rn(B, NH, S), 3 + rn(B, NH, S)
    c0 = n0 = m0 = None
    if init:
        c0, n0, m0 = 0.1 * rn(B, NH, DHQK, DHHV), 0.1 * rn(B, NH, DHQK), 0.3 * rn(B, NH)
    outs = []
    for noalloc in (False, True):
        H = torch.empty(B, NH, S, DHHV, dtype=torch.bfloat16, device=dev)
        n_out, m_out = torch.empty(B, NH, S, device=dev), torch.empty(B, NH, S, device=dev)
        c_last, n_last, m_last = torch.empty(B, NH, DHQK, DHHV, device=dev), torch.empty(B, NH, DHQK, device=dev), torch.empty(B, NH, device=dev)
        head = [ptr(q), ptr(k), ptr(v), ptr(i), ptr(f), ptr(c0), ptr(n0), ptr(m0), ptr(H), ptr(n_out), ptr(m_out),
                ptr(c_last), ptr(n_last), ptr(m_last)]
        tail = [B, NH, S, DHQK, DHHV, 1e-6, _lib.BF16, _lib.F32, gate, 1]
        if noalloc:
            rc = lib.mlstm_hip_chunkwise_fw_noalloc(*head, *tail, current_stream_ptr(dev))
            _lib.check(rc, "mlstm_hip_chunkwise_fw_noalloc")
        else:
            ws_bytes = lib.mlstm_hip_chunkwise_fw_workspace_bytes(B, NH, S, DHQK, DHHV, 0, _lib.PATH_AUTO, 0)
            assert 0 < ws_bytes <= _lib.NOALLOC_SCRATCH_BYTES
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            rc = lib.mlstm_hip_chunkwise_fw(*head, ptr(ws), ws_bytes, 0, *tail, _lib.PATH_AUTO, 0, _lib.NORM_NONE, 0.0, None, None,
                                    current_stream_ptr(dev))
            _lib.check(rc, "mlstm_hip_chunkwise_fw")
        torch.cuda.synchronize()
        outs.append((H, n_out, m_out, c_last, n_last, m_last))
    return outs


def test_noalloc_forward_matches_the_workspace_entry_point_on_two_calls_in_a_row():
    from mlstm_kernels_amd import _lib

    # first call: 8 heads x 2304 positions (ragged last chunk) at the xLSTM-7B head shape, about 21 MB of scratch;
    # second call: a smaller input, other head dimensions, sigmoid gate, initial state
    for (B, NH, S, DHQK, DHHV, seed, gate, init) in [(1, 8, 2300, 256, 512, 0, _lib.GATE_EXP, False),
                                                     (2, 2, 200, 128, 192, 1, _lib.GATE_SIG, True)]:
        ref, got = _call_both(B, NH, S, DHQK, DHHV, seed, gate, init)
        for name, a, b in zip(["H", "n_out", "m_out", "c_last", "n_last", "m_last"], ref, got):
            if gate == _lib.GATE_SIG and name == "m_out":
                continue  # written as zeros by both; compared below like the rest
            assert torch.equal(a, b), f"{name} differs between the two entry points (S={S})"
        assert not torch.isnan(got[0].float()).any()


def test_noalloc_forward_in_a_hip_graph_after_one_eager_call():
    """The entry point is meant for callers under HIP graph capture.  Its first call on a device looks the scratch
    address up and sets kernel attributes (host-side work that does not belong into a capture), so ONE eager call per
    device and shape comes first; after it the call is captured and replayed, with eager work between the replays:
    every replay reproduces the eager result bit for bit."""
    from mlstm_kernels_amd import _lib
    from mlstm_kernels_amd.torch.utils import current_stream_ptr, ptr

    lib = _lib.get_lib()
    dev = torch.device("cuda")
    B, NH, S, DHQK, DHHV = 1, 4, 1024, 256, 512
    g = torch.Generator(device=dev).manual_seed(7)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    q, k, v = rn(B, NH, S, DHQK).bfloat16(), rn(B, NH, S, DHQK).bfloat16(), rn(B, NH, S, DHHV).bfloat16()
    i, f = rn(B, NH, S), 3 + rn(B, NH, S)
    H = torch.empty(B, NH, S, DHHV, dtype=torch.bfloat16, device=dev)
    c_last, n_last, m_last = torch.empty(B, NH, DHQK, DHHV, device=dev), torch.empty(B, NH, DHQK, device=dev), torch.empty(B, NH, device=dev)

    def call():
        rc = lib.mlstm_hip_chunkwise_fw_noalloc(ptr(q), ptr(k), ptr(v), ptr(i), ptr(f), None, None, None, ptr(H), None, None,
                                                ptr(c_last), ptr(n_last), ptr(m_last), B, NH, S, DHQK, DHHV, 1e-6, _lib.BF16,
                                                _lib.F32, _lib.GATE_EXP, 1, current_stream_ptr(dev))
        _lib.check(rc, "mlstm_hip_chunkwise_fw_noalloc")

    call()  # the eager warm-up call
    torch.cuda.synchronize()
    H_ref, c_ref = H.clone(), c_last.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(3):
        H.zero_()
        c_last.zero_()
        q2 = (q.float() * 0.5).bfloat16()   # eager work of the program's own between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(H, H_ref) and torch.equal(c_last, c_ref), f"replay {rep} differs from the eager call"
    del q2


def test_noalloc_forward_rejects_shapes_beyond_the_static_scratch():
    from mlstm_kernels_amd import _lib
    from mlstm_kernels_amd.torch.utils import current_stream_ptr, ptr

    lib = _lib.get_lib()
    dev = torch.device("cuda")
    B, NH, S, DHQK, DHHV = 1, 8, 16384, 256, 512   # 8 heads x 64 kept states x 256 KiB = 128 MiB of states alone
    assert lib.mlstm_hip_chunkwise_fw_workspace_bytes(B, NH, S, DHQK, DHHV, 0, _lib.PATH_AUTO, 0) > _lib.NOALLOC_SCRATCH_BYTES
    q = torch.zeros(B, NH, S, DHQK, dtype=torch.bfloat16, device=dev)
    v = torch.zeros(B, NH, S, DHHV, dtype=torch.bfloat16, device=dev)
    g = torch.zeros(B, NH, S, device=dev)
    H = torch.empty_like(v)
    rc = lib.mlstm_hip_chunkwise_fw_noalloc(ptr(q), ptr(q), ptr(v), ptr(g), ptr(g), None, None, None, ptr(H), None, None,
                                            None, None, None, B, NH, S, DHQK, DHHV, 1e-6, _lib.BF16, _lib.F32,
                                            _lib.GATE_EXP, 1, current_stream_ptr(dev))
    assert rc != 0
    msg = lib.mlstm_hip_last_error().decode()
    assert "static scratch" in msg and "caller-provided workspace" in msg
