"""deepep_ll_dispatch_send_static (route scratch inside the library image, nothing allocated) against
deepep_ll_dispatch_send on the same inputs: every output bit for bit, on two calls in a row, the second
with a smaller batch.  Both batches are past 8192 (token, k) entries, where the send kernel reads the
chunk histograms that live in the scratch."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_static_scratch_send_equals_workspace_send():
    from deepep_efa_amd import _capi, ll_runtime, loopback
    lib = _capi.load()
    assert torch.cuda.is_available(), "this test needs the MI355X"
    r, rank, m, h, k, e = 4, 1, 1400, 512, 8, 64
    fmt = ll_runtime.ROW_FP8
    shape = ll_runtime.LLShape(r, rank, e, m, h, k, fmt)
    a = ll_runtime.LowLatencyState(shape)  # through the workspace entry point
    b = ll_runtime.LowLatencyState(shape)  # through the static-scratch entry point
    stream = torch.cuda.current_stream().cuda_stream
    for call, t in enumerate((1400, 1100)):  # 11200 and 8800 entries: chunks of 256 tokens
        assert t * k > 8192
        world = loopback.LoopbackWorld(r, rank, seed=100 + call)
        world.synthesise(t, h, k, e)
        x, topk = world.own_inputs()
        topk = topk.clone()
        topk[::17, 3] = -1  # a few dropped selections
        for st in (a, b):
            st.recv_staging.fill_(0xEE), st.send_slots.fill_(0xEE)
            st.send_count.fill_(-7), st.recv_count.fill_(-7), st.pair_slot.fill_(-7)
        a.dispatch_send(x, topk)
        _capi.check(lib.deepep_ll_dispatch_send_static(
            _capi.ptr(x), _capi.ptr(topk), t, h, k, e, r, rank, m, fmt, _capi.ptr(b.recv_staging),
            _capi.ptr(b.recv_count), _capi.ptr(b.send_slots), _capi.ptr(b.send_count), _capi.ptr(b.pair_slot), stream))
        torch.cuda.synchronize()
        assert int((a.pair_slot[:t] >= 0).sum()) == t * k - len(range(0, t, 17))  # the reference call did its work
        assert torch.equal(a.send_count, b.send_count)
        assert torch.equal(a.recv_count, b.recv_count)
        assert torch.equal(a.pair_slot, b.pair_slot)
        assert torch.equal(a.recv_staging, b.recv_staging)  # rows written and 0xEE elsewhere, byte for byte
        assert torch.equal(a.send_slots, b.send_slots)


def test_static_scratch_send_rejects_a_batch_beyond_its_scratch():
    from deepep_efa_amd import _capi
    lib = _capi.load()
    # 1 MiB of scratch holds ceil(T / 256) * E * 4 bytes at top-8: T = 300000 tokens of 256 experts do not fit
    rc = lib.deepep_ll_dispatch_send_static(None, None, 300000, 512, 8, 256, 8, 0, 300000, 1, None, None, None, None,
                                            None, None)
    assert rc != 0
    assert "static route scratch" in lib.deepep_last_error().decode()
