"""ucm_esa_retrieve_static - the entry point that allocates nothing (its candidate scores go to a scratch array
inside the library image) - against ucm_esa_retrieve, through the C ABI: identical indices, scores and counts, on
two calls in a row, the second with a smaller input, so that what the first call left in the shared scratch must not
show in the second's results."""
import numpy as np
import pytest
import torch

import synth

pytestmark = pytest.mark.gpu


def _both(ucm, dev, data, q, idx, topk):
    from ucm_amd import _lib

    batch, m = idx.shape
    stride = max(min(topk, m), 1)
    outs = []
    for static in (False, True):
        out_i = torch.full((batch, stride), -7, dtype=torch.int32, device=dev)
        out_s = torch.full((batch, stride), -7.0, dtype=torch.float32, device=dev)
        out_c = torch.full((batch,), -7, dtype=torch.int32, device=dev)
        stream = torch.cuda.current_stream().cuda_stream
        head = (data.data_ptr(), data.shape[0], data.shape[1], q.data_ptr(), idx.data_ptr(), batch, m, topk)
        tail = (out_i.data_ptr(), out_s.data_ptr(), out_c.data_ptr(), stride, stream)
        if static:
            # neither torch's allocator nor the driver hands out memory during the call (a hipMalloc inside the
            # library would not show in torch's own count, it does in the device's free memory)
            torch.cuda.synchronize()
            before, free_before = torch.cuda.memory_allocated(dev), torch.cuda.mem_get_info(dev)[0]
            _lib.call("ucm_esa_retrieve_static", *head, *tail)
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated(dev) == before
            assert torch.cuda.mem_get_info(dev)[0] == free_before
        else:
            ws = torch.zeros(batch * m, dtype=torch.float32, device=dev)
            _lib.call("ucm_esa_retrieve", *head, ws.data_ptr(), *tail)
        torch.cuda.synchronize()
        outs.append((out_i.cpu().numpy(), out_s.cpu().numpy().view(np.uint32), out_c.cpu().numpy()))
    return outs


def test_esa_retrieve_static_matches_workspace_variant(ucm, dev):
    from ucm_amd import _lib

    rows, dim = 3000, 1024
    data = torch.from_numpy(synth.normal_bf16_as_f32(9100, (rows, dim))).to(dev)
    for call, (batch, m, topk) in enumerate([(5, 2100, 300), (3, 200, 64)]):     # long lists first, then a smaller call
        q = torch.from_numpy(synth.normal_bf16_as_f32(9101 + call, (batch, dim))).to(dev)
        idx_h = np.stack([synth.permutation(9110 + 10 * call + r, rows)[:m] for r in range(batch)]).astype(np.int32)
        idx_h[:, m - 5 :] = -1
        idx_h[0, ::7] = -1
        idx = torch.from_numpy(idx_h).to(dev)
        (wi, ws, wc), (gi, gs, gc) = _both(ucm, dev, data, q, idx, topk)
        assert np.array_equal(gc, wc) and wc.min() > 0
        assert np.array_equal(gi, wi) and np.array_equal(gs, ws), call
    # a call beyond the built-in scratch is refused on the host, before anything is launched
    with pytest.raises(_lib.UcmHipError) as e:
        _lib.call("ucm_esa_retrieve_static", data.data_ptr(), rows, dim, data.data_ptr(), data.data_ptr(), 65, 8192, 4,
                  data.data_ptr(), data.data_ptr(), data.data_ptr(), 4, None)
    assert e.value.code == _lib.ENOTSUP and "scratch" in str(e.value)
