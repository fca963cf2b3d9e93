"""kge_margin_loss_static (the entry point that allocates nothing) against kge_margin_loss.

Collected last on purpose (file name): a failure here must not hide the parity tests."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(L, pos, neg, margin, sign):
    B, N = neg.shape
    dev = pos.device
    P = lambda t: C.c_void_p(t.data_ptr())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    for static in (False, True):
        loss = torch.full((1,), -7.0, device=dev)
        dpos, dneg = torch.full_like(pos, -7.0), torch.full_like(neg, -7.0)
        if static:
            rc = L.kge_margin_loss_static(P(pos), P(neg), B, N, margin, sign, P(loss), P(dpos), P(dneg), st)
        else:
            ws = torch.empty(max(int(L.kge_margin_loss_workspace(B, N)), 1), dtype=torch.uint8, device=dev)
            rc = L.kge_margin_loss(P(pos), P(neg), B, N, margin, sign, P(loss), P(dpos), P(dneg), P(ws), ws.numel(), st)
        assert rc == 0
        torch.cuda.synchronize()
        out.append((loss.cpu().numpy(), dpos.cpu().numpy(), dneg.cpu().numpy()))
    return out


def test_static_scratch_margin_loss_matches_the_workspace_form_on_two_calls_in_a_row():
    from cuke_amd import _lib
    L = _lib.lib()
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(5)
    # the second call is smaller: whatever the first left in the shared scratch must not leak into it
    for B, N, margin, sign in ((4096, 256, 1.0, 1.0), (1000, 37, 0.5, -1.0)):
        print(f"margin loss static: B={B} N={N}", flush=True)
        pos = torch.randn(B, generator=g).to(dev)
        neg = torch.randn(B, N, generator=g).to(dev)
        (l0, dp0, dn0), (l1, dp1, dn1) = _both(L, pos, neg, margin, sign)
        assert np.array_equal(l0, l1) and np.array_equal(dp0, dp1) and np.array_equal(dn0, dn1)
        ref = torch.clamp(margin - sign * (pos.double()[:, None] - neg.double()), min=0).mean().item()
        assert abs(float(l1[0]) - ref) <= 1e-6 * max(1.0, abs(ref))


def test_static_scratch_margin_loss_rejects_batches_beyond_its_limit_before_launching():
    from cuke_amd import _lib
    L = _lib.lib()
    fake = C.c_void_p(0x1000)
    assert L.kge_margin_loss_static(fake, fake, 65537, 4, 1.0, 1.0, fake, None, None, None) == -4
