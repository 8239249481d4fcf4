"""Payload rows on a pitch (TERRACE_ROW_PITCHED): the row buffers of a call are [n, pitch] bytes with `width` bytes of
data per row.  Every mover, the whole dispatch (both Hop-B forms, with and without a capacity) and the combine must
give, in the data part of every row, exactly what they give on packed rows -- which the other suites hold to the
oracle -- and must never write between a row's end and the next row."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import equal_quota_routing
from oracle import terrace_oracle as orc
from test_gpu_parity import DEV, announce

pytestmark = pytest.mark.gpu

POISON = 0xA5


def _pitched(rows: torch.Tensor, pitch_bytes: int) -> torch.Tensor:
    """The rows as a view of an [n, pitch] buffer whose every other byte is poison."""
    n, width = rows.shape
    base = torch.full((n, pitch_bytes), POISON, dtype=torch.uint8, device=rows.device).view(rows.dtype)
    base[:, :width] = rows
    return base[:, :width]


def _gap_untouched(view: torch.Tensor) -> bool:
    """Whether the bytes between each row's end and the next row still hold the poison."""
    n, width = view.shape
    whole = view.as_strided((n, view.stride(0)), (view.stride(0), 1))
    return bool((whole[:, width:].contiguous().view(torch.uint8) == POISON).all())


@pytest.fixture
def poisoned_outputs(monkeypatch):
    """Every row buffer the wrappers allocate on a pitch starts out full of poison and is remembered."""
    from terrace import _hip
    made = []
    plain = _hip.empty_rows

    def empty_rows(n, like):
        t = plain(n, like)
        if n > 1 and not t.is_contiguous():
            t.as_strided((n, t.stride(0)), (t.stride(0), 1)).view(torch.uint8).fill_(POISON)
            made.append(t)
        return t

    monkeypatch.setattr(_hip, "empty_rows", empty_rows)
    return made


@pytest.mark.parametrize("width,pitch,dtype", [(7392, 8192, torch.uint8), (1200, 2048, torch.bfloat16),
                                               (16, 1024, torch.float32), (1024, 2048, torch.float16),
                                               (3056, 3072, torch.uint8)])
def test_movers_on_a_pitch(width, pitch, dtype, poisoned_outputs):
    import terrace.ops as tops
    announce("pitched movers", width, pitch, dtype)
    g = torch.Generator().manual_seed(width)
    n_src, fan = 301, 3
    elems = width // torch.empty((), dtype=dtype).element_size()
    raw = torch.randint(0, 255, (n_src, width), generator=g, dtype=torch.uint8).view(dtype).reshape(n_src, elems)
    src = _pitched(raw.to(DEV), pitch)
    assert not src.is_contiguous()
    # gather with dead entries
    idx = torch.randint(-2, n_src + 2, (517,), generator=g)
    got = tops.gather_rows(src, idx.to(DEV))
    ok = (idx >= 0) & (idx < n_src)
    want = torch.where(ok[:, None], raw.view(torch.uint8).reshape(n_src, width)[idx.clamp(0, n_src - 1)],
                       torch.zeros((), dtype=torch.uint8))
    assert got.stride(0) * got.element_size() == pitch and torch.equal(got.cpu().view(torch.uint8).reshape(517, width), want)
    # scatter: a permutation of the places, some of them out of range
    n_dst = n_src * fan
    pos = torch.randperm(n_dst, generator=g).reshape(n_src, fan)
    pos[5, 1], pos[7, 0] = -1, n_dst + 3
    out = tops.scatter_rows(src, pos.to(DEV), n_dst)
    out_cpu = out.cpu().view(torch.uint8).reshape(n_dst, width)
    for r in (0, 5, 7, 100, n_src - 1):
        for f in range(fan):
            if 0 <= int(pos[r, f]) < n_dst:
                assert torch.equal(out_cpu[int(pos[r, f])], raw.view(torch.uint8).reshape(n_src, width)[r])
    live = (pos >= 0) & (pos < n_dst)
    flat_src = torch.arange(n_src)[:, None].expand(n_src, fan)[live]
    assert torch.equal(out_cpu[pos[live]], raw.view(torch.uint8).reshape(n_src, width)[flat_src])
    assert len(poisoned_outputs) == 2 and all(_gap_untouched(t) for t in poisoned_outputs)
    assert _gap_untouched(src)


@pytest.mark.parametrize("onepass", [False, True])
@pytest.mark.parametrize("capacity", [None, 40])
def test_dispatch_and_combine_on_a_pitch(onepass, capacity, poisoned_outputs):
    """fp8 rows with their block scales -- 7392 bytes on an 8 KB pitch, 528 bytes on a 1 KB pitch -- against the same
    dispatch on packed rows, plane by plane, and the combine over them against the oracle."""
    import terrace.ops as tops
    from terrace import configs, ta2a_fwd
    announce("pitched dispatch", onepass, capacity)
    for hidden, pitch, T in ((7168, 8192, 257), (512, 1024, 700)):
        world, rpn, E, k, M = 64, 8, 256, 8, 4
        g = torch.Generator().manual_seed(hidden + T)
        e = torch.from_numpy(equal_quota_routing(T, k, E, world // rpn, M, 11, False)).to(DEV)
        gates = torch.rand(T, k, generator=g).to(torch.bfloat16).to(DEV)
        packed = torch.from_numpy(orc.fp8_quantise_rows(torch.randn(T, hidden, generator=g).numpy())).to(DEV)
        x = _pitched(packed, pitch)
        dispatch = ta2a_fwd.loopback_dispatch_onepass if onepass else ta2a_fwd.loopback_dispatch
        a = dispatch(x, e, gates, world, E, rpn, M, capacity)
        b = dispatch(packed, e, gates, world, E, rpn, M, capacity)
        names = ("payload", "permuted") + (() if onepass else ("send_buf",))
        for n in names:
            ta, tb = getattr(a, n), getattr(b, n)
            assert ta.stride(0) == pitch and tb.is_contiguous(), n
            assert torch.equal(ta, tb), n
        assert torch.equal(a.place, b.place) and torch.equal(a.extras["where"], b.extras["where"])
        assert torch.equal(a.tokens_per_expert, b.tokens_per_expert)
        ya = ta2a_fwd.loopback_combine(a.permuted, a, fp8_hidden=hidden)
        yb = ta2a_fwd.loopback_combine(b.permuted, b, fp8_hidden=hidden)
        assert torch.equal(ya.view(torch.int16), yb.view(torch.int16))
        # and against the oracle's combine over the packed expert-order buffer
        want = orc.combine(b.permuted.cpu().numpy(), b.extras["where"].cpu().numpy(),
                           orc.bf16_to_f32(b.extras["gate_sorted"].view(torch.int16).cpu().numpy().view(np.uint16)),
                           "fp8", "bf16", hidden=hidden)
        assert np.array_equal(ya.view(torch.int16).cpu().numpy().view(np.uint16), want)
        assert poisoned_outputs and all(_gap_untouched(t) for t in poisoned_outputs)
        poisoned_outputs.clear()


def test_pitch_refusals():
    import terrace.ops as tops
    from terrace import _hip
    announce("pitched refusals")
    rows = torch.zeros((8, 1024), dtype=torch.uint8, device=DEV)
    idx = torch.arange(8, device=DEV)
    with pytest.raises(RuntimeError, match="invalid argument"):
        tops.gather_rows(rows[:, :100], idx)            # width not a multiple of 16 on a pitch
    wide = torch.zeros((8, 1040), dtype=torch.uint8, device=DEV)
    with pytest.raises(RuntimeError, match="invalid argument"):
        tops.gather_rows(wide[:, :512], idx)            # pitch not a whole number of kilobytes
    src = torch.zeros((4, 1024), dtype=torch.bfloat16, device=DEV)
    table = torch.zeros((1, 2), dtype=torch.int64, device=DEV)
    out = torch.zeros((1, 128), dtype=torch.bfloat16, device=DEV)
    rc = _hip.load().terrace_combine_pitched(_hip.ptr(src), 4, _hip.BF16, 100, _hip.ptr(table), None, 0, 1, 2, 128,
                                             _hip.ptr(out), _hip.BF16, _hip.stream(src.device))
    assert rc == _hip.EINVAL                                # rows closer together than they are wide
