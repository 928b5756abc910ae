"""GPU test of the entry point that allocates nothing (`ntfp8_quantize_delayed_batch_static`): its reduction
workspaces live in a static array inside the library's device image, for callers that cannot allocate device memory
(HIP graph capture, serving loops).  It must give what `ntfp8_quantize_delayed_batch` gives, bit for bit, on two calls
in a row, the second with smaller inputs (the array keeps whatever the first call left in it)."""
import pytest
import torch

from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().float().cpu().contiguous().view(torch.int32)


def _same(a, b):
    """fp32 values equal bit for bit; NaNs equal whatever their payload"""
    a, b = a.detach().float().cpu().reshape(-1), b.detach().float().cpu().reshape(-1)
    return bool(torch.all((a.view(torch.int32) == b.view(torch.int32)) | (a.isnan() & b.isnan())))


def _run(entry, xs, fmt, states, with_t, static):
    """One call of `entry` over the tensors xs; returns per tensor (bytes, transposed bytes or None, [amax, scale used])."""
    from nanotron_amd import _native as nt

    dev = xs[0].device
    descs = (nt.QuantDesc * len(xs))()
    if static:
        pool, st = None, nt.stream_ptr(dev)   # no workspaces from the caller
    else:
        pool, st = nt.workspace_pool(dev, len(xs))
    keep = []
    for i, (d, x, state, wt) in enumerate(zip(descs, xs, states, with_t)):
        cols = x.shape[-1]
        rows = x.numel() // cols
        out = torch.empty(x.shape, dtype=torch.uint8, device=dev)
        out_t = torch.empty((cols, rows), dtype=torch.uint8, device=dev) if wt else None
        sc = torch.zeros(2, dtype=torch.float32, device=dev)
        p = state.data_ptr()
        d.x, d.x_dtype, d.fmt, d.margin, d.history_len = x.data_ptr(), nt.TORCH_TO_NT[x.dtype], fmt, 0, state.numel() - 1
        d.rows, d.cols = rows, cols
        d.scale_state, d.amax_history, d.amax_out, d.scale_used_out = p, p + 4, sc.data_ptr(), sc.data_ptr() + 4
        d.out, d.out_t = out.data_ptr(), nt.ptr(out_t)
        d.workspace = None if static else pool[i].data_ptr()
        keep.append((out, out_t, sc))
    if static:
        # the call itself must leave device memory as it found it: outputs exist, the library was initialised
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(dev)[0]
    nt.check(entry(descs, len(xs), st), "quantize batch")
    if static:
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(dev)[0] == free_before, "the entry point that allocates nothing allocated"
    return keep


def test_static_scratch_entry_point_matches_the_allocating_one():
    from nanotron_amd import _native as nt

    dev = torch.device("cuda", 0)
    assert nt.lib.ntfp8_static_init(nt.stream_ptr(dev)) == 0
    # first call: 5 large tensors (bf16, one with a transposed copy, one ragged); second call: 3 small ones
    calls = [
        ([(4096, 4096), (4096, 6144), (1024, 768), (1000, 37), (2048, 1024)], [False, False, True, False, False]),
        ([(256, 128), (33, 7), (128, 256)], [False, False, True]),
    ]
    for fmt, ofmt in ((nt.E4M3, O.E4M3), (nt.E5M2, O.E5M2)):
        st_a = [torch.tensor([2.0 ** (3 + i)] + [0.0] * 16, device=dev) for i in range(5)]   # [scale, history]
        st_b = [s.clone() for s in st_a]
        for c, (shapes, with_t) in enumerate(calls):
            xs = [O.normal_tensor(900 + 10 * c + i, s, 0.5 + i, torch.bfloat16).to(dev) for i, s in enumerate(shapes)]
            if c == 1:
                xs[1].view(-1)[3] = float("nan")
            want = _run(nt.lib.ntfp8_quantize_delayed_batch, xs, fmt, st_a, with_t, static=False)
            got = _run(nt.lib.ntfp8_quantize_delayed_batch_static, xs, fmt, st_b, with_t, static=True)
            for i, ((o0, t0, s0), (o1, t1, s1)) in enumerate(zip(want, got)):
                assert torch.equal(o0, o1), (c, i)
                assert (t0 is None) == (t1 is None) and (t0 is None or torch.equal(t0, t1)), (c, i)
                assert torch.equal(_bits(s0), _bits(s1)), (c, i)
                assert torch.equal(_bits(st_a[i]), _bits(st_b[i])), (c, i)
                # and against the oracle: the held scale, saturating cast, NaN kept
                q = O.cast_to_fp8(xs[i].cpu(), s1[1].cpu(), ofmt)
                assert torch.equal(o1.cpu(), q), (c, i)
                a = O.amax(xs[i].cpu())
                assert _same(s1[0], a), (c, i)
    # more tensors than the static array has workspaces for: refused, nothing launched
    xs = [torch.ones(4, 4, dtype=torch.bfloat16, device=dev) for _ in range(nt.STATIC_MAX_TENSORS + 1)]
    sts = [torch.tensor([1.0] + [0.0] * 16, device=dev) for _ in xs]
    with pytest.raises(RuntimeError, match="size"):
        _run(nt.lib.ntfp8_quantize_delayed_batch_static, xs, nt.E4M3, sts, [False] * len(xs), static=True)
