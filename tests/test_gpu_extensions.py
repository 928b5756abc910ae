"""GPU parity of what this build adds around the reference's call sites: the bias inside the GEMM epilogue (the TODO
at src/nanotron/fp8/linear.py:62 and kernel.py:29-32), fp8 activations that autograd can carry (the TODO at
linear.py:63-64), both formats from one quantisation pass, evaluation passes that leave the scaling state alone,
and fp8 operands handed over as views."""
import pytest
import torch

from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu

REL_L2 = 1e-3


def _dt(fmt):
    from nanotron_amd.fp8 import DTypes

    return DTypes.FP8E4M3 if fmt == O.E4M3 else DTypes.FP8E5M2


def from_bytes(q_cpu, scale, fmt):
    from nanotron_amd.fp8 import FP8Tensor
    from nanotron_amd.fp8.meta import FP8Meta

    t = torch.Tensor._make_subclass(FP8Tensor, q_cpu.contiguous().cuda())
    t.fp8_meta = FP8Meta(torch.tensor(0.0, device="cuda"), torch.tensor(float(scale), dtype=torch.float32, device="cuda"),
                         _dt(fmt))
    return t


def _bits(t):
    return t.detach().float().cpu().contiguous().view(torch.int32)


def _same(a, b):
    """fp32 values equal bit for bit; NaNs equal whatever their payload (the GPU writes the quiet NaN 0x7fc00000)"""
    a, b = a.detach().float().cpu().reshape(-1), b.detach().float().cpu().reshape(-1)
    return bool(torch.all((a.view(torch.int32) == b.view(torch.int32)) | (a.isnan() & b.isnan())))


# ------------------------------------------------------------------------------------------ bias
@pytest.mark.parametrize("mnk", [(300, 272, 384), (4096, 1536, 1024), (64, 48, 32), (130, 250, 272), (5, 3, 7), (2304, 2048, 400)])
@pytest.mark.parametrize("bias_dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_bias_in_the_epilogue_integer_operands_bit_exact(mnk, bias_dtype):
    """All three GEMM kernels (large tiles with and without a half-tile tail, 128 x 128 tiles, one output per thread):
    D = round(fp32(acc * descale) + bias[n]).  Integer operands and integer bias: exact in fp32, so every output type
    must match the fp64 result rounded once."""
    from nanotron_amd.fp8.kernel import _gemm_nt

    M, N, K = mnk
    g = torch.Generator().manual_seed(M + N + K)
    one = torch.tensor(1.0)
    a = torch.randint(-4, 5, (M, K), generator=g).float()
    b = torch.randint(-4, 5, (N, K), generator=g).float()
    bias = torch.randint(-20, 21, (N,), generator=g).float().to(bias_dtype)
    A, B = from_bytes(O.cast_to_fp8(a, one, O.E5M2), 2.0, O.E5M2), from_bytes(O.cast_to_fp8(b, one, O.E4M3), 0.5, O.E4M3)
    want = (a.double() @ b.double().t()).float() + bias.float()
    for od in (torch.float32, torch.bfloat16, torch.float16):
        got = _gemm_nt(A, B, od, None, bias.cuda())
        assert torch.equal(got.cpu(), want.to(od)), (mnk, od)
    acc = torch.randint(-50, 50, (M, N), generator=g).float()
    accg = acc.cuda()
    _gemm_nt(A, B, torch.float32, accg, bias.cuda())
    assert torch.equal(accg.cpu(), want + acc)


def test_bias_fp32_output_equals_the_separate_addition():
    """For the reference's fp32 output, bias in the epilogue == `output + bias` (linear.py:65) bit for bit, on random
    operands (same accumulation, same two roundings)."""
    from nanotron_amd.fp8 import DTypes, FP8Tensor
    from nanotron_amd.fp8.kernel import fp8_matmul_kernel

    x = FP8Tensor(O.normal_tensor(1, (1024, 768), 1.0).cuda(), DTypes.FP8E4M3)
    w = FP8Tensor(O.normal_tensor(2, (640, 768), 0.02).cuda(), DTypes.FP8E4M3)
    b = O.normal_tensor(3, (640,), 0.3, torch.float32).cuda()
    plain = fp8_matmul_kernel(w, True, x, False, False)
    fused = fp8_matmul_kernel(w, True, x, False, False, bias=b)
    assert torch.equal(fused, plain + b)
    # bf16 output: one rounding instead of two
    fused16 = fp8_matmul_kernel(w, True, x, False, False, out_dtype=torch.bfloat16, bias=b)
    assert torch.equal(fused16, (plain + b).to(torch.bfloat16))


def test_bias_with_fp8_output():
    from nanotron_amd.fp8 import DTypes, FP8Tensor
    from nanotron_amd.fp8 import DelayedScaling
    from nanotron_amd.fp8.kernel import _gemm_nt, _gemm_nt_fp8

    def _state_with_scale(fmt, scale):
        st = DelayedScaling(_dt(fmt), history_len=4, device="cuda")
        st._buf[0] = float(scale)
        st.initialised = True
        return st

    def _clone_state(st):
        c = DelayedScaling(st.dtype, history_len=st.history_len, margin=st.margin, device="cuda")
        c._buf.copy_(st._buf)
        c.initialised = st.initialised
        return c

    for M, N, K in [(512, 272, 384), (96, 80, 64)]:
        x = FP8Tensor(O.normal_tensor(4, (M, K), 1.0).cuda(), DTypes.FP8E4M3)
        w = FP8Tensor(O.normal_tensor(5, (N, K), 0.05).cuda(), DTypes.FP8E4M3)
        b = O.normal_tensor(6, (N,), 0.5, torch.bfloat16).cuda()
        st = _state_with_scale(O.E4M3, 64.0)
        st2 = _clone_state(st)
        got = _gemm_nt_fp8(x, w, DTypes.FP8E4M3, st, True, b)
        want = FP8Tensor(_gemm_nt(x, w, torch.float32, None, b), DTypes.FP8E4M3, state=st2, with_transpose=True)
        assert torch.equal(got.as_subclass(torch.Tensor), want.as_subclass(torch.Tensor))
        assert torch.equal(got.transposed().as_subclass(torch.Tensor), want.transposed().as_subclass(torch.Tensor))
        assert torch.equal(_bits(got.fp8_meta.amax), _bits(want.fp8_meta.amax)) and torch.equal(_bits(st._buf), _bits(st2._buf))


@pytest.mark.parametrize("out_dtype", [None, torch.bfloat16])
def test_fp8linear_bias_forward_and_gradients(out_dtype):
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter

    M, K, N = 320, 256, 384
    x = O.normal_tensor(7, (M, K), 1.0, torch.float32)
    w = O.normal_tensor(8, (N, K), 0.05, torch.float32)
    b = O.normal_tensor(9, (N,), 0.2, torch.float32)
    gy = O.normal_tensor(10, (M, N), 1e-2, torch.float32)
    lin = FP8Linear(K, N, bias=True, device="cuda", out_dtype=out_dtype)
    lin.weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
    lin.bias.data = b.cuda()
    xg = x.cuda().requires_grad_(True)
    y = lin(xg)
    y.backward(gy.cuda().to(y.dtype))
    xq, wq = O.quantise_current(x, O.E4M3), O.quantise_current(w, O.E4M3)
    y_ref = O.linear_forward(xq, wq) + b                          # linear.py:65
    if out_dtype is None:
        assert y.dtype == torch.float32 and O.rel_l2(y.detach().cpu(), y_ref) <= REL_L2
    else:
        assert y.dtype == torch.bfloat16 and O.rel_l2(y.detach().float().cpu(), y_ref.to(torch.bfloat16).float()) <= REL_L2
    gyq = gy.to(y.dtype).float()
    assert lin.bias.grad.dtype == torch.float32 and lin.bias.grad.shape == (N,)
    assert torch.allclose(lin.bias.grad.cpu(), gyq.sum(0), rtol=1e-5, atol=1e-6)
    gq = O.quantise_current(gy.to(y.dtype), O.E5M2)
    assert O.rel_l2(xg.grad.cpu(), O.linear_dgrad(gq, wq)) <= REL_L2
    assert O.rel_l2(lin.weight.grad.cpu(), O.linear_wgrad(gq, xq)) <= REL_L2


# ------------------------------------------------------------------------------------------ inverse scales
def test_inverse_scale_entry_points_non_power_of_two():
    """The library takes the scale; Transformer Engine's functions take its reciprocal.  For powers of two the two
    forms agree bit for bit; for any other scale 1/(1/s) != s in general, which is why the inverse-scale forms exist."""
    from nanotron_amd import _native as nt

    g = torch.Generator().manual_seed(11)
    one = torch.tensor(1.0)
    M, N, K = 300, 272, 384
    a = torch.randint(-4, 5, (M, K), generator=g).float()
    b = torch.randint(-4, 5, (N, K), generator=g).float()
    aq, bq = O.cast_to_fp8(a, one, O.E4M3).cuda(), O.cast_to_fp8(b, one, O.E4M3).cuda()
    prod = (a.double() @ b.double().t()).float()
    for sa, sb in ((3.0, 0.3), (256.0, 0.125)):
        sat, sbt = torch.tensor(sa, device="cuda"), torch.tensor(sb, device="cuda")
        out = {}
        for inverse in (0, 1):
            d = (nt.GemmDesc * 1)()
            D = torch.empty(M, N, device="cuda")
            d[0].A, d[0].scale_a, d[0].B, d[0].scale_b, d[0].D = aq.data_ptr(), sat.data_ptr(), bq.data_ptr(), sbt.data_ptr(), D.data_ptr()
            d[0].M, d[0].N, d[0].K, d[0].scales_are_inverse = M, N, K, inverse
            nt.check(nt.lib.ntfp8_gemm_batch(d, 1, nt.stream_ptr(D.device)), "gemm")
            out[inverse] = D.cpu()
        f = torch.tensor
        assert torch.equal(out[1], prod * (f(sa) * f(sb)))
        assert torch.equal(out[0], prod * ((1 / f(sa)) * (1 / f(sb))))
        # handing the reciprocal to the inverse form reproduces the scale form exactly
        d = (nt.GemmDesc * 1)()
        D = torch.empty(M, N, device="cuda")
        ia, ib = (1 / sat).contiguous(), (1 / sbt).contiguous()
        d[0].A, d[0].scale_a, d[0].B, d[0].scale_b, d[0].D = aq.data_ptr(), ia.data_ptr(), bq.data_ptr(), ib.data_ptr(), D.data_ptr()
        d[0].M, d[0].N, d[0].K, d[0].scales_are_inverse = M, N, K, 1
        nt.check(nt.lib.ntfp8_gemm_batch(d, 1, nt.stream_ptr(D.device)), "gemm")
        assert torch.equal(D.cpu(), out[0])


# ------------------------------------------------------------------------------------------ both formats, one pass
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("shape", [(4096, 4096), (1000, 37), (5,), (257, 130)])
def test_dual_format_quantise_equals_two_single_passes(dtype, shape):
    from nanotron_amd import _native as nt
    from nanotron_amd.fp8 import DelayedScaling, DTypes, FP8Tensor

    if len(shape) == 2 and shape[0] == 4096 and dtype != torch.bfloat16:
        pytest.skip("benchmark tensor is bf16")
    dev = torch.device("cuda", 0)
    sts = {f: DelayedScaling(_dt(f), 16, 0, dev) for f in (O.E4M3, O.E5M2)}
    dual = {f: DelayedScaling(_dt(f), 16, 0, dev) for f in (O.E4M3, O.E5M2)}
    refs = {f: O.DelayedScaling(f) for f in (O.E4M3, O.E5M2)}
    for step in range(6):
        if len(shape) == 2 and shape[0] == 4096:
            x = O.student_t_outlier_tensor(1434 + step, shape)
        else:
            x = O.normal_tensor(100 + step, shape, 0.5 + step, dtype)
            if step == 3:
                x.view(-1)[0] = float("nan")
        xg = x.cuda()
        singles = {f: FP8Tensor(xg, _dt(f), state=sts[f]) for f in (O.E4M3, O.E5M2)}
        want = {f: refs[f].quantise(x) for f in (O.E4M3, O.E5M2)}
        if step == 0:   # first use of a role is current scaling (two passes): run it the ordinary way on the second pair too
            for f in (O.E4M3, O.E5M2):
                FP8Tensor(xg, _dt(f), state=dual[f])
            continue
        outs = {f: torch.empty(x.shape, dtype=torch.uint8, device=dev) for f in (O.E4M3, O.E5M2)}
        sc = torch.zeros(3, dtype=torch.float32, device=dev)   # amax, scale used e4m3, scale used e5m2
        ws, st = nt.workspace_and_stream(dev)
        p4, p5 = dual[O.E4M3]._buf.data_ptr(), dual[O.E5M2]._buf.data_ptr()
        nt.check(nt.lib.ntfp8_quantize_delayed_dual(xg.data_ptr(), nt.TORCH_TO_NT[dtype], x.numel(), 0, p4, p4 + 4, p5, p5 + 4, 16,
                                                    sc.data_ptr(), sc.data_ptr() + 4, sc.data_ptr() + 8,
                                                    outs[O.E4M3].data_ptr(), outs[O.E5M2].data_ptr(), ws.data_ptr(), st), "dual")
        for i, f in enumerate((O.E4M3, O.E5M2)):
            assert torch.equal(outs[f], singles[f].as_subclass(torch.Tensor)), (step, f)
            assert torch.equal(outs[f].cpu(), want[f].q), (step, f)
            assert _same(dual[f]._buf, sts[f]._buf), (step, f)
            assert _same(dual[f].scale, refs[f].scale) and _same(dual[f].amax_history, refs[f].hist), (step, f)
            assert _same(sc[1 + i], want[f].scale)
        assert _same(sc[0], want[O.E4M3].amax)
        assert int(ws.abs().sum().item()) == 0


# ------------------------------------------------------------------------------------------ evaluation passes
def test_evaluation_forward_leaves_the_scaling_state_alone():
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter

    M, K, N = 256, 384, 512
    lin = FP8Linear(K, N, bias=False, device="cuda", delayed_scaling=True, out_dtype=torch.bfloat16)
    w = O.normal_tensor(20, (N, K), 0.02, torch.float32)
    lin.weight = FP8Parameter(w.cuda(), DTypes.FP8E4M3)
    ref = O.DelayedScaling(O.E4M3)
    # before the role has seen anything, an evaluation pass scales from the tensor itself and records nothing
    lin.eval()
    x0 = O.normal_tensor(21, (M, K), 2.0)
    with torch.no_grad():
        y = lin(x0.cuda())
    assert not lin.scaling["input"].initialised and float(lin.scaling["input"].amax_history.abs().sum()) == 0.0
    assert O.rel_l2(y.float().cpu(), O.linear_forward(O.quantise_current(x0, O.E4M3), O.quantise_current(w, O.E4M3), torch.bfloat16).float()) <= REL_L2
    lin.train()
    for step in range(3):
        x = O.normal_tensor(22 + step, (M, K), 1.0 + step)
        lin(x.cuda())
        ref.quantise(x)
    before = lin.scaling["input"]._buf.clone()
    lin.eval()
    xe = O.normal_tensor(30, (M, K), 50.0)   # far larger than anything seen: would move the history
    with torch.no_grad():
        y = lin(xe.cuda())
    assert torch.equal(lin.scaling["input"]._buf, before)
    xq = O.Quantised(O.cast_to_fp8(xe, ref.scale, O.E4M3), O.amax(xe), ref.scale, O.E4M3)   # held scale, saturating
    assert O.rel_l2(y.float().cpu(), O.linear_forward(xq, O.quantise_current(w, O.E4M3), torch.bfloat16).float()) <= REL_L2
    lin.train()
    lin(xe.cuda())
    assert not torch.equal(lin.scaling["input"]._buf, before)


# ------------------------------------------------------------------------------------------ operands given as views
def test_fp8_operands_that_are_views():
    from nanotron_amd.fp8 import DTypes, FP8Tensor
    from nanotron_amd.fp8.kernel import _gemm_nt, _gemm_nt_batch

    x = FP8Tensor(O.normal_tensor(40, (512, 768), 1.0).cuda(), DTypes.FP8E4M3)
    w = FP8Tensor(O.normal_tensor(41, (640, 384), 0.05).cuda(), DTypes.FP8E4M3)
    xs = x[:, :384]                      # a strided view: loses the Python attribute
    xs.fp8_meta = x.fp8_meta
    wt = FP8Tensor(O.normal_tensor(42, (384, 640), 0.05).cuda(), DTypes.FP8E4M3)
    wv = wt.t()                          # [640, 384] view of a [384, 640] tensor
    wv.fp8_meta = wt.fp8_meta
    ref = O.gemm_nt(x.cpu().as_subclass(torch.Tensor)[:, :384].contiguous(), O.E4M3, x.fp8_meta.scale.cpu(),
                    w.cpu().as_subclass(torch.Tensor), O.E4M3, w.fp8_meta.scale.cpu())
    assert O.rel_l2(_gemm_nt(xs, w, torch.float32, None).cpu(), ref) <= REL_L2
    assert O.rel_l2(_gemm_nt_batch([(xs, w, torch.float32, None)])[0].cpu(), ref) <= REL_L2
    ref2 = O.gemm_nt(x.cpu().as_subclass(torch.Tensor)[:, :384].contiguous(), O.E4M3, x.fp8_meta.scale.cpu(),
                     wt.cpu().as_subclass(torch.Tensor).t().contiguous(), O.E4M3, wt.fp8_meta.scale.cpu())
    assert O.rel_l2(_gemm_nt(xs, wv, torch.float32, None).cpu(), ref2) <= REL_L2


# ------------------------------------------------------------------------------------------ fp8 activations + autograd
def test_two_layer_chain_with_fp8_activation_trains():
    """FP8Linear(out_dtype=E4M3) -> FP8Linear over 5 delayed-scaling steps, forward and backward, against the oracle:
    the activation between the layers exists only as fp8 bytes (quantised in the first GEMM's epilogue with the scale
    its "output" role holds); the second layer's dgrad reaches the first layer's backward through the gradient handle."""
    from nanotron_amd.fp8 import DTypes, FP8Linear, FP8Parameter, FP8Tensor

    M, K, H, N = 512, 384, 640, 272
    w1 = O.normal_tensor(50, (H, K), 0.05, torch.bfloat16)
    w2 = O.normal_tensor(51, (N, H), 0.05, torch.bfloat16)
    b1 = O.normal_tensor(52, (H,), 0.1, torch.bfloat16)
    l1 = FP8Linear(K, H, bias=True, device="cuda", dtype=torch.bfloat16, out_dtype=DTypes.FP8E4M3, delayed_scaling=True)
    l2 = FP8Linear(H, N, bias=False, device="cuda", dtype=torch.bfloat16, out_dtype=torch.bfloat16, delayed_scaling=True)
    l1.weight = FP8Parameter(w1.cuda(), DTypes.FP8E4M3)
    l2.weight = FP8Parameter(w2.cuda(), DTypes.FP8E4M3)
    l1.bias.data = b1.cuda()
    r = {k: O.DelayedScaling(O.E4M3) for k in ("x", "w1", "h", "w2")}
    r["g2"], r["g1"] = O.DelayedScaling(O.E5M2), O.DelayedScaling(O.E5M2)
    for step in range(5):
        x = O.normal_tensor(60 + step, (M, K), 1.0 + 0.5 * step)
        gy = O.normal_tensor(70 + step, (M, N), 1e-2)
        l1.requantize_weight()
        l2.requantize_weight()
        xg = x.cuda().requires_grad_(True)
        h = l1(xg)
        assert isinstance(h, FP8Tensor) and h.dtype == torch.uint8 and h.shape == (M, H)
        y = l2(h)
        sent = l2.fp8_grad_inputs_sent
        y.backward(gy.cuda())
        fp8_dh = l2.fp8_grad_inputs_sent > sent   # dh went back as e5m2 bytes out of the second layer's dgrad epilogue
        assert fp8_dh or step < 3                  # (once layer 1's gradient role is known on the host to hold a scale)
        # ---- oracle, forward
        xq, w1q, w2q = r["x"].quantise(x), r["w1"].quantise(w1), r["w2"].quantise(w2)
        h32 = O.linear_forward(xq, w1q) + b1.float()                 # fp32 result + bias, never rounded to 16 bits
        hq = r["h"].quantise(h32)
        assert O.rel_l2(O.cast_from_fp8(h.cpu().as_subclass(torch.Tensor), hq.scale, O.E4M3, torch.float32),
                        O.cast_from_fp8(hq.q, hq.scale, O.E4M3, torch.float32)) <= 2e-3   # bytes flip where the GEMMs' last bits differ
        assert torch.equal(_bits(h.fp8_meta.scale), _bits(hq.scale))
        for st, rf in ((l1.scaling["input"], r["x"]), (l1.scaling["weight"], r["w1"]), (l2.scaling["weight"], r["w2"])):
            assert torch.equal(_bits(st.scale), _bits(rf.scale)) and torch.equal(_bits(st.amax_history), _bits(rf.hist))
        # the output role follows the oracle except for the last bits of the GEMM: its scale (a power of two) must agree
        assert torch.equal(_bits(l1.scaling["output"].scale), _bits(r["h"].scale)), step
        hq_gpu = O.Quantised(h.cpu().as_subclass(torch.Tensor), h.fp8_meta.amax.cpu(), h.fp8_meta.scale.cpu(), O.E4M3)
        assert O.rel_l2(y.detach().float().cpu(), O.linear_forward(hq_gpu, w2q, torch.bfloat16).float()) <= REL_L2
        # ---- oracle, backward (from the bytes the GPU produced, so that only the GEMMs are compared)
        g2q = r["g2"].quantise(gy)
        # dh arrives at layer 1 as bf16 through the handle, or as e5m2 quantised from the fp32 result without that rounding
        dh = O.linear_dgrad(g2q, w2q, torch.float32 if fp8_dh else torch.bfloat16)
        assert O.rel_l2(l2.weight.main_grad.cpu(), O.linear_wgrad(g2q, hq_gpu)) <= REL_L2
        g1q = r["g1"].quantise(dh)
        st = l1.scaling["output_grad"]
        assert torch.equal(_bits(st.scale), _bits(r["g1"].scale)), step
        assert O.rel_l2(xg.grad.float().cpu(), O.linear_dgrad(g1q, w1q, torch.bfloat16).float()) <= 2e-3
        assert O.rel_l2(l1.weight.main_grad.cpu(), O.linear_wgrad(g1q, xq)) <= 2e-3
        # the bias gradient is summed from what layer 1's backward receives: bf16 dh, or the e5m2 values
        dh_seen = O.cast_from_fp8(g1q.q, g1q.scale, O.E5M2, torch.float32) if fp8_dh else dh.float()
        assert O.rel_l2(l1.bias.grad.float().cpu(), dh_seen.sum(0)) <= 4e-3
        l1.bias.grad = None


def test_fp8_output_without_consumer_gradient_and_with_two_consumers():
    from nanotron_amd.fp8 import DTypes, FP8Linear

    l1 = FP8Linear(256, 384, bias=False, device="cuda", out_dtype=DTypes.FP8E4M3)
    l2 = FP8Linear(384, 128, bias=False, device="cuda")
    l3 = FP8Linear(384, 192, bias=False, device="cuda")
    x = torch.randn(160, 256, device="cuda", requires_grad=True)
    h = l1(x)
    (l2(h).sum() + 2.0 * l3(h).sum()).backward()     # autograd sums both consumers' dX on the handle
    assert x.grad is not None and x.grad.shape == x.shape and bool(torch.isfinite(x.grad).all())
    assert l1.weight.grad is not None and l2.weight.grad is not None and l3.weight.grad is not None
    with torch.no_grad():
        h = l1(x)
        assert l2(h).shape == (160, 128)


# ------------------------------------------------------------------------------------------ overlapping streams
def test_quantisations_on_two_streams_at_once_equal_the_serial_results():
    """Calls that may overlap in time must use different reduction workspaces; the Python layer keeps one per (device,
    stream).  Two streams quantise different tensors over and over without waiting for each other: every result equals
    the one computed alone, bit for bit, and both workspaces are left zero."""
    from nanotron_amd import _native as nt
    from nanotron_amd.fp8 import DelayedScaling, DTypes, FP8Tensor

    dev = torch.device("cuda", 0)
    xs = [O.normal_tensor(40 + i, (2048, 4096), 10.0 ** (i - 2), torch.bfloat16).cuda() for i in range(4)]
    fmts = [DTypes.FP8E4M3, DTypes.FP8E5M2, DTypes.FP8E4M3, DTypes.FP8E5M2]

    def run(i, steps, out):
        st = DelayedScaling(fmts[i], 16, 0, dev)
        for s in range(steps):
            q = FP8Tensor(xs[(i + s) % 4], fmts[i], state=st)
            out.append((q.as_subclass(torch.Tensor).clone(), q.fp8_meta.amax.clone(), q.fp8_meta.scale.clone(), st._buf.clone()))

    serial = [[], []]
    for i in (0, 1):
        run(i, 12, serial[i])
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    both = [[], []]
    for s in streams:
        s.wait_stream(torch.cuda.current_stream())
    # the first quantisation of a role reads a flag on the host; interleave call by call so that the streams' kernels
    # are queued side by side
    states = [DelayedScaling(fmts[i], 16, 0, dev) for i in (0, 1)]
    for step in range(12):
        for i in (0, 1):
            with torch.cuda.stream(streams[i]):
                q = FP8Tensor(xs[(i + step) % 4], fmts[i], state=states[i])
                both[i].append((q.as_subclass(torch.Tensor).clone(), q.fp8_meta.amax.clone(), q.fp8_meta.scale.clone(),
                                states[i]._buf.clone()))
    torch.cuda.synchronize()
    for i in (0, 1):
        for step, (a, b) in enumerate(zip(serial[i], both[i])):
            assert torch.equal(a[0], b[0]), (i, step)
            for u, v in zip(a[1:], b[1:]):
                assert torch.equal(u.view(-1).view(torch.int32), v.view(-1).view(torch.int32)), (i, step)
    w0 = nt.workspace_and_stream(dev)[0]
    with torch.cuda.stream(streams[0]):
        w1 = nt.workspace_and_stream(dev)[0]
    with torch.cuda.stream(streams[1]):
        w2 = nt.workspace_and_stream(dev)[0]
    assert len({w0.data_ptr(), w1.data_ptr(), w2.data_ptr()}) == 3
    assert int(w1.view(torch.int32).abs().sum()) == 0 and int(w2.view(torch.int32).abs().sum()) == 0


# ------------------------------------------------------------------------------------------ beyond 2^31
def test_quantisation_of_more_than_two_to_the_31_elements():
    """Element counts are 64-bit end to end: a bf16 tensor of 2^31 + 12288 elements (4 GiB) is quantised with current
    scaling; the amax is found wherever it lies, the bytes at both ends equal the oracle's, the zeros in between
    stay zero."""
    from nanotron_amd.fp8 import DTypes, FP8Tensor

    n = (1 << 31) + 12288
    edge = 1 << 20
    x = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
    head = O.normal_tensor(71, (edge,), 1.0, torch.bfloat16)
    tail = O.normal_tensor(72, (edge,), 1.0, torch.bfloat16)
    x[:edge] = head.cuda()
    x[-edge:] = tail.cuda()
    x[(1 << 31) + 7] = -6.5          # the maximum lies behind the 2^31-th element
    tail[edge - 12288 + 7] = -6.5
    q = FP8Tensor(x, DTypes.FP8E4M3)
    assert float(q.fp8_meta.amax) == 6.5
    scale = q.fp8_meta.scale.cpu()
    assert float(scale) == float(O.update_scaling_factor(torch.tensor(6.5), torch.tensor(1.0), O.E4M3))
    raw = q.as_subclass(torch.Tensor)
    assert raw.shape == (n,)
    assert torch.equal(raw[:edge].cpu(), O.cast_to_fp8(head, scale, O.E4M3))
    assert torch.equal(raw[-edge:].cpu(), O.cast_to_fp8(tail, scale, O.E4M3))
    for lo in (edge, 1 << 30, (1 << 31) - (1 << 23)):
        assert int(raw[lo:lo + (1 << 22)].to(torch.int32).sum()) == 0
    del x, q, raw
    torch.cuda.empty_cache()


def test_gemm_with_an_operand_of_more_than_2_gib():
    """An A operand of 33024 x 65536 bytes does not fit the 32-bit buffer offsets of the 256-tile kernel; the library
    sends it to the kernel that addresses with 64-bit pointers.  Integer-valued operands: every output must be exact."""
    from nanotron_amd.fp8 import DTypes, FP8Tensor
    from nanotron_amd.fp8.kernel import _gemm_nt
    from nanotron_amd.fp8.meta import FP8Meta

    dev = torch.device("cuda", 0)
    M, N, K = 33024, 192, 65536
    codes = torch.tensor([0x00, 0x38, 0x40, 0xB8, 0xC0], dtype=torch.uint8, device=dev)   # 0, 1, 2, -1, -2 in e4m3
    vals = torch.tensor([0.0, 1.0, 2.0, -1.0, -2.0], device=dev)
    g = torch.Generator(device=dev).manual_seed(5)
    ia = torch.randint(0, 5, (M, K), generator=g, device=dev, dtype=torch.uint8)
    ib = torch.randint(0, 5, (N, K), generator=g, device=dev, dtype=torch.uint8)

    def fp8(idx):
        t = torch.Tensor._make_subclass(FP8Tensor, codes[idx.long()] if idx.numel() < (1 << 28) else _lookup(idx))
        t.fp8_meta = FP8Meta(torch.tensor(2.0, device=dev), torch.tensor(1.0, device=dev), DTypes.FP8E4M3)
        return t

    def _lookup(idx):   # row blocks, so that no int64 index tensor of 2 G elements is ever made
        out = torch.empty_like(idx)
        for r in range(0, idx.shape[0], 2048):
            out[r:r + 2048] = codes[idx[r:r + 2048].long()]
        return out

    a, b = fp8(ia), fp8(ib)
    assert a.numel() > (1 << 31)
    d = _gemm_nt(a, b, torch.float32, None)
    bf = vals[ib.long()]
    for r in (0, 8192, 16384, 24576, 32768 - 2048, 33024 - 2048):   # the last two blocks straddle / lie behind 2 GiB
        ref = vals[ia[r:r + 2048].long()] @ bf.t()                     # exact: |sum| <= 4 * 65536 < 2^24
        assert torch.equal(d[r:r + 2048], ref), r
