"""FP8 column- / row-parallel linears for a one-rank group: the constructor contract of the reference's
TensorParallelColumnLinear / TensorParallelRowLinear (src/nanotron/parallel/tensor_parallel/nn.py:46-176)
on the CPU, and on the GPU a LLaMA MLP block (src/nanotron/models/llama.py:227-246: gate_up column-parallel
with contiguous chunks, GLU, down row-parallel) against the oracle's quantised arithmetic."""
import os
import tempfile

import pytest
import torch
import torch.nn.functional as F

from oracle import fp8_oracle as O


class _FakeGroup:
    def __init__(self, n):
        self._n = n

    def size(self):
        return self._n


def _classes():
    from nanotron_amd.fp8.tensor_parallel import (FP8TensorParallelColumnLinear, FP8TensorParallelRowLinear,
                                                  TensorParallelLinearMode)

    return FP8TensorParallelColumnLinear, FP8TensorParallelRowLinear, TensorParallelLinearMode


# ------------------------------------------------------------------ host logic (CPU)
def test_mode_enum_formats_as_its_name():
    *_, Mode = _classes()
    assert str(Mode.ALL_REDUCE) == "ALL_REDUCE" and f"{Mode.REDUCE_SCATTER}" == "REDUCE_SCATTER"
    assert Mode.ALL_REDUCE is not Mode.REDUCE_SCATTER


def test_constructor_contract_on_cpu():
    Col, Row, Mode = _classes()
    col = Col(32, 48, None, Mode.ALL_REDUCE, bias=True, device="cpu", contiguous_chunks=(16, 32))
    assert (col.in_features, col.out_features, col.world_size) == (32, 48, 1)
    assert "unsharded_out_features=48" in col.extra_repr() and "tp_rank=0" in col.extra_repr()
    row = Row(48, 32, None, Mode.REDUCE_SCATTER, bias=False, device="cpu", async_communication=True)
    assert row.bias is None and "unsharded_in_features=48" in row.extra_repr()
    # CPU tensors take the plain linear, as the reference's FP8Linear does (src/nanotron/fp8/linear.py:53-54)
    x = torch.randn(5, 7, 32)
    assert torch.equal(col(x), F.linear(x, col.weight, col.bias))
    assert torch.equal(row(col(x)), F.linear(F.linear(x, col.weight, col.bias), row.weight))
    with pytest.raises(AssertionError):
        Col(32, 48, None, Mode.ALL_REDUCE, device="cpu", contiguous_chunks=(16, 16))
    with pytest.raises(AssertionError):
        Row(48, 32, None, Mode.ALL_REDUCE, device="cpu", contiguous_chunks=(16, 16))
    with pytest.raises(ValueError):
        Row(48, 32, None, Mode.ALL_REDUCE, device="cpu", async_communication=True)  # nn.py:145-146
    with pytest.raises(ValueError):
        Col(32, 48, None, "ALL_REDUCE", device="cpu")


def test_groups_of_more_than_one_rank_are_refused():
    Col, Row, Mode = _classes()
    for cls in (Col, Row):
        with pytest.raises(NotImplementedError, match="2 ranks"):
            cls(32, 48, _FakeGroup(2), Mode.ALL_REDUCE, device="cpu")
        assert cls(32, 48, _FakeGroup(1), Mode.ALL_REDUCE, device="cpu").world_size == 1


def test_accepts_a_real_one_rank_process_group():
    import torch.distributed as dist

    Col, Row, Mode = _classes()
    if dist.is_initialized():
        pytest.skip("a default process group already exists in this process")
    with tempfile.TemporaryDirectory() as d:
        dist.init_process_group("gloo", init_method="file://" + os.path.join(d, "rdzv"), rank=0, world_size=1)
        try:
            pg = dist.new_group([0])
            col = Col(16, 24, pg, Mode.REDUCE_SCATTER, device="cpu")
            row = Row(24, 16, pg, Mode.REDUCE_SCATTER, device="cpu")
            assert col.world_size == 1 and row.bias is not None and "tp_rank=0" in row.extra_repr()
            assert row(col(torch.randn(3, 16))).shape == (3, 16)
        finally:
            dist.destroy_process_group()


# ------------------------------------------------------------------ a LLaMA MLP block in FP8 (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("mode_name", ["ALL_REDUCE", "REDUCE_SCATTER"])
def test_llama_mlp_block_against_the_oracle(mode_name):
    from nanotron_amd.fp8 import DTypes, FP8Parameter

    Col, Row, Mode = _classes()
    mode = Mode[mode_name]
    S, B, H, I = 48, 2, 256, 384  # [seq, batch, hidden] activations, as the reference's blocks pass them
    x = O.normal_tensor(71, (S, B, H), 1.0, torch.bfloat16)
    w_gu = O.normal_tensor(72, (2 * I, H), 0.05, torch.float32)
    w_dn = O.normal_tensor(73, (H, I), 0.05, torch.float32)
    gy = O.normal_tensor(74, (S, B, H), 1e-2, torch.float32)
    gate_up = Col(H, 2 * I, None, mode, bias=False, device="cuda", contiguous_chunks=(I, I),
                  async_communication=mode is Mode.REDUCE_SCATTER, out_dtype=torch.bfloat16)
    down = Row(I, H, None, mode, bias=False, device="cuda", async_communication=mode is Mode.REDUCE_SCATTER)
    gate_up.weight = FP8Parameter(w_gu.cuda(), DTypes.FP8E4M3)
    down.weight = FP8Parameter(w_dn.cuda(), DTypes.FP8E4M3)

    def glu(t):
        g, u = torch.split(t, I, dim=-1)  # llama.py:196-198
        return F.silu(g) * u

    xg = x.cuda().requires_grad_(True)
    merged = gate_up(xg)
    assert merged.shape == (S, B, 2 * I) and merged.dtype == torch.bfloat16
    merged.retain_grad()
    out = down(glu(merged))
    assert out.shape == (S, B, H) and out.dtype == torch.float32
    out.backward(gy.cuda())

    # the same chain in the oracle's arithmetic, each linear on the operands the layer saw
    xq = O.quantise_current(x.reshape(-1, H), O.E4M3)
    wq_gu, wq_dn = O.quantise_current(w_gu, O.E4M3), O.quantise_current(w_dn, O.E4M3)
    merged_ref = O.linear_forward(xq, wq_gu, torch.bfloat16)
    assert O.rel_l2(merged.detach().float().cpu().reshape(-1, 2 * I), merged_ref.float()) <= 8e-3
    h = glu(merged.detach()).cpu()  # the block's own activations: the oracle follows from here
    hq = O.quantise_current(h.reshape(-1, I), O.E4M3)
    assert O.rel_l2(out.detach().cpu().reshape(-1, H), O.linear_forward(hq, wq_dn)) <= 1e-3
    gq = O.quantise_current(gy.reshape(-1, H), O.E5M2)
    assert O.rel_l2(down.weight.grad.cpu(), O.linear_wgrad(gq, hq)) <= 1e-3
    gm = merged.grad.detach().cpu().reshape(-1, 2 * I)  # upstream gradient of the column-parallel layer
    gmq = O.quantise_current(gm, O.E5M2)
    assert O.rel_l2(gate_up.weight.grad.cpu(), O.linear_wgrad(gmq, xq)) <= 1e-3
    assert xg.grad.shape == (S, B, H) and xg.grad.dtype == torch.bfloat16
    assert O.rel_l2(xg.grad.float().cpu().reshape(-1, H), O.linear_dgrad(gmq, wq_gu, torch.bfloat16).float()) <= 8e-3
