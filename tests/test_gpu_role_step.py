"""GPU: the fused role step (chunk pooling + role projection + argmax + index scan) against the oracle's
restatement of the torch ops the reference runs.

The kernel accumulates the projection in fp32 in its own order, so its logits agree with a library GEMM to
rounding; what must hold exactly: the roles are the argmax (with bias and forced globals) of the logits the
kernel itself reports, the index scan belongs to those roles, and the roles agree with the oracle's wherever
the oracle's decision is not a near tie."""
import numpy as np
import pytest
import torch

from oracle import nats_oracle as orc
from tests.gpu_util import say

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-5, torch.bfloat16: 3e-2}


def check_call(x, w, C, W, pre, carry, merge_max, bias, first_g, dtype):
    from neuralattentionsearch_amd import ops
    got = ops.role_step(x.cuda(), w.cuda(), C, W, pre_fill=pre, carry_in=None if carry is None else carry.cuda(),
                        merge_max=merge_max, global_bias=bias, force_first_global=first_g, with_logits=True,
                        with_scan=True)
    pooled, logits, carry_want, pad = orc.pooled_role_logits(x, w, C, pre_fill=pre, carry_in=carry, merge_max=merge_max)
    assert got["pad"] == pad
    tol = TOL[dtype]
    if carry_want is None:
        assert got["carry"] is None
    else:
        assert (got["carry"].float().cpu() - carry_want.float()).abs().max().item() <= tol
    if logits is None:
        assert got["roles"] is None
        return got["carry"].cpu() if got["carry"] is not None else None
    lg = got["logits"].cpu()
    assert lg.shape == logits.shape
    assert (lg.float() - logits.float()).abs().max().item() <= tol * max(1.0, logits.float().abs().max().item())
    # exact: roles = argmax of the kernel's own logits
    own = orc.roles_from_logits(lg, bias, force_first_global=first_g, force_last_global=pad != 0)
    roles = got["roles"].cpu().numpy()
    assert np.array_equal(roles, own)
    assert np.array_equal(got["token_states_info"].float().cpu().numpy(), orc.one_hot_roles(own, dtype=torch.float32).numpy())
    assert np.array_equal(got["end_idx"].cpu().numpy(), orc.next_global_index(own == orc.ROLE_GLOBAL))
    # agreement with the oracle's roles wherever its top two options are not within rounding of each other
    want = orc.roles_from_logits(logits, bias, force_first_global=first_g, force_last_global=pad != 0)
    biased = logits.float().clone()
    biased[..., 0] += bias
    top2 = biased.topk(2, dim=-1)[0]
    clear = ((top2[..., 0] - top2[..., 1]) > 4 * tol * max(1.0, logits.float().abs().max().item())).permute(0, 2, 1).numpy()
    assert np.array_equal(roles[clear], want[clear])
    if clear.size >= 96:
        assert clear.mean() > 0.5  # the comparison above is not vacuous
    return got["carry"].cpu() if got["carry"] is not None else None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("merge_max", [False, True])
@pytest.mark.parametrize("C,dim,H,lens", [(16, 512, 2, [100, 37, 1, 1, 1, 9, 16, 64, 3]), (64, 4096, 8, [1000, 24, 1, 1, 39, 128]),
                                          (8, 200, 3, [5, 2, 1, 30])])
def test_role_step_streams(dtype, merge_max, C, dim, H, lens):
    say("role step", dtype, merge_max, C, dim, H)
    g = torch.Generator().manual_seed(C + dim)
    w = (torch.randn(H * 3, dim, generator=g) * (4.0 / dim ** 0.5)).to(dtype)
    B, W = 2, 4 * C
    pre, carry, seen = 0, None, 0
    for n in lens:
        x = torch.randn(B, n, dim, generator=g).to(dtype)
        carry_new = check_call(x, w, C, W, pre, carry, merge_max, 0.1, seen < C, dtype)
        total = pre + n
        if total < C or total % C:
            carry = carry_new
        else:
            carry = None
        pre, seen = total % C, seen + n


def test_role_step_strided_input_and_errors():
    from neuralattentionsearch_amd import ops
    say("role step strided")
    g = torch.Generator().manual_seed(0)
    base = torch.randn(2, 70, 2 * 256, generator=g).bfloat16()
    x = base[:, :, :256]  # row stride 512
    w = torch.randn(6, 256, generator=g).bfloat16() * 0.2
    got = ops.role_step(x.cuda(), w.cuda(), 16, 32, with_logits=True)
    _, logits, _, _ = orc.pooled_role_logits(x.contiguous(), w, 16)
    assert (got["logits"].float().cpu() - logits.float()).abs().max().item() <= 3e-2 * max(1.0, logits.float().abs().max().item())
    with pytest.raises(ValueError):
        ops.role_step(x.cuda(), w.cuda(), 16, 32, pre_fill=3)  # an open chunk without its statistic
    with pytest.raises(NotImplementedError):
        ops.role_step(x.cuda(), w.cuda(), 12, 36)  # chunk size not a power of two
