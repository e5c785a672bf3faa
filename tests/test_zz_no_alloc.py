"""mie_conv_masked_noalloc: the workspace form of the masked conv whose workspace is an array in
the library's device image, for callers that cannot allocate.  Called through the C ABI and compared,
bit for bit, with mie_conv_masked_ws (a caller workspace of the same size) on two calls in a row,
the second on a smaller input; plus the size limit and the absence of any torch allocation."""
import pytest
import torch

from maskedincrementeval_amd import _lib, ops
from maskedincrementeval_amd.masked_types import TileMask
from maskedincrementeval_amd.synthetic import gaussian_delta, he_normal_conv_weight
from oracle import incr_oracle as io

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _dev(t):
    return ops.as_nhwc(t.to(DEV).contiguous(memory_format=torch.channels_last))


class _Case:
    """Inputs, filter, tile set and two sets of outputs / reservoirs for one conv shape."""

    def __init__(self, n, cin, cout, h, w, k, s, seed):
        p = k // 2
        self.n, self.cin, self.cout, self.h, self.w, self.k, self.s, self.p = n, cin, cout, h, w, k, s, p
        self.weight = he_normal_conv_weight(cout, cin, k, seed)
        self.filt = ops.ConvFilter(self.weight.permute(1, 2, 3, 0).contiguous().to(DEV))
        self.ho, self.wo = ops.conv_out_size(h, w, k, s, p)
        d, m = gaussian_delta(n, cin, h, w, 0.3, 0.5, seed=seed + 1)
        self.d_cpu = d
        self.d, self.m = _dev(d), m.to(DEV)
        self.ts = TileMask(n, self.ho, self.wo, DEV)
        ops.build_mask_tiles(self.m, None, n, h, w, _lib.FOOT_CONV, k, s, p, self.ts)
        r0 = torch.randn(n, cout, self.ho, self.wo, generator=torch.Generator().manual_seed(seed + 2))
        self.r0_cpu = r0
        self.res = [_dev(r0.clone()), _dev(r0.clone())]
        self.out = [ops.new_nhwc(n, cout, self.ho, self.wo, DEV), ops.new_nhwc(n, cout, self.ho, self.wo, DEV)]
        torch.cuda.synchronize()

    def args(self, which, x3=False):
        """x3: fp32 deltas multiplied as three bf16 terms (MIE_DTYPE_F32_BF16X3 and the filter copy packed for it)."""
        plain, mc = self.filt.for_dtype(torch.float32, x3=x3)
        return [self.d.data_ptr(), self.m.data_ptr(), self.cin, None, None, 0, self.h, self.w,
                plain.data_ptr(), mc.data_ptr(), self.cin, self.k, self.s, self.p, self.cout, self.ts.ref,
                self.out[which].data_ptr(), None, self.res[which].data_ptr(), _lib.ACT_RELU, 0.0,
                _lib.PATH_AUTO, _lib.DTYPE_F32_BF16X3 if x3 else _lib.DTYPE_F32]


def _stream():
    return torch.cuda.current_stream(torch.device(DEV)).cuda_stream


@pytest.mark.parametrize("x3", [False, True], ids=["fp32_instruction", "three_bf16_terms"])
def test_noalloc_matches_workspace_form_on_two_calls(x3):
    lib = _lib.lib()
    # 512 -> 256 on a 16x16 plane (4 tiles x 8 slabs, 16 chunks: split 8 ways), then a smaller 256 -> 128 conv
    # on an 8x24 plane (3 tiles x 4 slabs, 8 chunks): the second call finds the first call's partial sums
    big = _Case(1, 512, 256, 16, 16, 3, 1, seed=11)
    small = _Case(1, 256, 128, 8, 24, 3, 1, seed=21)
    ws = torch.full((_lib.NOALLOC_WS_BYTES // 4,), float("nan"), dtype=torch.float32, device=DEV)
    torch.cuda.synchronize()
    for case in (big, small):
        _lib.check(lib.mie_conv_masked_ws(*case.args(0, x3), ws.data_ptr(), ws.numel() * 4, _stream()))
        # no allocation: neither through torch's caching allocator nor behind its back (hipMalloc / hipFree in the
        # library would move the device's free byte count, which torch's statistics do not see)
        before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info(DEV)[0]
        _lib.check(lib.mie_conv_masked_noalloc(*case.args(1, x3), _stream()))
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats(DEV)["allocation.all.allocated"] == before
        assert torch.cuda.mem_get_info(DEV)[0] == free_before
        assert torch.equal(case.out[0], case.out[1]), "delta differs from the workspace form"
        assert torch.equal(case.res[0], case.res[1]), "reservoir differs from the workspace form"
        # and both are the conv: against the CPU oracle (fp32: rtol 1e-4, atol 1e-5)
        res = io.Reserve(case.r0_cpu.clone())
        ref = io.act_incr(torch.relu, res, io.conv_incr(case.d_cpu, case.weight, case.s, case.p))
        assert torch.allclose(case.out[1].cpu(), ref, rtol=1e-4, atol=1e-5)
        assert torch.allclose(case.res[1].cpu(), res.reservoir, rtol=1e-4, atol=1e-5)
    # the caller workspace was really used by the form compared against (the launches were split)
    assert torch.isfinite(ws[:16 * 16 * 256 * 2]).all()


def test_noalloc_runs_under_graph_capture():
    # the callers it is for: a captured HIP graph may not allocate.  After a warm-up call (which looks the array's
    # address up) the entry point is captured, replayed three times with the program's own work in between, and
    # every replay must reproduce the eager result bit for bit.
    lib = _lib.lib()
    case = _Case(1, 256, 128, 8, 24, 3, 1, seed=41)
    _lib.check(lib.mie_conv_masked_noalloc(*case.args(0), _stream()))          # warm-up, eager: the result to match
    torch.cuda.synchronize()
    want_out, want_res = case.out[0].clone(), case.res[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        _lib.check(lib.mie_conv_masked_noalloc(*case.args(1), side.cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(DEV)[0]
    with torch.cuda.graph(graph):
        _lib.check(lib.mie_conv_masked_noalloc(*case.args(1), _stream()))
    for _ in range(3):
        case.res[1].copy_(_dev(case.r0_cpu.clone()))       # the reservoir is updated in place: start each replay alike
        case.out[1].zero_()                                  # (inactive tiles are not written: they stay zero)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(case.out[1], want_out) and torch.equal(case.res[1], want_res)
    assert torch.cuda.mem_get_info(DEV)[0] >= free_before - (1 << 20)           # (the graph object itself is host-side)


def test_noalloc_rejects_outputs_beyond_its_workspace():
    lib = _lib.lib()
    case = _Case(1, 32, 64, 136, 136, 3, 1, seed=31)     # 2 planes of 136*136*64 floats > 8 MiB
    assert 2 * 136 * 136 * 64 * 4 > _lib.NOALLOC_WS_BYTES
    case.out[1].fill_(7.0)
    torch.cuda.synchronize()
    rc = lib.mie_conv_masked_noalloc(*case.args(1), _stream())
    assert rc == -3                                       # MIE_ERR_CAPACITY
    msg = lib.mie_last_error_string().decode()
    assert "exceeds the device-resident workspace" in msg and "mie_conv_masked" in msg
    torch.cuda.synchronize()
    assert torch.all(case.out[1] == 7.0)                  # nothing was launched
