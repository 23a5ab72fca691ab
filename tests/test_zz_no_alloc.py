"""The entry point that allocates nothing (onhip_conv2d_f32_noalloc) against the entry points it mirrors, through the
C ABI: two calls in a row on split-K problems, the second smaller than the first, so the second finds the first one's
partial sums in the built-in scratch array; then a problem whose partial sums do not fit, which must be refused."""
import ctypes as C

import numpy as np
import pytest

from onenew_amd import abi, datagen, hip
from onenew_amd.abi import ConvDesc

pytestmark = pytest.mark.gpu


def _desc(n, cin, hw, cout, k, pad, act=abi.RELU):
    d = ConvDesc()
    d.n, d.cin, d.h, d.w, d.cout, d.kh, d.kw = n, cin, hw, hw, cout, k, k
    d.stride_h = d.stride_w = 1
    d.pad_t = d.pad_l = d.pad_b = d.pad_r = pad
    d.group, d.has_bias, d.act_type, d.compute = 1, 1, act, abi.COMPUTE_F32
    return d


def _inputs(torch, tag, d):
    x = datagen.uniform(datagen.seed_for("noalloc", tag, "x"), (d.n, d.cin, d.h, d.w))
    w = datagen.normal(datagen.seed_for("noalloc", tag, "w"), (d.cout, d.cin, d.kh, d.kw), 0.0, (2.0 / (d.cin * d.kh * d.kw)) ** 0.5)
    b = datagen.normal(datagen.seed_for("noalloc", tag, "b"), (d.cout,), 0.0, 0.01)
    return [torch.from_numpy(a).cuda() for a in (x, w, b)]


def test_no_alloc_entry_point_matches_the_allocating_one():
    import torch
    assert torch.cuda.is_available(), "no GPU visible"
    hip.init(0)
    prev = hip.set_tuning(0)          # both entry points on the cost model's choice
    try:
        # few output tiles and a long reduction: the cost model cuts K into slices (partial sums in the scratch)
        for tag, d, packed in (("first", _desc(2, 512, 7, 512, 3, 1), True), ("second", _desc(1, 256, 14, 256, 3, 1), False),
                               ("third_1x1", _desc(1, 2048, 7, 512, 1, 0), False)):
            print(f"no-alloc case {tag}", flush=True)
            x, w, b = _inputs(torch, tag, d)
            wp = hip.pack_conv_weights(d, w) if packed else w
            ref = hip.conv2d_f32(d, x, wp, b, packed=packed)
            oh, ow = d.out_hw()
            out = torch.full((d.n, d.cout, oh, ow), float("nan"), dtype=torch.float32, device="cuda")
            torch.cuda.synchronize()
            used = hip.load().onhip_noalloc_scratch_launches()
            hip.conv2d_f32_noalloc(d, x, wp, out, b, packed=packed)
            torch.cuda.synchronize()
            # the case is only a test of the built-in array if the cost model did cut K for it
            assert hip.load().onhip_noalloc_scratch_launches() == used + 1, f"{tag}: the call did not use the built-in scratch array"
            got, want = out.cpu().numpy(), ref.cpu().numpy()
            assert np.isfinite(got).all()
            scale = float(np.abs(want).max())
            assert np.abs(got - want).max() <= 1e-4 * scale, tag          # the fp32 bar
            assert np.array_equal(got, want), tag                             # same tile, same split: the same bits
        # partial sums beyond the built-in array: refused, nothing written
        # (1 536 tiles of 64 x 64 are six rounds of 256; the cost model cuts K in five, 5 x 9.8 MB of partial sums)
        d = _desc(3, 1024, 40, 512, 3, 1)
        x = torch.zeros((d.n, d.cin, d.h, d.w), dtype=torch.float32, device="cuda")
        w = torch.zeros((d.cout, d.cin, 3, 3), dtype=torch.float32, device="cuda")
        b = torch.ones((d.cout,), dtype=torch.float32, device="cuda")
        out = torch.zeros((d.n, d.cout, 40, 40), dtype=torch.float32, device="cuda")
        rc = hip.load().onhip_conv2d_f32_noalloc(C.byref(d), x.data_ptr(), w.data_ptr(), 0, b.data_ptr(), None, out.data_ptr(), None)
        torch.cuda.synchronize()
        msg = hip.load().onhip_last_error().decode()
        print("big problem:", rc, msg, flush=True)
        assert rc == -3 and "built-in scratch" in msg, (rc, msg)
        assert float(out.abs().max()) == 0.0
    finally:
        hip.set_tuning(prev)
