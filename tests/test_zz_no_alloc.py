"""The entry point that allocates nothing (vxhip_packed_linear_forward_f32_noalloc): the same bits
as vxhip_packed_linear_forward_f32 through the C ABI, on calls in a row that share the library's
fixed scratch array, the second smaller than the first; no device memory is taken by a call; a
shape whose staging does not fit the array is refused with a message."""
import numpy as np
import pytest

import _cases as cases

pytestmark = pytest.mark.gpu


def test_no_alloc_entry_matches_the_allocating_one(oracle):
    import torch
    import volvoxai_amd as vx
    own = vx.Context(0, torch.cuda.current_stream())
    # (rows, k, n, group): a GEMM-sized call first, then smaller ones that reuse the same bytes of
    # the array: fewer rows through the GEMM, then the GEMV's operand-order staging, then a ragged K
    shapes = [(200, 1024, 264, 128), (40, 1024, 264, 128), (7, 1024, 264, 128), (32, 1000, 72, 32), (1, 4096, 96, 64),
              (130, 95, 33, 32)]
    for i, (rows, k, n, group) in enumerate(shapes):
        c = cases.packed_case(rows, k, n, group, 60 + i, True, special_rows=(rows >= 5))
        words = oracle.pack_w8_words(c["w"])
        pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group)
        xd = torch.from_numpy(c["x"]).cuda()
        st, want = pl.forward_f32(own, xd)
        own.synchronize()
        want_variant = own.last_variant
        out = torch.full((rows, n), -7.0, dtype=torch.float32, device="cuda")
        st2, _ = pl.forward_f32(own, xd, out=out, no_alloc=True)   # first call of this shape: code objects load
        own.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        out.fill_(-7.0)
        st3, _ = pl.forward_f32(own, xd, out=out, no_alloc=True)
        own.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "the call took or returned device memory"
        assert st == st2 == st3 == 0 and own.last_variant == want_variant
        got, want = out.cpu().numpy(), want.cpu().numpy()
        nan = np.isnan(want)
        assert (np.isnan(got) == nan).all() and (got.view(np.uint32)[~nan] == want.view(np.uint32)[~nan]).all(), shapes[i]
        _, ref = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], n, group)
        assert (got.view(np.uint32)[~nan] == ref.view(np.uint32)[~nan]).all()
        pl.close()
    # staging beyond the fixed 4 MiB: refused before anything is launched, output untouched
    k, n, rows = 4096, 32, 1100
    c = cases.packed_case(4, k, n, 128, 3)
    pl = vx.PackedLinear(oracle.pack_w8_words(c["w"]), c["scales"], c["bias"], k, n, 128)
    xd = torch.zeros((rows, k), dtype=torch.float32, device="cuda")
    out = torch.full((rows, n), -7.0, dtype=torch.float32, device="cuda")
    st, _ = pl.forward_f32(own, xd, out=out, no_alloc=True)
    assert st == -1 and b"fixed scratch" in vx.library().vxhip_last_error()
    assert bool((out == -7.0).all())
    st, _ = pl.forward_f32(own, xd[:1000], out=out[:1000], no_alloc=True)  # 1000 x 4096 + scales fits
    st2, want = pl.forward_f32(own, xd[:1000])
    own.synchronize()
    assert st == st2 == 0 and torch.equal(out[:1000].view(torch.int32), want.view(torch.int32))
    assert bool((out[1000:] == -7.0).all())
    pl.close()
    own.close()
