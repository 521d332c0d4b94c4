"""mmf_ternarize_pack_noalloc (the entry point that allocates nothing: its partial sums live in a device array of the
library) against mmf_ternarize_pack, through the C ABI: bit-identical packed codes and de-quantisation step, on two
calls in a row, the second with a smaller matrix (fewer partial sums than the first call left in the array), then a
third with another dtype; sizes beyond the stated maximum are rejected."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(lib, L, w):
    n, k = w.shape
    dev = w.device
    nbytes = lib.mmf_packed_bytes(n, k)
    outs = []
    for noalloc in (False, True):
        packed = torch.full((nbytes,), 0x5A, dtype=torch.uint8, device=dev)
        wdeq = torch.full((1,), -1.0, dtype=torch.float32, device=dev)
        if noalloc:
            rc = lib.mmf_ternarize_pack_noalloc(w.data_ptr(), L.dtype_id(w.dtype), n, k, packed.data_ptr(), wdeq.data_ptr(),
                                                L.stream())
        else:
            ws = torch.zeros(lib.mmf_ternarize_workspace_bytes(), dtype=torch.uint8, device=dev)
            rc = lib.mmf_ternarize_pack(w.data_ptr(), L.dtype_id(w.dtype), n, k, packed.data_ptr(), wdeq.data_ptr(),
                                        ws.data_ptr(), L.stream())
        assert rc == 0, rc
        torch.cuda.synchronize()
        outs.append((packed.cpu(), wdeq.cpu()))
    return outs


def test_ternarize_pack_noalloc_equals_ternarize_pack(dev):
    import matmulfreellm_amd._lib as L
    from oracle import quant as oq
    import matmulfreellm_amd.functional as F_
    lib = L.load()
    torch.manual_seed(70)
    cases = [((11264, 2048), torch.bfloat16),     # 1024 partial sums
             ((70, 300), torch.bfloat16),         # the next call is smaller: 6 partial sums, the rest of the array is stale
             ((2048, 5632), torch.float32),
             ((33, 129), torch.float16)]
    with torch.cuda.device(dev):
        for shape, dtype in cases:
            w = (torch.randn(*shape) * 0.02).to(dtype).to(dev)
            (p0, d0), (p1, d1) = _both(lib, L, w)
            assert torch.equal(p0, p1), f"packed codes differ for {shape} {dtype}"
            assert torch.equal(d0, d1), f"wdeq differs for {shape} {dtype}"
            t_ref, deq_ref = oq.ternary_codes(w.cpu())
            assert d1.item() == deq_ref.item()
            pw = F_.PackedWeight(p1.to(dev), d1.to(dev), shape[0], shape[1], shape[0])
            assert torch.equal(F_.unpack_ternary(pw).cpu(), t_ref)


def test_ternarize_pack_noalloc_rejects_what_it_cannot_take(dev):
    import matmulfreellm_amd._lib as L
    lib = L.load()
    with torch.cuda.device(dev):
        w = torch.zeros(64, 128, dtype=torch.bfloat16, device=dev)
        packed = torch.zeros(lib.mmf_packed_bytes(64, 128), dtype=torch.uint8, device=dev)
        wdeq = torch.zeros(1, dtype=torch.float32, device=dev)
        big = lib.mmf_ternarize_pack_noalloc_max_elements()
        assert big == 1 << 31
        assert lib.mmf_ternarize_pack_noalloc(w.data_ptr(), 1, 1 << 20, 1 << 12, packed.data_ptr(), wdeq.data_ptr(), L.stream()) == -2
        assert lib.mmf_ternarize_pack_noalloc(None, 1, 64, 128, packed.data_ptr(), wdeq.data_ptr(), L.stream()) == -1
        assert lib.mmf_ternarize_pack_noalloc(w.data_ptr(), 7, 64, 128, packed.data_ptr(), wdeq.data_ptr(), L.stream()) == -1
        assert lib.mmf_ternarize_pack_noalloc(w.data_ptr(), 1, 64, 128, packed.data_ptr() + 4, wdeq.data_ptr(), L.stream()) == -3
        torch.cuda.synchronize()
