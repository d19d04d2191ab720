"""The decode attention entry point that allocates nothing (bn_attn_mfma_decode_static, csrc/attn_mfma.h):
called through ctypes, its output is compared bit for bit with the existing entry point's (bn_attn_mfma,
which takes the split partials from buffers the caller allocates) on two calls in a row, the second with a
smaller input, so that what the first call left in the library's scratch array must not matter."""
import ctypes
import math
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

PAGE = 64
c_int, c_float, c_void_p = ctypes.c_int, ctypes.c_float, ctypes.c_void_p
ERR_SCRATCH = -3
SCRATCH_FLOATS = 4 * 1024 * 1024


def _library() -> ctypes.CDLL:
    from bitnet_c_amd.csrc import build
    lib = build.load("attn_mfma")
    lib.bn_attn_mfma_decode_static.restype = c_int
    lib.bn_attn_mfma_decode_static.argtypes = [
        c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int,
        c_int, c_float, c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p]
    lib.bn_attn_mfma.restype = c_int
    lib.bn_attn_mfma.argtypes = [
        c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
        c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p,
        c_void_p]
    return lib


def _case(seed, lens, H, Hkv, hs):
    """A paged bf16 cache (blocked pages) with random keys and values for sequences of the given lengths (the new
    token included), pages in random order, unused pages NaN; one query row per sequence."""
    g = torch.Generator().manual_seed(seed)
    rnd = random.Random(seed)
    B = len(lens)
    width = max((l + PAGE - 1) // PAGE for l in lens)
    n_pages = sum((l + PAGE - 1) // PAGE for l in lens) + 2
    free = list(range(n_pages))
    rnd.shuffle(free)
    kp = torch.full((n_pages, Hkv, PAGE, hs), float("nan"), dtype=torch.bfloat16)
    vp = torch.full((n_pages, Hkv, hs, PAGE), float("nan"), dtype=torch.bfloat16)
    bt = torch.zeros((B, width), dtype=torch.int32)
    ks, vs = [], []
    for s, l in enumerate(lens):
        k = torch.randn((l, Hkv, hs), generator=g).to(torch.bfloat16)
        v = torch.randn((l, Hkv, hs), generator=g).to(torch.bfloat16)
        ks.append(k)
        vs.append(v)
        for i in range((l + PAGE - 1) // PAGE):
            p = free.pop()
            bt[s, i] = p
            n = min(PAGE, l - PAGE * i)
            kp[p, :, :n] = k[PAGE * i:PAGE * i + n].transpose(0, 1)
            vp[p, :, :, :n] = v[PAGE * i:PAGE * i + n].permute(1, 2, 0)
    q = torch.randn((B, H * hs), generator=g).to(torch.bfloat16)
    from bitnet_c_amd import ops
    kp, vp = ops.to_blocked_pages(kp, vp)          # the order in which the matrix-core kernels read a page
    return q.cuda(), kp.cuda(), vp.cuda(), bt.cuda(), torch.tensor(lens, dtype=torch.int32).cuda(), ks, vs


def _plain(q, ks, vs, H, Hkv, hs, scale):
    rows = []
    for s, (k, v) in enumerate(zip(ks, vs)):
        qs = q[s].float().cpu().view(H, hs)
        for h in range(H):
            kh = h // (H // Hkv)
            p = torch.softmax((k[:, kh].float() @ qs[h]) * scale, dim=0)
            rows.append(p @ v[:, kh].float())
    return torch.stack(rows).view(len(ks), H * hs)


def test_decode_attention_without_allocation_equals_the_allocating_entry_point():
    lib = _library()
    H, Hkv, hs, GT = 8, 2, 128, 4
    scale = 1.0 / math.sqrt(hs)
    stream = torch.cuda.current_stream().cuda_stream
    # the second call is smaller in every way: fewer sequences, shorter, fewer splits
    for seed, lens, n_splits, chunk in ((1, [700, 1, 64, 65, 300, 1500, 129], 6, 256), (2, [130, 40, 257], 3, 128)):
        q, kp, vp, bt, d_lens, ks, vs = _case(seed, lens, H, Hkv, hs)
        B = len(lens)
        assert n_splits * chunk >= bt.shape[1] * PAGE
        part_o = torch.empty((B * H * n_splits, hs), dtype=torch.float32, device="cuda")
        part_ml = torch.empty((B * H * n_splits, 2), dtype=torch.float32, device="cuda")
        want = torch.full((B, H * hs), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = lib.bn_attn_mfma(q.data_ptr(), H * hs, want.data_ptr(), H * hs, kp.data_ptr(), vp.data_ptr(), bt.data_ptr(),
                              bt.shape[1], d_lens.data_ptr(), None, B, B, H, Hkv, hs, GT, 0, scale, n_splits, chunk,
                              part_o.data_ptr(), part_ml.data_ptr(), None, 0, 0, None, None, stream)
        assert rc == 0
        got = torch.full((B, H * hs), float("nan"), dtype=torch.bfloat16, device="cuda")

        def static_call(out):
            return lib.bn_attn_mfma_decode_static(q.data_ptr(), H * hs, out.data_ptr(), H * hs, kp.data_ptr(), vp.data_ptr(),
                                                  bt.data_ptr(), bt.shape[1], d_lens.data_ptr(), B, H, Hkv, hs, GT, 0, scale,
                                                  n_splits, chunk, None, 0, 0, None,
                                                  torch.cuda.current_stream().cuda_stream)
        assert static_call(got) == 0
        torch.cuda.synchronize()
        assert torch.equal(got.cpu(), want.cpu()), seed
        # It allocates nothing: the call goes past torch's allocator, so what is compared is the driver's own count of
        # free device memory, around a call after the one that looked the array's address up.
        again = torch.full((B, H * hs), float("nan"), dtype=torch.bfloat16, device="cuda")
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        assert static_call(again) == 0
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(again.cpu(), want.cpu()), seed
        # Under graph capture (a caller that cannot allocate): recorded after the warm call, replayed three times with
        # eager work between the replays, every replay the eager result.
        captured = torch.full((B, H * hs), float("nan"), dtype=torch.bfloat16, device="cuda")
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            rc = static_call(captured)
        assert rc == 0
        for replay in range(3):
            captured.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(captured.cpu(), want.cpu()), (seed, replay)
            assert static_call(again) == 0                     # the array's contents between replays do not matter
            torch.cuda.synchronize()
        # and both are the plain formula's result within the rounding of the bf16 softmax weights
        ref = _plain(q, ks, vs, H, Hkv, hs, scale)
        assert bool(((got.float().cpu() - ref).abs() <= ref.abs() * 2.0 ** -8 + 5 * 2.0 ** -9).all()), seed
    # The limit from both sides: the most partials that fit (419 sequences x 11 heads x 7 splits x 130 floats are 114
    # floats short of the array; the head size plus two never divides its size) run and equal the allocating entry
    # point's result; one sequence more is refused.
    H2, n_splits2, chunk2 = 11, 7, 64
    rnd = random.Random(5)
    lens2 = [rnd.randrange(1, 7 * 64 + 1) for _ in range(420)]
    q2, kp2, vp2, bt2, d_lens2, _, _ = _case(3, lens2, H2, H2, hs)
    assert 419 * H2 * n_splits2 * (hs + 2) <= SCRATCH_FLOATS < 420 * H2 * n_splits2 * (hs + 2)
    po = torch.empty((419 * H2 * n_splits2, hs), dtype=torch.float32, device="cuda")
    pm = torch.empty((419 * H2 * n_splits2, 2), dtype=torch.float32, device="cuda")
    want2 = torch.zeros((420, H2 * hs), dtype=torch.bfloat16, device="cuda")
    got2 = torch.zeros((420, H2 * hs), dtype=torch.bfloat16, device="cuda")
    assert lib.bn_attn_mfma(q2.data_ptr(), H2 * hs, want2.data_ptr(), H2 * hs, kp2.data_ptr(), vp2.data_ptr(), bt2.data_ptr(),
                            bt2.shape[1], d_lens2.data_ptr(), None, 419, 419, H2, H2, hs, 1, 0, scale, n_splits2, chunk2,
                            po.data_ptr(), pm.data_ptr(), None, 0, 0, None, None, stream) == 0
    fits = lambda n, out: lib.bn_attn_mfma_decode_static(
        q2.data_ptr(), H2 * hs, out.data_ptr(), H2 * hs, kp2.data_ptr(), vp2.data_ptr(), bt2.data_ptr(), bt2.shape[1],
        d_lens2.data_ptr(), n, H2, H2, hs, 1, 0, scale, n_splits2, chunk2, None, 0, 0, None, stream)
    assert fits(419, got2) == 0
    torch.cuda.synchronize()
    assert torch.equal(got2.cpu(), want2.cpu()) and float(got2[:419].float().abs().sum()) > 0
    assert fits(420, got2) == ERR_SCRATCH
    torch.cuda.synchronize()
    assert float(got2[419].float().abs().sum()) == 0.0            # nothing was launched for the call that was refused
    # far more partials than the array holds: refused, nothing launched, the output untouched
    B = SCRATCH_FLOATS // (H * 64 * (hs + 2)) + 1
    out = torch.zeros((1, H * hs), dtype=torch.bfloat16, device="cuda")
    rc = lib.bn_attn_mfma_decode_static(q.data_ptr(), H * hs, out.data_ptr(), H * hs, kp.data_ptr(), vp.data_ptr(),
                                        bt.data_ptr(), bt.shape[1], d_lens.data_ptr(), B, H, Hkv, hs, GT, 0, scale, 64,
                                        64, None, 0, 0, None, stream)
    assert rc == ERR_SCRATCH
    torch.cuda.synchronize()
    assert float(out.float().abs().sum()) == 0.0
