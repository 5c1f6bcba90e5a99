"""flexattn_fwd_noalloc (the forward that keeps its block map in a device array of the library and
allocates nothing) against flexattn_fwd with a caller-allocated map, through the C ABI: identical
bits for o, l, m (same kernels, same map contents), on two calls in a row, the second one smaller
and with another mask, so that whatever the first call left in the array must not matter."""
import ctypes as C
import math

import pytest
import torch

from flex_attention_tpu_amd import _lib

pytestmark = pytest.mark.gpu


def _inputs(B, Hq, Hkv, S, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, S, D, generator=g).to(dtype).cuda()
    k = torch.randn(B, Hkv, S, D, generator=g).to(dtype).cuda()
    v = torch.randn(B, Hkv, S, D, generator=g).to(dtype).cuda()
    return q, k, v


def _both(lib, q, k, v, mask, keep, score=None):
    """(o, l, m) of flexattn_fwd with a map built into fresh tensors, and of flexattn_fwd_noalloc."""
    B, Hq, S, D = q.shape
    Hkv = k.shape[1]
    dt = _lib.BF16 if q.dtype == torch.bfloat16 else _lib.F32
    bq, bk = _lib.tile_shape(_lib.PASS_FWD, dt, D)
    nq, nk = S // bq, S // bk
    dev = q.device
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    state = torch.empty(nq, nk, dtype=torch.uint8, device=dev)
    kv_cnt = torch.empty(nq, dtype=torch.int32, device=dev)
    kv_idx = torch.empty(nq, nk, dtype=torch.int32, device=dev)
    rc = lib.flexattn_build_block_mask(C.byref(mask), S, S, bq, bk, state.data_ptr(), kv_cnt.data_ptr(), kv_idx.data_ptr(),
                                       None, None, stream)
    assert rc == 0, lib.flexattn_last_error_string()
    out = []
    for entry, bm in ((lib.flexattn_fwd, _lib.BlockMapC(state.data_ptr(), kv_cnt.data_ptr(), kv_idx.data_ptr(), None, None,
                                                       nq, nk, bq, bk)),
                      (lib.flexattn_fwd_noalloc, _lib.BlockMapC())):
        o = torch.full_like(q, float("nan"))
        l = torch.full((B, Hq, S), float("nan"), dtype=torch.float32, device=dev)
        m = torch.full_like(l, float("nan"))
        p = _lib.FwdParamsC(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), l.data_ptr(), m.data_ptr(),
                            B, Hq, Hkv, S, S, D, dt, 1.0 / math.sqrt(D), 0, 0, score or _lib.ScoreSpecC(), mask, bm)
        # a first call loads the kernels' code objects (the runtime may take device memory for that once);
        # the call that is measured is the second one: neither torch's allocator nor the driver (free bytes
        # of the device, which a hipMalloc inside the library would lower) may see an allocation
        rc = entry(C.byref(p), stream)
        assert rc == 0, lib.flexattn_last_error_string()
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        rc = entry(C.byref(p), stream)
        assert rc == 0, lib.flexattn_last_error_string()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.cuda.mem_get_info()[0] >= free_before, "device memory was allocated during the call"
        out.append((o, l, m))
    del keep
    return out


def _same(a, b):
    for name, x, y in zip("olm", a, b):
        assert not torch.isnan(x.float()).any(), name
        assert torch.equal(x, y), f"{name}: flexattn_fwd_noalloc differs from flexattn_fwd"


def test_noalloc_forward_equals_forward_with_a_caller_map(lib):
    # first call: 2048 tokens, documents + causal, GQA, bf16 (generated stream, persistent or not)
    S = 2048
    lens = [700, 1, 835, 512]
    doc = torch.repeat_interleave(torch.arange(len(lens)), torch.tensor(lens)).to(torch.int32).cuda()
    mask = _lib.MaskSpecC(_lib.MASK_CAUSAL | _lib.MASK_DOC, 0, 0, 0, doc.data_ptr(), doc.data_ptr())
    q, k, v = _inputs(2, 8, 2, S, 128, torch.bfloat16, 1)
    ref, got = _both(lib, q, k, v, mask, doc)
    _same(ref, got)
    # second call, smaller, another mask and a score function: shorter lists over the first call's leftovers
    S = 384
    mask = _lib.MaskSpecC(_lib.MASK_CAUSAL | _lib.MASK_WINDOW, 200, 0, 0, None, None)
    q, k, v = _inputs(1, 4, 4, S, 128, torch.bfloat16, 2)
    ref, got = _both(lib, q, k, v, mask, None, _lib.ScoreSpecC(_lib.SCORE_SOFTCAP, 20.0, 0.0, 0, 0, 0, None))
    _same(ref, got)
    # third call: the fp32 kernels (their own tile granularity), no mask
    q, k, v = _inputs(1, 2, 2, 256, 64, torch.float32, 3)
    ref, got = _both(lib, q, k, v, _lib.MaskSpecC(), None)
    _same(ref, got)


def test_noalloc_forward_under_graph_capture(lib):
    """The use the entry point is meant for: captured into a HIP graph (after one eager call, which looks up the
    resident array's address), replayed several times with new inputs in the same buffers and eager work in
    between; every replay must give the bits of flexattn_fwd on the same inputs."""
    S, D = 1024, 128
    lens = [300, 724]
    doc = torch.repeat_interleave(torch.arange(len(lens)), torch.tensor(lens)).to(torch.int32).cuda()
    mask = _lib.MaskSpecC(_lib.MASK_CAUSAL | _lib.MASK_DOC, 0, 0, 0, doc.data_ptr(), doc.data_ptr())
    q, k, v = _inputs(2, 4, 2, S, D, torch.bfloat16, 11)
    B, Hq, Hkv = 2, 4, 2
    o = torch.empty_like(q)
    l = torch.empty(B, Hq, S, dtype=torch.float32, device="cuda")
    m = torch.empty_like(l)
    p = _lib.FwdParamsC(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), l.data_ptr(), m.data_ptr(),
                        B, Hq, Hkv, S, S, D, _lib.BF16, 1.0 / math.sqrt(D), 0, 0, _lib.ScoreSpecC(), mask, _lib.BlockMapC())
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # eager warm-up on the stream the capture will use
        assert lib.flexattn_fwd_noalloc(C.byref(p), C.c_void_p(side.cuda_stream)) == 0, lib.flexattn_last_error_string()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        rc = lib.flexattn_fwd_noalloc(C.byref(p), C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.flexattn_last_error_string()
    for seed in (12, 13, 14):
        qn, kn, vn = _inputs(B, Hq, Hkv, S, D, torch.bfloat16, seed)
        q.copy_(qn); k.copy_(kn); v.copy_(vn)
        o.fill_(float("nan")); l.fill_(float("nan")); m.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = (o.clone(), l.clone(), m.clone())
        ref, _ = _both(lib, qn, kn, vn, mask, doc)   # (eager work between the replays, the resident map rebuilt by it)
        _same(ref, got)


def test_noalloc_forward_rejects_what_exceeds_the_resident_map(lib):
    dummy = torch.empty(16, device="cuda")
    p = _lib.FwdParamsC()
    p.q = p.k = p.v = p.o = dummy.data_ptr()
    p.B, p.Hq, p.Hkv, p.D, p.dtype, p.sm_scale = 1, 1, 1, 128, _lib.BF16, 1.0
    bq, bk = _lib.tile_shape(_lib.PASS_FWD, _lib.BF16, 128)
    p.Sq, p.Sk = 512 * bq, 512 * bk
    assert lib.flexattn_fwd_noalloc(C.byref(p), None) == _lib.EINVAL
    assert b"exceed" in lib.flexattn_last_error_string()
