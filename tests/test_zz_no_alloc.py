"""The attention entry point that allocates nothing (cdm_attn_fwd_static_bf16: K / V tile images in a device array
built into the library) against the entry point it is a variant of (cdm_attn_fwd_bf16 with a caller-owned
workspace), through the C ABI.  Both run the same kernels, so the outputs must agree bit for bit; the oracle check
of the operator itself is in test_gpu_kernels.py.  Two calls in a row share the array: the second, smaller one must
not see anything the first one left behind."""
import pytest
import torch

import oracle as O
from cosmos_amd import _lib, rotary
from gpu_util import BF16_COS, BF16_REL, assert_close, dev

pytestmark = pytest.mark.gpu


def _call_pair(lib, n, H, Hkv, hd, seed, causal_prefix=0):
    g = torch.Generator().manual_seed(seed)
    d, dkv = H * hd, Hkv * hd
    qkv = (torch.randn((n, d + 2 * dkv), generator=g) * 0.5).to(torch.bfloat16).to(dev())
    q, k, v = qkv[:, :d], qkv[:, d:d + dkv], qkv[:, d + dkv:]
    pos = O.text_positions(3, n)
    cos, sin = O.mrope_cos_sin(pos, hd, (hd // 4, 3 * hd // 8, 3 * hd // 8))
    cos, sin = cos.contiguous().to(dev()), sin.contiguous().to(dev())
    st = torch.cuda.current_stream().cuda_stream
    need = lib.cdm_attn_workspace_bytes(n, Hkv, hd)
    ws = torch.empty(need, dtype=torch.uint8, device=dev())
    want = torch.empty((n, d), dtype=torch.bfloat16, device=dev())
    rc = lib.cdm_attn_fwd_bf16(q.data_ptr(), qkv.stride(0), k.data_ptr(), qkv.stride(0), v.data_ptr(), qkv.stride(0),
                               cos.data_ptr(), sin.data_ptr(), want.data_ptr(), d, n, H, Hkv, hd, ws.data_ptr(), need,
                               None, causal_prefix, st)
    _lib.check(rc, "cdm_attn_fwd_bf16")
    got = torch.full((n, d), float("nan"), dtype=torch.bfloat16, device=dev())
    static = lambda: lib.cdm_attn_fwd_static_bf16(q.data_ptr(), qkv.stride(0), k.data_ptr(), qkv.stride(0), v.data_ptr(),
                                                  qkv.stride(0), cos.data_ptr(), sin.data_ptr(), got.data_ptr(), d, n, H, Hkv,
                                                  hd, None, causal_prefix, st)
    _lib.check(static(), "cdm_attn_fwd_static_bf16")      # the first call on a device resolves the array's address
    torch.cuda.synchronize()
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    # "allocates nothing" at the level of the device, not only of torch's caching allocator (which a hipMalloc inside the
    # library would bypass): the free memory the driver reports must not drop across the call
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    _lib.check(static(), "cdm_attn_fwd_static_bf16")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] >= free_before, "device memory was allocated inside cdm_attn_fwd_static_bf16"
    return qkv, cos.cpu(), sin.cpu(), got, want


def test_static_scratch_entry_point_matches_workspace_entry_point():
    lib = _lib.load()
    assert lib.cdm_attn_static_scratch_bytes() == 32 << 20
    # first call: 1,500 tokens x 4 K/V heads x 128 (ragged last tile); second call: smaller, other head geometry
    for (n, H, Hkv, hd, seed, P) in [(1500, 8, 4, 128, 1, 0), (333, 4, 4, 64, 2, 0), (700, 2, 1, 128, 3, 130)]:
        qkv, cos, sin, got, want = _call_pair(lib, n, H, Hkv, hd, seed, P)
        assert torch.equal(got, want), f"static-scratch attention differs from the workspace form at n={n}"
        # and against the oracle on a few rows, so that a failure of both forms cannot pass as agreement
        d, dkv = H * hd, Hkv * hd
        x = qkv.float().cpu()
        rows = torch.tensor([0, 1, n // 2, n - 1] + ([P - 1, P] if P else []))
        qr = O.apply_mrope(x[:, :d].view(n, H, hd), cos, sin)[rows]
        kr = O.apply_mrope(x[:, d:d + dkv].view(n, Hkv, hd), cos, sin)
        kv_end = O.hybrid_kv_end(n, P)[rows] if P else None
        ref = O.attention_rows(qr, kr, x[:, d + dkv:].view(n, Hkv, hd), kv_end).reshape(len(rows), d)
        assert_close(got[rows.to(dev())], ref, BF16_COS, BF16_REL, f"static-scratch attention n={n}")


def test_static_scratch_entry_point_under_graph_capture():
    """The use the entry point is for: recorded into a HIP graph (after cdm_attn_static_scratch_bytes(), which resolves
    the built-in array on the current device outside the capture), replayed on new inputs - several times, with eager
    work and synchronisations in between - and compared bit for bit with the eager call on the same inputs."""
    lib = _lib.load()
    n, H, Hkv, hd = 900, 4, 2, 128
    d, dkv = H * hd, Hkv * hd
    assert lib.cdm_attn_static_scratch_bytes() == 32 << 20
    g = torch.Generator().manual_seed(11)
    qkv = torch.zeros((n, d + 2 * dkv), dtype=torch.bfloat16, device=dev())
    cos, sin = O.mrope_cos_sin(O.text_positions(0, n), hd, (32, 48, 48))
    cos, sin = cos.contiguous().to(dev()), sin.contiguous().to(dev())
    out = torch.zeros((n, d), dtype=torch.bfloat16, device=dev())
    q, k, v = qkv[:, :d], qkv[:, d:d + dkv], qkv[:, d + dkv:]

    def call(dst):
        rc = lib.cdm_attn_fwd_static_bf16(q.data_ptr(), qkv.stride(0), k.data_ptr(), qkv.stride(0), v.data_ptr(), qkv.stride(0),
                                          cos.data_ptr(), sin.data_ptr(), dst.data_ptr(), d, n, H, Hkv, hd, None, 0,
                                          torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "cdm_attn_fwd_static_bf16")
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        call(out)
    for rep in range(3):
        qkv.copy_((torch.randn(qkv.shape, generator=g) * 0.5).to(torch.bfloat16))
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        eager = torch.empty_like(out)
        call(eager)
        torch.cuda.synchronize()
        assert bool(torch.isfinite(out.float()).all())
        assert torch.equal(out, eager), f"replay {rep} differs from the eager call"


def test_static_scratch_entry_point_rejects_what_does_not_fit():
    lib = _lib.load()
    fake = 0x10000
    # 56,320 tokens x 32 heads x 128 need 923 MB of tile images
    rc = lib.cdm_attn_fwd_static_bf16(fake, 4096, fake, 4096, fake, 4096, None, None, fake, 4096, 56320, 32, 32, 128, None,
                                      0, None)
    assert rc == _lib.ERR_BAD_SHAPE and "scratch" in _lib.last_error()
