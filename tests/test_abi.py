"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares, and
rejects bad arguments on the host before touching a device."""
import ctypes as C
import os
import re

import pytest
import torch

from cosmos_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HAS_GPU = torch.cuda.is_available()


def header_functions(crosscheck=False):
    """Function names the header declares for the product library (or, crosscheck=True, inside its
    ``#ifdef CDM_CROSSCHECK`` sections: the extra exports of the cross-check build)."""
    text = open(os.path.join(ROOT, "include", "cosmos_dm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    guarded = "".join(re.findall(r"#ifdef CDM_CROSSCHECK(.*?)#endif", text, flags=re.S))
    plain = re.sub(r"#ifdef CDM_CROSSCHECK.*?#endif", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cdm_[a-z0-9_]+)\s*\(", guarded if crosscheck else plain)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = header_functions()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/cosmos_dm.h but not exported"
    assert set(names) == set(_lib.SIGNATURES), "ctypes signatures and header disagree"
    # the product library carries no process-wide knob; the cross-check build exports it on top of the same ABI
    extra = header_functions(crosscheck=True)
    assert extra == sorted(_lib.CROSSCHECK_SIGNATURES) == ["cdm_set_variant"]
    assert not hasattr(lib, "cdm_set_variant")
    xlib = _lib.load_crosscheck()
    for n in names + extra:
        assert hasattr(xlib, n), f"{n} missing from the cross-check build"
    assert xlib.cdm_set_variant(b"nope", 0) == _lib.ERR_BAD_ARG
    assert xlib.cdm_source_hash() == lib.cdm_source_hash()
    assert lib.cdm_version() >= 100
    # two tile images of 128 padded tokens x 2 heads x 64 channels (bf16) + one fp32 key-norm bound per (head, tile)
    assert lib.cdm_attn_workspace_bytes(100, 2, 64) == 2 * 128 * 2 * 64 * 2 + 2 * 2 * 4


def test_loaded_library_was_built_from_the_present_sources(tmp_path):
    """The loader never runs a stale build: the library carries the hash of the sources it was built from, readable
    from the file without loading it, and load() rebuilds the in-tree library when that hash differs."""
    from cosmos_amd import build as B
    lib = _lib.load()
    want = B.source_hash()
    assert len(want) == 16 and lib.cdm_source_hash().decode() == want
    assert B.built_hash(_lib.lib_path()) == want
    stale = tmp_path / "stale.so"
    stale.write_bytes(b"\x7fELF....CDM_SRC_HASH=0123456789abcdef....")
    assert B.built_hash(str(stale)) == "0123456789abcdef" != want
    assert B.built_hash(str(tmp_path / "missing.so")) == ""


def test_bad_arguments_are_rejected_on_the_host():
    lib = _lib.load()
    fake = 0x10000   # aligned, never dereferenced: validation fails first
    assert lib.cdm_adaln_rmsnorm_bf16(None, fake, None, None, fake, 4, 64, 1e-6, None) == _lib.ERR_BAD_ARG
    assert "null" in _lib.last_error()
    assert lib.cdm_adaln_rmsnorm_bf16(fake, fake, None, None, fake, 4, 60, 1e-6, None) == _lib.ERR_BAD_SHAPE
    assert lib.cdm_adaln_rmsnorm_bf16(fake + 2, fake, None, None, fake, 4, 64, 1e-6, None) == _lib.ERR_BAD_ALIGN
    assert lib.cdm_adaln_rmsnorm_bf16(fake, fake, fake + 4, None, fake, 4, 64, 1e-6, None) == _lib.ERR_BAD_ALIGN      # shift
    g = lambda **kw: lib.cdm_gemm_bf16(kw.get("A", fake), kw.get("lda", 128), fake, 128, kw.get("W2", None), fake, 256, 8, 256,
                                       kw.get("K", 128), kw.get("epi", 0), kw.get("R", None), 256, None, None, None,
                                       kw.get("rope_cols", 0), kw.get("hd", 0), None)
    assert g(A=None) == _lib.ERR_BAD_ARG
    assert g(K=96, lda=96) == _lib.ERR_BAD_SHAPE
    assert g(epi=7) == _lib.ERR_BAD_ARG
    assert g(epi=_lib.EPI_SWIGLU) == _lib.ERR_BAD_ARG            # W2 missing
    assert g(epi=_lib.EPI_GATE_RESIDUAL) == _lib.ERR_BAD_ARG     # R missing
    assert g(epi=_lib.EPI_ROPE_QK) == _lib.ERR_BAD_ARG           # tables missing
    assert g(lda=100) == _lib.ERR_BAD_ARG                        # stride < K
    assert lib.cdm_attn_fwd_bf16(fake, 64, fake, 64, fake, 64, None, None, fake, 64, 16, 1, 1, 48, fake, 1 << 20, None, 0, None) == _lib.ERR_BAD_SHAPE
    assert lib.cdm_attn_fwd_bf16(fake, 64, fake, 64, fake, 64, None, None, fake, 64, 16, 1, 1, 64, fake, 16, None, 0, None) == _lib.ERR_BAD_ARG
    assert "workspace" in _lib.last_error()
    # the entry point that allocates nothing rejects shapes whose tile images exceed its built-in scratch
    assert lib.cdm_attn_static_scratch_bytes() == 32 << 20
    assert lib.cdm_attn_fwd_static_bf16(fake, 4096, fake, 4096, fake, 4096, None, None, fake, 4096, 56320, 32, 32, 128, None, 0,
                                        None) == _lib.ERR_BAD_SHAPE
    assert "scratch" in _lib.last_error()
    assert lib.cdm_attn_fwd_static_bf16(fake, 64, fake, 64, fake, 64, None, None, fake, 64, 0, 1, 1, 64, None, 0, None) == _lib.OK
    assert lib.cdm_mrope_qk_bf16(fake, 64, None, 0, fake, fake, 4, 1, 32, None) == _lib.ERR_BAD_SHAPE
    assert lib.cdm_quant_rows_e4m3(fake, 128, fake, fake, 4, 100, None) == _lib.ERR_BAD_SHAPE
    # empty inputs are accepted without work
    assert lib.cdm_attn_fwd_bf16(fake, 64, fake, 64, fake, 64, fake, None, fake, 64, 16, 1, 1, 64, fake, 1 << 20, None, 0, None) == _lib.ERR_BAD_ARG   # cos without sin
    assert lib.cdm_attn_fwd_bf16(fake, 64, fake, 64, fake, 64, None, None, fake, 64, 0, 1, 1, 64, None, 0, None, 0, None) == _lib.OK
    # QK-norm descriptor: segments must cover the sequence, 1..8 segments, positive eps, both tables present
    import ctypes as C
    ends = (C.c_int64 * 2)(8, 12)
    qn = _lib.QkNorm(fake, fake, ends, 2, 1e-6)
    args = (fake, 64, fake, 64, fake, 64, None, None, fake, 64, 16, 1, 1, 64, fake, 1 << 20)
    assert lib.cdm_attn_fwd_bf16(*args, C.addressof(qn), 0, None) == _lib.ERR_BAD_ARG      # covers 12 of 16 tokens
    assert "segments cover" in lib.cdm_last_error().decode()
    qn = _lib.QkNorm(fake, None, ends, 2, 1e-6)
    assert lib.cdm_attn_fwd_bf16(*args, C.addressof(qn), 0, None) == _lib.ERR_BAD_ARG
    ends = (C.c_int64 * 2)(8, 16)
    qn = _lib.QkNorm(fake, fake, ends, 9, 1e-6)
    assert lib.cdm_attn_fwd_bf16(*args, C.addressof(qn), 0, None) == _lib.ERR_BAD_ARG
    assert lib.cdm_attn_fwd_bf16(*args, None, 17, None) == _lib.ERR_BAD_ARG                  # causal prefix > n_tokens
    pk = (fake, 64, None, None, fake, fake, 64, 16, 1, 1, 64, None)
    assert lib.cdm_attn_fwd_packed_bf16(*pk, fake, -64, 0, None, None, 0, None) == _lib.ERR_BAD_SHAPE       # negative prefix length
    assert lib.cdm_attn_fwd_packed_bf16(*pk, None, 64, 0, None, None, 0, None) == _lib.ERR_BAD_ARG          # prefix size without images
    assert lib.cdm_attn_fwd_packed_bf16(*pk, fake, 64, 4, None, None, 0, None) == _lib.ERR_UNSUPPORTED      # prefix images + causal prefix
    qn = _lib.QkNorm(fake, fake, ends, 2, 0.0)
    assert lib.cdm_attn_fwd_bf16(*args, C.addressof(qn), 0, None) == _lib.ERR_BAD_ARG
    # grouped-query attention: the K/V head count must divide the query head count
    gq = lambda H, Hkv: lib.cdm_attn_fwd_bf16(fake, 64 * H, fake, 64 * max(Hkv, 1), fake, 64 * max(Hkv, 1), None, None, fake,
                                              64 * H, 16, H, Hkv, 64, fake, 1 << 24, None, 0, None)
    assert gq(6, 4) == _lib.ERR_BAD_SHAPE and "divide" in _lib.last_error()
    assert gq(6, 0) == _lib.ERR_BAD_SHAPE
    assert lib.cdm_attn_fwd_packed_bf16(fake, 384, None, None, fake, fake, 384, 16, 6, 4, 64, None, None, 0, 0, None,
                                        None, 0, None) == _lib.ERR_BAD_SHAPE
    assert lib.cdm_attn_fwd_packed_bf16(*pk, None, 0, 0, None, fake + 4, 1 << 20, None) == _lib.ERR_BAD_ARG   # misaligned split scratch
    # the split of the last round: nothing below two whole rounds of workgroups per XCD, nothing on a whole number of rounds
    assert lib.cdm_attn_split_scratch_bytes(4096, 16, 128) == 0
    assert lib.cdm_attn_split_scratch_bytes(57344, 32, 128) == 0
    assert lib.cdm_attn_split_scratch_bytes(56320, 32, 128) == 8 * 16 * 2 * 256 * (256 + 4)      # 16 query blocks x 2 ranges per XCD
    assert lib.cdm_attn_split_scratch_bytes(56832, 32, 128) == 0      # 24 blocks left: no plan ends in half a round or less
    assert lib.cdm_attn_split_scratch_bytes(29440, 32, 128) == 8 * 12 * 8 * 256 * (256 + 4)
    assert lib.cdm_attn_split_scratch_bytes(56832, 30, 128) == 0
    assert lib.cdm_attn_fwd_packed_bf16(*pk, None, 0, 0, fake + 2, None, 0, None) == _lib.ERR_BAD_ALIGN       # misaligned row_amax
    # edge linear: strides must cover the rows
    assert lib.cdm_linear_bias_bf16(fake, 8, fake, 64, None, fake, 64, 4, 64, 64, None) == _lib.ERR_BAD_ARG
    assert lib.cdm_linear_bias_bf16(fake, 64, fake, 64, fake + 1, fake, 64, 4, 64, 64, None) == _lib.ERR_BAD_ALIGN
    assert lib.cdm_linear_bias_bf16(fake, 64, fake, 64, None, fake, 64, 0, 64, 64, None) == _lib.OK          # no rows: nothing to launch
    # partial row maxima: only the SwiGLU epilogue of the e4m3 GEMM writes them; the quantiser that reads them checks its table
    f8 = lambda epi, amax, ld: lib.cdm_gemm_fp8(fake, 256, fake, fake, 256, fake, fake, fake, fake, 256, 8, 256, 256, epi, None, 0,
                                                None, None, None, 0, 0, amax, ld, None)
    assert f8(_lib.EPI_NONE, fake, 4) == _lib.ERR_BAD_ARG and "SWIGLU" in _lib.last_error()
    assert f8(_lib.EPI_SWIGLU, fake, 3) == _lib.ERR_BAD_ARG            # 256 columns need 4 entries per row
    assert lib.cdm_quant_rows_from_parts_e4m3(fake, 128, None, 4, 4, fake, fake, 4, 128, None) == _lib.ERR_BAD_ARG
    assert lib.cdm_quant_rows_from_parts_e4m3(fake, 128, fake, 2, 4, fake, fake, 4, 128, None) == _lib.ERR_BAD_ARG
    assert lib.cdm_quant_rows_from_parts_e4m3(fake, 128, fake, 4, 4, fake, fake, 4, 100, None) == _lib.ERR_BAD_SHAPE
    assert lib.cdm_quant_rows_from_parts_e4m3(fake, 128, fake, 4, 4, fake, fake, 0, 128, None) in (_lib.OK, _lib.ERR_NO_DEVICE)
    # the workspace holds K/V heads only
    assert lib.cdm_attn_workspace_bytes(100, 2, 64) * 3 == lib.cdm_attn_workspace_bytes(100, 6, 64)
    # QKV projection with fused tile images: head_dim 128 (or 64 with even head counts), segments tile the sequence on 64-token boundaries,
    # the workspace must hold the images, and the general GEMM entry points refuse its epilogue code
    W = (C.c_void_p * 2)(fake, fake)

    def qp(starts, lens, hd=128, ws=1 << 24, H=2, Hkv=2, qkn=None):
        st, ln = (C.c_int64 * len(starts))(*starts), (C.c_int64 * len(lens))(*lens)
        return lib.cdm_grouped_gemm_qkv_pack_bf16(fake, 256, W, 256, fake, H * hd, st, ln, len(starts), 256, H, Hkv, hd, None, None,
                                                  qkn, fake, ws, None)
    assert qp([0], [100], hd=32) == _lib.ERR_UNSUPPORTED
    assert qp([0], [100], hd=64, H=3, Hkv=3) == _lib.ERR_UNSUPPORTED and "even head counts" in _lib.last_error()
    assert qp([0], [100], hd=64) in (_lib.OK, _lib.ERR_NO_DEVICE, _lib.ERR_LAUNCH)      # accepted: fails only for want of a device
    assert qp([0, 100], [100, 28]) == _lib.ERR_UNSUPPORTED and "multiple of 64" in _lib.last_error()
    assert qp([0, 128], [64, 64]) == _lib.ERR_UNSUPPORTED           # a gap between the segments
    assert qp([0], [100], ws=1024) == _lib.ERR_BAD_ARG and "workspace" in _lib.last_error()
    assert qp([0], [100], H=3, Hkv=2) == _lib.ERR_BAD_SHAPE
    # the K-norm descriptor must have the projection's segments
    e2 = (C.c_int64 * 2)(64, 128)
    qn2 = _lib.QkNorm(fake, fake, e2, 2, 1e-6)
    assert qp([0], [128], qkn=C.addressof(qn2)) == _lib.ERR_BAD_ARG and "segments" in _lib.last_error()
    e1 = (C.c_int64 * 1)(100)
    qn1 = _lib.QkNorm(fake, fake, e1, 1, 1e-6)
    assert qp([0], [128], qkn=C.addressof(qn1)) == _lib.ERR_BAD_ARG and "does not end" in _lib.last_error()
    qn0 = _lib.QkNorm(fake, fake, e1, 1, 0.0)
    assert qp([0], [100], qkn=C.addressof(qn0)) == _lib.ERR_BAD_ARG and "eps" in _lib.last_error()
    assert g(epi=5) == _lib.ERR_BAD_ARG and "qkv_pack" in _lib.last_error()


def test_step_arguments_are_validated_on_the_host():
    lib = _lib.load()
    fake = 0x10000
    coef = (C.c_float * 6)(1, 1, 0, 1, 1, 0)
    outs = (C.c_void_p * 2)(fake, fake + 64)
    hist = (C.c_void_p * 1)(fake + 128)
    call = lambda n_hist=1, n_out=2, outs=outs: lib.cdm_cfg_step_f32(fake, fake, None, 1.0, hist, n_hist, coef, outs, n_out, 0, None)
    assert call() == _lib.OK                                   # n = 0: accepted without work
    assert call(n_out=0) == _lib.ERR_BAD_ARG and call(n_out=4) == _lib.ERR_BAD_ARG
    assert call(n_hist=5) == _lib.ERR_BAD_ARG
    same = (C.c_void_p * 2)(fake, fake)
    assert call(outs=same) == _lib.ERR_BAD_ARG and "coincide" in _lib.last_error()
    odd = (C.c_void_p * 2)(fake, fake + 4)
    assert call(outs=odd) == _lib.ERR_BAD_ARG


@pytest.mark.skipif(HAS_GPU, reason="needs a host without a GPU")
def test_valid_call_without_a_device_reports_no_device():
    lib = _lib.load()
    fake = 0x10000
    assert lib.cdm_device_count() == 0
    assert lib.cdm_adaln_rmsnorm_bf16(fake, fake, None, None, fake, 4, 64, 1e-6, None) == _lib.ERR_NO_DEVICE
    assert lib.cdm_gemm_bf16(fake, 128, fake, 128, None, fake, 256, 8, 256, 128, 0, None, 0, None, None, None, 0, 0,
                             None) == _lib.ERR_NO_DEVICE
    assert "no HIP device" in _lib.last_error()


def test_ops_refuse_cpu_tensors():
    from cosmos_amd import ops
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.adaln_rmsnorm(x, torch.ones(64, dtype=torch.bfloat16))
