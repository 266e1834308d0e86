"""Host-side checks that need no GPU: the C ABI library loads and exports every symbol the
header declares, compute calls fail loudly without a device (no CPU fallback), the product
package never touches the oracle, and artifact validation reports bad task graphs."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "fusekit_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fk_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import fusekit_amd.native as fk
    names = _declared()
    assert len(names) >= 40
    missing = [n for n in names if not hasattr(fk.lib, n)]
    assert not missing, missing
    assert "gfx950" in fk.version()


def test_compute_fails_loudly_without_a_device():
    import fusekit_amd.native as fk
    if fk.has_device():
        pytest.skip("a HIP device is present")
    with pytest.raises(fk.FusekitError) as e:
        fk.DeviceBuffer(16)
    assert e.value.status == fk.FK_ERR_HIP and "no CPU path" in str(e.value)
    w = fk.Weight(1, 1, 1, 8, 64, 4, 64)
    assert fk.lib.fk_qgemv(C.byref(w), C.c_void_p(1), None, C.c_void_p(1), None) == fk.FK_ERR_HIP
    h = C.c_uint64()
    assert fk.lib.fk_load_dispatcher(None, None, C.byref(h)) == fk.FK_ERR_HIP


def test_artifact_validation_precedes_device_use(tmp_path):
    """A bad task graph is reported as such on any machine (version gate, unknown kernel)."""
    import fusekit_amd.native as fk
    h = C.c_uint64()
    missing = str(tmp_path / "missing.json").encode()
    assert fk.lib.fk_load_dispatcher(None, missing, C.byref(h)) == fk.FK_ERR_NOT_FOUND
    p = tmp_path / "task_graph.json"
    p.write_text('{"version": 1, "tasks": []}')
    assert fk.lib.fk_load_dispatcher(None, str(p).encode(), C.byref(h)) == fk.FK_ERR_INVALID
    assert b"version" in fk.lib.fk_last_error()
    p.write_text('{"version": 2, "tasks": [{"id": 0, "kernel": "fusekit_not_a_kernel_f3"}]}')
    assert fk.lib.fk_load_dispatcher(None, str(p).encode(), C.byref(h)) == fk.FK_ERR_INVALID
    assert b"fusekit_not_a_kernel_f3" in fk.lib.fk_last_error()
    p.write_text('{"version": 2, "tasks": [')
    assert fk.lib.fk_load_dispatcher(None, str(p).encode(), C.byref(h)) == fk.FK_ERR_IO
    assert fk.lib.fk_load_dispatcher(str(tmp_path / "kernel.hsaco").encode(), None, C.byref(h)) == fk.FK_ERR_NOT_FOUND


def test_product_never_imports_or_links_the_oracle():
    pkg = os.path.join(ROOT, "fusekit_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")) or f == "Makefile":
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)
                assert "_work/" not in text and "_work\"" not in text, os.path.join(dirpath, f)


def test_decoder_config_byte_accounting():
    from fusekit_amd.decoder import DENSE_4B, DecoderConfig
    cfg = DecoderConfig(**DENSE_4B)
    per_layer = 2560 * (4096 + 1024 + 1024) + 4096 * 2560 + 3 * 9728 * 2560
    assert per_layer == 100925440
    assert cfg.layer_param_bytes() == int(per_layer * 0.5625)
    assert cfg.n_layers * cfg.layer_param_bytes() == 2043740160          # 4-bit g64 layer weights per token
    assert cfg.token_bytes(512) == 2043740160 + 777912320 + 75497472     # + tied bf16 LM head + KV at ctx 512
    assert DecoderConfig(**DENSE_4B, bits=8).n_layers * DecoderConfig(**DENSE_4B, bits=8).layer_param_bytes() == 3860398080
    assert DecoderConfig(**DENSE_4B, bits=16).n_layers * DecoderConfig(**DENSE_4B, bits=16).layer_param_bytes() == 7266631680


def test_target_description_without_a_gpu():
    """T1: fk_target_describe answers with the published MI355X figures when no device is visible."""
    import ctypes as C
    import os
    lib = C.CDLL(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "fusekit_amd", "libfusekit_hip.so"))

    class Target(C.Structure):
        _fields_ = [("arch", C.c_char * 32), ("from_device", C.c_uint32), ("compute_units", C.c_uint32),
                    ("xcds", C.c_uint32), ("wave_size", C.c_uint32), ("simds_per_cu", C.c_uint32),
                    ("vgprs_per_lane", C.c_uint32), ("lds_bytes_per_cu", C.c_uint32), ("workgroup_threads", C.c_uint32),
                    ("gemm_min_rows", C.c_uint32), ("gemm_rows_per_pass", C.c_uint32), ("hbm_bytes", C.c_uint64),
                    ("hbm_peak_bytes_per_s", C.c_double), ("mfma_bf16_peak_flops", C.c_double)]
    t = Target()
    assert lib.fk_target_describe(C.byref(t)) == 0
    assert t.arch.startswith(b"gfx950") and t.wave_size == 64 and t.workgroup_threads == 256
    if not t.from_device:
        assert (t.compute_units, t.xcds, t.lds_bytes_per_cu) == (256, 8, 160 * 1024)
        assert t.hbm_peak_bytes_per_s == 8.0e12 and t.hbm_bytes == 288 << 30


def test_two_launch_layer_admission_rules_need_no_device():
    """The shape rules of the two-launch layer, the LDS budget among them, are checked before any device is asked:
    a bf16 layer of hidden 4096 / intermediate 14336 needs more than half a CU's LDS per workgroup, so its 512
    workgroups could not all be resident (the hand-overs need that) -- refused as unsupported, on any machine."""
    import fusekit_amd.native as fk
    u = C.c_uint32
    st = fk.lib.fk_xcd_layer_supported(u(4096), u(14336), u(32), u(8), u(128), u(1024), u(16), u(64))
    assert st == fk.FK_ERR_UNSUPPORTED and b"resident" in fk.lib.fk_last_error()
    st = fk.lib.fk_xcd_layer_supported(u(4096), u(12288), u(32), u(8), u(128), u(1024), u(16), u(64))
    assert st == fk.FK_ERR_UNSUPPORTED and b"resident" in fk.lib.fk_last_error()
    st = fk.lib.fk_xcd_layer_supported(u(2560), u(9728), u(32), u(4), u(128), u(1024), u(4), u(64))
    assert st == fk.FK_ERR_UNSUPPORTED and b"8 KV heads" in fk.lib.fk_last_error()
    # the 4B-class shape passes every rule; without a device the answer is then "no HIP device"
    st = fk.lib.fk_xcd_layer_supported(u(2560), u(9728), u(32), u(8), u(128), u(1024), u(4), u(64))
    assert st == (fk.FK_OK if fk.has_device() else fk.FK_ERR_HIP), fk.lib.fk_last_error()
    # the 8B class: in 4 bits its tiles (up to 1792 quantisation groups) fit the flavour with the pass loop; in 8 bits
    # two workgroups of the MLP launch do not fit a CU
    st = fk.lib.fk_xcd_layer_supported(u(4096), u(14336), u(32), u(8), u(128), u(1024), u(4), u(64))
    assert st == (fk.FK_OK if fk.has_device() else fk.FK_ERR_HIP), fk.lib.fk_last_error()
    st = fk.lib.fk_xcd_layer_supported(u(4096), u(14336), u(32), u(8), u(128), u(1024), u(8), u(64))
    assert st == fk.FK_ERR_UNSUPPORTED and b"resident" in fk.lib.fk_last_error()
    # a tile beyond 2048 groups per matrix is refused (hidden 4096 in groups of 32: 28 rows x 128 groups)
    st = fk.lib.fk_xcd_layer_supported(u(4096), u(14336), u(32), u(8), u(128), u(1024), u(4), u(32))
    assert st == fk.FK_ERR_UNSUPPORTED and b"quantisation groups" in fk.lib.fk_last_error()


def test_expert_and_low_rank_attention_launch_admission_rules_need_no_device():
    """fk_xcd_moe_supported / fk_xcd_mla_supported answer the shape rules on any machine; a shape that passes them all is
    then asked of the device."""
    import fusekit_amd.native as fk
    u = C.c_uint32
    ok = fk.FK_OK if fk.has_device() else fk.FK_ERR_HIP
    moe = lambda *a: fk.lib.fk_xcd_moe_supported(*[u(v) for v in a])
    assert moe(2048, 1408, 2816, 64, 6, 4, 64) == ok, fk.lib.fk_last_error()
    assert moe(2048, 1408, 2816, 64, 6, 8, 64) == fk.FK_ERR_UNSUPPORTED and b"4-bit" in fk.lib.fk_last_error()
    assert moe(2048, 1408, 2816, 128, 6, 4, 64) == fk.FK_ERR_UNSUPPORTED and b"64 experts" in fk.lib.fk_last_error()
    assert moe(2048, 1408, 4224, 64, 6, 4, 64) == fk.FK_ERR_UNSUPPORTED and b"at most 8" in fk.lib.fk_last_error()
    assert moe(2048, 1400, 2800, 64, 6, 4, 64) == fk.FK_ERR_UNSUPPORTED and b"multiples of 128" in fk.lib.fk_last_error()
    assert moe(4096, 2048, 4096, 64, 6, 4, 64) == fk.FK_ERR_UNSUPPORTED and b"chunks" in fk.lib.fk_last_error()
    mla = lambda *a: fk.lib.fk_xcd_mla_supported(*[u(v) for v in a])
    assert mla(2048, 16, 512, 64, 128, 128, 1024, 4, 64) == ok, fk.lib.fk_last_error()
    assert mla(2048, 12, 512, 64, 128, 128, 1024, 4, 64) == fk.FK_ERR_UNSUPPORTED and b"heads" in fk.lib.fk_last_error()
    assert mla(2048, 16, 512, 64, 128, 128, 1024, 8, 64) == fk.FK_ERR_UNSUPPORTED and b"4-bit" in fk.lib.fk_last_error()
    assert mla(2048, 16, 448, 64, 128, 128, 1024, 4, 64) == fk.FK_ERR_UNSUPPORTED and b"latent" in fk.lib.fk_last_error()
    assert fk.xcd_moe_scratch_bytes(1408) == 8 * 64 * 4 + 8 * 1408 * 2
