"""CPU-side checks (no GPU, no compute calls): the C-ABI library loads and exports every symbol the
header declares, the ctypes mirror of trn_attn_desc matches the C layout, argument validation that
happens before any launch returns the documented status codes, and the module protocol's host logic."""
import ctypes as C
import os
import re
import subprocess

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "trinity_hip.h")


@pytest.fixture(scope="module")
def lib():
    from triton_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from triton_amd import build
        build.build(verbose=False)
    return _lib.load()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(trn_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    from triton_amd import _lib
    names = declared_functions()
    assert names, "no declarations parsed from the header"
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/trinity_hip.h but not exported"
    assert sorted(_lib.EXPORTS) == names


def test_version_and_status_names(lib):
    assert lib.trn_version() >= 100
    assert lib.trn_status_name(0) == b"TRN_OK"
    assert lib.trn_status_name(-5) == b"TRN_E_UNSUPPORTED"
    assert lib.trn_status_name(-99) == b"TRN_E_UNKNOWN"


def test_attn_desc_layout_matches_c(tmp_path):
    """Compile a tiny C program against the header and compare sizeof/offsetof with ctypes."""
    from triton_amd._lib import AttnDesc
    fields = [f[0] for f in AttnDesc._fields_]
    src = tmp_path / "layout.c"
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', 'int main(void){',
             'printf("%zu\\n", sizeof(trn_attn_desc));']
    lines += [f'printf("%zu\\n", offsetof(trn_attn_desc, {f}));' for f in fields]
    lines += ['return 0;}']
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", str(src), "-o", str(exe)], check=True)
    out = [int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()]
    assert out[0] == C.sizeof(AttnDesc)
    for f, off in zip(fields, out[1:]):
        assert getattr(AttnDesc, f).offset == off, f


def _desc(**kw):
    from triton_amd._lib import AttnDesc
    d = AttnDesc()
    base = dict(batch=1, n_q_heads=4, n_kv_heads=2, seq_q=8, seq_kv=8, head_dim=64, scale=0.125, causal=1,
                q_stride_b=2048, q_stride_h=512, q_stride_s=64, k_stride_b=1024, k_stride_h=512, k_stride_s=64,
                v_stride_b=1024, v_stride_h=512, v_stride_s=64, o_stride_b=2048, o_stride_h=512, o_stride_s=64, tau=1.0)
    base.update(kw)
    for k, v in base.items():
        setattr(d, k, v)
    return d


def test_validation_rejects_before_launch(lib):
    """Every call below fails validation, so no kernel is launched and no device is touched."""
    p = C.c_void_p(0x1000)       # non-null, 16-byte aligned dummy; never dereferenced on these paths
    fwd = lambda d, q=p: lib.trn_attn_fwd_f16(C.byref(d), q, p, p, p, None, None, None, None, None)
    assert fwd(_desc(), None) == -1                                   # TRN_E_NULL
    assert fwd(_desc(head_dim=32)) == -5                              # TRN_E_UNSUPPORTED
    assert fwd(_desc(n_q_heads=3)) == -2                              # heads not a multiple of kv heads
    assert fwd(_desc(seq_kv=4)) == -2                                 # causal with fewer keys than queries
    assert fwd(_desc(scale=0.0)) == -5
    assert fwd(_desc(q_stride_s=32)) == -3                            # TRN_E_STRIDE
    assert fwd(_desc(k_stride_h=516)) == -4                           # pitch not 16-byte aligned
    assert fwd(_desc(), C.c_void_p(0x1008)) == -4                     # pointer not 16-byte aligned
    assert lib.trn_attn_fwd_f16(C.byref(_desc()), p, p, p, p, None, None, p, None, None) == -1   # noise without lse_pert
    assert lib.trn_attn_colstats_f16(C.byref(_desc()), p, p, p, None, None, None, None) == -1    # no output
    assert lib.trn_attn_colstats_f16(C.byref(_desc(q_norm=1)), p, p, p, None, p, None, None) == -5
    rms = lambda cols, ld, x=p: lib.trn_rmsnorm_f16(x, None, p, 1, 4, cols, 0, ld, 0, ld, 0, 0.0, None)
    assert rms(12, 12) == -2 and rms(64, 32) == -3 and rms(64, 68) == -4 and rms(64, 64, None) == -1
    assert lib.trn_rmsnorm_f16(None, None, None, 1, 0, 64, 0, 64, 0, 64, 0, 0.0, None) == 0      # zero rows: no-op
    g = lambda **kw: lib.trn_prenorm_qkv_f16(p, None, p, p, p, p, p, p, *[kw.get(k, v) for k, v in dict(
        tokens=16, hidden=64, n_q=64, n_kv=64, head_dim=64, ldx=64, ldwq=64, ldwk=64, ldwv=64, qh=64, qs=64, kh=64,
        ks=64, vh=64, vs=64).items()], 0.0, 1, None)
    assert g(hidden=60) == -2 and g(n_q=96) == -2 and g(ldx=32) == -3 and g(ldwq=68) == -4 and g(qs=32) == -3
    assert g(tokens=0) == 0


def test_kernel_name_follows_the_launch_rules(lib):
    """trn_attn_fwd_kernel_name answers from the same rules the launch uses (no device involved): the workgroup shape
    of the 16x16x32 kernel by problem size, the kernel with score perturbation, the decode kernel with its column
    shares."""
    def name(with_noise=0, **kw):
        S, Skv, D, H = kw.get("seq_q", 8), kw.get("seq_kv", kw.get("seq_q", 8)), kw.get("head_dim", 64), kw.get("n_q_heads", 4)
        kw.setdefault("seq_kv", Skv)
        strides = dict(q_stride_b=H * S * D, q_stride_h=S * D, q_stride_s=D, o_stride_b=H * S * D, o_stride_h=S * D, o_stride_s=D,
                       k_stride_b=kw.get("n_kv_heads", 2) * Skv * D, k_stride_h=Skv * D, k_stride_s=D,
                       v_stride_b=kw.get("n_kv_heads", 2) * Skv * D, v_stride_h=Skv * D, v_stride_s=D)
        return lib.trn_attn_fwd_kernel_name(C.byref(_desc(**strides, **kw)), with_noise).decode()
    llama = dict(n_q_heads=32, n_kv_heads=8, head_dim=128)
    assert name(seq_q=4096, **llama) == "trn::attn_fwd16_kernel<128, 8, false>"         # two rounds of wide workgroups
    assert name(seq_q=2048, **llama) == "trn::attn_fwd16_kernel<128, 8, true>"          # a single round: paired tiles
    assert name(seq_q=1024, **llama) == "trn::attn_fwd16_kernel<128, 4, false>"         # pairs would cover half the chip
    assert name(seq_q=4096, causal=0, **llama) == "trn::attn_fwd16_kernel<128, 8, false>"
    assert name(seq_q=2048, n_q_heads=71, n_kv_heads=1, head_dim=64) == "trn::attn_fwd16_kernel<64, 4, false>"
    assert name(1, seq_q=4096, **llama) == "trn::attn_fwd_kernel<128, 8, true>"
    assert name(1, seq_q=512, **llama) == "trn::attn_fwd_kernel<128, 4, true>"
    assert name(seq_q=16, seq_kv=1040, causal=0, **llama) == "trn::attn_decode_kernel<128, 4, 0>"
    assert name(1, seq_q=16, seq_kv=1040, causal=0, n_q_heads=71, n_kv_heads=71, head_dim=64) == "trn::attn_decode_kernel<64, 2, 1>"
    assert name(seq_q=16, seq_kv=100, causal=0, **llama) == "trn::attn_decode_kernel<128, 1, 0>"    # short cache
    assert name(seq_q=16, seq_kv=1040, causal=0, n_q_heads=160, n_kv_heads=8, head_dim=128) == "trn::attn_decode_kernel<128, 1, 0>"
    assert name(head_dim=32) == ""                                                                 # invalid descriptor


def test_validation_of_the_workspace_statistics_and_linear_entry_points(lib):
    """As above: every call fails validation before anything is launched."""
    p = C.c_void_p(0x1000)
    d = _desc()
    ws = lambda w, n: lib.trn_attn_fwd_ws_f16(C.byref(d), p, p, p, p, None, None, None, None, w, n, None)
    assert ws(C.c_void_p(0x1010), 4096) == -4                          # workspace not 256-byte aligned
    assert lib.trn_attn_fwd_ws_f16(C.byref(d), None, p, p, p, None, None, None, None, p, 4096, None) == -1
    assert lib.trn_attn_workspace_bytes(C.byref(_desc(head_dim=32))) == 0      # invalid shape: no workspace
    assert lib.trn_attn_workspace_bytes(None) == 0
    st = lambda dd, s1, s2: lib.trn_attn_fwd_stats_f16(C.byref(dd), p, p, p, p, None, None, None, None, s1, s2, None)
    assert st(d, None, None) == -1                                     # no statistics output
    assert st(_desc(q_norm=1), p, None) == -5                          # fused query norm is not offered with statistics
    assert st(_desc(seq_q=64, seq_kv=64), p, None) == -1               # more than 32 queries: lse is the hand-over buffer
    vps = lambda *xs: (C.c_void_p * len(xs))(*xs)
    i64 = lambda *xs: (C.c_int64 * len(xs))(*xs)
    lin = lambda tokens=4, hidden=64, ldx=64, k=1, n=(64,), ldw=(64,), ldo=(64,), w=None: lib.trn_linear_f16(
        p, tokens, hidden, ldx, k, w if w is not None else vps(*([0x1000] * len(n))), i64(*n), i64(*ldw), vps(*([0x1000] * len(n))), i64(*ldo), None, None)
    assert lin(k=0) == -2 and lin(k=4) == -2 and lin(hidden=60) == -2 and lin(n=(12,), ldw=(12,), ldo=(12,)) == -2
    assert lin(ldx=32) == -3 and lin(ldw=(32,)) == -3 and lin(ldo=(68,)) == -4
    assert lin(w=vps(None)) == -1 and lin(tokens=0) == 0
    gate = lambda rows=4, cols=64, ld=64, kind=0, c1=p: lib.trn_gate_f16(c1, p, p, rows, cols, ld, ld, ld, kind, None)
    assert gate(cols=12) == -2 and gate(kind=2) == -2 and gate(ld=32) == -3 and gate(ld=68) == -4
    assert gate(c1=None) == -1 and gate(rows=0) == 0


def test_no_workspace_exceeds_the_static_scratch_array(lib):
    """trn_attn_fwd_noalloc_f16 rejects a problem whose workspace is larger than the library's static array.  With
    the present split rule that cannot happen; this sweep of trn_attn_workspace_bytes over the decode shapes (host
    arithmetic, nothing is launched) is what trips when a change to the rule makes it possible."""
    import re
    hdr = open(os.path.join(ROOT, "include", "trinity_hip.h")).read()
    m = re.search(r"#define TRN_ATTN_NOALLOC_SCRATCH_BYTES \((\d+)u << (\d+)\)", hdr)
    capacity = int(m.group(1)) << int(m.group(2))
    largest = 0
    for D in (64, 128):
        for heads in (1, 2, 3, 7, 8, 16, 31, 32, 63, 64, 71, 100, 127, 128, 200):
            for batch in (1, 2, 5):
                for sq in (1, 16, 32):
                    for skv in (64, 1024, 1040, 4112, 16384, 131072, 1 << 20):
                        d = _desc(batch=batch, n_q_heads=heads, n_kv_heads=1, seq_q=sq, seq_kv=skv, head_dim=D,
                                  q_stride_b=heads * sq * D, q_stride_h=sq * D, q_stride_s=D, k_stride_b=skv * D,
                                  k_stride_h=skv * D, k_stride_s=D, v_stride_b=skv * D, v_stride_h=skv * D, v_stride_s=D,
                                  o_stride_b=heads * sq * D, o_stride_h=sq * D, o_stride_s=D, causal=0)
                        largest = max(largest, lib.trn_attn_workspace_bytes(C.byref(d)))
    assert 0 < largest <= capacity, (largest, capacity)


def test_attention_split_rule_on_the_host(lib):
    """trn_attn_workspace_bytes: keys are split from 4096 keys with at most 16 heads, from 8192 with more, never with 128
    heads or more or with more than 32 queries per head; the size is counters + heads x shares x 32 x (head_dim + 4) floats."""
    def need(heads, sq, skv, D=128, batch=1):
        d = _desc(batch=batch, n_q_heads=heads, n_kv_heads=1, seq_q=sq, seq_kv=skv, head_dim=D, causal=0,
                  q_stride_b=heads * sq * D, q_stride_h=sq * D, q_stride_s=D, k_stride_b=skv * D, k_stride_h=skv * D,
                  k_stride_s=D, v_stride_b=skv * D, v_stride_h=skv * D, v_stride_s=D, o_stride_b=heads * sq * D,
                  o_stride_h=sq * D, o_stride_s=D)
        return lib.trn_attn_workspace_bytes(C.byref(d))
    for heads, sq, skv, D, split in ((8, 16, 4096, 128, True), (8, 16, 4095, 128, False), (16, 1, 4096, 64, True),
                                     (17, 16, 8191, 128, False), (17, 16, 8192, 128, True), (32, 16, 1040, 128, False),
                                     (71, 16, 8192, 64, True), (127, 16, 8192, 128, True), (128, 16, 1 << 20, 128, False),
                                     (8, 33, 16384, 128, False)):
        assert (need(heads, sq, skv, D) > 0) == split, (heads, sq, skv, D)
    assert need(64, 16, 4096, batch=2) == 0 and need(4, 16, 4096, batch=2) > 0      # the head count is batch x heads
    # 32 heads, 8208 keys: 8 shares of 33 blocks; 8 heads, 4112 keys: 16 shares of 9 blocks, the last one short (15 shares)
    assert need(32, 16, 8208) == 256 + 32 * 8 * 32 * 132 * 4
    assert need(8, 16, 4112) == 256 + 8 * 15 * 32 * 132 * 4


def test_statistics_split_rule_on_the_host(lib):
    """trn_attn_stats_workspace_bytes: the long-cache rule (few heads, many keys, at most 32 queries per head) is host
    arithmetic; where it says split, the size is that of the attention's own split workspace."""
    def need(heads, sq, skv, D=128, fn=lib.trn_attn_stats_workspace_bytes):
        d = _desc(batch=1, n_q_heads=heads, n_kv_heads=1, seq_q=sq, seq_kv=skv, head_dim=D, causal=0,
                  q_stride_b=heads * sq * D, q_stride_h=sq * D, q_stride_s=D, k_stride_b=skv * D, k_stride_h=skv * D,
                  k_stride_s=D, v_stride_b=skv * D, v_stride_h=skv * D, v_stride_s=D, o_stride_b=heads * sq * D,
                  o_stride_h=sq * D, o_stride_s=D)
        return fn(C.byref(d))
    for heads, sq, skv, D, split in ((8, 16, 8192, 128, True), (8, 16, 8191, 128, False), (16, 16, 8192, 64, True),
                                     (16, 16, 8192, 128, False), (16, 16, 16384, 128, True), (4, 16, 4096, 128, True),
                                     (4, 16, 4095, 128, False), (2, 16, 4096, 64, True), (17, 4, 65536, 128, False),
                                     (32, 16, 65536, 128, False), (32, 16, 16384, 64, True), (71, 16, 65536, 64, False),
                                     (8, 33, 16384, 128, False), (8, 1, 1040, 128, False)):
        got = need(heads, sq, skv, D)
        assert (got > 0) == split, (heads, sq, skv, D, got)
        if split:
            assert got == need(heads, sq, skv, D, lib.trn_attn_workspace_bytes)
    assert lib.trn_attn_stats_workspace_bytes(None) == 0


def test_a_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    from triton_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libtrinity_hip.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib.load()


def test_wrappers_raise_python_exceptions_on_cpu_tensors():
    from triton_amd import ops
    x = torch.zeros(4, 64, dtype=torch.float16)
    with pytest.raises(ValueError, match="GPU tensor"):
        ops.rmsnorm(x, None, x.clone(), 0.0)
    q = torch.zeros(1, 2, 8, 64, dtype=torch.float16)
    with pytest.raises(ValueError):
        ops.attention(q, q, q, q, 1.0, True)


def test_module_protocol_host_logic():
    from triton_amd import modules
    from triton_amd.modules import keyformer, prenorm, qknorm, rms, roco, vanilla
    for mod in (keyformer, prenorm, qknorm, rms, roco, vanilla):
        assert mod.TENSOR_PARAMS == sorted(mod.TENSOR_PARAMS, key=lambda s: s) and mod.BLOCK_PARAMS == []
        assert callable(mod.forward)
    # names the reference's drivers know (vanilla_llama_benchmark.py:42-77, keyformer_llama_benchmark.py:74-79)
    assert modules.get("vanilla", "decode", head_dim=128).TENSOR_PARAMS == ["K_cache", "O2", "V_cache", "WK", "WQ", "WV", "X"]
    assert "noise" in modules.get("keyformer", "decode", head_dim=128).TENSOR_PARAMS
    assert {"C_out1", "C_out2"} <= set(modules.get("roco", "decode", head_dim=64).TENSOR_PARAMS)
    with pytest.raises(KeyError):
        modules.get("nope")
    m = modules.get("vanilla")
    with pytest.raises(TypeError):
        m.forward(torch.zeros(1))                       # too few tensors
    with pytest.raises(ValueError):
        modules.get("roco", stats="variance")
    assert modules.get("roco", stats="mean_std").TENSOR_PARAMS == modules.get("roco").TENSOR_PARAMS


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run(["python", os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_flop_and_byte_conventions():
    from triton_amd import configs
    assert configs.attn_flops(1, 32, 4096, 4096, 128, True) == 137438953472
    assert configs.rmsnorm_bytes(4096, 4096) == 67117056
    assert configs.qkv_gemm_flops(2048, 4096, 4096, 1024) == 103079215104
    assert configs.attn_flops(1, 71, 2048, 2048, 64, True) == 38117834752
