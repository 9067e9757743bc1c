"""The C-ABI library on a machine without a GPU: it loads, exports every symbol include/pith_hip.h
declares, its argument structs have the layout the Python binding assumes, and every entry point
rejects bad arguments with an error code before touching the device."""

import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pith_hip.h")

from pithtrain_amd import _C  # noqa: E402


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pith_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _C.lib()
    declared = _declared_symbols()
    assert len(declared) >= 9
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in pith_hip.h but not exported"
    assert sorted(_C.SYMBOLS) == declared, "python binding table and header disagree"
    assert lib.pith_version() >= 100
    assert lib.pith_error_name(-2) == b"PITH_ERR_BAD_SHAPE"


def test_struct_layouts_match_the_header(tmp_path):
    """sizeof/offsetof from a C compile of the header against the ctypes Structures."""
    pairs = {
        "pith_combine_args": _C.CombineArgs,
        "pith_attn_fwd_args": _C.AttnFwdArgs,
        "pith_attn_delta_args": _C.AttnDeltaArgs,
        "pith_attn_bwd_args": _C.AttnBwdArgs,
        "pith_norm_rope_args": _C.NormRopeArgs,
        "pith_mla_assemble_args": _C.MlaAssembleArgs,
        "pith_device_info_t": _C.DeviceInfo,
    }
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "pith_hip.h"', "int main(void){"]
    for cname, st in pairs.items():
        lines.append(f'printf("{cname} %zu\\n", sizeof({cname}));')
        for fname, _ in st._fields_:
            lines.append(f'printf("{cname}.{fname} %zu\\n", offsetof({cname}, {fname}));')
    lines.append("return 0;}")
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    got = dict(line.split() for line in out.strip().splitlines())
    for cname, st in pairs.items():
        assert int(got[cname]) == ctypes.sizeof(st), cname
        for fname, _ in st._fields_:
            assert int(got[f"{cname}.{fname}"]) == getattr(st, fname).offset, f"{cname}.{fname}"


def test_device_info_without_a_device():
    lib = _C.lib()
    assert lib.pith_device_info(0, None) == _C.PITH_ERR_NULL_POINTER
    info = _C.DeviceInfo()
    rc = lib.pith_device_info(0, ctypes.byref(info))
    import torch

    if torch.cuda.is_available():
        assert rc == _C.PITH_OK and info.compute_units > 0
    else:  # no GPU here: the runtime's error is reported, nothing crashes
        assert rc == _C.PITH_ERR_LAUNCH and lib.pith_last_error().startswith(b"pith_device_info")


def _fwd_args(**kw):
    base = dict(q=16, k=16, v=16, o=16, lse=16, B=1, Sq=64, Skv=64, Hq=4, Hkv=2, Dqk=128, Dv=128,
                q_bs=64 * 4 * 128, k_bs=64 * 2 * 128, v_bs=64 * 2 * 128, o_bs=64 * 4 * 128,
                lse_bs=4 * 64, lse_hs=64, scale=0.088, causal=0)  # fmt: skip
    base.update(kw)
    return _C.AttnFwdArgs(**base)


@pytest.mark.parametrize(
    "kw,code",
    [
        (dict(q=None), _C.PITH_ERR_NULL_POINTER),
        (dict(Sq=0), _C.PITH_ERR_BAD_SHAPE),
        (dict(Hq=3), _C.PITH_ERR_BAD_SHAPE),
        (dict(causal=1, Skv=32), _C.PITH_ERR_UNSUPPORTED),
        (dict(Dqk=96), _C.PITH_ERR_UNSUPPORTED),
        (dict(Dqk=192, Dv=192), _C.PITH_ERR_UNSUPPORTED),
        (dict(k=8), _C.PITH_ERR_MISALIGNED),
        (dict(q_bs=100), _C.PITH_ERR_MISALIGNED),
    ],
)
def test_attn_fwd_rejects_bad_arguments(kw, code):
    lib = _C.lib()
    rc = lib.pith_attn_fwd(ctypes.byref(_fwd_args(**kw)), None)
    assert rc == code, lib.pith_last_error()
    assert lib.pith_last_error().startswith(b"pith_attn_fwd")
    with pytest.raises(_C.PithError) as e:
        _C.check(rc)
    assert e.value.code == code


def test_null_args_struct_is_rejected_everywhere():
    lib = _C.lib()
    for name in ("pith_combine", "pith_attn_fwd", "pith_attn_bwd_delta", "pith_attn_bwd_dkdv", "pith_attn_bwd_dq"):
        assert getattr(lib, name)(None, None) == _C.PITH_ERR_NULL_POINTER, name
    assert lib.pith_cast_f32_bf16(None, None, 8, None) == _C.PITH_ERR_NULL_POINTER
    assert lib.pith_cast_f32_bf16(16, 16, 12, None) == _C.PITH_ERR_BAD_SHAPE


def test_combine_and_bwd_validation():
    lib = _C.lib()
    c = _C.CombineArgs(out1=16, lse1=16, out2=16, lse2=16, out=16, lse_out=16, dtype1=0, dtype2=1, dtype_out=1,
                       base=0, B=1, S=8, H=2, D=128, out1_bs=2048, out2_bs=2048, out_bs=2048, lse1_bs=16, lse1_hs=8,
                       lse2_bs=16, lse2_hs=8, lse_out_bs=16, lse_out_hs=8)  # fmt: skip
    c.dtype2 = 7
    assert lib.pith_combine(ctypes.byref(c), None) == _C.PITH_ERR_BAD_DTYPE
    c.dtype2, c.base = 1, 5
    assert lib.pith_combine(ctypes.byref(c), None) == _C.PITH_ERR_BAD_DTYPE
    c.base, c.D = 0, 100
    assert lib.pith_combine(ctypes.byref(c), None) == _C.PITH_ERR_BAD_SHAPE
    b = _C.AttnBwdArgs(q=16, k=16, v=16, dout=16, lse=16, delta=16, dq=None, dk=16, dv=16, B=1, Sq=64, Skv=64, Hq=4,
                       Hkv=4, Dqk=128, Dv=128, scale=0.1)  # fmt: skip
    assert lib.pith_attn_bwd_dq(ctypes.byref(b), None) == _C.PITH_ERR_NULL_POINTER  # dq missing
    b.dk = None
    assert lib.pith_attn_bwd_dkdv(ctypes.byref(b), None) == _C.PITH_ERR_NULL_POINTER
    d = _C.AttnDeltaArgs(o=16, dout=16, delta=16, B=1, S=8, H=2, D=96)
    assert lib.pith_attn_bwd_delta(ctypes.byref(d), None) == _C.PITH_ERR_UNSUPPORTED


def _norm_rope_args(**kw):
    base = dict(x=16, weight=16, cos=16, sin=16, dout=16, out=16, dweight=16, workspace=None, workspace_bytes=0,
                B=2, S=64, H=4, D=128, x_bs=64 * 4 * 128, out_bs=64 * 4 * 128, dout_bs=64 * 4 * 128, cs_bs=64 * 128,
                eps=1e-6, weight_dtype=_C.PITH_BF16)  # fmt: skip
    base.update(kw)
    return _C.NormRopeArgs(**base)


@pytest.mark.parametrize(
    "kw,code",
    [
        (dict(x=None), _C.PITH_ERR_NULL_POINTER),
        (dict(cos=None), _C.PITH_ERR_NULL_POINTER),
        (dict(H=0), _C.PITH_ERR_BAD_SHAPE),
        (dict(D=96), _C.PITH_ERR_UNSUPPORTED),
        (dict(D=1024), _C.PITH_ERR_UNSUPPORTED),
        (dict(weight_dtype=9), _C.PITH_ERR_BAD_DTYPE),
        (dict(x=12), _C.PITH_ERR_MISALIGNED),
        (dict(cs_bs=6), _C.PITH_ERR_MISALIGNED),
        (dict(x_bs=1024), _C.PITH_ERR_BAD_SHAPE),
        (dict(cs_bs=128), _C.PITH_ERR_BAD_SHAPE),
    ],
)
def test_norm_rope_rejects_bad_arguments(kw, code):
    lib = _C.lib()
    for fn in (lib.pith_norm_rope_fwd, lib.pith_norm_rope_bwd):
        rc = fn(ctypes.byref(_norm_rope_args(**kw)), None)
        assert rc == code, lib.pith_last_error()
        assert lib.pith_last_error().startswith(b"pith_norm_rope")


def test_norm_rope_backward_needs_its_workspace():
    lib = _C.lib()
    assert lib.pith_norm_rope_fwd(None, None) == _C.PITH_ERR_NULL_POINTER
    assert lib.pith_norm_rope_bwd(None, None) == _C.PITH_ERR_NULL_POINTER
    a = _norm_rope_args()
    need = lib.pith_norm_rope_bwd_workspace_bytes(ctypes.byref(a))
    assert need > 0 and need % (128 * 4) == 0
    assert lib.pith_norm_rope_bwd(ctypes.byref(a), None) == _C.PITH_ERR_BAD_SHAPE  # no workspace given
    assert b"workspace" in lib.pith_last_error()
    a.workspace, a.workspace_bytes = 16, need - 4
    assert lib.pith_norm_rope_bwd(ctypes.byref(a), None) == _C.PITH_ERR_BAD_SHAPE
    assert lib.pith_norm_rope_bwd(ctypes.byref(_norm_rope_args(dout=None)), None) == _C.PITH_ERR_NULL_POINTER
    assert lib.pith_norm_rope_bwd(ctypes.byref(_norm_rope_args(dweight=None)), None) == _C.PITH_ERR_NULL_POINTER
    # the two-tensor launch: both structs are validated, B must agree, weights both or neither
    ok = _norm_rope_args(workspace=16, workspace_bytes=need)
    assert lib.pith_norm_rope_fwd_pair(ctypes.byref(ok), None, None) == _C.PITH_ERR_NULL_POINTER
    assert lib.pith_norm_rope_bwd_pair(None, ctypes.byref(ok), None) == _C.PITH_ERR_NULL_POINTER
    for fn in (lib.pith_norm_rope_fwd_pair, lib.pith_norm_rope_bwd_pair):
        assert fn(ctypes.byref(ok), ctypes.byref(_norm_rope_args(D=96)), None) == _C.PITH_ERR_UNSUPPORTED
        other_b = _norm_rope_args(B=3, workspace=16, workspace_bytes=1 << 30)
        assert fn(ctypes.byref(ok), ctypes.byref(other_b), None) == _C.PITH_ERR_BAD_SHAPE
        assert b"differ in B" in lib.pith_last_error()
        assert fn(ctypes.byref(ok), ctypes.byref(_norm_rope_args(weight=None)), None) == _C.PITH_ERR_UNSUPPORTED
    # without a weight there is nothing to reduce, hence no workspace
    assert lib.pith_norm_rope_bwd_workspace_bytes(ctypes.byref(_norm_rope_args(weight=None))) == 0


def _mla_assemble_args(**kw):
    base = dict(q=16, kv=16, k_pe=16, cos=16, sin=16, position_ids=None, q_out=16, k_out=16, v_out=16,
                dq_out=16, dk_out=16, dv_out=16, B=2, S=8, H=16, Dn=128, Dr=64, Dv=128, P=64,
                q_bs=8 * 16 * 192, kv_bs=8 * 16 * 256, k_pe_bs=8 * 576, k_pe_rs=576, pos_bs=8)  # fmt: skip
    base.update(kw)
    return _C.MlaAssembleArgs(**base)


@pytest.mark.parametrize(
    "kw,code",
    [
        (dict(cos=None), _C.PITH_ERR_NULL_POINTER),
        (dict(q_out=None), _C.PITH_ERR_NULL_POINTER),
        (dict(S=0), _C.PITH_ERR_BAD_SHAPE),
        (dict(P=0), _C.PITH_ERR_BAD_SHAPE),
        (dict(Dr=24), _C.PITH_ERR_UNSUPPORTED),
        (dict(Dn=100), _C.PITH_ERR_UNSUPPORTED),
        (dict(sin=8), _C.PITH_ERR_MISALIGNED),
        (dict(position_ids=4), _C.PITH_ERR_MISALIGNED),
    ],
)
def test_mla_assemble_rejects_bad_arguments(kw, code):
    lib = _C.lib()
    for fn in (lib.pith_mla_assemble_fwd, lib.pith_mla_assemble_bwd):
        rc = fn(ctypes.byref(_mla_assemble_args(**kw)), None)
        assert rc == code, lib.pith_last_error()
        assert lib.pith_last_error().startswith(b"pith_mla_assemble")


def test_mla_assemble_direction_specific_validation():
    lib = _C.lib()
    assert lib.pith_mla_assemble_fwd(None, None) == _C.PITH_ERR_NULL_POINTER
    assert lib.pith_mla_assemble_bwd(None, None) == _C.PITH_ERR_NULL_POINTER
    fwd, bwd = lib.pith_mla_assemble_fwd, lib.pith_mla_assemble_bwd
    assert fwd(ctypes.byref(_mla_assemble_args(kv=None)), None) == _C.PITH_ERR_NULL_POINTER
    assert bwd(ctypes.byref(_mla_assemble_args(dk_out=None)), None) == _C.PITH_ERR_NULL_POINTER
    assert fwd(ctypes.byref(_mla_assemble_args(k_pe_rs=32)), None) == _C.PITH_ERR_BAD_SHAPE
    assert fwd(ctypes.byref(_mla_assemble_args(k_pe_rs=580)), None) == _C.PITH_ERR_MISALIGNED
    assert fwd(ctypes.byref(_mla_assemble_args(q_bs=1024)), None) == _C.PITH_ERR_BAD_SHAPE
    # the backward stages every head's rope gradient in LDS: H * Dr is limited
    assert bwd(ctypes.byref(_mla_assemble_args(H=512)), None) == _C.PITH_ERR_UNSUPPORTED


def test_operators_refuse_cpu_tensors():
    """No CPU fallback: the product path raises instead of computing somewhere else."""
    import torch

    from pithtrain_amd.operators.mla.hip import _mla_fwd
    from pithtrain_amd.operators.ring_attention.mla import _online_softmax_combine_log2

    q = torch.zeros(1, 64, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="need tensors on a GPU"):
        _mla_fwd(q, q, q, 0.1, causal=True)
    lse = torch.zeros(1, 2, 64)
    with pytest.raises(RuntimeError, match="need tensors on a GPU"):
        _online_softmax_combine_log2(q, lse, q, lse)
    from pithtrain_amd.operators.norm_rope import qk_norm_rope

    w = torch.ones(128, dtype=torch.bfloat16)
    cs = torch.zeros(1, 64, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="need tensors on a GPU"):
        qk_norm_rope(q, q, w, w, cs, cs, 1e-6)
    from pithtrain_amd.operators.mla_assemble import mla_assemble_qkv

    x = torch.zeros(1, 4, 2, 192, dtype=torch.bfloat16)
    kv = torch.zeros(1, 4, 2, 256, dtype=torch.bfloat16)
    table = torch.zeros(8, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="need tensors on a GPU"):
        mla_assemble_qkv(x, kv, torch.zeros(1, 4, 1, 64, dtype=torch.bfloat16), table, table, None)


def test_ring_schedule_matches_oracle_schedule():
    """Host logic: the product's step schedule equals the oracle's independent restatement."""
    from oracle import ring_oracle as R
    from pithtrain_amd.operators.ring_attention.local import ring_schedule

    for layout in ("contiguous", "zigzag"):
        for C in (1, 2, 3, 4, 8):
            for r in range(C):
                ours = [(s.kv_rank, s.causal, s.q_rows, s.kv_rows) for s in ring_schedule(r, C, 64, layout)]
                assert ours == R._steps(r, C, 64, layout)


_ASM_CACHE = {}


def _kernel_asm(src, tmp_dir):
    """gfx950 assembly of one kernel source (compiled once per test session)."""
    from pithtrain_amd import build as B

    if src not in _ASM_CACHE:
        out = os.path.join(str(tmp_dir), src + ".s")
        cmd = [B._hipcc(), *B.HIPCC_FLAGS, "-I", B.INCLUDE_DIR, "-I", B.SRC_DIR, "--cuda-device-only", "-S",
               os.path.join(B.SRC_DIR, src), "-o", out]  # fmt: skip
        subprocess.run(cmd, check=True, capture_output=True)
        with open(out) as f:
            _ASM_CACHE[src] = f.read()
    return _ASM_CACHE[src]


def test_m0_is_touched_only_by_the_direct_load_statements(tmp_path_factory):
    """csrc/attn_tiles.h sets M0 inside inline assembly (the LDS destination of global_load_lds), which
    the compiler cannot be told about. Compile every kernel source to gfx950 assembly and check that
    no instruction OUTSIDE the inline-assembly regions (;;#ASMSTART ... ;;#ASMEND) mentions M0, i.e. that the
    compiler keeps no M0 state of its own that those statements could corrupt."""
    from concurrent.futures import ThreadPoolExecutor

    from pithtrain_amd import build as B

    tmp = tmp_path_factory.getbasetemp()

    def offending(src):
        bad, in_asm = [], False
        for line in _kernel_asm(src, tmp).splitlines():
            code = line.split(";")[0]
            if "#ASMSTART" in line:
                in_asm = True
            elif "#ASMEND" in line:
                in_asm = False
            elif not in_asm and re.search(r"\bm0\b", code):
                bad.append(f"{src}: {line.strip()}")
        return bad

    users = [s for s in B.SOURCES if "attn_tiles.h" in open(os.path.join(B.SRC_DIR, s)).read()
             or "attn_bwd_common.h" in open(os.path.join(B.SRC_DIR, s)).read()
             or "attn_fwd_common.h" in open(os.path.join(B.SRC_DIR, s)).read()]  # fmt: skip
    assert users
    with ThreadPoolExecutor(max_workers=8) as pool:
        bad = [b for res in pool.map(offending, users) for b in res]
    assert not bad, "compiler-generated M0 use next to inline M0 writes:\n" + "\n".join(bad[:10])


def test_ds_storing_dkdv_kernel_waits_for_its_tile_loads_only(tmp_path_factory):
    """The dK/dV kernel that also stores its dS tiles ends an interval with `s_waitcnt vmcnt(4)`: the tile
    requests of the interval must have landed, its four dS stores may stay in flight. Vector memory operations
    retire in issue order, so this is only right if, in the steady-state loop of the storing waves, every load is
    issued before the first store, exactly four stores follow, and no register spill traffic (which counts in
    vmcnt as well) sits in the loop. Checked on the compiler's output."""
    from pithtrain_amd import build as B  # noqa: F401

    text = _kernel_asm("attn_bwd_dkdv_d128.hip", tmp_path_factory.getbasetemp())
    lines = text.splitlines()
    waits = [i for i, l in enumerate(lines) if re.search(r"s_waitcnt vmcnt\(4\)\s*$", l) and "s_barrier" in lines[i + 1]]
    assert len(waits) == 6, (
        f"expected one steady-state wait per storing kernel variant (no mask, mask with ascending and with descending "
        f"query walk; 2 output types each), got {len(waits)}"
    )
    for w in waits:
        head = max(i for i in range(w) if "Inner Loop Header" in lines[i])
        label = re.match(r"\.(LBB\d+_\d+):", lines[head]).group(1)
        body = lines[head:w]
        ops = [l.split()[0] for l in body if re.match(r"\s+(global_|scratch_|buffer_|flat_)", l)]
        assert not [o for o in ops if o.startswith(("scratch_", "buffer_", "flat_"))], f"spill or foreign memory traffic in the loop: {ops}"
        stores = [i for i, o in enumerate(ops) if o.startswith("global_store")]
        assert len(stores) == 4, f"the loop must issue exactly the four dS stores, found {len(stores)}"
        assert stores == list(range(len(ops) - 4, len(ops))), f"a load is issued after a store: {ops}"
        assert any(o.startswith("global_load_lds") for o in ops[: stores[0]]), "the tile requests must precede the stores"
        # blocks of the same loop that the compiler placed out of line (ragged-tile requests) hold loads only
        end = next(i for i in range(w, len(lines)) if "s_endpgm" in lines[i])
        in_loop_blocks = []
        cur = None
        for l in lines[w:end]:
            m = re.match(r"\.(LBB\d+_\d+):(.*)", l)
            if m:
                cur = f"Header=B{label[2:]}" in m.group(2)
            elif cur and re.match(r"\s+(global_store|scratch_)", l):
                in_loop_blocks.append(l.strip())
        assert not in_loop_blocks, f"stores or spills in out-of-line blocks of the loop: {in_loop_blocks}"
