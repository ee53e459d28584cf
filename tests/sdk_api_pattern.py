"""Test-only: HIP runtime API callback records with a fixed argument pattern, the reference's rows
for them (through oracle/_ref/sdk_ref_driver) and the engine's rows in the same text form."""
import ctypes as C
import os
import struct
import subprocess

from kineto_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SDK_REF_DRIVER = os.path.join(ROOT, "oracle", "_ref", "sdk_ref_driver")
ARENA = 0x700000000000   # the driver maps zero pages here: pointer arguments may be followed by the SDK

_sim = None


def sim():
    global _sim
    if _sim is None:
        lib = C.CDLL(os.path.join(ROOT, "tests", "host_sim", "libktjsim.so"))
        lib.ktjsim_sdk_api_args_size.restype = C.c_uint64
        lib.ktjsim_sdk_api_last_op.restype = C.c_uint32
        lib.ktjsim_sdk_api_kind_hip_runtime.restype = C.c_uint32
        lib.ktjsim_sdk_api_row.restype = C.c_uint32
        lib.ktjsim_sdk_api_row.argtypes = [C.c_uint32, C.c_uint64, C.c_char_p, C.c_uint64, C.c_uint64, C.c_uint32, C.c_uint32,
                                           C.POINTER(abi.RuntimeRec)]
        lib.ktjsim_sdk_api_record_create.restype = C.c_void_p
        lib.ktjsim_sdk_api_record_create.argtypes = [C.c_uint32, C.c_uint32, C.c_uint64, C.c_char_p]
        lib.ktjsim_sdk_api_record_free.argtypes = [C.c_void_p]
        _sim = lib
    return _sim


def n_ops():
    return sim().ktjsim_sdk_api_last_op()


def args_bytes(op):
    """Every 8-byte word of the argument union is a different address inside the arena: a pointer
    argument can be followed, and integer arguments take the halves of those words as values."""
    n = sim().ktjsim_sdk_api_args_size()
    return b"".join(struct.pack("<Q", ARENA + 0x1000 * op + 8 * k) for k in range(n // 8)) + b"\0" * (n % 8)


def correlation(op):
    return (1 << 33) + 7 * op


def reference_lines():
    ops = range(n_ops())
    req = struct.pack("<IQ", 2, len(ops)) + b"".join(struct.pack("<IIQ", op, 0, correlation(op)) + args_bytes(op) for op in ops)
    out = subprocess.run([SDK_REF_DRIVER], input=req, stdout=subprocess.PIPE, check=True, timeout=300).stdout.decode("latin1")
    lines = [line for line in out.split("\n") if line]
    assert lines[0].startswith("kind hip_runtime_api=") and len(lines) == 1 + 2 * len(ops)
    # the SDK's rendering of the arguments is kept for the rows that read arguments
    return [lines[0]] + [line for k, line in enumerate(lines[1:]) if k % 2 == 0 or not lines[k].startswith("default")]


def engine_line(op, domain):
    """The engine's row for the same call (kineto_amd/csrc/sdk_api_rows.h), in the driver's text form.
    Also returns the record, for the argument values that the reference only keeps as text."""
    r = abi.RuntimeRec()
    kind = sim().ktjsim_sdk_api_row(op, correlation(op), args_bytes(op), 111, 222, 3, 4, C.byref(r))
    assert (r.id, r.begin, r.end, r.cid, r.pid, r.tid, r.kind) == (correlation(op), 111, 222, op, 3, 4, kind)
    head = f"id={r.id} domain={domain} cid={r.cid}"
    if kind == 1:
        k = r.u.kernel
        assert k.kernel_name_id == abi.KTJ_NONE
        line = (f"kernel {head} grid={k.grid[0]},{k.grid[1]},{k.grid[2]} workgroup={k.workgroup[0]},{k.workgroup[1]},{k.workgroup[2]} "
                f"gss={k.group_segment_size} stream={k.stream} faddr=0 function=0")
    elif kind == 2:
        c = r.u.copy
        line = f"copy {head} size={c.size} kind={C.c_int32(c.copy_kind).value} stream={c.stream}"
    elif kind == 3:
        line = f"malloc {head} size={r.u.malloc_.size}"
    else:
        line = f"default {head}"
    return line, r
