"""CPU: the oracle against the reference's own ChromeTraceLogger / JsonTypedMetadataVisitor / fmt,
compiled from the reference sources by oracle/Makefile into oracle/_ref.  Skipped where that
library has not been built (it cannot be built without /root/reference)."""
import ctypes as C
import math
import random
import struct

import pytest

import kat_cases
import oracle_glue as og
from kineto_amd import abi

pytestmark = pytest.mark.skipif(not og.have_ref(), reason="oracle/_ref/libktj_ref.so not built")


@pytest.mark.parametrize("cfg,n", [(1, 10000), (2, 20000), (3, 30000), (4, 30000), (5, 4000), (1, 1), (2, 7)])
def test_synthetic_configs_byte_identical(cfg, n):
    sp, release = abi.synth_stream(cfg, n, **og.ref_stream_args())
    o = og.OracleRun(sp)
    mine = o.output()
    theirs = og.ref_render(sp, o)
    o.close()
    release()
    assert mine == theirs


@pytest.mark.parametrize("case", kat_cases.SUBSTRING_CASES + [kat_cases.case_rocm_sync_trace], ids=lambda c: c.__name__)
def test_hand_made_cases_byte_identical(case):
    sp = kat_cases.build_for_real_logger(case, og.ref_stream_args())
    o = og.OracleRun(sp)
    mine = o.output()
    theirs = og.ref_render(sp, o)
    o.close()
    assert mine == theirs


@pytest.mark.parametrize("seed", range(24))
def test_random_streams_byte_identical(seed):
    """Every record class, activity type and edge value the engine accepts, mixed at random: the
    oracle's document against the real logger's."""
    import random_streams
    sp = kat_cases.build_for_real_logger(lambda: (random_streams.random_stream(seed, wide_ids=seed % 2 == 1), None),
                                         og.ref_stream_args())
    o = og.OracleRun(sp)
    mine = o.output()
    theirs = og.ref_render(sp, o)
    o.close()
    if mine != theirs:
        i = next((k for k in range(min(len(mine), len(theirs))) if mine[k] != theirs[k]), min(len(mine), len(theirs)))
        raise AssertionError(f"byte {i}: oracle {mine[max(0, i - 80):i + 60]!r} reference {theirs[max(0, i - 80):i + 60]!r}")


def test_double_formatting_matches_fmt():
    ref, ora = og.load_ref(), og.load_oracle()
    b1, b2 = C.create_string_buffer(64), C.create_string_buffer(64)
    rng = random.Random(11)
    vals = [0.0, -0.0, 1.5, 2.5, 3.125e-05, 0.4375, 1e15, 1e16, 1e-4, 1e-5, 5e-324, 1.7976931348623157e308,
            2.2250738585072014e-308, float("inf"), float("-inf"), float("nan"), 9007199254740993.0, 0.1, 1 / 3, 1e22, 1e23]
    vals += [2.0 ** e for e in range(-1074, 1024, 3)]
    for _ in range(150000):
        r = rng.random()
        if r < 0.4:
            v = struct.unpack("<d", struct.pack("<Q", rng.getrandbits(64)))[0]
        elif r < 0.6:
            v = rng.randrange(1, 1 << 40) / rng.randrange(1, 1 << 30)
        elif r < 0.8:
            v = rng.randrange(0, 1000001) / 1e6
        else:
            v = rng.randrange(1, 1 << 53) * 2.0 ** rng.randrange(-80, 40)
        if not math.isnan(v):
            vals.append(v)
    for v in vals:
        n1 = ora.ktj_oracle_fmt_double(v, b1)
        n2 = ref.ktj_ref_fmt_double(v, b2)
        assert b1.raw[:n1] == b2.raw[:n2], (v, b1.raw[:n1], b2.raw[:n2])


def test_schema_key_orders_are_the_reference_maps_order():
    """The synthetic schemas list their keys in the order the reference's unordered_map iterates
    them after the documented insertion order."""
    ref = og.load_ref()
    out = C.create_string_buffer(4096)

    def order(keys):
        arr = (C.c_char_p * len(keys))(*[k.encode() for k in keys])
        n = ref.ktj_ref_metadata_order(arr, len(keys), out, 4096)
        import re
        return re.findall(r'"([^"]+)": \d+', out.raw[:n].decode())

    assert order(["Sequence number", "Fwd thread id", "Record function id", "Ev Idx"]) == \
        ["Ev Idx", "Record function id", "Fwd thread id", "Sequence number"]
    assert order(["grid", "block", "registers per thread", "shared memory", "occupancy"]) == \
        ["occupancy", "registers per thread", "block", "shared memory", "grid"]
    # and the generator really emits them in that order
    sp, release = abi.synth_stream(5, 3)
    s = sp.contents
    sch = s.schemas[s.n_schemas - 1]
    blob = C.string_at(s.str_blob, s.str_off[s.n_strings])
    keys = []
    for f in range(sch.n_fields):
        k = s.fields[sch.first_field + f].key_id
        keys.append(blob[s.str_off[k]:s.str_off[k + 1]].decode())
    release()
    assert keys == ["occupancy", "registers per thread", "block", "shared memory", "grid"]


def test_generic_add_metadata_raw_json_path():
    """test/GenericTraceActivityMetadataTest.cpp:88-111, 144-178: addMetadata stores fmt text as RawJson."""
    ref = og.load_ref()
    out = C.create_string_buffer(4096)
    keys = (C.c_char_p * 1)(b"ratio")
    kinds = (C.c_int * 1)(1)
    iv = (C.c_int64 * 1)(0)
    dv = (C.c_double * 1)(1.5)
    sv = (C.c_char_p * 1)(None)
    n = ref.ktj_ref_generic_metadata(1, keys, kinds, iv, dv, sv, out, 4096)
    assert out.raw[:n] == b'"ratio": 1.5'
    kinds[0] = 4
    iv[0] = -1
    keys[0] = b"big"
    n = ref.ktj_ref_generic_metadata(1, keys, kinds, iv, dv, sv, out, 4096)
    assert out.raw[:n] == b'"big": 18446744073709551615'
