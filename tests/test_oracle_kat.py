"""CPU: the oracle against known-answer strings (observed from the real logger / asserted by the
reference's own tests)."""
import pytest

import kat_cases
import oracle_glue as og


@pytest.mark.parametrize("case", kat_cases.SUBSTRING_CASES, ids=lambda c: c.__name__)
def test_known_answers(case):
    b, expect = case()
    o = og.OracleRun(b.build())
    out = o.output().decode("latin1")
    o.close()
    for e in expect:
        assert e in out, f"missing {e!r} in\n{out}"


@pytest.mark.parametrize("quoted", [False, True])
def test_collective_metadata_expectations_of_the_reference_test(quoted):
    """libkineto/test/OutputJsonTest.cpp:186-225: the document parses as JSON and the kernel's args
    and "distributedInfo" equal the expected objects, for quoted and bare string values alike."""
    import json
    b, _ = kat_cases.case_collective_reference_test(quoted)
    o = og.OracleRun(b.build())
    trace = json.loads(o.output().decode())
    o.close()
    args = [e["args"] for e in trace["traceEvents"] if e.get("name") == "nccl:all_reduce"]
    assert args == [kat_cases.COLLECTIVE_REF_ARGS]
    assert trace["distributedInfo"] == kat_cases.COLLECTIVE_REF_DIST


def test_rocm_sync_trace_counts():
    b, counts = kat_cases.case_rocm_sync_trace()
    o = og.OracleRun(b.build())
    out = o.output().decode("latin1")
    acts, n = o.activities()
    assert n == 15
    o.close()
    for k, v in counts.items():
        assert out.count(k) == v, (k, out.count(k), v)


def test_header_and_footer_bytes():
    """Header/footer whitespace observed from the real logger."""
    from stream_builder import StreamBuilder
    b = StreamBuilder(host_name="vm", trace_name="/tmp/x.json")
    o = og.OracleRun(b.build())
    out = o.output().decode()
    o.close()
    assert out.startswith(' {\n    "schemaVersion": 1,\n    "deviceProperties": [],\n    \n      "host_name": "vm",\n'
                          '    "displayTimeUnit": "ms",\n    "baseTimeNanoseconds": 1790857026000000000,\n    "traceEvents": [\n    ')
    assert out.endswith('\n  ],"traceName": "/tmp/x.json" }')


def test_leaf_functions():
    import ctypes as C
    lib = og.load_oracle()
    buf = C.create_string_buffer(64)
    for ns, want in ((0, b"0.000"), (1234, b"1.234"), (999, b"0.999"), (1000, b"1.000"), (123456789012, b"123456789.012")):
        n = lib.ktj_oracle_fmt_ts(ns, buf)
        assert buf.raw[:n] == want
    for v, want in ((1.5, b"1.5"), (2.5, b"2.5"), (3.125e-05, b"3.125e-05"), (0.4375, b"0.4375"), (0.0001, b"0.0001"),
                    (1e15, b"1000000000000000"), (1e16, b"1e+16"), (0.00001, b"1e-05"), (64.0, b"64"), (-0.0, b"-0"),
                    (5e-324, b"5e-324"), (1.7976931348623157e308, b"1.7976931348623157e+308"), (1 / 3, b"0.3333333333333333"),
                    (2.0 ** -24, b"5.960464477539063e-08")):
        n = lib.ktj_oracle_fmt_double(v, buf)
        assert buf.raw[:n] == want, (v, buf.raw[:n], want)
    for t, want in enumerate(["cpu_op", "user_annotation", "gpu_user_annotation", "gpu_memcpy", "gpu_memset", "kernel",
                              "external_correlation", "cuda_runtime"]):
        assert lib.ktj_oracle_type_name(t).decode() == want


def test_name_pipeline_exhaustive_two_bytes():
    """All 1- and 2-byte names: brute force against a direct Python statement of the three steps
    (output_json.cpp:72-78, 103-112, 86-91)."""
    import ctypes as C
    lib = og.load_oracle()
    out = C.create_string_buffer(32)

    def py(name):
        s = name.replace(b"\\", b"/").replace(b"\n", b"")
        if any(c < 0x20 or c > 0x7e for c in s):
            return b"unknown"
        return s.replace(b'"', b'\\"')

    for a in range(256):
        for bb in [None] + list(range(0, 256, 1)):
            name = bytes([a]) if bb is None else bytes([a, bb])
            n = lib.ktj_oracle_sanitize_name(name, len(name), out)
            assert out.raw[:n] == py(name), name
    n = lib.ktj_oracle_sanitize_name(b"kernel", 6, out)
    assert out.raw[:n] == b"Kernel"


def test_clock_conversion_exact():
    """(int64)((double)(t - t0a) * (long double)scale) + t0 against exact integer arithmetic:
    product of two 53-bit significands rounded to 64 bits (nearest even), then truncated."""
    import ctypes as C
    import random
    from fractions import Fraction
    from kineto_amd import abi
    lib = og.load_oracle()
    rng = random.Random(7)

    def exact(t, t0a, t0, scale):
        if t <= t0a:
            return 0
        dt = float(t - t0a)                      # int -> double, round to nearest even (Python does the same)
        p = Fraction(dt) * Fraction(scale)       # exact product
        if p == 0:
            return t0
        # round to 64 significant bits, ties to even
        e = p.numerator.bit_length() - p.denominator.bit_length()
        if Fraction(2) ** e > p:
            e -= 1
        q = p / Fraction(2) ** (e - 63)          # in [2^63, 2^64)
        fl = q.numerator // q.denominator
        rem = q - fl
        if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
            fl += 1
        val = Fraction(fl) * Fraction(2) ** (e - 63)
        return int(val) + t0                     # truncation toward zero (val > 0)

    for _ in range(3000):
        t0a = rng.randrange(0, 1 << 40)
        t = t0a + rng.choice([rng.randrange(-3, 4), rng.randrange(1, 1 << 20), rng.randrange(1, 1 << 45), rng.randrange(1, 1 << 60)])
        t = max(t, 0)
        scale = rng.choice([1.0, 1.000001, 0.999999, rng.uniform(0.25, 4.0), 2.0 ** -10])
        t0 = rng.randrange(-(1 << 40), 1 << 60)
        m = abi.ClockModel(t0a, t0, scale, 0, 1, 1)
        assert lib.ktj_oracle_convert_ts(C.byref(m), t) == exact(t, t0a, t0, scale), (t, t0a, t0, scale)
