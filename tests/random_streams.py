"""Seeded random ktj_stream objects that mix every record class, type and edge value the engine
accepts: used for differential tests (host build of the formatting core, and the GPU engine,
against the oracle)."""
import random
import struct

from kineto_amd import abi
from stream_builder import B, StreamBuilder

TYPES = list(range(29))  # every ActivityType
I64_MIN, I64_MAX = -(1 << 63), (1 << 63) - 1


def _name(rng):
    r = rng.random()
    if r < 0.08:
        return rng.choice(["kernel", "Stream Sync", "", "unknown", "Kernel", " ", "\n"])
    alphabet = "abcXYZ019_:<>(), *&[]"
    if r < 0.35:
        alphabet += '"\\\n\t'
    if r < 0.15:
        alphabet += "\x01\x7f\xe9"
    n = rng.choice([1, 3, 7, 8, 9, 15, 16, 17, 31, 40, 63, 64, 65, 120, 300, 700])
    return "".join(rng.choice(alphabet) for _ in range(n))


def _i64(rng):
    return rng.choice([0, 1, -1, 7, 999, 1000, 1001, 99999999, 100000000, 10**16 - 1, 10**16, I64_MAX, I64_MIN,
                       rng.randrange(-10**6, 10**6), rng.randrange(I64_MIN, I64_MAX)])


def _f64(rng):
    v = rng.choice([0.0, -0.0, 1.5, 2.5, 0.1, 1e-5, 1e-4, 123456.789, 1e15, 1e16, 1e22, 5e-324, 1.7976931348623157e308,
                    float("inf"), float("-inf"), float("nan"), rng.random(), rng.uniform(-1e9, 1e9),
                    struct.unpack("<d", struct.pack("<Q", rng.getrandbits(64)))[0]])
    return v


def random_stream(seed, n_generic=40, n_runtime=40, n_device=60, wide_ids=False, unique_runtime_ids=False):
    rng = random.Random(seed)
    lo, hi = B + 1000, B + 10**7
    window = (lo, hi) if rng.random() < 0.7 else (B + 3 * 10**6, B + 6 * 10**6)
    b = StreamBuilder(window=window, host_name="rnd", end_time=hi + 5)
    rng_memset = random.Random(seed * 7919 + 13)   # memset rows: the view's extra fields, and the CUDA >= 12 key set or not
    b.create_flags = abi.KTJ_CREATE_CUDA12_ARGS if rng_memset.random() < 0.5 else 0
    if rng.random() < 0.5:
        b.clock = abi.ClockModel(rng.randrange(0, 1000), rng.randrange(-500, 500), rng.choice([1.0, 1.000001, 0.999]), rng.randrange(-50, 50),
                                 rng.choice([0, 1]), rng.choice([0, 1, 2]))
    apis = ["hipLaunchKernel", "hipMemcpyAsync", "hipMalloc", "hipGraphLaunch", None, "hipFree", 'odd "api"\\name']
    b.api(apis, flow_start=rng.sample(range(len(apis)), 4), malloc_cid=rng.choice([2, abi.KTJ_NONE]))
    names = [_name(rng) for _ in range(12)] + ["hccl::all_reduce", "record_param_comms"]

    def t():
        return rng.choice([rng.randrange(lo - 500, hi + 500), rng.randrange(lo, hi), 0, lo, hi])

    # schemas
    def random_fields(n_max):
        """Fields of every kind; now and then a run of them sits inside a dict, and all of them in another."""
        fields = []
        for _k in range(rng.randrange(0, n_max)):
            typ = rng.choice([0, 1, 2, 3, 4, 5, 6, abi.F_STR_ARRAY, abi.F_SHAPES, abi.F_UNSUPPORTED])
            cnt = rng.randrange(1, 5) if typ == abi.F_I64_ARRAY else rng.randrange(0, 4) if typ == abi.F_STR_ARRAY else 0 if typ == abi.F_UNSUPPORTED else 1
            fields.append((_name(rng)[:12] or "k", typ, cnt))
        if rng.random() < 0.5:
            i = rng.randrange(0, len(fields) + 1)
            j = rng.randrange(i, len(fields) + 1)
            fields[j:j] = [(None, abi.F_DICT_END, 0)]
            fields[i:i] = [(_name(rng)[:8] or "d", abi.F_DICT_BEGIN, 0)]
        if rng.random() < 0.3:
            fields = [("all", abi.F_DICT_BEGIN, 0)] + fields + [(None, abi.F_DICT_END, 0)]
        return fields

    def random_shapes():
        def shape():
            return [_i64(rng) for _ in range(rng.randrange(0, 4))]
        return [([shape() for _ in range(rng.randrange(1, 4))] if rng.random() < 0.3 else shape()) for _ in range(rng.randrange(0, 4))]

    schemas = [None, b.schema([(None, abi.F_RAW, 1)])]
    for _ in range(4):
        fields = random_fields(6)
        schemas.append((b.schema(fields), fields))
    # collective metadata: entries with random subsets of the keys, schemas that start with a reference to one
    n_coll = rng.choice([0, 0, 1, 5])
    for _ in range(n_coll):
        vals = {}
        for key in abi.COLLECTIVE_KEYS:
            if rng.random() < 0.6:
                v = rng.choice(["0", "8", "default_pg", '"default_pg"', "[0, 1]", '"x"', '"', '""', "a\\b", "tp", "allreduce", "Float"])
                if key == "pg_desc" and rng.random() < 0.5:
                    v = rng.choice(["default_pg", '"default_pg"'])
                if key == "pg_name":
                    v = rng.choice(["0", "1", "2", '"3"', "4", "5", "group six", ""])
                vals[key] = v
        b.add_collective(**vals)
    if n_coll:
        for _ in range(3):
            fields = [(None, abi.F_COLLECTIVE, 1)] + random_fields(3)
            schemas.append((b.schema(fields), fields))
        schemas.append((b.schema([(None, abi.F_COLLECTIVE, 1), (None, abi.F_RAW, 1)]), [(None, abi.F_COLLECTIVE, 1), (None, abi.F_RAW, 1)]))
    pids, tids = [0, 1, 7, -3, 4242], [0, 5, -5, 4243, I64_MIN, I64_MAX, 10**12]
    if wide_ids:  # deviceId values that do not fit the record's 32-bit field
        pids += [2**40, -(2**33) - 5]
    ids = list(range(1, 30))
    if wide_ids:
        ids += [(1 << 32) + 3, (1 << 31) + 1, 0xFFFFFFFFFFFFFFFF, 0xFFFFFFFF00000001, 1 << 40]
    for _ in range(n_generic):
        sch = rng.choice(schemas)
        values, sid = (), None
        if isinstance(sch, int):
            sid = sch
            values = [b.s(rng.choice(['"k": 1', "   ", "", "\n", '"a": "b\\c"', _name(rng)]))]
        elif sch is not None:
            sid, fields = sch
            values = []
            for _key, typ, cnt in fields:
                if typ == abi.F_COLLECTIVE:
                    values.append(rng.choice(list(range(n_coll)) + [n_coll, 2**40]))
                elif typ == abi.F_F64:
                    values.append(_f64(rng))
                elif typ in (abi.F_STR, abi.F_RAW):
                    values.append(b.s(_name(rng)))
                elif typ == abi.F_STR_ARRAY:
                    values += [b.s(_name(rng)) for _ in range(cnt)]
                elif typ == abi.F_SHAPES:
                    values.append(rng.choice([b.shapes(random_shapes()), 2**50]))   # now and then a slot that points nowhere
                elif typ in (abi.F_DICT_BEGIN, abi.F_DICT_END, abi.F_UNSUPPORTED):
                    pass
                elif typ == abi.F_BOOL:
                    values.append(rng.randrange(3))
                elif typ == abi.F_I64_ARRAY:
                    values += [_i64(rng) for _ in range(cnt)]
                else:
                    values.append(_i64(rng))
        s0 = t()
        b.add_generic(rng.choice(names + [None]), rng.choice(TYPES + [0, 0, 0, 9, 15, 17, 28, 28, 5, 5, 13, 13]), s0, s0 + rng.choice([0, 1, 999, 1000, -3, 10**5]),
                      rng.choice(pids), rng.choice(tids), id=rng.choice([0, -2, 5, 6, 7, 8, 2**31 - 1, -(2**31)] + ids[:8]),
                      schema=sid, values=values, flow_id=rng.choice([0, 0, 1, 77, 2**32 - 1, 2**40 + 3, -4]), flow_type=rng.choice([0, 1, 2, 3]),
                      flow_start=rng.random() < 0.5, linked=rng.choice([None, None, 5, -9, 2**40 + 1]))
    # with unique_runtime_ids no two runtime rows share a correlation id (the engine then keeps what
    # each row wrote for the device rows in its single pass); device rows still repeat ids
    unique_pool = rng.sample(range(1, max(4 * n_runtime, 64)), n_runtime) if unique_runtime_ids else None
    for k_rt in range(n_runtime):
        kind = rng.randrange(4)
        s0 = t()
        kw = {}
        if kind == 1:
            kw = dict(grid=[rng.choice([0, 1, 7, 2**32 - 1]) for _ in range(3)], workgroup=[rng.choice([1, 64, 1024]) for _ in range(3)],
                      lds=rng.choice([0, 65536, 2**40]), stream=rng.choice([0, 0x7000, 0x8000, 0x9000]),
                      kernel_name=rng.choice([None, None, _name(rng)]))
        elif kind == 2:
            kw = dict(src=rng.getrandbits(48), dst=rng.choice([0, rng.getrandbits(64)]), size=rng.choice([0, 4096, 2**35]),
                      stream=rng.choice([0, 0x7000, 0xA000]), copy_kind=rng.choice([0, 1, 2, 3, 4, 0xFFFFFFFF]))
        elif kind == 3:
            kw = dict(ptr=rng.getrandbits(47), size=rng.choice([0, 777, 2**33]))
        b.add_runtime(unique_pool[k_rt] if unique_pool else rng.choice(ids), s0, s0 + rng.choice([0, 5, 5000, -7]), rng.choice([0, 1, 2, 3, 4, 5, 6, 9, 10**6]),
                      rng.choice([10, 11]), rng.choice([20, 21, 22]), kind=kind, **kw)
    for _ in range(n_device):
        dom = rng.choice([0, 0, 0, 1, 1, 2, 7])
        s0 = t()
        b.add_device(rng.choice((unique_pool[:40] if unique_pool else []) + ids + [100, 101, 0]), s0, s0 + rng.choice([0, 1, 2, 900, 10**5]), domain=dom,
                     op=rng.choice([0, 1, 2, 3, 4, 9]), device=rng.choice([0, 0, 1, -1]), name=rng.choice(names + [None]),
                     queue=rng.choice([0, 1, 2, 3, 2**63 + 5]), stream=rng.choice([0, 0, 0, 5, 0x7000]), nbytes=rng.choice([0, 1000, 2**40]),
                     memory_kind=rng_memset.randrange(0, 10), channel_type=rng_memset.randrange(0, 4))
    for _ in range(rng.randrange(0, 40)):
        b.add_extcorr(rng.choice((unique_pool[:30] if unique_pool else []) + ids + [0xFFFFFFFFFFFFFFFF]), rng.choice([5, 6, 7, 8, 0, 2**31 - 1, 0xFFFFFFFF80000000, 2**40, 12345]))
    if rng.random() < 0.5:  # user-domain correlation: GPU user-annotation spans
        for _ in range(rng.randrange(1, 40)):
            b.add_usercorr(rng.choice((unique_pool[:20] if unique_pool else []) + ids + [100, 0]), rng.choice([5, 6, 7, 8, 0, 2**31 - 1, 0xFFFFFFFF80000000, 2**40, 12345]))
    if rng.random() < 0.5:
        b.add_device_info(0, 5000000, 'GPU "zero"', "GPU 0", B + 10)
        b.add_resource_info(5, 5, 0, 'stream "5"', False, B + 10)
        b.add_resource_info(4243, 4243, 4242, "worker", True, B + 11)
        b.add_overhead_info("CUPTI overhead", B + 12)
        b.add_span(lo, hi, 3, 1, "PyTorch Profiler", "pfx")
    return b
