"""Known-answer cases for the logger path.  Every expected string below was either observed from
the real ChromeTraceLogger (built from the reference sources) or is a literal the reference's own
tests assert; the source is named per case.  Used on the CPU against the oracle and on the GPU
against the engine."""
from kineto_amd import abi
from stream_builder import B, StreamBuilder

T = abi  # type constants live in abi as plain ints below
CPU_OP, GPU_MEMCPY, KERNEL, RUNTIME = 0, 3, 5, 7


def case_logger_events():
    """Observed from the real logger: CPU op, linked runtime row with flow start, kernel with a name
    that needs sanitising, orphan kernel with unprintable name, 'kernel' rename, blank metadata."""
    b = StreamBuilder()
    b.api([None] * 12 + ["hipLaunchKernel"], flow_start=[12])
    b.add_generic("aten::mm", CPU_OP, B + 1234, B + 5678, 4242, 4243, id=7)
    b.add_runtime(7, B + 2000, B + 3000, 12, 4242, 4243, kind=0)
    b.add_extcorr(7, 7)
    b.add_generic('void f<"q", a\\b>(int)\n', KERNEL, B + 4000, B + 4500, 0, 3, id=7, flow_id=7, flow_type=2)
    b.add_generic("bad\x01name", KERNEL, B + 6000, B + 5997, 0, -5, id=99, flow_id=99, flow_type=2)
    sch = b.schema([(None, abi.F_RAW, 1)])
    b.add_generic("kernel", GPU_MEMCPY, B + 7000, B + 7100, 0, 3, id=0, schema=sch, values=[b.s("   ")])
    expect = [
        '"cat": "cpu_op",\n    "name": "aten::mm",\n    "pid": 4242,\n    "tid": 4243,\n    "ts": 1.234,\n    "dur": 4.444\n    ,\n    "args": {\n      "External id": 7\n    }',
        '"External id": 7,"cid": 12, "correlation": 7',
        '"ph": "s",\n    "id": 7,\n    "pid": 4242,\n    "tid": 4243,\n    "ts": 2.000,\n    "cat": "ac2g",\n    "name": "ac2g"\n    \n  },',
        '"name": "void f<\\"q\\", a/b>(int)"',
        '"name": "ac2g"\n    , "bp": "e"\n  },',
        '"name": "unknown",\n    "pid": 0,\n    "tid": 5,\n    "ts": 6.000,\n    "dur": 0.000\n    \n  },\n  {\n    "ph": "f",\n    "id": 99,',
        '"cat": "gpu_memcpy",\n    "name": "Kernel",\n    "pid": 0,\n    "tid": 3,\n    "ts": 7.000,\n    "dur": 0.100\n    \n  },',
    ]
    return b, expect


def case_trace_span():
    """Observed from the real logger (TraceSpan 'PyTorch Profiler', +1000..+900000, opCount 1, iter 0)."""
    b = StreamBuilder(end_time=B + 900000)
    b.add_span(B + 1000, B + 900000, 1, 0, "PyTorch Profiler")
    expect = [
        '"ph": "X",\n    "cat": "Trace",\n    "name": "PyTorch Profiler (0)",\n    "pid": "Spans",\n    "tid": "PyTorch Profiler",\n    "ts": 1.000,\n    "dur": 899.000\n    ,\n    "args": {\n      "Op count": 1\n    }\n  },',
        '"ph": "M",\n    "name": "process_sort_index",\n    "ts": 1.000,\n    "pid": "Spans",\n    "tid": 0,\n    "args": {\n      "sort_index": 536870912\n    }',
        '"s": "g",\n    "name": "Iteration Start: PyTorch Profiler",\n    "pid": "Traces",\n    "tid": "Trace PyTorch Profiler",\n    "ts": 1.000',
        '"name": "Record Window End",\n    "pid": "",\n    "tid": "",\n    "ts": 900.000\n    \n  }\n  ],"traceName": "t.json" }',
    ]
    return b, expect


def case_benchmark_cpu_op():
    """benchmarks/json_output_benchmark.cpp:181-197 through the real logger: duplicate keys are
    emitted as they are, the logger's own External id first."""
    b = StreamBuilder()
    sch = b.schema([("Sequence number", abi.F_I64, 1), ("Input Dims", abi.F_STR, 1), ("External id", abi.F_RAW, 1)])
    b.add_generic("aten::conv2d", CPU_OP, B + 10, B + 20, 12345, 67890, id=2, schema=sch,
                  values=[1, b.s("[[32, 64, 28, 28], [64, 64, 3, 3]]"), b.s("3")])
    return b, ['"External id": 2,"Sequence number": 1, "Input Dims": "[[32, 64, 28, 28], [64, 64, 3, 3]]", "External id": 3']


def case_typed_kernel_args():
    """Observed from the real logger; key order is the reference's unordered_map order for keys
    inserted as grid, block, registers per thread, shared memory, occupancy."""
    b = StreamBuilder()
    sch = b.schema([("occupancy", abi.F_F64, 1), ("registers per thread", abi.F_U64, 1), ("block", abi.F_I64_ARRAY, 3),
                    ("shared memory", abi.F_I64, 1), ("grid", abi.F_I64_ARRAY, 3)])
    b.add_generic("k1", KERNEL, B + 10, B + 20, 0, 1, id=1, schema=sch, values=[0.00003125, 64, 256, 1, 1, 163840, 128, 1, 1],
                  flow_id=5, flow_type=2)
    b.add_generic("k2", KERNEL, B + 30, B + 40, 0, 1, id=2, schema=sch, values=[0.4375, 64, 256, 1, 1, 163840, 128, 1, 1])
    expect = [
        '"occupancy": 3.125e-05, "registers per thread": 64, "block": [256, 1, 1], "shared memory": 163840, "grid": [128, 1, 1]',
        '"occupancy": 0.4375, "registers per thread": 64',
        '"ph": "f",\n    "id": 5,',
    ]
    return b, expect


def case_typed_metadata_pins():
    """Literals asserted by libkineto/test/TypedMetadataTest.cpp:164-178, 240 and
    GenericTraceActivityMetadataTest.cpp:144-178 (strings pass through unescaped except for the
    logger's later backslash/newline pass)."""
    b = StreamBuilder()
    sch = b.schema([("count", abi.F_I64, 1), ("ids", abi.F_I64_ARRAY, 2), ("label", abi.F_STR, 1), ("ratio", abi.F_F64, 1),
                    ("enabled", abi.F_BOOL, 1), ("big", abi.F_U64, 1), ("raw", abi.F_RAW, 1), ("neg", abi.F_I64, 1),
                    ("special", abi.F_STR, 1), ("nan", abi.F_F64, 1)])
    b.add_generic("op", CPU_OP, B + 1, B + 2, 1, 2, id=0, schema=sch,
                  values=[5, 1, 2, b.s("label"), 1.5, 1, 0xFFFFFFFFFFFFFFFF, b.s("[1, 2, 3]"), -7,
                          b.s('quote " slash \\ newline\n'), float("nan")])
    expect = ['"count": 5, "ids": [1, 2], "label": "label", "ratio": 1.5, "enabled": true, "big": 18446744073709551615, '
              '"raw": [1, 2, 3], "neg": -7, "special": "quote " slash / newline", "nan": "nan"']
    return b, expect


def case_typed_metadata_collections():
    """libkineto/test/TypedMetadataTest.cpp:145-178 (string array, nested dict with a field after
    it), :186-200 (a dict inside a dict with siblings on both sides), :209 (a type the visitor does
    not know), :229-244 (uint64 and InputShapes)."""
    b = StreamBuilder()
    D, E = (abi.F_DICT_BEGIN, 0), (abi.F_DICT_END, 0)
    one = b.schema([("count", abi.F_I64, 1), ("ids", abi.F_I64_ARRAY, 2), ("label", abi.F_STR, 1), ("ratio", abi.F_F64, 1),
                    ("enabled", abi.F_BOOL, 1), ("names", abi.F_STR_ARRAY, 2), ("special", abi.F_STR, 1),
                    ("nested",) + D, ("nested_count", abi.F_I64, 1), ("nested_other", abi.F_I64, 1), (None,) + E,
                    ("after_nested", abi.F_I64, 1)])
    b.add_generic("op1", CPU_OP, B + 1, B + 2, 1, 2, id=0, schema=one,
                  values=[5, 1, 2, b.s("label"), 1.5, 1, b.s("a"), b.s("b"), b.s('quote " slash \\ newline\n'), 7, 8, 9])
    two = b.schema([("outer",) + D, ("count", abi.F_I64, 1), ("inner",) + D, ("enabled", abi.F_BOOL, 1), (None,) + E,
                    ("ratio", abi.F_F64, 1), (None,) + E, ("after_nested", abi.F_I64, 1)])
    b.add_generic("op2", CPU_OP, B + 3, B + 4, 1, 2, id=0, schema=two, values=[1, 1, 2.5, 9])
    three = b.schema([("count", abi.F_I64, 1), ("pair", abi.F_UNSUPPORTED, 0), ("address", abi.F_U64, 1),
                      ("input_dims", abi.F_SHAPES, 1), ("empty", abi.F_STR_ARRAY, 0), ("first",) + D, (None,) + E,
                      ("strides", abi.F_SHAPES, 1)])
    dims = b.shapes([[2, 2], [[4, 1], [4, 1]]])
    strides = b.shapes([[], [[]], [[7], [], [-1, 0, 9223372036854775807]], [1]])
    b.add_generic("op3", CPU_OP, B + 5, B + 6, 1, 2, id=0, schema=three, values=[5, 0xFFFFFFFFFFFFFFFF, dims, strides])
    # a dict as the first and only field, and a schema of brackets alone
    four = b.schema([("occupancy",) + D, ("active_blocks_per_multiprocessor", abi.F_I64, 1), ("limiting_factors", abi.F_STR, 1), (None,) + E])
    b.add_generic("op4", CPU_OP, B + 7, B + 8, 1, 2, id=0, schema=four, values=[4, b.s("warps, registers")])
    expect = ['"count": 5, "ids": [1, 2], "label": "label", "ratio": 1.5, "enabled": true, "names": ["a", "b"], '
              '"special": "quote " slash / newline", "nested": {"nested_count": 7, "nested_other": 8}, "after_nested": 9',
              '"outer": {"count": 1, "inner": {"enabled": true}, "ratio": 2.5}, "after_nested": 9',
              '"count": 5, "pair": "<unsupported metadata type>", "address": 18446744073709551615, '
              '"input_dims": [[2, 2], [[4, 1], [4, 1]]], "empty": [], "first": {}, '
              '"strides": [[], [[]], [[7], [], [-1, 0, 9223372036854775807]], [1]]',
              '"occupancy": {"active_blocks_per_multiprocessor": 4, "limiting_factors": "warps, registers"}']
    return b, expect


def case_cuda_shaped_kernel_args():
    """The typed metadata of a CUDA kernel activity (libkineto/src/CuptiActivity.h:499-576): fifteen
    fields, the last a dict of nine, as a schema of a generic kernel record."""
    b = StreamBuilder()
    D, E = (abi.F_DICT_BEGIN, 0), (abi.F_DICT_END, 0)
    sch = b.schema([("queued", abi.F_U64, 1), ("device", abi.F_I64, 1), ("context", abi.F_U64, 1), ("stream", abi.F_I64, 1),
                    ("correlation", abi.F_U64, 1), ("registers per thread", abi.F_U64, 1), ("shared memory", abi.F_I64, 1),
                    ("blocks per SM", abi.F_F64, 1), ("warps per SM", abi.F_F64, 1), ("grid", abi.F_I64_ARRAY, 3),
                    ("block", abi.F_I64_ARRAY, 3), ("est. achieved occupancy %", abi.F_I64, 1),
                    ("occupancy",) + D, ("active_blocks_per_multiprocessor", abi.F_I64, 1), ("limiting_factors", abi.F_STR, 1),
                    ("block_limit_regs", abi.F_I64, 1), ("block_limit_shared_mem", abi.F_I64, 1), ("block_limit_warps", abi.F_I64, 1),
                    ("block_limit_blocks", abi.F_I64, 1), ("block_limit_barriers", abi.F_I64, 1),
                    ("allocated_registers_per_block", abi.F_I64, 1), ("allocated_shared_mem_per_block", abi.F_U64, 1), (None,) + E])
    for k in range(3):
        b.add_generic("void gemm<float>(int)", KERNEL, B + 100 * k, B + 100 * k + 40, 0, 7, id=50 + k, schema=sch,
                      values=[0, 0, 1, 7, 50 + k, 64 + k, 49152, 0.5945945945945946, 4.756756756756757, 88, 1, 1, 256, 1, 1, 38,
                              3, b.s("registers"), 3, 4, 8, 32, 16, 16384 + k, 49152], flow_id=50 + k, flow_type=2)
    expect = ['"queued": 0, "device": 0, "context": 1, "stream": 7, "correlation": 50, "registers per thread": 64, '
              '"shared memory": 49152, "blocks per SM": 0.5945945945945946, "warps per SM": 4.756756756756757, '
              '"grid": [88, 1, 1], "block": [256, 1, 1], "est. achieved occupancy %": 38, '
              '"occupancy": {"active_blocks_per_multiprocessor": 3, "limiting_factors": "registers", "block_limit_regs": 3, '
              '"block_limit_shared_mem": 4, "block_limit_warps": 8, "block_limit_blocks": 32, "block_limit_barriers": 16, '
              '"allocated_registers_per_block": 16384, "allocated_shared_mem_per_block": 49152}']
    return b, expect


def case_names():
    """Observed from the real logger: UTF-8, TAB and DEL make the whole name 'unknown'; printable
    punctuation is untouched; newlines vanish; quotes are escaped after backslashes became slashes."""
    b = StreamBuilder()
    names = [b"caf\xc3\xa9", b"tab\there", b"del\x7f", b"sp ace~!", b"nl\nonly\n", b'q""x\\\\']
    for i, n in enumerate(names):
        b.add_generic(n, CPU_OP, B + 10 * i, B + 10 * i + 5, 1, 1, id=0)
    expect = ['"name": "unknown"', '"name": "sp ace~!"', '"name": "nlonly"', '"name": "q\\"\\"x//"']
    return b, expect


def case_resource_infos():
    """libkineto/test/OutputJsonTest.cpp:154-179, 227-255: HOST_THREAD display name, escaping of quoted
    resource names; RocmActivityProfilerTest.cpp:967-975: GPU labels and sort index."""
    b = StreamBuilder()
    b.add_resource_info(12345, 12345, 99, "worker", host_thread=True)
    b.add_resource_info(-7, 3, 0, 'str"eam\\x')
    b.add_device_info(3, 3 + 5000000, "python", "GPU 3")
    b.add_overhead_info("CUPTI Overhead")
    expect = ['"name": "thread_name",\n    "ts": 0.000,\n    "pid": 99,\n    "tid": 12345,\n    "args": {\n      "name": "thread 12345 (worker)"\n    }',
              '"tid": 7,\n    "args": {\n      "name": "str\\"eam/x"\n    }',
              '"name": "process_labels",\n    "ts": 0.000,\n    "pid": 3,\n    "tid": 0,\n    "args": {\n      "labels": "GPU 3"\n    }',
              '"sort_index": 5000003', '"pid": -1,\n    "tid": 0,\n    "args": {\n      "sort_index": 16777226\n    }']
    return b, expect


def case_rocm_sync_trace():
    """The 15-activity trace of libkineto/test/RocmActivityProfilerTest.cpp:315-397: names, counts and
    resource ids (kernels on queue 1, copies on queue 2, no runtime row carries a stream)."""
    b = StreamBuilder(window=(B, B + 300), end_time=B + 300)
    b.api(["hipLaunchKernel", "hipMemcpy"], flow_start=[0, 1])
    pid, tid = 4000, 4001
    for i, (nm, s0, e0, cid) in enumerate([("op1", 20, 50, 1), ("op2", 30, 40, 2), ("op3", 100, 150, 3), ("op4", 160, 180, 4),
                                           ("op5", 190, 210, 4)]):
        b.add_generic(nm, CPU_OP, B + s0, B + e0, pid, tid, id=cid)
    b.add_runtime(1, B + 33, B + 38, 0, pid, tid, kind=1)
    b.add_runtime(2, B + 110, B + 120, 1, pid, tid, kind=2, size=1)
    b.add_runtime(3, B + 130, B + 145, 0, pid, tid, kind=1)
    b.add_runtime(4, B + 165, B + 175, 1, pid, tid, kind=2, size=1)
    b.add_runtime(5, B + 195, B + 205, 0, pid, tid, kind=1)
    b.add_device(1, B + 50, B + 70, domain=0, name="kernel", queue=1)
    b.add_device(2, B + 140, B + 150, domain=1, op=2, queue=2)
    b.add_device(3, B + 160, B + 220, domain=0, name="kernel", queue=1)
    b.add_device(4, B + 230, B + 250, domain=1, op=3, queue=2)
    b.add_device(5, B + 260, B + 280, domain=0, name="kernel", queue=1)
    expect_counts = {'"name": "hipLaunchKernel"': 3, '"name": "Memcpy HtoD (Host -> Device)"': 1,
                     '"name": "Memcpy DtoH (Device -> Host)"': 1, '"name": "Kernel"': 3, '"ph": "X"': 15,
                     '"pid": 0,\n    "tid": 1,\n    "ts"': 6, '"pid": 0,\n    "tid": 2,\n    "ts"': 4}
    return b, expect_counts


def case_instant_and_stream_sync():
    """Instant events (handleGenericInstantEvent, output_json.cpp:660-677: name and metadata printed
    as they are) and Stream Sync rows (output_json.cpp:913-943, 1008-1013: own row at tid + 1000000,
    announced once per (device, row), flow events on the same row).  Expected strings follow the
    reference's templates; the whole document is compared with the real logger where it is built."""
    CPU_INSTANT_EVENT, CUDA_SYNC = 9, 15
    b = StreamBuilder()
    frag = b.schema([(None, abi.F_RAW, 1)])
    b.add_generic('mark "a"\\b', CPU_INSTANT_EVENT, B + 100, B + 100, 7, 8, id=3, schema=frag,
                  values=[b.s('"note": "x\\y"')])
    b.add_generic("plain mark", CPU_INSTANT_EVENT, B + 150, B + 150, 7, 8)
    b.add_generic("Stream Sync", CUDA_SYNC, B + 2000, B + 2500, 0, 5, id=11, flow_id=11, flow_type=2)
    b.add_generic("Stream Sync", CUDA_SYNC, B + 1000, B + 1200, 0, 5, id=12)        # earlier in time: this one announces the row
    b.add_generic("Stream Sync", CUDA_SYNC, B + 3000, B + 3100, 1, 5, id=13)        # other device: own announcement
    b.add_generic("Event Sync", CUDA_SYNC, B + 4000, B + 4100, 0, 5, id=14)         # other name: stays on the stream's row
    b.add_generic("Stream Sync", KERNEL, B + 5000, B + 5100, 0, 5, id=15)           # other type: stays too
    expect = [
        '"ph": "i",\n    \n    "cat": "cpu_instant_event",\n    "s": "t",\n    "name": "mark "a"\\b",\n    "pid": 7,\n    "tid": 8,\n    "ts": 0.100\n    ,\n    "args": {\n      "note": "x\\y"\n    }\n  },',
        '"name": "plain mark",\n    "pid": 7,\n    "tid": 8,\n    "ts": 0.150\n    \n  },',
        '"name": "thread_name", "ph": "M", "ts": 1.000, "pid": 0, "tid": 1000005,\n    "args": {\n      "name": "stream 5 (sync)"\n    }\n  },\n  {\n    "name": "thread_sort_index", "ph": "M", "ts": 1.000, "pid": 0, "tid": 1000005,\n    "args": {\n      "sort_index": 5\n    }\n  },\n  {\n    "ph": "X",\n    "cat": "cuda_sync",\n    "name": "Stream Sync",\n    "pid": 0,\n    "tid": 1000005,\n    "ts": 1.000,',
        '"ph": "f",\n    "id": 11,\n    "pid": 0,\n    "tid": 1000005,\n    "ts": 2.000,',
        '"ts": 3.000, "pid": 1, "tid": 1000005,',
        '"name": "Event Sync",\n    "pid": 0,\n    "tid": 5,',
        '"cat": "kernel",\n    "name": "Stream Sync",\n    "pid": 0,\n    "tid": 5,',
    ]
    return b, expect


def case_counter_events():
    """Counter events (handleCounterEvent + writeCounterEvent, output_json.cpp:679-716, 294-316).
    Hardware counters print one event per value on the device's counter track, the other counter
    kinds one event with every value; values go through fmt "{}" and non-finite ones stay bare;
    names are printed as they are; neither an External id nor a flow event follows.  Expected
    strings follow the reference's templates; the whole document is compared with the real
    logger where it is built."""
    MTIA_COUNTERS, XPU_SCOPE_PROFILER, HARDWARE_COUNTERS = 17, 26, 28
    b = StreamBuilder()
    two = b.schema([("sm__cycles", abi.F_F64, 1), ('odd "name"\\x', abi.F_F64, 1)])
    mixed = b.schema([("skipped int", abi.F_I64, 1), ("busy", abi.F_F64, 1), (None, abi.F_RAW, 1), ("idle", abi.F_F64, 1)])
    specials = b.schema([("a", abi.F_F64, 1), ("b", abi.F_F64, 1), ("c", abi.F_F64, 1), ("d", abi.F_F64, 1), ("e", abi.F_F64, 1)])
    b.add_generic("ignored name", HARDWARE_COUNTERS, B + 1000, B + 1000, 3, -9, id=5, schema=two, values=[1.5, 2e-7],
                  flow_id=5, flow_type=2)
    b.add_generic('mtia "c"\\n', MTIA_COUNTERS, B + 2000, B + 2500, 1, 4, id=6, schema=mixed,
                  values=[12, 0.25, b.s('"x": 1'), 1e21], flow_id=6, flow_type=2, flow_start=True)
    b.add_generic("scope", XPU_SCOPE_PROFILER, B + 3000, B + 3000, 2, 2, schema=specials,
                  values=[float("inf"), float("-inf"), float("nan"), -0.0, 123456789012345680.0])
    b.add_generic("no values", MTIA_COUNTERS, B + 4000, B + 4000, 1, 4)
    b.add_generic("no values hw", HARDWARE_COUNTERS, B + 4500, B + 4500, 1, 4)
    b.add_generic("before base", XPU_SCOPE_PROFILER, B - 50, B - 50, 2, 2, schema=two, values=[3.0, 4.0])
    expect = [
        '\n  {\n    "ph": "C",\n    "cat": "hardware_counters",\n    "name": "sm__cycles",\n    "pid": "GPU 3 Counters",\n    "tid": 9,\n    "ts": 1.000,\n    "args": {\n      "": 1.5\n    }\n  },'
        '\n  {\n    "ph": "C",\n    "cat": "hardware_counters",\n    "name": "odd "name"\\x",\n    "pid": "GPU 3 Counters",\n    "tid": 9,\n    "ts": 1.000,\n    "args": {\n      "": 2e-07\n    }\n  },',
        '\n  {\n    "ph": "C",\n    "cat": "mtia_counters",\n    "name": "mtia "c"\\n",\n    "pid": 1,\n    "tid": 4,\n    "ts": 2.000,\n    "args": {\n      "busy": 0.25,"idle": 1e+21\n    }\n  },',
        '"name": "scope",\n    "pid": 2,\n    "tid": 2,\n    "ts": 3.000,\n    "args": {\n      "a": inf,"b": -inf,"c": nan,"d": -0,"e": 1.2345678901234568e+17\n    }\n  },',
        '"name": "no values",\n    "pid": 1,\n    "tid": 4,\n    "ts": 4.000,\n    "args": {\n      \n    }\n  },',
        '"name": "before base",\n    "pid": 2,\n    "tid": 2,\n    "ts": 0.000,\n    "args": {\n      "sm__cycles": 3,"odd "name"\\x": 4\n    }\n  },',
    ]
    return b, expect


COLLECTIVE_REF_VALUES = dict(collective_name="allreduce", dtype="Float", pg_name="0", pg_desc="default_pg", in_split="[1, 2]",
                             out_split="[3, 4]", group_ranks="[0, 1, 2, 3, 4, 5, 6, 7]", in_tensors_start="[[4096, 8192]]",
                             out_tensors_start="[[12288]]")
COLLECTIVE_REF_NUMBERS = dict(in_msg_nelems="1024", out_msg_nelems="512", group_size="8", rank="0", src_rank="1", dst_rank="2",
                              seq="3", comms_id="4")
# expectedArgs / expectedDistInfo of libkineto/test/OutputJsonTest.cpp:188-219
COLLECTIVE_REF_ARGS = {"Collective name": "allreduce", "In msg nelems": 1024, "Out msg nelems": 512, "Group size": 8,
                       "dtype": "Float", "Input Tensors start": "[[4096, 8192]]", "Output Tensors start": "[[12288]]",
                       "In split size": "[1, 2]", "Out split size": "[3, 4]", "Process Group Name": "0",
                       "Process Group Description": "default_pg", "Process Group Ranks": "[0, 1, 2, 3, 4, 5, 6, 7]",
                       "Src Rank": 1, "Dst Rank": 2, "Seq": 3, "Comms Id": 4}
COLLECTIVE_REF_DIST = {"backend": "nccl", "rank": 0, "world_size": 8, "pg_count": 1,
                       "pg_config": [{"pg_name": "0", "pg_desc": "default_pg", "backend_config": "cuda:nccl", "pg_size": 8,
                                      "ranks": "[0, 1, 2, 3, 4, 5, 6, 7]"}],
                       "nccl_version": "unknown"}


def case_collective_reference_test(quoted=False):
    """The trace of libkineto/test/OutputJsonTest.cpp:81-130: one CONCURRENT_KERNEL activity linked to
    a record_param_comms op; string values arrive with surrounding quotes (`quoted`) or bare.  The
    activity arrives with its linked op resolved, so the record itself carries the collective
    metadata."""
    b = StreamBuilder(end_time=B + 300)
    q = (lambda v: '"%s"' % v) if quoted else (lambda v: v)
    k = b.add_collective(**{key: q(v) for key, v in COLLECTIVE_REF_VALUES.items()}, **COLLECTIVE_REF_NUMBERS)
    own = b.schema([(None, abi.F_COLLECTIVE, 1)])
    b.add_generic("nccl:all_reduce", KERNEL, B + 100, B + 200, 0, 0, schema=own, values=[k], linked=0)
    expect = [
        '"name": "nccl:all_reduce",\n    "pid": 0,\n    "tid": 0,\n    "ts": 0.100,\n    "dur": 0.100\n    ,\n    "args": {\n      '
        '"Collective name": "allreduce","In msg nelems": 1024,"Out msg nelems": 512,"Group size": 8,"dtype": "Float",'
        '"Input Tensors start": "[[4096, 8192]]","Output Tensors start": "[[12288]]","In split size": "[1, 2]",'
        '"Out split size": "[3, 4]","Process Group Name": "0","Process Group Description": "default_pg",'
        '"Process Group Ranks": "[0, 1, 2, 3, 4, 5, 6, 7]","Dst Rank": 2,"Src Rank": 1,"Seq": 3,"Comms Id": 4\n    }\n  },',
        '\n  ],\n  "distributedInfo": {"backend": "nccl", "rank": 0, "world_size": 8, "pg_count": 1, "pg_config": ['
        '{"pg_name": "0", "pg_desc": "default_pg", "backend_config": "cuda:nccl", "pg_size": 8, '
        '"ranks": "[0, 1, 2, 3, 4, 5, 6, 7]"}], "nccl_version": "unknown"},"traceName": "t.json" }',
    ]
    return b, expect


def case_collective_reference_test_quoted():
    return case_collective_reference_test(quoted=True)


def case_collective_joined():
    """Collective metadata through the join (output_json.cpp:718-835, 899-908, 1030-1064): kernel rows
    print the values of the record_param_comms op their correlation id leads to; copies and kernels
    linked to other ops do not; the first kernel in emission order that names the default process
    group fills "distributedInfo", every group is listed once (first entry of a name stays); an
    MTIA event named hccl::... reports backend "hccl"; a kernel outside the window counts for
    nothing.  Expected strings follow the reference's templates; the whole document is compared
    with the real logger where it is built."""
    MTIA_CCP_EVENTS = 13
    b = StreamBuilder(window=(B, B + 10**6), end_time=B + 10**6)
    b.api(["hipLaunchKernel", "hipMemcpyAsync"], flow_start=[0, 1])
    typed = [(None, abi.F_COLLECTIVE, 1), ("Collective name", abi.F_STR, 1), ("Seq", abi.F_I64, 1)]
    sch = b.schema(typed)
    bare = b.schema([(None, abi.F_COLLECTIVE, 1)])
    plain = b.schema([("Seq", abi.F_I64, 1)])
    groups = [("7", "tp_group", "4", "[0, 1, 2, 3]"), ("0", "default_pg", "8", "[0, 1, 2, 3, 4, 5, 6, 7]"),
              ("12", "pp", "2", "[0, 4]"), ("3", 'dp "x"', "2", "[0, 1]"), ("0", "shadowed", "9", "[9]")]
    colls = []
    for i, (name, desc, size, ranks) in enumerate(groups):
        colls.append(b.add_collective(collective_name='"allgather"' if i % 2 else "allgather", in_msg_nelems=str(100 + i),
                                      out_msg_nelems=str(200 + i), group_size=size, dtype="Half", pg_name=name, pg_desc=desc,
                                      group_ranks=ranks, rank=str(5), seq=str(i), comms_id=str(1 << 40)))
    partial = b.add_collective(collective_name="broadcast", in_msg_nelems="1", pg_name="21", pg_desc="default_pg",
                               in_split="[1]", src_rank="3", rank="6")   # no dtype: none of the five; no out split: no splits
    empty = b.add_collective()                                            # nothing at all: group "" is still listed
    ops = colls + [partial, empty]
    pid, tid = 500, 501
    for i, k in enumerate(ops):                                           # CPU ops, ids 1..7
        b.add_generic("record_param_comms", CPU_OP, B + 1000 * i, B + 1000 * i + 500, pid, tid, id=i + 1, schema=sch if i < 5 else bare,
                      values=[k, b.s("allgather"), i] if i < 5 else [k])
    b.add_generic("aten::add", CPU_OP, B + 9000, B + 9500, pid, tid, id=8, schema=plain, values=[77])
    for corr in range(1, 11):
        b.add_extcorr(100 + corr, min(corr, 8))
        b.add_runtime(100 + corr, B + 20000 + corr, B + 20010 + corr, 0, pid, tid, kind=1, grid=[1, 1, 1], workgroup=[64, 1, 1], stream=0x7000)
    # kernels: emission order is by (device, stream index, start); arrival order is deliberately different
    b.add_device(104, B + 50000, B + 50100, domain=0, name="ncclDevKernel_dp", queue=1)          # group 3
    b.add_device(101, B + 40000, B + 40100, domain=0, name="ncclDevKernel_tp", queue=1)          # group 7: first in time on its stream
    b.add_device(102, B + 60000, B + 60100, domain=0, name="ncclDevKernel_default", queue=1)     # group 0 default_pg
    b.add_device(105, B + 30000, B + 30100, domain=0, name="ncclDevKernel_shadow", queue=1)      # group 0 again, other description: seen first
    b.add_device(103, B + 70000, B + 70100, domain=0, name="ncclDevKernel_pp", queue=1)
    b.add_device(106, B + 80000, B + 80100, domain=0, name="ncclDevKernel_partial", queue=1)
    b.add_device(107, B + 90000, B + 90100, domain=0, name="ncclDevKernel_empty", queue=1)
    b.add_device(108, B + 95000, B + 95100, domain=0, name="vector_add", queue=1)                # linked to aten::add
    b.add_device(102, B + 96000, B + 96100, domain=1, op=2, queue=1)                               # a copy linked to a collective op
    b.add_device(103, B + 2 * 10**6, B + 2 * 10**6 + 5, domain=0, name="late", queue=1)           # outside the window
    b.add_device(109, B + 97000, B + 97100, domain=0, name="vector_mul", queue=1)                # ids above 108 lead to aten::add too
    k_h = b.add_collective(collective_name="all_reduce", in_msg_nelems="4", out_msg_nelems="4", group_size="2", dtype="Int",
                           pg_name="h0", pg_desc="hccl_pg", group_ranks="[0, 1]", rank="1")
    own = b.schema([(None, abi.F_COLLECTIVE, 1), (None, abi.F_RAW, 1)])
    b.add_generic("hccl::all_reduce", MTIA_CCP_EVENTS, B + 100, B + 200, 0, 1, id=40, schema=own, values=[k_h, b.s('"x": 1')], linked=3)
    b.add_generic("not_hccl", MTIA_CCP_EVENTS, B + 300, B + 400, 0, 1, id=41, schema=own, values=[k_h, b.s('"y": 2')], linked=3)
    b.add_generic("hccl::unlinked", MTIA_CCP_EVENTS, B + 500, B + 600, 0, 1, id=42, schema=own, values=[k_h, b.s('"z": 3')])
    expect = [
        '"name": "hccl::all_reduce",\n    "pid": 0,\n    "tid": 1,\n    "ts": 0.100,\n    "dur": 0.100\n    ,\n    "args": {\n      "External id": 3,"x": 1,'
        '"Collective name": "all_reduce","In msg nelems": 4,"Out msg nelems": 4,"Group size": 2,"dtype": "Int","Process Group Name": "h0",'
        '"Process Group Description": "hccl_pg","Process Group Ranks": "[0, 1]"\n    }\n  },',
        '"name": "not_hccl",\n    "pid": 0,\n    "tid": 1,\n    "ts": 0.300,\n    "dur": 0.100\n    ,\n    "args": {\n      "External id": 3,"y": 2\n    }\n  },',
        '"args": {\n      "External id": 42,"z": 3\n    }\n  },',
        '"name": "ncclDevKernel_shadow",',
        '"correlation": 105, "kind": "Dispatch Kernel", "grid": [1, 1, 1], "block": [64, 1, 1],"Collective name": "allgather","In msg nelems": 104,'
        '"Out msg nelems": 204,"Group size": 9,"dtype": "Half","Process Group Name": "0","Process Group Description": "shadowed",'
        '"Process Group Ranks": "[9]","Seq": 4,"Comms Id": 1099511627776\n    }\n  },',
        '"correlation": 106, "kind": "Dispatch Kernel", "grid": [1, 1, 1], "block": [64, 1, 1],"In msg nelems"',
        '"correlation": 106, "kind": "Dispatch Kernel", "grid": [1, 1, 1], "block": [64, 1, 1],"Process Group Name": "21","Process Group Description": "default_pg","Src Rank": 3\n    }',
        '"correlation": 107, "kind": "Dispatch Kernel", "grid": [1, 1, 1], "block": [64, 1, 1]\n    }',
        '"correlation": 108, "kind": "Dispatch Kernel", "grid": [1, 1, 1], "block": [64, 1, 1]\n    }',
        '"distributedInfo": {"backend": "nccl", "rank": 5, "world_size": 8, "pg_count": 7, "pg_config": [',
        '{"pg_name": "0", "pg_desc": "shadowed", "backend_config": "cuda:nccl", "pg_size": 9, "ranks": "[9]"}',
        '{"pg_name": "h0", "pg_desc": "hccl_pg", "backend_config": "mtia:hccl", "pg_size": 2, "ranks": "[0, 1]"}',
        '{"pg_name": "", "pg_desc": "", "backend_config": "cuda:nccl", "pg_size": , "ranks": ""}',
        '{"pg_name": "3", "pg_desc": "dp "x"", "backend_config": "cuda:nccl", "pg_size": 2, "ranks": "[0, 1]"}',
        '], "nccl_version": "unknown"},"traceName": "t.json" }',
    ]
    absent = ['"correlation": 106, "kind": "Dispatch Kernel", "grid": [1, 1, 1], "block": [64, 1, 1],"In msg nelems"']
    expect = [e for e in expect if e not in absent]
    return b, expect


def case_gpu_user_annotation_reference_test():
    """The trace of libkineto/test/RocmActivityProfilerTest.cpp:770-833: one CPU annotation, two
    kernels correlated with it in the user domain; an extra GPU_USER_ANNOTATION activity covers
    both kernels on their device and queue: ts = first kernel's, duration = end of the second -
    start of the first, correlation id and name of the CPU annotation.  It is printed one ns early
    and two ns longer (output_json.cpp:862-869) with the annotation's id as External id."""
    b = StreamBuilder(window=(B, B + 300), end_time=B + 300)
    L = B + 20
    b.add_generic("annotation", CPU_OP, L, L + 10, 4000, 4001, id=1)
    b.add_usercorr(1, 1)
    b.add_device(1, L + 5, L + 10, domain=0, name="kernel", queue=1)
    b.add_usercorr(1, 1)
    b.add_device(1, L + 15, L + 25, domain=0, name="kernel", queue=1)
    expect = [
        # kernel 1: ts = begin + 1 = 26 ns; kernel 2 ends at 45 ns: span 26..45, printed from 25 for 21
        '"ph": "X",\n    "cat": "gpu_user_annotation",\n    "name": "annotation",\n    "pid": 0,\n    "tid": 1,\n    "ts": 0.025,\n    "dur": 0.021\n    ,\n    "args": {\n      "External id": 1\n    }\n  },',
        '"cat": "kernel",\n    "name": "Kernel",\n    "pid": 0,\n    "tid": 1,\n    "ts": 0.026,\n    "dur": 0.004',
        '"cat": "kernel",\n    "name": "Kernel",\n    "pid": 0,\n    "tid": 1,\n    "ts": 0.036,\n    "dur": 0.009',
    ]
    return b, expect


def case_gpu_user_annotations():
    """GPU user annotations over several streams and annotations (GenericActivityProfiler.cpp:277-327,
    423-433): one span per (device, stream, annotation); rows outside the window, rows whose
    correlation has no user record and user records that name no CPU activity add nothing; the
    last user record of a correlation id and the last CPU activity of an id are the ones used; a
    row that starts at time 0 makes the next row's start replace the span's (start rule :304-306)."""
    b = StreamBuilder(window=(0, B + 10**6), end_time=B + 10**6)
    b.add_generic("step A", 1, B + 10, B + 500, 7, 8, id=50)                  # USER_ANNOTATION
    b.add_generic("step B (shadowed)", 1, B + 20, B + 600, 7, 8, id=51)
    b.add_generic('step B "final"', 1, B + 30, B + 700, 7, 8, id=51)          # same id: this one is looked up
    b.add_generic("no kernels", 1, B + 40, B + 800, 7, 8, id=52)
    b.add_generic("zero", 1, B + 50, B + 900, 7, 8, id=0)                     # id 0: no External id printed
    for corr, ext in [(1, 50), (2, 50), (3, 51), (4, 51), (5, 99), (6, 50), (3, 52), (3, 51), (7, 0), (8, 0), (9, 0), (10, 50)]:
        b.add_usercorr(corr, ext)
    b.add_device(2, B + 3000, B + 3500, domain=0, name="k2", queue=1)         # A on queue 1 (later in time, first in arrival)
    b.add_device(1, B + 1000, B + 1200, domain=0, name="k1", queue=1)         # A on queue 1: earliest
    b.add_device(6, B + 2000, B + 9000, domain=1, op=2, queue=2)              # A on queue 2 (a copy)
    b.add_device(3, B + 4000, B + 4100, domain=0, name="k3", queue=1)         # B on queue 1
    b.add_device(4, B + 100, B + 200, domain=0, name="k4", queue=1, device=1) # B on another device
    b.add_device(5, B + 5000, B + 5100, domain=0, name="k5", queue=1)         # annotation 99 does not exist
    b.add_device(11, B + 6000, B + 6100, domain=0, name="k11", queue=1)       # no user record
    b.add_device(10, B + 2 * 10**6, B + 2 * 10**6 + 9, domain=0, name="late", queue=3)  # outside the window
    b.add_device(7, 40, 60, domain=2, stream=9, queue=5, nbytes=16)           # memset rows start at `begin`
    b.add_device(8, 0, 30, domain=2, stream=9, queue=5, nbytes=16)            # starts at time 0 ...
    b.add_device(9, 70, 90, domain=2, stream=9, queue=5, nbytes=16)           # ... so this start replaces it
    expect = [
        '"cat": "gpu_user_annotation",\n    "name": "step A",\n    "pid": 0,\n    "tid": 1,\n    "ts": 1.000,\n    "dur": 2.501\n    ,\n    "args": {\n      "External id": 50\n    }',
        '"cat": "gpu_user_annotation",\n    "name": "step A",\n    "pid": 0,\n    "tid": 2,\n    "ts": 2.000,\n    "dur": 7.001\n    ,\n    "args": {\n      "External id": 50\n    }',
        '"cat": "gpu_user_annotation",\n    "name": "step B \\"final\\"",\n    "pid": 0,\n    "tid": 1,\n    "ts": 4.000,\n    "dur": 0.101\n    ,',
        '"cat": "gpu_user_annotation",\n    "name": "step B \\"final\\"",\n    "pid": 1,\n    "tid": 1,\n    "ts": 0.100,\n    "dur": 0.101\n    ,',
        '"cat": "gpu_user_annotation",\n    "name": "zero",\n    "pid": 0,\n    "tid": 9,\n    "ts": 0.000,\n    "dur": 0.022\n    \n  },',
    ]
    return b, expect


SUBSTRING_CASES = [case_gpu_user_annotation_reference_test, case_gpu_user_annotations, case_collective_reference_test, case_collective_reference_test_quoted, case_collective_joined, case_counter_events, case_instant_and_stream_sync, case_logger_events, case_trace_span, case_benchmark_cpu_op, case_typed_kernel_args,
                   case_typed_metadata_pins, case_typed_metadata_collections, case_cuda_shaped_kernel_args, case_names, case_resource_infos]


def build_for_real_logger(case, ref_args):
    """Builds a hand-made case so that the real logger can render it: every absolute time is
    shifted by the difference between the real logger's base time (wall clock, `ref_args` from
    oracle_glue.ref_stream_args()) and the default one, and the header carries this machine's
    host name."""
    import stream_builder
    delta = ref_args["base_time_ns"] - stream_builder.B
    b, _ = case()
    b.base += delta
    b.window = (b.window[0] + delta, b.window[1] + delta)
    b.end_time += delta
    for r in b.generic:
        r.start_ns += delta; r.end_ns += delta
    for r in b.runtime:
        r.begin += delta; r.end += delta
    for r in b.device:
        r.begin += delta; r.end += delta
    for lst in (b.device_infos, b.resource_infos, b.overhead_infos):
        for x in lst:
            x.time_ns += delta
    for x in b.spans:
        x.start_ns += delta; x.end_ns += delta
    b.meta = [("host_name", '"%s"' % ref_args["host_name"])]
    return b.build()
