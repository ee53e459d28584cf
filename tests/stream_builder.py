"""Hand-made ktj_stream objects for known-answer and edge-case tests (ctypes, no computation)."""
import ctypes as C
import struct

from kineto_amd import abi

B = abi.DEFAULT_BASE_TIME_NS


class StreamBuilder:
    def __init__(self, base=B, trace_name="t.json", host_name=None, window=(None, None), end_time=None):
        self.base = base
        self.trace_name = trace_name
        self.meta = []
        if host_name is not None:
            self.meta.append(("host_name", '"%s"' % host_name))
        self.strings = []
        self.fields = []
        self.schemas = []
        self.args = []
        self.cid_names = []
        self.flow_start = []
        self.malloc_cid = abi.KTJ_NONE
        self.clock = abi.ClockModel(0, 0, 1.0, 0, 0, 0)
        self.window = (base if window[0] is None else window[0], base + 10**12 if window[1] is None else window[1])
        self.end_time = self.window[1] if end_time is None else end_time
        self.generic, self.runtime, self.device, self.extcorr = [], [], [], []
        self.device_infos, self.resource_infos, self.overhead_infos, self.spans = [], [], [], []
        self.collectives = []
        self.usercorr = []
        self.create_flags = 0   # the ktj_create flags that change the document (KTJ_CREATE_CUDA12_ARGS)
        self._keep = []

    # ---- dictionary / schemas ----
    def s(self, text):
        b = text if isinstance(text, bytes) else text.encode("latin1")
        self.strings.append(b)
        return len(self.strings) - 1

    def schema(self, fields):
        """fields: list of (key or None, type, count)"""
        first = len(self.fields)
        for key, typ, cnt in fields:
            self.fields.append((abi.KTJ_NONE if key is None else self.s(key), typ, cnt))
        self.schemas.append((first, len(fields)))
        return len(self.schemas) - 1

    def add_collective(self, **values):
        """One record_param_comms op's metadata values (abi.COLLECTIVE_KEYS, as getMetadataValue()
        returns them); returns the index for the slot of a leading F_COLLECTIVE field."""
        m = abi.CollectiveMeta()
        for k, v in values.items():
            assert k in abi.COLLECTIVE_KEYS, k
            setattr(m, k, v.encode("latin1") if isinstance(v, str) else v)
        self.collectives.append(m)
        return len(self.collectives) - 1

    def arg_slots(self, values):
        off = len(self.args)
        for v in values:
            if isinstance(v, float):
                v = struct.unpack("<Q", struct.pack("<d", v))[0]
            self.args.append(v & 0xFFFFFFFFFFFFFFFF)
        return off

    def shapes(self, value):
        """Encodes an InputShapes value (a list whose entries are a shape, e.g. [2, 2], or a list of
        shapes, e.g. [[4, 1], [4, 1]]; an empty entry is an empty shape) in the args blob and returns
        the slot index for a F_SHAPES field (include/ktj.h: KTJ_F_SHAPES)."""
        enc = [len(value)]
        for entry in value:
            if entry and isinstance(entry[0], (list, tuple)):
                enc.append(abi.SHAPE_LIST | len(entry))
                for shape in entry:
                    enc += [len(shape)] + list(shape)
            else:
                enc += [len(entry)] + list(entry)
        return self.arg_slots(enc)

    def api(self, names, flow_start=(), malloc_cid=abi.KTJ_NONE):
        self.cid_names = [abi.KTJ_NONE if n is None else self.s(n) for n in names]
        self.flow_start = list(flow_start)
        self.malloc_cid = malloc_cid

    # ---- records ----
    def add_generic(self, name, typ, start, end, device, resource, id=0, schema=None, values=(), flow_id=0,
                    flow_type=0, flow_start=False, linked=None):
        r = abi.GenericRec()
        r.start_ns, r.end_ns, r.resource = start, end, resource
        wide = not -(1 << 31) <= device < (1 << 31)  # travels in the slot before the record's values
        r.id, r.device = id, 0 if wide else device
        r.name_id = abi.KTJ_NONE if name is None else self.s(name)
        r.type = typ
        r.flow_id, r.flow_type = flow_id, flow_type
        r.flags = (1 if flow_start else 0) | (2 if linked is not None else 0) | (abi.KTJ_GF_WIDE_DEVICE if wide else 0)
        r.linked_id = 0 if linked is None else C.c_int32(linked & 0xFFFFFFFF).value
        r.schema_id = abi.KTJ_NONE if schema is None else schema
        if wide:
            self.arg_slots([device])
        r.args_off = self.arg_slots(values) if schema is not None else (len(self.args) if wide else 0)
        self.generic.append(r)
        return r

    def add_runtime(self, id, begin, end, cid, pid, tid, kind=0, **kw):
        r = abi.RuntimeRec()
        r.id, r.begin, r.end, r.cid, r.pid, r.tid, r.kind = id, begin, end, cid, pid, tid, kind
        if kind == 1:
            g = kw.get("grid", (0, 0, 0)); w = kw.get("workgroup", (0, 0, 0))
            for i in range(3):
                r.u.kernel.grid[i] = g[i]; r.u.kernel.workgroup[i] = w[i]
            r.u.kernel.group_segment_size = kw.get("lds", 0)
            r.u.kernel.stream = kw.get("stream", 0)
            r.u.kernel.kernel_name_id = abi.KTJ_NONE if kw.get("kernel_name") is None else self.s(kw["kernel_name"])
        elif kind == 2:
            r.u.copy.src, r.u.copy.dst = kw.get("src", 0), kw.get("dst", 0)
            r.u.copy.size, r.u.copy.stream = kw.get("size", 0), kw.get("stream", 0)
            r.u.copy.copy_kind = kw.get("copy_kind", 0)
        elif kind == 3:
            r.u.malloc_.ptr, r.u.malloc_.size = kw.get("ptr", 0), kw.get("size", 0)
        self.runtime.append(r)
        return r

    def add_device(self, id, begin, end, domain=0, op=0, device=0, name=None, queue=0, stream=0, nbytes=0,
                   memory_kind=abi.KTJ_MEMKIND_DEVICE, channel_type=0):
        """A device row.  For a memset row (domain 2) the fields are read through the ktj_memset_rec
        view: queue = context | channel id << 32, stream = stream | graph id << 32, op and the name's
        string id are the two halves of the graph node id (add_memset spells that out)."""
        d = abi.DeviceRec()
        d.id, d.begin, d.end, d.domain, d.op, d.device = id, begin, end, domain, op, device
        if domain == abi.KTJ_DOM_MEMSET:
            d.domain = domain | (channel_type & 0xFF) << 16 | (memory_kind & 0xFF) << 24
        d.name_id = abi.KTJ_NONE if name is None else self.s(name)
        d.queue, d.stream, d.bytes = queue, stream, nbytes
        self.device.append(d)
        return d

    def add_memset(self, id, begin, end, device=0, context=0, stream=0, nbytes=0, memory_kind=abi.KTJ_MEMKIND_DEVICE,
                   graph_id=0, graph_node_id=0, channel_id=0, channel_type=0):
        m = abi.MemsetRec()
        m.id, m.begin, m.end, m.domain, m.device = id, begin, end, abi.KTJ_DOM_MEMSET, device
        m.channel_type, m.memory_kind = channel_type, memory_kind
        m.graph_node_lo, m.graph_node_hi = graph_node_id & 0xFFFFFFFF, graph_node_id >> 32
        m.context, m.channel_id, m.stream, m.graph_id, m.bytes = context, channel_id, stream, graph_id, nbytes
        d = abi.DeviceRec.from_buffer_copy(bytes(m))
        self.device.append(d)
        return d

    def add_extcorr(self, corr, ext):
        self.extcorr.append(abi.ExtCorrRec(corr, ext))

    def add_usercorr(self, corr, ext):
        self.usercorr.append(abi.ExtCorrRec(corr & 0xFFFFFFFFFFFFFFFF, ext & 0xFFFFFFFFFFFFFFFF))

    def add_device_info(self, id, sort_index, name, label, t=None):
        self.device_infos.append(abi.DeviceInfo(id, sort_index, name.encode(), label.encode(), self.base if t is None else t))

    def add_resource_info(self, id, sort_index, device_id, name, host_thread=False, t=None):
        self.resource_infos.append(abi.ResourceInfo(id, sort_index, device_id, name.encode(), 1 if host_thread else 0, 0,
                                                    self.base if t is None else t))

    def add_overhead_info(self, name, t=None):
        self.overhead_infos.append(abi.OverheadInfo(name.encode(), self.base if t is None else t))

    def add_span(self, start, end, op_count, iteration, name, prefix=""):
        self.spans.append(abi.TraceSpan(start, end, op_count, iteration, name.encode(), prefix.encode()))

    # ---- assemble ----
    def _arr(self, ctype, items):
        a = (ctype * max(len(items), 1))(*items)
        self._keep.append(a)
        return a

    def build(self):
        st = abi.Stream()
        st.base_time_ns = self.base
        st.trace_name = self.trace_name.encode()
        st.device_properties = b""
        kv = []
        for k, v in self.meta:
            kv += [k.encode(), v.encode()]
        st.meta_kv = self._arr(C.c_char_p, kv)
        st.n_meta = len(self.meta)
        blob = b"".join(self.strings)
        offs = [0]
        for x in self.strings:
            offs.append(offs[-1] + len(x))
        bb = C.create_string_buffer(blob, max(len(blob), 1))
        self._keep.append(bb)
        st.str_blob = C.cast(bb, C.c_void_p)
        st.str_off = self._arr(C.c_uint64, offs)
        st.n_strings = len(self.strings)
        st.fields = self._arr(abi.Field, [abi.Field(*f) for f in self.fields])
        st.n_fields = len(self.fields)
        st.schemas = self._arr(abi.SchemaDesc, [abi.SchemaDesc(*x) for x in self.schemas])
        st.n_schemas = len(self.schemas)
        st.args = self._arr(C.c_uint64, self.args)
        st.n_args = len(self.args)
        st.cid_name_ids = self._arr(C.c_uint32, self.cid_names)
        st.n_cids = len(self.cid_names)
        st.flow_start_cids = self._arr(C.c_uint32, self.flow_start)
        st.n_flow_start = len(self.flow_start)
        st.malloc_cid = self.malloc_cid
        st.create_flags = self.create_flags
        st.clock = self.clock
        st.window_start_ns, st.window_end_ns = self.window
        st.end_time_ns = self.end_time
        for name, ctype, items in (("generic", abi.GenericRec, self.generic), ("runtime", abi.RuntimeRec, self.runtime),
                                   ("device", abi.DeviceRec, self.device), ("extcorr", abi.ExtCorrRec, self.extcorr),
                                   ("usercorr", abi.ExtCorrRec, self.usercorr),
                                   ("device_infos", abi.DeviceInfo, self.device_infos),
                                   ("resource_infos", abi.ResourceInfo, self.resource_infos),
                                   ("overhead_infos", abi.OverheadInfo, self.overhead_infos),
                                   ("spans", abi.TraceSpan, self.spans), ("collectives", abi.CollectiveMeta, self.collectives)):
            setattr(st, name, self._arr(ctype, items))
            setattr(st, "n_" + name, len(items))
        self._keep.append(st)
        return C.pointer(st)
