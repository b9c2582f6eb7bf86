"""Writer for MegCC `.tiny` model files: the FlatBuffers binary of runtime/schema/model.fbs that
`mgb-to-tinynn` exports (compiler/lib/Target/TinyNN/exporter.cpp) and the TinyNN runtime parses
(runtime/src/parse.c). Pure Python, no flatbuffers package: the wire format is written directly.

A model is described with plain dicts/lists (see `write_model`); field numbers follow the order of
declaration in the schema. Scalars equal to their schema default are left out of the table, as the
FlatBuffers builders do, so readers must apply the defaults.
"""
import struct

import numpy as np

# schema enums (runtime/schema/model.fbs)
FLOAT32, FLOAT16, INT32, INT8, INT16, UINT8, QINT8, QINT32, QUINT8 = 0, 1, 2, 3, 4, 5, 100, 101, 102
FORMAT_NCHW, FORMAT_NHWC, FORMAT_NCHW4, FORMAT_NCHW8, FORMAT_OIHW = range(5)
(DEVICE_BARE_METAL, DEVICE_ARM64, DEVICE_ARM32, DEVICE_ARM64_V82, DEVICE_ARM32_V82,
 DEVICE_OPENCL_MALI, DEVICE_WEB_ASSEMBLY, DEVICE_GFX950) = range(8)
TENSOR, WEIGHT = 0, 1
MEMFORWARD_RESHAPE, MEMFORWARD_SUBTENSOR, MEMFORWARD_DIMSHUFFLE = 0, 1, 2
INSTRUCTION_IDS = {"Opr": 1, "DevMemAlloc": 2, "DevMemFree": 3, "MemForward": 4}

_ITEMSIZE = {FLOAT32: 4, FLOAT16: 2, INT32: 4, INT8: 1, INT16: 2, UINT8: 1, QINT8: 1, QINT32: 4,
             QUINT8: 1}

_SCALARS = {"i8": "<b", "u8": "<B", "bool": "<B", "i32": "<i", "u32": "<I", "i64": "<q",
            "u64": "<Q", "f32": "<f"}


class _Table:
    """fields: (number, kind, value[, schema default]); kind is a scalar kind or one of
    table / string / ints / bytes / tables / strings (the last five are reached by offset)."""

    def __init__(self, fields):
        self.fields = []
        for f in fields:
            number, kind, value = f[:3]
            if value is None:
                continue
            if len(f) > 3 and kind in _SCALARS and value == f[3]:
                continue
            self.fields.append((number, kind, value))


class _Writer:
    def __init__(self):
        self.buf = bytearray()

    def _pad_to(self, align, after=0):
        """pads so that position + `after` is a multiple of `align`"""
        while (len(self.buf) + after) % align:
            self.buf.append(0)

    def _patch(self, at, target):
        struct.pack_into("<I", self.buf, at, target - at)

    def string(self, s):
        raw = s.encode()
        self._pad_to(4)
        pos = len(self.buf)
        self.buf += struct.pack("<I", len(raw)) + raw + b"\0"
        return pos

    def scalars(self, fmt, size, values, align=4):
        self._pad_to(max(align, 4), after=4)  # the elements, not the count, get the alignment
        pos = len(self.buf)
        self.buf += struct.pack("<I", len(values))
        if isinstance(values, (bytes, bytearray)):
            self.buf += values
        else:
            self.buf += struct.pack("<%d%s" % (len(values), fmt), *values)
        return pos

    def offsets(self, children, write_child):
        self._pad_to(4)
        pos = len(self.buf)
        self.buf += struct.pack("<I", len(children)) + b"\0" * (4 * len(children))
        for i, child in enumerate(children):
            self._patch(pos + 4 + 4 * i, write_child(child))
        return pos

    def table(self, t):
        sized = []
        for number, kind, value in t.fields:
            size = struct.calcsize(_SCALARS[kind]) if kind in _SCALARS else 4
            sized.append((size, number, kind, value))
        sized.sort(key=lambda f: (-f[0], f[1]))
        slots = (max(f[1] for f in sized) + 1) if sized else 0
        vt_bytes = 4 + 2 * slots
        at, where = 4, {}
        for size, number, kind, value in sized:
            at = (at + size - 1) // size * size
            where[number] = at
            at += size
        tab_bytes = at
        self._pad_to(8, after=vt_bytes)
        vt_pos = len(self.buf)
        self.buf += struct.pack("<HH", vt_bytes, tab_bytes)
        self.buf += struct.pack("<%dH" % slots, *[where.get(i, 0) for i in range(slots)])
        pos = len(self.buf)
        self.buf += struct.pack("<i", pos - vt_pos) + b"\0" * (tab_bytes - 4)
        later = []
        for size, number, kind, value in sized:
            if kind in _SCALARS:
                struct.pack_into(_SCALARS[kind], self.buf, pos + where[number], value)
            else:
                later.append((pos + where[number], kind, value))
        for at, kind, value in later:
            if kind == "table":
                target = self.table(value)
            elif kind == "string":
                target = self.string(value)
            elif kind == "ints":
                target = self.scalars("i", 4, [int(v) for v in value])
            elif kind == "bytes":  # tensor data: 16-byte aligned in the file
                target = self.scalars("b", 1, bytes(value), align=16)
            elif kind == "small_bytes":
                target = self.scalars("b", 1, bytes(value))
            elif kind == "tables":
                target = self.offsets(value, self.table)
            elif kind == "strings":
                target = self.offsets(value, self.string)
            else:
                raise ValueError(kind)
            self._patch(at, target)
        return pos


def _dtype(d):
    """(type enum, scale or None[, zero point])"""
    kind, scale = d[0], d[1] if len(d) > 1 else None
    zero = d[2] if len(d) > 2 else 0
    param = None
    if scale is not None:
        param = _Table([(0, "f32", float(scale), 1.0), (1, "u8", int(zero), 0)])
    return _Table([(0, "i8", _signed8(kind), 0), (1, "table", param)])


def _signed8(v):
    return v - 256 if v > 127 else v


def _layout(dims, stride=None, fmt=FORMAT_NCHW):
    dims = [int(d) for d in dims]
    if stride is None:
        stride, s = [], 1
        for d in reversed(dims):
            stride.insert(0, s)
            s *= d
    return _Table([(0, "ints", dims), (1, "ints", stride), (2, "i8", fmt, 0)])


def _weight(w):
    data = w["data"]
    if isinstance(data, np.ndarray):
        data = np.ascontiguousarray(data).tobytes()
    return _Table([
        (0, "table", _dtype(w["dtype"])),
        (1, "table", _layout(w["dims"], w.get("stride"), w.get("format", FORMAT_NCHW))),
        (2, "i32", w.get("use_count", 0), 0),
        (3, "bytes", data),
        (4, "string", w["name"]),
        (5, "u32", w.get("checksum", 0), 0),
        (6, "bool", int(w.get("compressed", False)), 0),
    ])


def _tensor(t):
    return _Table([
        (0, "table", _dtype(t["dtype"])),
        (1, "table", _layout(t["dims"], t.get("stride"), t.get("format", FORMAT_NCHW))),
        (2, "i64", int(t.get("offset", 0)), 0),
        (3, "bool", int(t.get("dynamic", False)), 0),
        (4, "i32", t.get("use_count", 0), 0),
        (5, "string", t.get("name", "")),
    ])


def _instruction(kind, f):
    if kind == "Opr":
        ws = _Table([(0, "i64", int(f.get("workspace_size", 0)), 0),
                     (1, "i64", int(f.get("workspace_offset", 0)), 0)])
        return _Table([
            (0, "string", f.get("name", "")),
            (1, "string", f["type"]),
            (2, "ints", f["inputs"]),
            (3, "small_bytes", [int(v) for v in f["input_types"]]),
            (4, "ints", f["outputs"]),
            (5, "table", ws),
            (6, "i32", f.get("init_id", -1), -1),
            (7, "i32", f.get("kernel_id", 0), 0),
            (8, "i32", f.get("workspace_id", -1), -1),
            (9, "i32", f.get("deduce_id", -1), -1),
        ])
    if kind == "MemForward":
        return _Table([(0, "i32", f["input"], 0), (1, "i32", f["output"], 0),
                       (2, "i32", f.get("offset", 0), 0), (3, "i8", f.get("type", 0), 0)])
    if kind in ("DevMemAlloc", "DevMemFree"):
        return _Table([(0, "i32", f["tensor"], 0)])
    raise ValueError("instruction %r is not written by this module" % kind)


def _device_model(d):
    kinds = [INSTRUCTION_IDS[k] for k, _ in d["instructions"]]
    return _Table([
        (0, "i8", d.get("device", DEVICE_BARE_METAL), 0),
        (1, "tables", [_tensor(t) for t in d["tensors"]]),
        (2, "small_bytes", kinds),
        (3, "tables", [_instruction(k, f) for k, f in d["instructions"]]),
        (4, "u64", int(d.get("tensor_memory", 0)), 0),
        (5, "ints", d.get("inputs", [])),
        (6, "ints", d.get("outputs", [])),
        (7, "ints", d.get("weight_outputs", [])),
        (8, "strings", d.get("weight_output_names", [])),
    ])


def write_model(model):
    """model = {name, model_id, const_shape,
                weights: [{name, dtype: (enum, scale|None), dims, data, [stride, format,
                           use_count, checksum, compressed]}],
                device_models: [{device, tensor_memory, inputs, outputs,
                                 [weight_outputs, weight_output_names],
                                 tensors: [{name, dtype, dims, offset, [stride, format, dynamic,
                                            use_count]}],
                                 instructions: [("Opr", {name, type, inputs, input_types, outputs,
                                                         [workspace_size, workspace_offset,
                                                          init_id, kernel_id, workspace_id,
                                                          deduce_id]}),
                                                ("MemForward", {input, output, [offset, type]}),
                                                ...]}]}
    Returns the file contents as bytes."""
    w = _Writer()
    w.buf += b"\0" * 4  # root offset
    root = w.table(_Table([
        (0, "tables", [_weight(x) for x in model.get("weights", [])]),
        (1, "tables", [_device_model(d) for d in model["device_models"]]),
        (2, "bool", int(model.get("const_shape", True)), 0),
        (3, "string", model.get("name", "")),
        (4, "u64", int(model.get("model_id", 0)), 0),
    ]))
    struct.pack_into("<I", w.buf, 0, root)
    return bytes(w.buf)


class _WeightId(int):
    """index into the weight pool (a plain int is an index into the tensor pool)"""


class ModelBuilder:
    """Collects a static-shape model through the same calls as runtime.Model (tensor, weight,
    alias, opr, mark_input, mark_output) and serialises it the way the MegCC exporter does: one
    device model, tensors with offsets from the static memory plan, one Opr instruction per
    kernel call (Opr.type = kernel symbol, compiler/lib/Target/TinyNN/exporter.cpp:374-380), a
    MemForward instruction per view. The plan is the PUSHDOWN plan of the operators' lifetimes
    (time step = Opr index; outputs stay alive to the end); model inputs are not in the arena."""

    def __init__(self, name="model", device=DEVICE_BARE_METAL, alignment=64, kernel_table=None):
        """kernel_table: {symbol: (kernel_id, init_id, workspace_id)}, the indices of the kernel
        tables the TinyNN runtime was built with (kernels[] / init_kernels[] / workspace_func[] of
        the exporter's kernels.c, compiler/lib/Target/TinyNN/KernelExporter.cpp:15-66). With a
        table every Opr carries those ids and a workspace sized by the kernel's own _workspace
        function, planned into the arena for the one step the Opr runs (the compiler evaluates
        that function at compile time, compiler/lib/KernelGen/Jit/JitExe.cpp:67-123; the runtime
        points Opr.workspace at arena + offset, runtime/src/init.c:478-484). Without a table
        kernel_id is the Opr's position and no workspace is planned (the model runtime of this
        library binds kernels by symbol and keeps one workspace of its own)."""
        self.name, self.device, self.alignment = name, device, alignment
        self.kernel_table = kernel_table
        self.tensors, self.weights, self.instructions = [], [], []
        self.inputs, self.outputs = [], []
        self._root, self._first, self._last = [], [], []
        self._nr_opr = 0

    @staticmethod
    def _dtype(type_enum, scale):
        return (type_enum, float(scale)) if type_enum >= QINT8 else (type_enum, None)

    def tensor(self, name, shape, type_enum, scale=1.0):
        self.tensors.append(dict(name=name, dtype=self._dtype(type_enum, scale),
                                 dims=list(shape), offset=0, use_count=0))
        self._root.append(-1)
        self._first.append(-1)
        self._last.append(-1)
        return len(self.tensors) - 1

    def weight(self, name, array, type_enum, scale=1.0):
        array = np.ascontiguousarray(array)
        self.weights.append(dict(name=name, dtype=self._dtype(type_enum, scale),
                                 dims=list(array.shape), data=array, use_count=0))
        return _WeightId(len(self.weights) - 1)

    def alias(self, name, of, shape):
        src = self.tensors[of]
        tid = self.tensor(name, shape, src["dtype"][0], src["dtype"][1] or 1.0)
        self._root[tid] = of
        self.instructions.append(("MemForward", dict(input=of, output=tid, offset=0,
                                                     type=MEMFORWARD_RESHAPE)))
        return tid

    def view(self, name, of, shape, strides, offset=0, kind=MEMFORWARD_SUBTENSOR):
        """strided window into tensor `of` (element strides, first element `offset` elements
        in): the tensor carries the strides, a MemForward of type `kind` the byte offset"""
        src = self.tensors[of]
        tid = self.tensor(name, shape, src["dtype"][0], src["dtype"][1] or 1.0)
        self.tensors[tid]["stride"] = [int(s) for s in strides]
        self._root[tid] = of
        self.instructions.append(("MemForward", dict(
            input=of, output=tid, offset=int(offset) * _ITEMSIZE[src["dtype"][0]], type=kind)))
        return tid

    def _root_of(self, t):
        while self._root[t] >= 0:
            t = self._root[t]
        return t

    def opr(self, symbol, inputs, outputs):
        k = self._nr_opr
        for t in inputs:
            if isinstance(t, _WeightId):
                self.weights[t]["use_count"] += 1
                continue
            self.tensors[t]["use_count"] += 1
            r = self._root_of(t)
            self._last[r] = max(self._last[r], k)
        for t in outputs:
            r = self._root_of(t)
            if self._first[r] < 0:
                self._first[r] = k
            self._last[r] = max(self._last[r], k)
        fields = dict(
            name="%s:%d" % (symbol, k), type=symbol, inputs=[int(t) for t in inputs],
            input_types=[WEIGHT if isinstance(t, _WeightId) else TENSOR for t in inputs],
            outputs=list(outputs), kernel_id=k)
        if self.kernel_table is not None:
            if symbol not in self.kernel_table:
                raise KeyError("the runtime's kernel tables hold no %s" % symbol)
            fields["kernel_id"], fields["init_id"], fields["workspace_id"] = self.kernel_table[symbol]
            fields["workspace_size"] = self._workspace_bytes(symbol, inputs)
        self.instructions.append(("Opr", fields))
        self._nr_opr += 1

    def _workspace_bytes(self, symbol, inputs):
        """what the kernel's _workspace function answers for these operands (shapes, dtypes and
        scales only: no tensor memory is touched)"""
        import ctypes as C

        from . import abi, runtime
        tensors = []
        for t in inputs:
            info = self.weights[t] if isinstance(t, _WeightId) else self.tensors[t]
            kind, scale = info["dtype"]
            tensors.append(abi.make_tensor(None, info["dims"], kind, scale if scale is not None else 1.0,
                                           info["name"].encode(), info.get("stride")))
        size = C.c_size_t(0)
        desc = runtime.parse_symbol(symbol)
        runtime.check(runtime.lib().megcc_gfx950_call_workspace(
            C.byref(desc), abi.tensor_array(tensors), len(tensors), 1, C.byref(size)), "workspace of " + symbol)
        return size.value

    def mark_input(self, t):
        self.inputs.append(t)

    def mark_output(self, t):
        if t not in self.outputs:
            self.outputs.append(t)

    def finalize(self):
        pass

    def to_dict(self):
        from . import runtime
        planned = [t for t in range(len(self.tensors))
                   if self._root[t] < 0 and self._first[t] >= 0 and t not in self.inputs]
        outs = {self._root_of(t) for t in self.outputs}
        begin = [self._first[t] for t in planned]
        end = [self._nr_opr + 1 if t in outs else self._last[t] + 1 for t in planned]
        size = []
        for t in planned:
            info = self.tensors[t]
            size.append(int(np.prod(info["dims"])) * _ITEMSIZE[info["dtype"][0]])
        # workspaces: alive for the one step of their Opr
        with_ws = [(k, f) for k, f in enumerate(f for kind, f in self.instructions if kind == "Opr")
                   if f.get("workspace_size", 0) > 0]
        for k, f in with_ws:
            begin.append(k)
            end.append(k + 1)
            size.append(f["workspace_size"])
        offsets, arena, _ = runtime.plan_memory(begin, end, size, self.alignment)
        for t, off in zip(planned, offsets):
            self.tensors[t]["offset"] = int(off)
        for (k, f), off in zip(with_ws, offsets[len(planned):]):
            f["workspace_offset"] = int(off)
        for t in range(len(self.tensors)):  # views report their root's offset
            if self._root[t] >= 0:
                self.tensors[t]["offset"] = self.tensors[self._root_of(t)]["offset"]
        return dict(name=self.name, model_id=0, const_shape=True, weights=self.weights,
                    device_models=[dict(device=self.device, tensor_memory=arena,
                                        tensors=self.tensors, instructions=self.instructions,
                                        inputs=self.inputs, outputs=self.outputs)])

    def to_bytes(self):
        return write_model(self.to_dict())
