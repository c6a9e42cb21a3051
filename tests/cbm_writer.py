"""Writer of the CatBoost binary model format (.cbm) for test models, in plain Python.

TEST INFRASTRUCTURE ONLY: it turns the dict that oracle/cbm_reader.read_cbm returns (and that
oracle.OracleModel takes) back into bytes, so that synthetic models, CTR features and value tables
included, reach the shipped library through its own file reader and the oracle without passing through
any product code. Format: catboost/libs/model/model.cpp:1113-1228 (b"CBM1", core size, flatbuffer
TModelCore, model parts), schemas catboost/libs/model/flatbuffers/{model,features,ctr_data}.fbs; the
static CTR provider part is TCtrData::Save (catboost/libs/model/ctr_data.cpp:12-22).

The flatbuffer is laid out front to back: a table first, the things it points to after it (offsets in
a flatbuffer are unsigned and forward, the offset to a vtable is signed).
"""
import struct

import numpy as np

FORMAT_STRING = "FlabuffersModel_v1"  # sic, model.cpp:53


class _Out:
    def __init__(self):
        self.b = bytearray()

    def align(self, n, ahead=0):
        while (len(self.b) + ahead) % n:
            self.b.append(0)

    def patch(self, at, target):
        struct.pack_into("<I", self.b, at, target - at)

    # ---- children: each returns the position its parent points at
    def string(self, s):
        raw = s.encode("utf-8") if isinstance(s, str) else bytes(s)
        self.align(4)
        pos = len(self.b)
        self.b += struct.pack("<I", len(raw)) + raw + b"\0"
        return pos

    def vector(self, values, dtype, align=None):
        a = np.ascontiguousarray(values, dtype=dtype)
        align = max(4, align or a.dtype.itemsize)
        self.align(align, ahead=4)
        pos = len(self.b)
        self.b += struct.pack("<I", a.size) + a.tobytes()
        return pos

    def struct_vector(self, raw, count):
        self.align(4)
        pos = len(self.b)
        self.b += struct.pack("<I", count) + bytes(raw)
        return pos

    def offsets(self, emitters):
        """Vector of offsets to tables or strings; `emitters` write the elements afterwards."""
        self.align(4)
        pos = len(self.b)
        self.b += struct.pack("<I", len(emitters)) + b"\0" * (4 * len(emitters))
        for i, emit in enumerate(emitters):
            self.patch(pos + 4 + 4 * i, emit())
        return pos

    def table(self, fields):
        """fields: {slot: ("b"|"B"|"i"|"f"|"d", value)} for scalars, {slot: callable} for children."""
        slots = max(fields) + 1 if fields else 0
        layout, size = {}, 4
        for slot in sorted(fields):
            f = fields[slot]
            width = 4 if callable(f) else struct.calcsize("<" + f[0])
            size = (size + width - 1) // width * width
            layout[slot] = size
            size += width
        self.align(2)
        vt = len(self.b)
        self.b += struct.pack("<HH", 4 + 2 * slots, size)
        for slot in range(slots):
            self.b += struct.pack("<H", layout.get(slot, 0))
        self.align(8)
        pos = len(self.b)
        self.b += b"\0" * size
        struct.pack_into("<i", self.b, pos, pos - vt)
        for slot, f in fields.items():
            if not callable(f):
                struct.pack_into("<" + f[0], self.b, pos + layout[slot], f[1])
        for slot in sorted(fields):
            f = fields[slot]
            if callable(f):
                self.patch(pos + layout[slot], f())
        return pos


def _finish(root_emitter):
    out = _Out()
    out.b += b"\0" * 8  # root offset, padding that keeps 8-byte alignment for what follows
    out.patch(0, root_emitter(out))
    return bytes(out.b)


def _ctr_base(out, base):
    def projection():
        fields = {0: lambda: out.vector(base["cat_features"], np.int32)}
        if len(base["float_splits"]):
            raw = b"".join(struct.pack("<if", int(f), float(b)) for f, b in base["float_splits"])
            fields[1] = lambda raw=raw: out.struct_vector(raw, len(base["float_splits"]))
        if len(base["one_hot_splits"]):
            raw = b"".join(struct.pack("<ii", int(f), int(v)) for f, v in base["one_hot_splits"])
            fields[2] = lambda raw=raw: out.struct_vector(raw, len(base["one_hot_splits"]))
        return out.table(fields)

    return out.table({0: projection, 1: ("b", int(base["ctr_type"])),
                      2: ("i", int(base["target_border_classifier_idx"]))})


def _strings(out, items):
    return out.offsets([(lambda s=s: out.string(s)) for s in items])


def _model_core(out, model):
    def cat_feature(c):
        return out.table({0: ("i", c["index"]), 1: ("i", c["flat_index"]),
                          2: lambda: out.string(c.get("feature_id", "")), 3: ("B", 1 if c.get("used", True) else 0)})

    def float_feature(f):
        return out.table({0: ("B", 1 if f.get("has_nans") else 0), 1: ("i", f["index"]), 2: ("i", f["flat_index"]),
                          3: lambda: out.vector(f["borders"], np.float32),
                          4: lambda: out.string(f.get("feature_id", "")), 5: ("b", int(f.get("nan_treatment", 0)))})

    def one_hot_feature(o):
        return out.table({0: ("i", o["cat_index"]), 1: lambda: out.vector(o["values"], np.int32),
                          2: lambda: _strings(out, o.get("string_values", []))})

    def ctr_feature(c):
        def model_ctr():
            return out.table({0: lambda: _ctr_base(out, c["base"]), 1: ("i", int(c["target_border_idx"])),
                              2: ("f", float(c["prior_num"])), 3: ("f", float(c["prior_denom"])),
                              4: ("f", float(c["shift"])), 5: ("f", float(c["scale"]))})

        return out.table({0: model_ctr, 1: lambda: out.vector(c["borders"], np.float32)})

    def tables_of(items, emit):
        return lambda: out.offsets([(lambda x=x: emit(x)) for x in items])

    def trees():
        bias = np.asarray(model["bias"], np.float64)
        fields = {
            0: ("i", int(model["approx_dimension"])),
            1: lambda: out.vector(model["tree_splits"], np.int32),
            2: lambda: out.vector(model["tree_sizes"], np.int32),
            3: lambda: out.vector(model["tree_start_offsets"], np.int32),
            4: tables_of(model.get("cat_features", []), cat_feature),
            5: tables_of(model.get("float_features", []), float_feature),
            6: tables_of(model.get("one_hot_features", []), one_hot_feature),
            7: tables_of(model.get("ctr_features", []), ctr_feature),
            8: lambda: out.vector(model["leaf_values"], np.float64),
            9: lambda: out.vector(model.get("leaf_weights", []), np.float64),
            14: ("d", float(model.get("scale", 1.0))),
            16: lambda: out.vector(bias, np.float64),
        }
        if len(model.get("step_nodes", [])):
            nodes = np.ascontiguousarray(model["step_nodes"], np.uint16)
            fields[10] = lambda: out.struct_vector(nodes.tobytes(), nodes.shape[0])
            fields[11] = lambda: out.vector(model["node_id_to_leaf_id"], np.uint32)
        return out.table(fields)

    def key_value(k, v):
        return out.table({0: lambda: out.string(k), 1: lambda: out.string(v)})

    info = sorted(model.get("info", {}).items())
    parts = ["static_provider_v1"] if model.get("ctr_tables") else []
    return out.table({0: lambda: out.string(FORMAT_STRING), 1: trees,
                      2: lambda: out.offsets([(lambda kv=kv: key_value(*kv)) for kv in info]),
                      3: lambda: _strings(out, parts)})


def _save_size(n):
    """SaveSize, util/ysaveload.h:262-275."""
    return struct.pack("<I", n) if n < 0xFFFFFFFF else struct.pack("<IQ", 0xFFFFFFFF, n)


def _ctr_value_table(table):
    def root(out):
        return out.table({0: lambda: _ctr_base(out, table["base"]),
                          1: lambda: out.vector(table["index_hash_raw"], np.uint8, align=8),
                          2: lambda: out.vector(table["ctr_blob"], np.uint8, align=8),
                          3: ("i", int(table["counter_denominator"])), 4: ("i", int(table["target_classes_count"]))})

    return _finish(root)


def write_cbm(model):
    """Bytes of a .cbm file for `model` (keys as oracle/cbm_reader.read_cbm returns them)."""
    core = _finish(lambda out: _model_core(out, model))
    data = b"CBM1" + _save_size(len(core)) + core
    tables = model.get("ctr_tables", [])
    if tables:
        data += _save_size(len(tables))
        for t in tables:
            raw = _ctr_value_table(t)
            data += _save_size(len(raw)) + raw
    return data
