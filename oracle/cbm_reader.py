"""Independent reader of the CatBoost binary model format (.cbm) for the CPU oracle.

TEST INFRASTRUCTURE ONLY: the shipped library has its own C++ reader; this one exists so that the
oracle sees a model through code that shares nothing with the product.

Format (catboost/libs/model/model.cpp:41-53, 1179-1228): b"CBM1", core size as ui32 (0xffffffff
followed by ui64 for big cores, util/ysaveload.h:277-296), a flatbuffer with root TModelCore
(catboost/libs/model/flatbuffers/model.fbs:48-54), then optional trailing model parts. The schemas
carry no explicit field ids, so the vtable slot of a field is its declaration order.
"""
import struct

import numpy as np

FORMAT_STRING = "FlabuffersModel_v1"  # sic, model.cpp:53


class _Table:
    def __init__(self, buf, pos):
        self.buf = buf
        self.pos = pos
        (soff,) = struct.unpack_from("<i", buf, pos)
        self.vt = pos - soff
        (self.vt_size,) = struct.unpack_from("<H", buf, self.vt)

    def _field(self, slot):
        off = 4 + 2 * slot
        if off >= self.vt_size:
            return 0
        (f,) = struct.unpack_from("<H", self.buf, self.vt + off)
        return f

    def scalar(self, slot, fmt, default):
        f = self._field(slot)
        if not f:
            return default
        return struct.unpack_from("<" + fmt, self.buf, self.pos + f)[0]

    def _indirect(self, slot):
        f = self._field(slot)
        if not f:
            return None
        loc = self.pos + f
        (rel,) = struct.unpack_from("<I", self.buf, loc)
        return loc + rel

    def string(self, slot):
        p = self._indirect(slot)
        if p is None:
            return None
        (n,) = struct.unpack_from("<I", self.buf, p)
        return bytes(self.buf[p + 4:p + 4 + n]).decode("utf-8", errors="replace")

    def table(self, slot):
        p = self._indirect(slot)
        return None if p is None else _Table(self.buf, p)

    def vector(self, slot, dtype, per_element=1):
        """Vector of scalars, or of structs made of `per_element` scalars of `dtype`."""
        p = self._indirect(slot)
        if p is None:
            return np.zeros(0, dtype=dtype)
        (n,) = struct.unpack_from("<I", self.buf, p)
        return np.frombuffer(self.buf, dtype=dtype, count=n * per_element, offset=p + 4).copy()

    def vector_len(self, slot):
        p = self._indirect(slot)
        if p is None:
            return 0
        return struct.unpack_from("<I", self.buf, p)[0]

    def tables(self, slot):
        p = self._indirect(slot)
        if p is None:
            return []
        (n,) = struct.unpack_from("<I", self.buf, p)
        out = []
        for i in range(n):
            loc = p + 4 + 4 * i
            (rel,) = struct.unpack_from("<I", self.buf, loc)
            out.append(_Table(self.buf, loc + rel))
        return out

    def strings(self, slot):
        p = self._indirect(slot)
        if p is None:
            return []
        (n,) = struct.unpack_from("<I", self.buf, p)
        out = []
        for i in range(n):
            loc = p + 4 + 4 * i
            (rel,) = struct.unpack_from("<I", self.buf, loc)
            q = loc + rel
            (m,) = struct.unpack_from("<I", self.buf, q)
            out.append(bytes(self.buf[q + 4:q + 4 + m]).decode("utf-8", errors="replace"))
        return out


def _read_ctr_base(t):
    """TModelCtrBase (ctr_data.fbs:15-19) with its TFeatureCombination (features.fbs:71-75)."""
    base = {"cat_features": np.zeros(0, np.int32), "float_splits": [], "one_hot_splits": [],
            "ctr_type": 0, "target_border_classifier_idx": 0}
    if t is None:
        return base
    proj = t.table(0)
    if proj is not None:
        base["cat_features"] = proj.vector(0, np.int32)
        raw = proj.vector(1, np.uint32, per_element=2).reshape(-1, 2)
        base["float_splits"] = [(int(np.int32(r[0])), np.array([r[1]], np.uint32).view(np.float32)[0]) for r in raw]
        raw = proj.vector(2, np.int32, per_element=2).reshape(-1, 2)
        base["one_hot_splits"] = [(int(r[0]), int(r[1])) for r in raw]
    base["ctr_type"] = t.scalar(1, "b", 0)
    base["target_border_classifier_idx"] = t.scalar(2, "i", 0)
    return base


def ctr_base_key(base):
    """Hashable identity of a TModelCtrBase (its operator==, online_ctr.h:182-186)."""
    return (tuple(int(c) for c in base["cat_features"]),
            tuple((f, np.float32(b).tobytes()) for f, b in base["float_splits"]),
            tuple(base["one_hot_splits"]), int(base["ctr_type"]), int(base["target_border_classifier_idx"]))


def _read_size(data, pos):
    """LoadSize, util/ysaveload.h:277-296."""
    (n,) = struct.unpack_from("<I", data, pos)
    pos += 4
    if n == 0xFFFFFFFF:
        (n,) = struct.unpack_from("<Q", data, pos)
        pos += 8
    return n, pos


def _read_static_ctr_provider(data, pos):
    """TCtrData::Load (ctr_data.cpp:24-34): count, then (size, flatbuffer TCtrValueTable) per table."""
    count, pos = _read_size(data, pos)
    tables = []
    for _ in range(count):
        n, pos = _read_size(data, pos)
        buf = data[pos:pos + n]
        pos += n
        (root,) = struct.unpack_from("<I", buf, 0)
        t = _Table(buf, root)
        tables.append({"base": _read_ctr_base(t.table(0)), "index_hash_raw": t.vector(1, np.uint8),
                       "ctr_blob": t.vector(2, np.uint8), "counter_denominator": t.scalar(3, "i", 0),
                       "target_classes_count": t.scalar(4, "i", 0)})
    return tables, pos


def read_cbm(data):
    """Parses .cbm bytes into a dict of numpy arrays (keys follow the flatbuffer field names)."""
    data = memoryview(bytes(data))
    if len(data) < 8 or bytes(data[:4]) != b"CBM1":
        raise ValueError("Incorrect model file descriptor")
    (size,) = struct.unpack_from("<I", data, 4)
    pos = 8
    if size == 0xFFFFFFFF:
        (size,) = struct.unpack_from("<Q", data, 8)
        pos = 16
    if pos + size > len(data):
        raise ValueError("truncated model core")
    core = data[pos:pos + size]
    (root,) = struct.unpack_from("<I", core, 0)
    mc = _Table(core, root)
    fmt = mc.string(0)
    if fmt != FORMAT_STRING:
        raise ValueError("Unsupported model format: %r" % (fmt,))
    info = {}
    for kv in mc.tables(2):
        info[kv.string(0)] = kv.string(1)
    parts = mc.strings(3)
    t = mc.table(1)
    model = {"info": info, "model_part_ids": parts}
    if t is None:
        raise ValueError("model has no trees table")
    dim = t.scalar(0, "i", 0)
    model["approx_dimension"] = dim
    model["tree_splits"] = t.vector(1, np.int32)
    model["tree_sizes"] = t.vector(2, np.int32)
    model["tree_start_offsets"] = t.vector(3, np.int32)
    cats = []
    for c in t.tables(4):
        cats.append({"index": c.scalar(0, "i", -1), "flat_index": c.scalar(1, "i", -1),
                     "feature_id": c.string(2) or "", "used": bool(c.scalar(3, "B", 1))})
    floats = []
    for f in t.tables(5):
        floats.append({"has_nans": bool(f.scalar(0, "B", 0)), "index": f.scalar(1, "i", -1),
                       "flat_index": f.scalar(2, "i", -1), "borders": f.vector(3, np.float32),
                       "feature_id": f.string(4) or "", "nan_treatment": f.scalar(5, "b", 0)})
    onehots = []
    for o in t.tables(6):
        onehots.append({"cat_index": o.scalar(0, "i", -1), "values": o.vector(1, np.int32),
                        "string_values": o.strings(2)})
    model["cat_features"] = cats
    model["float_features"] = floats
    model["one_hot_features"] = onehots
    model["ctr_feature_count"] = t.vector_len(7)
    ctrs = []
    for c in t.tables(7):  # TCtrFeature / TModelCtr, ctr_data.fbs:21-33
        mc_ctr = c.table(0)
        ctrs.append({"base": _read_ctr_base(mc_ctr.table(0)), "target_border_idx": mc_ctr.scalar(1, "i", 0),
                     "prior_num": mc_ctr.scalar(2, "f", 0.0), "prior_denom": mc_ctr.scalar(3, "f", 1.0),
                     "shift": mc_ctr.scalar(4, "f", 0.0), "scale": mc_ctr.scalar(5, "f", 1.0),
                     "borders": c.vector(1, np.float32)})
    model["ctr_features"] = ctrs
    model["leaf_values"] = t.vector(8, np.float64)
    model["leaf_weights"] = t.vector(9, np.float64)
    model["step_nodes"] = t.vector(10, np.uint16, per_element=2).reshape(-1, 2)
    model["node_id_to_leaf_id"] = t.vector(11, np.uint32)
    model["text_feature_count"] = t.vector_len(12)
    model["estimated_feature_count"] = t.vector_len(13)
    model["scale"] = t.scalar(14, "d", 1.0)
    bias = t.scalar(15, "d", 0.0)
    multi_bias = t.vector(16, np.float64)
    # TModelTrees::SetScaleAndBias, model.cpp:711-722
    if multi_bias.size:
        model["bias"] = multi_bias
    else:
        if not (dim == 1 or bias == 0):
            raise ValueError("Inappropriate dimension of bias")
        model["bias"] = np.full(dim, bias, dtype=np.float64)
    model["repacked_bins_in_file"] = t.vector(17, np.uint32)
    model["embedding_feature_count"] = t.vector_len(18)
    # trailing model parts, model.cpp:1201-1226; only the static CTR provider is read
    model["ctr_tables"] = []
    part_pos = pos + size
    for part in parts:
        if part != "static_provider_v1":
            break
        tables, part_pos = _read_static_ctr_provider(data, part_pos)
        model["ctr_tables"] = tables
    return model


def read_cbm_file(path):
    with open(path, "rb") as f:
        return read_cbm(f.read())
