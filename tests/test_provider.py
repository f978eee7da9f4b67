"""The backend provider (volvoxai_amd/provider) driven through a test double of the
runtime side of the reference's provider SPI (tests/provider_host/mock_host.c).

Without a GPU: registration, package reading and every refusal.  With a GPU: whole
packages from graph.json + SafeTensors to output bytes, against the literal KAT of
tests/parity/external/quantized_oracle.py:34-41,89-103 and against the oracle.
"""
import ctypes as C
import json
import struct
from pathlib import Path

import numpy as np
import pytest

import _cases as cases

I8, U8 = cases.DTYPE_I8, cases.DTYPE_U8

ROOT = Path(__file__).resolve().parent.parent
PROVIDER = ROOT / "volvoxai_amd" / "lib" / "libvxhip_provider.so"
MOCK = ROOT / "tests" / "provider_host" / "libvx_mock_host.so"

pytestmark = pytest.mark.skipif(not (PROVIDER.exists() and MOCK.exists()),
                                reason="provider and mock host are built where the reference's headers are present")

DT = {"u8": 5, "i8": 6, "i32": 16, "f32": 18}
ARITH = {"dynamic_i8": 1, "f16": 2, "f32": 3, "f32_fast": 4, "dynamic_i4": 5}
ST = {-1: "INVALID_ARGUMENT", -4: "IO_ERROR", -5: "INVALID_GRAPH", -6: "BACKEND_UNAVAILABLE", -7: "BACKEND_UNSUPPORTED"}


class MockRun(C.Structure):
    _fields_ = [("graph_path", C.c_char_p), ("weight_path", C.c_char_p), ("packed_arithmetic", C.c_int32),
                ("input_name", C.c_char_p), ("input_dtype", C.c_int32), ("rank", C.c_uint32),
                ("input_shape", C.c_int64 * 8), ("lead_max", C.c_int64 * 8), ("input", C.c_void_p),
                ("input_bytes", C.c_uint64), ("output_name", C.c_char_p), ("output_dtype", C.c_int32),
                ("output_last", C.c_int64), ("output", C.c_void_p), ("output_capacity", C.c_uint64),
                ("executions", C.c_int32),
                ("status", C.c_int32), ("failed_stage", C.c_int32), ("output_bytes", C.c_uint64),
                ("writes", C.c_int32), ("sink_mismatch", C.c_int32), ("compile_attested", C.c_int32),
                ("execute_attested", C.c_int32), ("identities_echoed", C.c_int32),
                ("attested_arithmetic", C.c_int32), ("maximum_tensor_bytes", C.c_uint64),
                ("maximum_resident_bytes", C.c_uint64), ("message", C.c_char * 256),
                ("compile_route", C.c_char * 512), ("execute_route", C.c_char * 512), ("device", C.c_char * 128)]


class ModelSource(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("graph_path", C.c_char_p), ("weight_paths", C.POINTER(C.c_char_p)),
                ("weight_path_count", C.c_size_t), ("bank_residency", C.c_void_p), ("bank_residency_count", C.c_size_t)]


@pytest.fixture(scope="module")
def host():
    import volvoxai_amd as vx
    vx.library()  # brings in the HIP runtime in the right order
    mock = C.CDLL(str(MOCK), mode=C.RTLD_GLOBAL)
    provider = C.CDLL(str(PROVIDER))
    mock.mock_host_registered_name.restype = C.c_char_p
    mock.mock_host_run.argtypes = [C.POINTER(MockRun)]
    provider.volvoxai_hip_gfx950_inspect_package.argtypes = [
        C.POINTER(ModelSource), C.c_int32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_int32),
        C.c_char_p, C.c_size_t]
    return mock, provider, None


def write_safetensors(path, tensors):
    names = {np.dtype(np.int8): "I8", np.dtype(np.uint8): "U8", np.dtype(np.int32): "I32",
             np.dtype(np.uint32): "U32", np.dtype(np.float32): "F32"}
    header, blobs, offset = {}, [], 0
    for name, arr in tensors.items():
        if name == "__metadata__":  # free-form strings beside the tensors
            header[name] = dict(arr)
            continue
        arr = np.ascontiguousarray(arr)
        dtype = names[arr.dtype]
        if name.endswith("#as_i32"):  # packed words are stored as I32
            name, dtype = name[:-7], "I32"
        raw = arr.tobytes()
        header[name] = {"dtype": dtype, "shape": list(arr.shape), "data_offsets": [offset, offset + len(raw)]}
        blobs.append(raw)
        offset += len(raw)
    text = json.dumps(header, separators=(",", ":")).encode()
    text += b" " * (-len(text) % 8)
    Path(path).write_bytes(struct.pack("<Q", len(text)) + text + b"".join(blobs))


def qlinear_package(tmp, x_shape, w, scales, zps, bias, s_in, zp_in, s_out, zp_out, in_dtype="int8", out_dtype="int8",
                    mutate=None, op="QLinear", rows_symbol=False):
    d_out, d_in = w.shape
    np_of = {"int8": np.int8, "uint8": np.uint8}
    graph = {
        "format": "volvox-graph/v1", "dimensions": {},
        "inputs": {"hidden_q": {"shape": list(x_shape), "dtype": in_dtype}},
        "nodes": [{"id": "projection", "opType": op,
                   "inputs": {"input": "hidden_q", "weight": "projection.weight", "bias": "projection.bias"},
                   "outputs": {"out": {"tensor": "projected_q", "shape": list(x_shape[:-1]) + [d_out], "dtype": out_dtype}},
                   "params": {}}],
        "outputs": ["projected_q"],
        "quantization": {"format": "volvox-affine-safetensors/v1", "tensors": {
            "hidden_q": {"scheme": "per_tensor", "scale_tensor": "__quant__.hidden.scale",
                         "zero_point_tensor": "__quant__.hidden.zero_point"},
            "projection.weight": {"scheme": "per_axis", "axis": 0, "scale_tensor": "__quant__.projection.weight.scale",
                                  "zero_point_tensor": "__quant__.projection.weight.zero_point"},
            "projected_q": {"scheme": "per_tensor", "scale_tensor": "__quant__.projected.scale",
                            "zero_point_tensor": "__quant__.projected.zero_point"}}},
        "execution": {"stateless": {}, "entrypoints": [{"name": "evaluate", "effect": 1, "allowed_ranges": [1],
                                                         "inputs": ["hidden_q"], "outputs": ["projected_q"]}]}}
    tensors = {
        "projection.weight": w, "projection.bias": np.asarray(bias, np.int32),
        "__quant__.hidden.scale": np.array([s_in], np.float32),
        "__quant__.hidden.zero_point": np.array([zp_in], np_of[in_dtype]),
        "__quant__.projection.weight.scale": np.asarray(scales, np.float32),
        "__quant__.projection.weight.zero_point": np.asarray(zps).astype(w.dtype),
        "__quant__.projected.scale": np.array([s_out], np.float32),
        "__quant__.projected.zero_point": np.array([zp_out], np_of[out_dtype])}
    if rows_symbol:
        graph["dimensions"] = {"rows": {"min": 1, "max": 64}}
        graph["inputs"]["hidden_q"]["shape"][0] = "rows"
        graph["nodes"][0]["outputs"]["out"]["shape"][0] = "rows"
    if mutate:
        mutate(graph, tensors)
    tmp.mkdir(parents=True, exist_ok=True)
    (tmp / "graph.json").write_text(json.dumps(graph, separators=(",", ":")) + "\n")
    write_safetensors(tmp / "model.safetensors", tensors)
    return tmp / "graph.json", tmp / "model.safetensors"


def packed_package(tmp, x_shape, words, scales, bias, group, bits=8, mutate=None):
    n = words.shape[0]
    graph = {
        "format": "volvox-graph/v1", "dimensions": {},
        "inputs": {"x": {"shape": list(x_shape), "dtype": "float32"}},
        "nodes": [{"id": "packed", "opType": "PackedLinear",
                   "inputs": {"input": "x", "weight": "w", "scale": "s", "bias": "b"},
                   "outputs": {"out": {"tensor": "logits", "shape": list(x_shape[:-1]) + [n], "dtype": "float32"}},
                   "params": {"group_size": group, "weight_bits": bits}}],
        "outputs": ["logits"],
        "execution": {"stateless": {}, "entrypoints": [{"name": "evaluate", "effect": 1, "allowed_ranges": [1],
                                                         "inputs": ["x"], "outputs": ["logits"]}]}}
    tensors = {"w#as_i32": words.astype(np.uint32), "s": scales.astype(np.float32), "b": bias.astype(np.float32)}
    if mutate:
        mutate(graph, tensors)
    tmp.mkdir(parents=True, exist_ok=True)
    (tmp / "graph.json").write_text(json.dumps(graph, separators=(",", ":")))
    write_safetensors(tmp / "model.safetensors", tensors)
    return tmp / "graph.json", tmp / "model.safetensors"


def chain_package(tmp, x_shape, in_name, in_dtype, nodes, tensors, affine):
    """A graph whose nodes form a chain.  nodes: (id, opType, extra inputs, output tensor, d_out, dtype,
    params); affine: byte tensor or weight name -> (scale tensor, zero-point tensor[, axis])."""
    lead = list(x_shape[:-1])
    graph_nodes, current = [], in_name
    for node_id, op, extra, out_name, d_out, dtype, params in nodes:
        graph_nodes.append({"id": node_id, "opType": op, "inputs": dict({"input": current}, **extra),
                            "outputs": {"out": {"tensor": out_name, "shape": lead + [d_out], "dtype": dtype}},
                            "params": params})
        current = out_name
    table = {}
    for name, ref in affine.items():
        table[name] = {"scheme": "per_tensor", "scale_tensor": ref[0], "zero_point_tensor": ref[1]}
        if len(ref) == 3:
            table[name].update(scheme="per_axis", axis=ref[2])
    graph = {"format": "volvox-graph/v1", "dimensions": {},
             "inputs": {in_name: {"shape": list(x_shape), "dtype": in_dtype}},
             "nodes": graph_nodes, "outputs": [current],
             "execution": {"stateless": {}, "entrypoints": [{"name": "evaluate", "effect": 1, "allowed_ranges": [1],
                                                             "inputs": [in_name], "outputs": [current]}]}}
    if table:
        graph["quantization"] = {"format": "volvox-affine-safetensors/v1", "tensors": table}
    tmp.mkdir(parents=True, exist_ok=True)
    (tmp / "graph.json").write_text(json.dumps(graph, separators=(",", ":")))
    write_safetensors(tmp / "model.safetensors", tensors)
    return tmp / "graph.json", tmp / "model.safetensors"


def sandwich(tmp, x_shape, c1, c2=None, mutate=None):
    """QuantizeLinear -> QLinear [-> QLinear] -> DequantizeLinear over f32 rows; c1/c2 are
    cases.qlinear_random_case dictionaries (int8 throughout, c2 reads what c1 writes)."""
    tensors = {"in.s": np.array([c1["s_in"]], np.float32), "in.z": np.array([c1["zp_in"]], np.int8),
               "w1": c1["w"], "w1.s": c1["scales"], "w1.z": c1["zps"].astype(np.int8), "b1": c1["bias"],
               "h.s": np.array([c1["s_out"]], np.float32), "h.z": np.array([c1["zp_out"]], np.int8)}
    affine = {"xq": ("in.s", "in.z"), "w1": ("w1.s", "w1.z", 0), "hq": ("h.s", "h.z")}
    nodes = [("q", "QuantizeLinear", {"scale": "in.s", "zero_point": "in.z"}, "xq", c1["w"].shape[1], "int8", {}),
             ("fc1", "QLinear", {"weight": "w1", "bias": "b1"}, "hq", c1["w"].shape[0], "int8", {})]
    last, last_d, last_affine = "hq", c1["w"].shape[0], ("h.s", "h.z")
    if c2 is not None:
        tensors.update({"w2": c2["w"], "w2.s": c2["scales"], "w2.z": c2["zps"].astype(np.int8), "b2": c2["bias"],
                        "y.s": np.array([c2["s_out"]], np.float32), "y.z": np.array([c2["zp_out"]], np.int8)})
        affine.update({"w2": ("w2.s", "w2.z", 0), "yq": ("y.s", "y.z")})
        nodes.append(("fc2", "QGemm", {"weight": "w2", "bias": "b2"}, "yq", c2["w"].shape[0], "int8", {}))
        last, last_d, last_affine = "yq", c2["w"].shape[0], ("y.s", "y.z")
    nodes.append(("dq", "DequantizeLinear", {"scale": last_affine[0], "zero_point": last_affine[1]}, "y", last_d,
                  "float32", {}))
    if mutate:
        mutate(nodes, tensors, affine)
    return chain_package(tmp, x_shape, "x", "float32", nodes, tensors, affine), last_d


def inspect(host, graph, weights, arithmetic="f32"):
    """weights: one SafeTensors path, or a list of them (a sharded package)."""
    _, provider, _ = host
    files = list(weights) if isinstance(weights, (list, tuple)) else [weights]
    paths = (C.c_char_p * len(files))(*[str(f).encode() for f in files])
    src = ModelSource(C.sizeof(ModelSource), str(graph).encode(), paths, len(files), None, 0)
    d_in, d_out, packed = C.c_uint32(0), C.c_uint32(0), C.c_int32(0)
    msg = C.create_string_buffer(256)
    st = provider.volvoxai_hip_gfx950_inspect_package(C.byref(src), ARITH[arithmetic], C.byref(d_in), C.byref(d_out),
                                                      C.byref(packed), msg, 256)
    return st, d_in.value, d_out.value, packed.value, msg.value.decode()


def run(host, graph, weights, x, in_name, in_dtype, out_name, out_dtype, d_out, arithmetic="f32", lead_max=None,
        executions=1, threads=0, batch_proof=None):
    mock, _, _ = host
    x = np.ascontiguousarray(x)
    out_np = {"i8": np.int8, "u8": np.uint8, "f32": np.float32}[out_dtype]
    y = np.zeros(x.shape[:-1] + (d_out,), out_np)
    r = MockRun()
    r.graph_path, r.weight_path = str(graph).encode(), str(weights).encode()
    r.packed_arithmetic = ARITH[arithmetic]
    r.input_name, r.input_dtype, r.rank = in_name.encode(), DT[in_dtype], x.ndim
    for i, e in enumerate(x.shape):
        r.input_shape[i] = e
    for i, e in enumerate(lead_max or []):
        r.lead_max[i] = e
    r.input, r.input_bytes = x.ctypes.data, x.nbytes
    r.output_name, r.output_dtype, r.output_last = out_name.encode(), DT[out_dtype], d_out
    r.output, r.output_capacity, r.executions = y.ctypes.data, y.nbytes, executions
    if batch_proof is not None:
        mock.mock_host_run_batch.argtypes = [C.POINTER(MockRun), C.c_int32]
        mock.mock_host_run_batch(C.byref(r), 1 if batch_proof else 0)
    elif threads:
        mock.mock_host_run_concurrent.argtypes = [C.POINTER(MockRun), C.c_int32]
        mock.mock_host_run_concurrent(C.byref(r), threads)
    else:
        mock.mock_host_run(C.byref(r))
    return r, y


@pytest.fixture(scope="module")
def registered(host):
    mock, provider, _ = host
    if not mock.mock_host_registered_name():
        register = C.cast(provider.volvoxai_hip_gfx950_backend_register, C.c_void_p)
        mock.mock_host_register.argtypes = [C.c_void_p]
        assert mock.mock_host_register(register) == 0, "registration was refused"
        assert mock.mock_host_register(register) == -1, "a second registration under the same name must be refused"
    return host


KAT = dict(x=np.array([[-1, -1, -1], [-3, -3, -3]], np.int8),
           w=np.array([[2, 1, 1], [-3, -2, -3], [127] * 3, [-128] * 3], np.int8),
           zps=[1, -3, 2, -1], scales=[.5, .5, 1, 1], bias=[0, 0, 0, 0], s_in=1.0, zp_in=-2, s_out=1.0, zp_out=3,
           want=np.array([[4, 4, 127, -128], [2, 2, -128, 127]], np.int8))


# ---- no GPU needed ---------------------------------------------------------------------------------

def test_registration_passes_the_descriptor_checks(registered):
    mock, _, _ = registered
    assert mock.mock_host_registered_name() == b"hip-gfx950"
    assert mock.mock_host_shape_domain_support() == 1  # FULL


def test_reads_qlinear_and_packed_packages(registered, tmp_path):
    k = KAT
    g, w = qlinear_package(tmp_path / "q", k["x"].shape, k["w"], k["scales"], k["zps"], k["bias"], k["s_in"], k["zp_in"],
                           k["s_out"], k["zp_out"])
    assert inspect(registered, g, w)[:4] == (0, 3, 4, 0)
    for op in ("QGemm", "QMatMul"):
        g, w = qlinear_package(tmp_path / op, k["x"].shape, k["w"], k["scales"], k["zps"], k["bias"], k["s_in"],
                               k["zp_in"], k["s_out"], k["zp_out"], op=op)
        assert inspect(registered, g, w)[0] == 0
    c = cases.packed_case(3, 96, 5, 32, 1)
    from oracle.pyoracle import Oracle
    words = Oracle().pack_w8_words(c["w"])
    g, w = packed_package(tmp_path / "p", c["x"].shape, words, c["scales"], c["bias"], 32)
    assert inspect(registered, g, w, "dynamic_i8")[:4] == (0, 96, 5, 1)


def _drop(path):
    def f(graph, tensors):
        node = graph
        for key in path[:-1]:
            node = node[key]
        del node[path[-1]]
    return f


@pytest.mark.parametrize("name,mutate,status", [
    ("format", lambda g, t: g.__setitem__("format", "volvox-graph/v0"), -5),
    ("two writers of one tensor", lambda g, t: g["nodes"].append(dict(g["nodes"][0], id="again")), -5),
    ("other op", lambda g, t: g["nodes"][0].__setitem__("opType", "Linear"), -7),
    ("no table", _drop(["quantization"]), -5),
    ("table extra field", lambda g, t: g["quantization"].__setitem__("scales", [1.0]), -5),
    ("descriptor extra field", lambda g, t: g["quantization"]["tensors"]["hidden_q"].__setitem__("scale", 0.5), -5),
    ("missing zero point", _drop(["quantization", "tensors", "projected_q", "zero_point_tensor"]), -5),
    ("weight per_tensor", lambda g, t: g["quantization"]["tensors"]["projection.weight"].update(scheme="per_tensor"), -5),
    ("weight axis 1", lambda g, t: g["quantization"]["tensors"]["projection.weight"].update(axis=1), -7),
    ("negative axis spelling", lambda g, t: g["quantization"]["tensors"]["projection.weight"].update(axis=-2), 0),
    ("scale not positive", lambda g, t: t.__setitem__("__quant__.projected.scale", np.array([0.0], np.float32)), -5),
    ("scale nan", lambda g, t: t.__setitem__("__quant__.hidden.scale", np.array([np.nan], np.float32)), -5),
    ("zero point dtype", lambda g, t: t.__setitem__("__quant__.hidden.zero_point", np.array([0], np.uint8)), -5),
    ("scale count", lambda g, t: t.__setitem__("__quant__.projection.weight.scale", np.ones(3, np.float32)), -5),
    ("same tensor twice", lambda g, t: g["quantization"]["tensors"]["hidden_q"].update(
        zero_point_tensor="__quant__.hidden.scale"), -5),
    ("weight shape", lambda g, t: t.__setitem__("projection.weight", np.zeros((4, 5), np.int8)), -5),
    ("bias dtype", lambda g, t: t.__setitem__("projection.bias", np.zeros(4, np.float32)), -5),
    ("dangling weight", lambda g, t: t.pop("projection.weight"), -5),
    # representations the v1 format retired (docs/w8a8-safetensors.md:176-188, :100-102)
    ("retired graph field", lambda g, t: g.__setitem__("weights_quantization", {"projection.weight": "int8"}), -5),
    ("retired storage field", lambda g, t: g.__setitem__("weights_quantization_storage", "safetensors"), -5),
    ("inline input quantization", lambda g, t: g["inputs"]["hidden_q"].__setitem__("quantization", {"scale": 0.5}), -5),
    ("node outputs_quantization", lambda g, t: g["nodes"][0].__setitem__("outputs_quantization", {"out": {}}), -5),
    ("retired safetensors metadata", lambda g, t: t.__setitem__("__metadata__", {"weights_quantization": "int8"}), -5),
    ("unrelated safetensors metadata", lambda g, t: t.__setitem__("__metadata__", {"exported_by": "a test"}), 0),
])
def test_qlinear_package_refusals(registered, tmp_path, name, mutate, status):
    k = KAT
    g, w = qlinear_package(tmp_path / "q", k["x"].shape, k["w"], k["scales"], k["zps"], k["bias"], k["s_in"], k["zp_in"],
                           k["s_out"], k["zp_out"], mutate=mutate)
    st, *_, msg = inspect(registered, g, w)
    assert st == status, f"{name}: {ST.get(st, st)} {msg!r}"
    assert (st == 0) == (msg == "")


def test_packed_package_refusals(registered, tmp_path):
    from oracle.pyoracle import Oracle
    c = cases.packed_case(3, 96, 5, 32, 1)
    words = Oracle().pack_w8_words(c["w"])
    g, w = packed_package(tmp_path / "a", c["x"].shape, words, c["scales"], c["bias"], 32)
    for arithmetic in ("f32", "f16", "f32_fast", "dynamic_i4"):
        assert inspect(registered, g, w, arithmetic)[0] == -7  # only DYNAMIC_I8 is this arithmetic
    g, w = packed_package(tmp_path / "b", c["x"].shape, words, c["scales"], c["bias"], 32, bits=5)
    assert inspect(registered, g, w, "dynamic_i8")[0] == -7
    # four-bit weights are offered, with their own word count: W8 words under weight_bits 4 are malformed
    g, w = packed_package(tmp_path / "b4", c["x"].shape, words, c["scales"], c["bias"], 32, bits=4)
    assert inspect(registered, g, w, "dynamic_i8")[0] == -5
    w4 = Oracle().pack_w4_words(cases.four_bit(c["w"]))
    g, w = packed_package(tmp_path / "b4ok", c["x"].shape, w4, c["scales"], c["bias"], 32, bits=4)
    assert inspect(registered, g, w, "dynamic_i8")[:4] == (0, 96, 5, 1)
    g, w = packed_package(tmp_path / "c", c["x"].shape, words, c["scales"], c["bias"], 48)
    assert inspect(registered, g, w, "dynamic_i8")[0] == -5
    g, w = packed_package(tmp_path / "d", c["x"].shape, words[:, :-1], c["scales"], c["bias"], 32)
    assert inspect(registered, g, w, "dynamic_i8")[0] == -5
    g, w = packed_package(tmp_path / "e", c["x"].shape, words, c["scales"][:, :-1], c["bias"], 32)
    assert inspect(registered, g, w, "dynamic_i8")[0] == -5


def test_reads_node_chains(registered, tmp_path):
    c1 = cases.qlinear_random_case(4, 48, 24, 5, I8, I8, I8, False)
    c2 = cases.qlinear_random_case(4, 24, 10, 6, I8, I8, I8, False)
    c2["s_in"], c2["zp_in"] = c1["s_out"], c1["zp_out"]
    (g, w), d_out = sandwich(tmp_path / "ok", (4, 48), c1, c2)
    assert inspect(registered, g, w)[:4] == (0, 48, 10, 0)

    # a node may read any earlier tensor, but the weight it names must fit what it reads: the second
    # linear (24 inputs) on the quantized graph input (48 wide) is refused for its shapes
    (g, w), _ = sandwich(tmp_path / "dag", (4, 48), c1, c2)
    doc = json.loads(g.read_text())
    doc["nodes"][2]["inputs"]["input"] = "xq"
    g.write_text(json.dumps(doc))
    assert inspect(registered, g, w)[0] == -5
    # a node that reads a tensor nobody provides, or one a LATER node writes
    doc["nodes"][2]["inputs"]["input"] = "nowhere"
    g.write_text(json.dumps(doc))
    st, *_, msg = inspect(registered, g, w)
    assert st == -5 and "neither a graph input nor an earlier node" in msg
    doc["nodes"][2]["inputs"]["input"] = doc["nodes"][3]["outputs"]["out"]["tensor"]
    g.write_text(json.dumps(doc))
    assert inspect(registered, g, w)[0] == -5
    # a graph output no node writes
    (g, w), _ = sandwich(tmp_path / "out", (4, 48), c1, c2)
    doc = json.loads(g.read_text())
    doc["outputs"] = ["xq", "missing"]
    g.write_text(json.dumps(doc))
    st, *_, msg = inspect(registered, g, w)
    assert st == -5 and "missing" in msg

    def other_parameters(nodes, tensors, affine):  # the node and the table disagree about the input's scale
        tensors["in.s2"] = np.array([0.5], np.float32)
        nodes[0] = ("q", "QuantizeLinear", {"scale": "in.s2", "zero_point": "in.z"}, "xq", 48, "int8", {})
    (g, w), _ = sandwich(tmp_path / "bad", (4, 48), c1, mutate=other_parameters)
    assert inspect(registered, g, w)[0] == -5

    def widen(nodes, tensors, affine):  # a boundary node may not change the row length
        nodes[0] = ("q", "QuantizeLinear", {"scale": "in.s", "zero_point": "in.z"}, "xq", 49, "int8", {})
    (g, w), _ = sandwich(tmp_path / "wide", (4, 48), c1, mutate=widen)
    assert inspect(registered, g, w)[0] == -5

    def unknown(nodes, tensors, affine):
        nodes.insert(2, ("act", "QGELU", {}, "gq", 24, "int8", {}))
    (g, w), _ = sandwich(tmp_path / "op", (4, 48), c1, mutate=unknown)
    assert inspect(registered, g, w)[0] == -7


def test_sharded_weight_files(registered, tmp_path):
    """The model source may name several SafeTensors files (docs/w8a8-safetensors.md:84-108): a tensor
    is looked up across all of them and must exist exactly once."""
    from oracle.pyoracle import Oracle
    c = cases.packed_case(3, 96, 5, 32, 1)
    words = Oracle().pack_w8_words(c["w"])
    g, w = packed_package(tmp_path / "one", c["x"].shape, words, c["scales"], c["bias"], 32)
    a, b = tmp_path / "one" / "a.safetensors", tmp_path / "one" / "b.safetensors"
    write_safetensors(a, {"w#as_i32": words.astype(np.uint32)})
    write_safetensors(b, {"s": c["scales"].astype(np.float32), "b": c["bias"].astype(np.float32)})
    assert inspect(registered, g, [a, b], "dynamic_i8")[:4] == (0, 96, 5, 1)
    assert inspect(registered, g, [b, a], "dynamic_i8")[:4] == (0, 96, 5, 1)
    assert inspect(registered, g, [a], "dynamic_i8")[0] == -5          # scales and bias are missing
    assert inspect(registered, g, [a, b, w], "dynamic_i8")[0] == -5    # every tensor now exists twice
    assert inspect(registered, g, [a, tmp_path / "absent.safetensors"], "dynamic_i8")[0] == -4


def test_readers_survive_mutated_documents_under_sanitizers(tmp_path):
    """The JSON and SafeTensors readers, built with AddressSanitizer and UBSan (host code only), fed every
    truncation and thousands of byte mutations of a valid package: each is parsed or refused, none read
    out of bounds (the program aborts on the first finding)."""
    import subprocess
    from oracle.pyoracle import Oracle
    here = Path(__file__).parent / "provider_host"
    built = subprocess.run(["make", "-C", str(here), "parser_mutations"], capture_output=True, text=True)
    if built.returncode != 0:
        pytest.skip("sanitizer build unavailable: " + built.stderr[-200:])
    c = cases.packed_case(3, 96, 5, 32, 1)
    g, w = packed_package(tmp_path / "p", c["x"].shape, Oracle().pack_w8_words(c["w"]), c["scales"], c["bias"], 32)
    r = subprocess.run([str(here / "parser_mutations"), str(g), str(w), str(tmp_path / "mutant.bin")],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "parsed" in r.stdout and "refused" in r.stdout


def test_package_reading_survives_mutated_graphs_under_sanitizers(tmp_path):
    """The whole package reading -- planner, ports, fused linears, the decoder route -- built from the
    provider's sources with AddressSanitizer and UBSan (host code only; no device is touched) and fed
    truncations, byte pokes, digit and name edits and random corruptions of three valid graph
    documents: a graph with branches and several ports, a boundary/linear chain, a decoder.  Every
    mutant is accepted or refused; the program aborts on the first finding."""
    import os
    import subprocess
    import test_provider_decode as decode_tests
    from volvoxai_amd.decoder import DecoderConfig, init_weights
    here = Path(__file__).parent / "provider_host"
    built = subprocess.run(["make", "-C", str(here), "planner_mutations"], capture_output=True, text=True)
    if built.returncode != 0:
        pytest.skip("sanitizer build unavailable: " + built.stderr[-200:])
    a, b, c, q, _ = forked_cases(3)
    packages = [("dynamic_i8",) + tuple(forked_package(tmp_path / "forked", [3], a, b, c, q))]
    (g, w), _ = sandwich(tmp_path / "chain", (3, 96), cases.qlinear_random_case(3, 96, 40, 34, I8, I8, I8, False))
    packages.append(("f32", g, w))
    cfg = DecoderConfig(layers=2, hidden=128, q_heads=2, kv_heads=1, head_dim=64, inter=128, vocab=40, group=64, max_seq=16)
    packages.append(("dynamic_i8",) + tuple(decode_tests.decoder_package(tmp_path / "decoder", cfg, init_weights(cfg, 3), 2, 8)))
    # (leak checking needs ptrace, which a sandbox may refuse; out-of-bounds and use-after-free checks do not)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    for arithmetic, graph, weights in packages:
        r = subprocess.run([str(here / "planner_mutations"), str(ARITH[arithmetic]), str(tmp_path / "mutant.json"),
                            str(graph), str(weights)], capture_output=True, text=True, timeout=300, env=env)
        assert r.returncode == 0, (str(graph), r.stderr[-2000:])
        assert "accepted" in r.stdout and "refused" in r.stdout


def test_malformed_documents_are_refused(registered, tmp_path):
    k = KAT
    g, w = qlinear_package(tmp_path / "q", k["x"].shape, k["w"], k["scales"], k["zps"], k["bias"], k["s_in"], k["zp_in"],
                           k["s_out"], k["zp_out"])
    good = g.read_text()
    for bad in (good[:-3], good.replace('"nodes"', '"format"', 1), good + "{}", "[1,2", '{"a":1,"a":2}'):
        g.write_text(bad)
        assert inspect(registered, g, w)[0] == -5
    g.write_text(good)
    w.write_bytes(w.read_bytes()[:20])
    assert inspect(registered, g, w)[0] == -4
    assert inspect(registered, tmp_path / "nothing.json", w)[0] == -4


@pytest.mark.skipif(__import__("torch").cuda.is_available(), reason="covers the box without a GPU")
def test_without_a_device_the_provider_is_unavailable(registered, tmp_path):
    k = KAT
    g, w = qlinear_package(tmp_path / "q", k["x"].shape, k["w"], k["scales"], k["zps"], k["bias"], k["s_in"], k["zp_in"],
                           k["s_out"], k["zp_out"])
    r, _ = run(registered, g, w, k["x"], "hidden_q", "i8", "projected_q", "i8", 4)
    assert r.status == -6 and r.failed_stage == 1 and r.writes == 0


# ---- on the GPU ---------------------------------------------------------------------------------------

@pytest.mark.gpu
def test_literal_kat_package_end_to_end(registered, tmp_path):
    k = KAT
    g, w = qlinear_package(tmp_path / "q", k["x"].shape, k["w"], k["scales"], k["zps"], k["bias"], k["s_in"], k["zp_in"],
                           k["s_out"], k["zp_out"])
    r, y = run(registered, g, w, k["x"], "hidden_q", "i8", "projected_q", "i8", 4, executions=2)
    assert r.status == 0, r.message
    assert (y == k["want"]).all()
    assert r.writes == 2 and r.compile_attested and r.execute_attested and r.identities_echoed
    assert b"provider=hip-gfx950" in r.compile_route and b"hip.qlinear" in r.execute_route
    assert b"gfx950" in r.device and r.maximum_resident_bytes >= 1024 and r.maximum_tensor_bytes == 8


@pytest.mark.gpu
@pytest.mark.parametrize("rows,k,n,in_dtype,w_dtype", [(1, 64, 48, "int8", np.int8), (33, 200, 72, "uint8", np.int8),
                                                        (300, 512, 256, "int8", np.uint8)])
def test_qlinear_package_matches_oracle(registered, oracle, tmp_path, rows, k, n, in_dtype, w_dtype):
    rng = np.random.default_rng(rows)
    lo, hi = (-128, 128) if in_dtype == "int8" else (0, 256)
    x = rng.integers(lo, hi, (2, rows, k)).astype(np.int8 if in_dtype == "int8" else np.uint8)
    wlo, whi = (-127, 128) if w_dtype == np.int8 else (0, 256)
    wt = rng.integers(wlo, whi, (n, k)).astype(w_dtype)
    scales = (rng.uniform(0.002, 0.01, n) / np.sqrt(k) * 8).astype(np.float32)
    zps = rng.integers(-3, 4, n) if w_dtype == np.int8 else rng.integers(120, 136, n)
    bias = rng.integers(-2000, 2000, n).astype(np.int32)
    zp_in = 3 if in_dtype == "int8" else 131
    g, w = qlinear_package(tmp_path / "q", x.shape, wt, scales, zps, bias, 0.04, zp_in, 0.05, -5, in_dtype=in_dtype,
                           rows_symbol=True)
    r, y = run(registered, g, w, x, "hidden_q", "i8" if in_dtype == "int8" else "u8", "projected_q", "i8", n,
               lead_max=[64, 0])
    assert r.status == 0, r.message
    dt = {np.int8: 6, np.uint8: 5}
    ok, want = oracle.qlinear(x.reshape(-1, k), wt, bias, scales, np.asarray(zps, np.int32), 0.04, zp_in, 0.05, -5,
                              6 if in_dtype == "int8" else 5, dt[w_dtype], 6)[:2]
    assert ok == 1 and (y.reshape(-1, n) == want).all()


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["q-dense-rank2", "q-dense-rank3"])
def test_reference_shape_contract_cases(registered, oracle, tmp_path, case):
    """The two q-dense success cases of the reference's shape-contract vectors
    (tests/contracts/shape_vectors/quantized_vectors.json): shapes, dtypes and quantization
    parameters as given there, tensor contents seeded here, bytes against the oracle."""
    spec = {"q-dense-rank2": dict(x_shape=(2, 4), in_dtype="int8", w_shape=(3, 4), w_dtype=np.int8,
                                  scales=[0.02, 0.03, 0.04], zps=[0, 0, 0], s_in=0.1, zp_in=0, out_dtype="uint8",
                                  s_out=0.05, zp_out=128),
            "q-dense-rank3": dict(x_shape=(2, 5, 4), in_dtype="uint8", w_shape=(2, 4), w_dtype=np.uint8,
                                  scales=[0.01, 0.02], zps=[127, 127], s_in=0.1, zp_in=128, out_dtype="int8",
                                  s_out=0.05, zp_out=0)}[case]
    rng = np.random.default_rng(len(case))
    signed_in = spec["in_dtype"] == "int8"
    x = rng.integers(-128 if signed_in else 0, 128 if signed_in else 256, spec["x_shape"]).astype(
        np.int8 if signed_in else np.uint8)
    signed_w = spec["w_dtype"] == np.int8
    wt = rng.integers(-127 if signed_w else 0, 128 if signed_w else 256, spec["w_shape"]).astype(spec["w_dtype"])
    bias = rng.integers(-50, 50, spec["w_shape"][0]).astype(np.int32)
    g, w = qlinear_package(tmp_path / "q", x.shape, wt, spec["scales"], spec["zps"], bias, spec["s_in"], spec["zp_in"],
                           spec["s_out"], spec["zp_out"], in_dtype=spec["in_dtype"], out_dtype=spec["out_dtype"])
    out_code = "u8" if spec["out_dtype"] == "uint8" else "i8"
    r, y = run(registered, g, w, x, "hidden_q", "i8" if signed_in else "u8", "projected_q", out_code, wt.shape[0])
    assert r.status == 0, r.message
    ok, want = oracle.qlinear(x.reshape(-1, x.shape[-1]), wt, bias, np.asarray(spec["scales"], np.float32),
                              np.asarray(spec["zps"], np.int32), spec["s_in"], spec["zp_in"], spec["s_out"],
                              spec["zp_out"], 6 if signed_in else 5, 6 if signed_w else 5, DT[out_code])[:2]
    assert ok == 1 and (y.reshape(want.shape) == want).all()


@pytest.mark.gpu
def test_qlinear_package_with_unprovable_accumulator_is_refused_at_compile(registered, tmp_path):
    k = 40000  # 40000 * 255 * 255 > INT32_MAX
    x = np.zeros((1, k), np.uint8)
    wt = np.full((8, k), 255, np.uint8)
    g, w = qlinear_package(tmp_path / "q", x.shape, wt, np.full(8, 0.01, np.float32), np.zeros(8), np.zeros(8), 0.04, 0,
                           0.05, 0, in_dtype="uint8")
    r, _ = run(registered, g, w, x, "hidden_q", "u8", "projected_q", "i8", 8)
    assert r.status == -5 and r.failed_stage == 3 and r.writes == 0 and b"int32" in r.message


@pytest.mark.gpu
@pytest.mark.parametrize("rows,k,n,group", [(3, 96, 5, 32), (1, 4096, 512, 128), (40, 1000, 264, 64)])
def test_packed_linear_package_matches_oracle(registered, oracle, tmp_path, rows, k, n, group):
    c = cases.packed_case(rows, k, n, group, rows + k)
    words = oracle.pack_w8_words(c["w"])
    g, w = packed_package(tmp_path / "p", c["x"].shape, words, c["scales"], c["bias"], group)
    r, y = run(registered, g, w, c["x"], "x", "f32", "logits", "f32", n, arithmetic="dynamic_i8")
    assert r.status == 0, r.message
    _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], n, group)
    assert (y.view(np.uint32) == want.view(np.uint32)).all()
    assert r.attested_arithmetic == ARITH["dynamic_i8"] and b"hip.packed-linear" in r.execute_route
    # the same package under another arithmetic is refused before anything is allocated
    r2, _ = run(registered, g, w, c["x"], "x", "f32", "logits", "f32", n, arithmetic="f32")
    assert r2.status == -7 and r2.failed_stage == 3 and r2.writes == 0


@pytest.mark.gpu
@pytest.mark.parametrize("rows,k,n,group", [(3, 96, 5, 32), (1, 4096, 512, 128), (40, 1000, 264, 64)])
def test_packed_linear_w4_package_matches_oracle(registered, oracle, tmp_path, rows, k, n, group):
    c = cases.packed_case(rows, k, n, group, rows + k)
    words = oracle.pack_w4_words(cases.four_bit(c["w"]))
    g, w = packed_package(tmp_path / "p4", c["x"].shape, words, c["scales"], c["bias"], group, bits=4)
    r, y = run(registered, g, w, c["x"], "x", "f32", "logits", "f32", n, arithmetic="dynamic_i8")
    assert r.status == 0, r.message
    _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], n, group, bits=4)
    assert (y.view(np.uint32) == want.view(np.uint32)).all()
    assert b"hip.packed-linear" in r.execute_route


@pytest.mark.gpu
@pytest.mark.parametrize("rows,two", [(3, False), (40, True), (1, True)])
def test_quantize_linear_dequantize_chain_matches_oracle(registered, oracle, tmp_path, rows, two):
    """QuantizeLinear -> QLinear (-> QGemm) -> DequantizeLinear in one compiled model: every node's
    bytes are the oracle's, and the intermediate tensors never leave the device (the bytes in front
    of the DequantizeLinear are never stored at all)."""
    c1 = cases.qlinear_random_case(rows, 200, 96, 15, I8, I8, I8, False)
    c2 = cases.qlinear_random_case(rows, 96, 36, 16, I8, I8, I8, False) if two else None
    x = np.random.default_rng(3).normal(0, 40 * c1["s_in"], (rows, 200)).astype(np.float32)
    x[0, :4] = [np.nan, np.inf, -np.inf, 0.5 * c1["s_in"]]
    if two:
        c2["s_in"], c2["zp_in"] = c1["s_out"], c1["zp_out"]
    (g, w), d_out = sandwich(tmp_path / "c", x.shape, c1, c2)
    r, y = run(registered, g, w, x, "x", "f32", "y", "f32", d_out)
    assert r.status == 0, r.message
    ok, q = oracle.quantize(x, c1["s_in"], c1["zp_in"], I8)
    ok1, h = oracle.qlinear(q, c1["w"], c1["bias"], c1["scales"], c1["zps"], c1["s_in"], c1["zp_in"], c1["s_out"],
                            c1["zp_out"], I8, I8, I8)
    assert ok == 1 and ok1 == 1
    last = c1
    if two:
        ok2, h = oracle.qlinear(h, c2["w"], c2["bias"], c2["scales"], c2["zps"], c2["s_in"], c2["zp_in"], c2["s_out"],
                                c2["zp_out"], I8, I8, I8)
        assert ok2 == 1
        last = c2
    _, want = oracle.dequantize(h, last["s_out"], last["zp_out"], I8)
    assert (y.view(np.uint32) == want.view(np.uint32)).all()
    assert (b"nodes=4" if two else b"nodes=3") in r.execute_route
    # the boundary nodes ride in the linears next to them (nobody else reads those bytes): one launch per QLinear
    assert r.compile_route.endswith(b"route=hip.quantize-linear+qlinear>hip.qlinear+dequantize-linear" if two else
                                    b"route=hip.quantize-linear+qlinear+dequantize-linear")
    assert b"route=hip.qlinear." in r.execute_route  # the last launch of the execution is the linear's own


def requantize_chain(tmp, rows, mutate=None):
    """QuantizeLinear -> QLinear -> RequantizeLinear (I8 -> U8, other scale) -> QLinear -> DequantizeLinear."""
    c1 = cases.qlinear_random_case(rows, 128, 64, 41, I8, I8, I8, True)
    c2 = cases.qlinear_random_case(rows, 64, 48, 42, U8, I8, I8, True)
    tensors = {"in.s": np.array([c1["s_in"]], np.float32), "in.z": np.array([c1["zp_in"]], np.int8),
               "w1": c1["w"], "w1.s": c1["scales"], "w1.z": c1["zps"].astype(np.int8), "b1": c1["bias"],
               "h.s": np.array([c1["s_out"]], np.float32), "h.z": np.array([c1["zp_out"]], np.int8),
               "r.s": np.array([c2["s_in"]], np.float32), "r.z": np.array([c2["zp_in"]], np.uint8),
               "w2": c2["w"], "w2.s": c2["scales"], "w2.z": c2["zps"].astype(np.int8), "b2": c2["bias"],
               "y.s": np.array([c2["s_out"]], np.float32), "y.z": np.array([c2["zp_out"]], np.int8)}
    affine = {"xq": ("in.s", "in.z"), "w1": ("w1.s", "w1.z", 0), "hq": ("h.s", "h.z"), "rq": ("r.s", "r.z"),
              "w2": ("w2.s", "w2.z", 0), "yq": ("y.s", "y.z")}
    nodes = [("q", "QuantizeLinear", {"scale": "in.s", "zero_point": "in.z"}, "xq", 128, "int8", {}),
             ("fc1", "QLinear", {"weight": "w1", "bias": "b1"}, "hq", 64, "int8", {}),
             ("bridge", "RequantizeLinear", {}, "rq", 64, "uint8", {}),
             ("fc2", "QLinear", {"weight": "w2", "bias": "b2"}, "yq", 48, "int8", {}),
             ("dq", "DequantizeLinear", {"scale": "y.s", "zero_point": "y.z"}, "y", 48, "float32", {})]
    if mutate:
        mutate(nodes, tensors, affine)
    return chain_package(tmp, (rows, 128), "x", "float32", nodes, tensors, affine), c1, c2


def test_reads_requantize_nodes(registered, tmp_path):
    """RequantizeLinear between two QLinear nodes is read with the descriptors of its two byte tensors; a
    float side, a changed width or a missing descriptor is refused."""
    (g, w), _, _ = requantize_chain(tmp_path / "ok", 3)
    assert inspect(registered, g, w)[0] == 0

    def to_float(nodes, tensors, affine):
        nodes[2] = nodes[2][:5] + ("float32",) + nodes[2][6:]

    def widen(nodes, tensors, affine):
        nodes[2] = nodes[2][:4] + (80,) + nodes[2][5:]

    def undescribed(nodes, tensors, affine):
        del affine["rq"]

    for name, mutate in (("float", to_float), ("wide", widen), ("bare", undescribed)):
        (g, w), _, _ = requantize_chain(tmp_path / name, 3, mutate)
        assert inspect(registered, g, w)[0] == -5, name


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [1, 37])
def test_requantize_chain_matches_oracle(registered, oracle, tmp_path, rows):
    """The five-node chain through the provider: the f32 rows are those of the oracle's five operators in
    turn (the bridge changes type, scale and zero point between the two linears)."""
    (g, w), c1, c2 = requantize_chain(tmp_path / "c", rows)
    x = np.random.default_rng(5).normal(0, 40 * c1["s_in"], (rows, 128)).astype(np.float32)
    r, y = run(registered, g, w, x, "x", "f32", "y", "f32", 48)
    assert r.status == 0, r.message
    _, xq = oracle.quantize(x, c1["s_in"], c1["zp_in"], I8)
    ok1, h = oracle.qlinear(xq, c1["w"], c1["bias"], c1["scales"], c1["zps"], c1["s_in"], c1["zp_in"], c1["s_out"], c1["zp_out"],
                            I8, I8, I8)
    ok2, rq = oracle.requantize_linear(h, c1["s_out"], c1["zp_out"], c2["s_in"], c2["zp_in"], I8, U8)
    ok3, q = oracle.qlinear(rq, c2["w"], c2["bias"], c2["scales"], c2["zps"], c2["s_in"], c2["zp_in"], c2["s_out"], c2["zp_out"],
                            U8, I8, I8)
    assert ok1 == ok2 == ok3 == 1
    _, want = oracle.dequantize(q, c2["s_out"], c2["zp_out"], I8)
    assert (y.view(np.uint32) == want.view(np.uint32)).all()
    assert b"hip.requantize-linear" in r.compile_route and b"nodes=5" in r.execute_route


@pytest.mark.gpu
def test_packed_linear_chain_matches_oracle(registered, oracle, tmp_path):
    """Two PackedLinear nodes (W8 then W4) back to back: the f32 rows of the first are what the second
    prepares and multiplies."""
    a = cases.packed_case(9, 256, 130, 64, 41)
    b = cases.packed_case(9, 130, 40, 32, 42)
    wa, wb = oracle.pack_w8_words(a["w"]), oracle.pack_w4_words(cases.four_bit(b["w"]))
    nodes = [("up", "PackedLinear", {"weight": "wa", "scale": "sa", "bias": "ba"}, "h", 130, "float32",
              {"group_size": 64, "weight_bits": 8}),
             ("down", "PackedLinear", {"weight": "wb", "scale": "sb", "bias": "bb"}, "y", 40, "float32",
              {"group_size": 32, "weight_bits": 4})]
    tensors = {"wa#as_i32": wa, "sa": a["scales"], "ba": a["bias"], "wb#as_i32": wb, "sb": b["scales"], "bb": b["bias"]}
    g, w = chain_package(tmp_path / "mlp", a["x"].shape, "x", "float32", nodes, tensors, {})
    r, y = run(registered, g, w, a["x"], "x", "f32", "y", "f32", 40, arithmetic="dynamic_i8")
    assert r.status == 0, r.message
    _, h = oracle.packed_linear(a["x"], wa, a["scales"], a["bias"], 130, 64)
    _, want = oracle.packed_linear(h, wb, b["scales"], b["bias"], 40, 32, bits=4)
    assert (y.view(np.uint32) == want.view(np.uint32)).all()
    assert r.attested_arithmetic == ARITH["dynamic_i8"] and b"nodes=2" in r.execute_route


@pytest.mark.gpu
def test_contexts_of_one_compiled_model_run_concurrently(registered, oracle, tmp_path):
    """Four threads, each with its own context on the same compiled instance, eight executions each."""
    c = cases.packed_case(24, 1024, 520, 128, 9)
    words = oracle.pack_w8_words(c["w"])
    g, w = packed_package(tmp_path / "p", c["x"].shape, words, c["scales"], c["bias"], 128)
    r, y = run(registered, g, w, c["x"], "x", "f32", "logits", "f32", 520, arithmetic="dynamic_i8", executions=8,
               threads=4)
    assert r.status == 0 and r.writes == 8
    _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], 520, 128)
    assert (y.view(np.uint32) == want.view(np.uint32)).all()


@pytest.mark.gpu
def test_scheduler_batch_runs_as_one_invocation(registered, oracle, tmp_path):
    """Six requests of [1, 3, K] stacked along a symbolic axis 0: one provider invocation, six lane
    sinks, every lane the slice the oracle computes; without the core's independence proof the
    frozen contract stays at B = 1."""
    batch, inner, k, n, group = 6, 3, 384, 200, 128
    c = cases.packed_case(batch * inner, k, n, group, 21)
    x = c["x"].reshape(batch, inner, k)
    words = oracle.pack_w8_words(c["w"])
    g, w = packed_package(tmp_path / "p", (1, inner, k), words, c["scales"], c["bias"], group)
    r, y = run(registered, g, w, x, "x", "f32", "logits", "f32", n, arithmetic="dynamic_i8", lead_max=[16, 0],
               batch_proof=True)
    assert r.status == 0, r.message
    assert r.writes == batch and r.execute_attested and r.attested_arithmetic == 16  # frozen max_batch
    _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], n, group)
    assert (y.reshape(-1, n).view(np.uint32) == want.view(np.uint32)).all()
    r2, _ = run(registered, g, w, x, "x", "f32", "logits", "f32", n, arithmetic="dynamic_i8", lead_max=[16, 0],
                batch_proof=False)
    assert r2.status == -7 and r2.attested_arithmetic == 1 and r2.writes == 0


@pytest.mark.gpu
def test_bindings_are_validated_before_anything_runs(registered, tmp_path):
    k = KAT
    g, w = qlinear_package(tmp_path / "q", k["x"].shape, k["w"], k["scales"], k["zps"], k["bias"], k["s_in"], k["zp_in"],
                           k["s_out"], k["zp_out"])
    r, _ = run(registered, g, w, k["x"], "hidden_q", "i8", "projected_q", "i8", 4)
    assert r.status == 0
    wrong = np.zeros((2, 3), np.uint8)
    r, _ = run(registered, g, w, wrong, "hidden_q", "u8", "projected_q", "i8", 4)  # dtype differs from the graph's
    assert r.status == -1 and r.writes == 0
    r, _ = run(registered, g, w, k["x"], "other", "i8", "projected_q", "i8", 4)
    assert r.status == -1 and r.writes == 0


# ---- graphs that are not chains ----------------------------------------------------------------

class MockPort(C.Structure):
    _fields_ = [("name", C.c_char_p), ("dtype", C.c_int32), ("last", C.c_int64), ("data", C.c_void_p),
                ("bytes", C.c_uint64), ("written", C.c_int32)]


class MockGraphRun(C.Structure):
    _fields_ = [("graph_path", C.c_char_p), ("weight_path", C.c_char_p), ("packed_arithmetic", C.c_int32),
                ("rank", C.c_uint32), ("lead", C.c_int64 * 8), ("lead_max0", C.c_int64), ("batch", C.c_int32),
                ("input_count", C.c_int32), ("output_count", C.c_int32), ("inputs", MockPort * 8),
                ("outputs", MockPort * 8),
                ("status", C.c_int32), ("failed_stage", C.c_int32), ("writes", C.c_int32), ("sink_mismatch", C.c_int32),
                ("message", C.c_char * 256), ("execute_route", C.c_char * 512)]


def forked_package(tmp, lead, a, b, c, q, rows_symbol=False):
    """Two inputs, three outputs: x -> PackedLinear A -> ya;  x -> PackedLinear B -> h -> PackedLinear C
    -> yc (x is read twice);  u -> QuantizeLinear -> uq -> QLinear -> vq (an independent branch)."""
    lead = list(lead)
    shape = lambda d: lead + [d]

    def packed(node_id, fed, out_name, case, prefix):
        return {"id": node_id, "opType": "PackedLinear",
                "inputs": {"input": fed, "weight": prefix + ".w", "scale": prefix + ".s", "bias": prefix + ".b"},
                "outputs": {"out": {"tensor": out_name, "shape": shape(case["n"]), "dtype": "float32"}},
                "params": {"group_size": case["group"], "weight_bits": 8}}

    nodes = [packed("A", "x", "ya", a, "a"), packed("B", "x", "h", b, "b"),
             {"id": "quant", "opType": "QuantizeLinear", "inputs": {"input": "u", "scale": "u.s", "zero_point": "u.z"},
              "outputs": {"out": {"tensor": "uq", "shape": shape(q["w"].shape[1]), "dtype": "int8"}}, "params": {}},
             packed("C", "h", "yc", c, "c"),
             {"id": "fc", "opType": "QLinear", "inputs": {"input": "uq", "weight": "q.w", "bias": "q.b"},
              "outputs": {"out": {"tensor": "vq", "shape": shape(q["w"].shape[0]), "dtype": "int8"}}, "params": {}}]
    graph = {"format": "volvox-graph/v1", "dimensions": {"rows": {"min": 1, "max": 64}} if rows_symbol else {},
             "inputs": {"x": {"shape": shape(a["k"]), "dtype": "float32"},
                        "u": {"shape": shape(q["w"].shape[1]), "dtype": "float32"}},
             "nodes": nodes, "outputs": ["yc", "vq", "ya"],
             "quantization": {"format": "volvox-affine-safetensors/v1", "tensors": {
                 "uq": {"scheme": "per_tensor", "scale_tensor": "u.s", "zero_point_tensor": "u.z"},
                 "q.w": {"scheme": "per_axis", "axis": 0, "scale_tensor": "q.w.s", "zero_point_tensor": "q.w.z"},
                 "vq": {"scheme": "per_tensor", "scale_tensor": "v.s", "zero_point_tensor": "v.z"}}}}
    from oracle.pyoracle import Oracle
    orc = Oracle()
    tensors = {"u.s": np.array([q["s_in"]], np.float32), "u.z": np.array([q["zp_in"]], np.int8),
               "q.w": q["w"], "q.b": q["bias"], "q.w.s": q["scales"], "q.w.z": q["zps"].astype(np.int8),
               "v.s": np.array([q["s_out"]], np.float32), "v.z": np.array([q["zp_out"]], np.int8)}
    for prefix, case in (("a", a), ("b", b), ("c", c)):
        tensors[prefix + ".w#as_i32"] = orc.pack_w8_words(case["w"])
        tensors[prefix + ".s"], tensors[prefix + ".b"] = case["scales"], case["bias"]
    tmp.mkdir(parents=True, exist_ok=True)
    (tmp / "graph.json").write_text(json.dumps(graph, separators=(",", ":")))
    write_safetensors(tmp / "model.safetensors", tensors)
    return tmp / "graph.json", tmp / "model.safetensors"


def forked_cases(rows):
    a = cases.packed_case(rows, 384, 200, 128, 31)
    b = cases.packed_case(rows, 384, 130, 64, 32)
    c = cases.packed_case(rows, 130, 72, 32, 33)
    q = cases.qlinear_random_case(rows, 96, 40, 34, I8, I8, I8, False)
    u = np.random.default_rng(35).normal(0, 20, (rows, 96)).astype(np.float32)
    return a, b, c, q, u


def forked_expectation(oracle, a, b, c, q, u):
    _, ya = oracle.packed_linear(a["x"], oracle.pack_w8_words(a["w"]), a["scales"], a["bias"], a["n"], a["group"])
    _, h = oracle.packed_linear(a["x"], oracle.pack_w8_words(b["w"]), b["scales"], b["bias"], b["n"], b["group"])
    _, yc = oracle.packed_linear(h, oracle.pack_w8_words(c["w"]), c["scales"], c["bias"], c["n"], c["group"])
    _, uq = oracle.quantize(u, q["s_in"], q["zp_in"], I8)
    ok, vq = oracle.qlinear(uq, q["w"], q["bias"], q["scales"], q["zps"], q["s_in"], q["zp_in"], q["s_out"], q["zp_out"],
                            I8, I8, I8)
    assert ok == 1
    return ya, yc, vq


def run_forked(host, g, w, lead, a, q, u, batch=0, lead_max0=0):
    mock, _, _ = host
    rows = int(np.prod(lead))
    x = np.ascontiguousarray(a["x"])
    outs = {"yc": np.zeros((rows, 72), np.float32), "vq": np.zeros((rows, 40), np.int8), "ya": np.zeros((rows, 200), np.float32)}
    r = MockGraphRun()
    r.graph_path, r.weight_path, r.packed_arithmetic = str(g).encode(), str(w).encode(), ARITH["dynamic_i8"]
    r.rank = len(lead) + 1
    for i, e in enumerate(lead):
        r.lead[i] = e
    r.lead_max0, r.batch = lead_max0, batch
    r.input_count, r.output_count = 2, 3
    r.inputs[0] = MockPort(b"x", DT["f32"], 384, x.ctypes.data, x.nbytes, 0)
    r.inputs[1] = MockPort(b"u", DT["f32"], 96, u.ctypes.data, u.nbytes, 0)
    for k, (name, dt) in enumerate((("ya", "f32"), ("yc", "f32"), ("vq", "i8"))):
        r.outputs[k] = MockPort(name.encode(), DT[dt], outs[name].shape[1], outs[name].ctypes.data, outs[name].nbytes, 0)
    mock.mock_host_run_graph.argtypes = [C.POINTER(MockGraphRun)]
    mock.mock_host_run_graph(C.byref(r))
    return r, outs


def test_reads_graphs_with_branches_and_several_ports(registered, tmp_path):
    a, b, c, q, _ = forked_cases(6)
    g, w = forked_package(tmp_path / "fork", (6,), a, b, c, q)
    assert inspect(registered, g, w, "dynamic_i8")[:4] == (0, 384, 72, 1)  # first input, first output
    doc = json.loads(g.read_text())
    doc["inputs"]["u"]["shape"] = [7, 96]  # another row count than x
    g.write_text(json.dumps(doc))
    st, *_, msg = inspect(registered, g, w, "dynamic_i8")
    assert st == -7 and "leading extents" in msg


@pytest.mark.gpu
def test_forked_graph_two_inputs_three_outputs(registered, oracle, tmp_path):
    """A graph that is not a chain: one input read by two linears, a second input with its own
    branch, three outputs declared in another order than they are computed; every output equals the
    oracle's composition of its branch, and each is written once under its own name and type."""
    rows = 37
    a, b, c, q, u = forked_cases(rows)
    g, w = forked_package(tmp_path / "fork", (rows,), a, b, c, q)
    r, outs = run_forked(registered, g, w, (rows,), a, q, u)
    assert r.status == 0 and r.failed_stage == 0, (r.status, r.failed_stage, r.message)
    ya, yc, vq = forked_expectation(oracle, a, b, c, q, u)
    assert (outs["ya"].view(np.uint32) == ya.view(np.uint32)).all()
    assert (outs["yc"].view(np.uint32) == yc.view(np.uint32)).all()
    assert (outs["vq"] == vq).all()
    assert r.writes == 3 and b"nodes=5" in r.execute_route


@pytest.mark.gpu
def test_forked_graph_as_one_scheduler_batch(registered, oracle, tmp_path):
    """The same graph with a symbolic axis 0: five requests of [1, 3, d] stacked into one
    invocation, every lane's sink receiving its slice of each of the three outputs."""
    batch, inner = 5, 3
    rows = batch * inner
    a, b, c, q, u = forked_cases(rows)
    g, w = forked_package(tmp_path / "fork", (1, inner), a, b, c, q)
    r, outs = run_forked(registered, g, w, (batch, inner), a, q, u, batch=1, lead_max0=16)
    assert r.status == 0 and r.failed_stage == 0, (r.status, r.failed_stage, r.message)
    ya, yc, vq = forked_expectation(oracle, a, b, c, q, u)
    assert (outs["ya"].view(np.uint32) == ya.view(np.uint32)).all()
    assert (outs["yc"].view(np.uint32) == yc.view(np.uint32)).all()
    assert (outs["vq"] == vq).all()
    assert r.writes == 3 * batch
