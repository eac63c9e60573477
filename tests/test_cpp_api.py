"""C++ API (include/turboquant/*.h), the 25-symbol C API (include/turboquant_c/turboquant_c.h)
and the TQ8 safetensors layout.

CPU part: the handle-based C entry points, and this library's safetensors reader/writer checked
in both directions against the independent `safetensors` Python package.
GPU part: a C++ program drives quantize_weight / TurboQuantLinear / dequantize_weight_gpu /
write_tq_safetensors and its results are compared with the CPU oracle; tq_model_dequant is run
on a model directory assembled here.
"""
import ctypes
import json
import os
import subprocess

import numpy as np
import pytest
from safetensors import safe_open
from safetensors.numpy import load_file, save_file

import __graft_entry__ as entry

BIN = os.path.join(entry.ROOT, "tests", "cpp", "bin")


def _run(name, *args):
    exe = os.path.join(BIN, name)
    assert os.path.exists(exe), "build the test programs first (python __graft_entry__.py)"
    p = subprocess.run([exe, *args], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, f"{name} failed:\n{p.stdout}\n{p.stderr}"
    return p.stdout


def _metadata(path):
    with safe_open(path, framework="np") as f:
        return f.metadata() or {}


# --------------------------------------------------------------------------- CPU
def test_c_api_program(tmp_path):
    """Reference tests/c_api/*.c cases, compiled as C99 against turboquant_c.h."""
    assert "c api ok" in _run("test_c_api", str(tmp_path))


def test_safetensors_reader_and_writer_against_python_package(tmp_path):
    rng = np.random.default_rng(5)
    tensors = {
        "a.packed_primary": rng.integers(0, 256, (7, 16), dtype=np.uint8),
        "a.norms": rng.standard_normal(7).astype(np.float32),
        "a.seeds": np.array([0xDEADBEEF, 0, 512], dtype=np.uint32),
        "half": rng.standard_normal((3, 5)).astype(np.float16),
        "wide": rng.standard_normal((2, 2, 3)),
        "i64": rng.integers(-2**40, 2**40, (4,), dtype=np.int64),
        "flags": np.array([True, False, True]),
        "scalar": np.array(3.5, dtype=np.float32),
        "empty": np.zeros((0, 4), dtype=np.float32),
        "unié\"quote\\": np.arange(6, dtype=np.int32).reshape(2, 3),
    }
    md = {"quantization_method": "turboquant", "note": "line\nbreak \"q\" ü", "tq_version": "1"}
    src, dst = str(tmp_path / "in.safetensors"), str(tmp_path / "out.safetensors")
    save_file(tensors, src, metadata=md)
    assert f"{len(tensors)} tensors" in _run("st_roundtrip", "copy", src, dst)
    back = load_file(dst)                      # our writer, their reader
    assert set(back) == set(tensors)
    for k, v in tensors.items():
        assert back[k].dtype == v.dtype and back[k].shape == v.shape, k
        assert np.array_equal(back[k], v), k
    assert _metadata(dst) == md
    out = _run("st_roundtrip", "meta", dst)
    assert "quantization_method=turboquant" in out and "tq_version=1" in out
    # header is 8-byte aligned as the format recommends
    n = int.from_bytes(open(dst, "rb").read(8), "little")
    assert n % 8 == 0


def test_reader_rejects_malformed_files(tmp_path):
    bad = tmp_path / "bad.safetensors"
    bad.write_bytes((100).to_bytes(8, "little") + b"{}")
    p = subprocess.run([os.path.join(BIN, "st_roundtrip"), "copy", str(bad), str(tmp_path / "o")],
                       capture_output=True, text=True)
    assert p.returncode == 1 and "error" in p.stderr
    hdr = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode()
    bad.write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\0" * 8)       # data too short
    p = subprocess.run([os.path.join(BIN, "st_roundtrip"), "copy", str(bad), str(tmp_path / "o")],
                       capture_output=True, text=True)
    assert p.returncode == 1
    assert _run("st_roundtrip", "meta", str(tmp_path / "missing.safetensors")) == ""


def test_reader_survives_corrupted_headers(tmp_path):
    """Every way of corrupting the header of a valid file ends in a clean error (exit code 1) or in
    a successful parse, never in a crash: reversed, oversized and negative offsets, shapes that
    overflow, unknown dtypes, missing keys, wrong JSON types, truncation at every length class,
    and a few hundred random byte flips (fixed seed).  The same corpus was run through a build
    of the reader with the address and undefined-behaviour sanitizers without findings."""
    import copy
    import random
    import struct
    good = tmp_path / "good.safetensors"
    save_file({"a.weight": np.arange(128, dtype=np.float32).reshape(8, 16), "b": np.arange(10, dtype=np.uint8)},
              str(good), metadata={"k": 'v"x\\y'})
    raw = good.read_bytes()
    hl = struct.unpack("<Q", raw[:8])[0]
    header, data = json.loads(raw[8:8 + hl]), raw[8 + hl:]

    def pack(h, d=data):
        hb = json.dumps(h).encode()
        return struct.pack("<Q", len(hb)) + hb + d

    def mutate(fn):
        h = copy.deepcopy(header)
        fn(h)
        return pack(h)

    cases = [raw[:4], struct.pack("<Q", 2 ** 62) + raw[8:], struct.pack("<Q", hl + 1000) + raw[8:],
             struct.pack("<Q", 0) + raw[8:], pack(header, data[:5]),
             mutate(lambda h: h["a.weight"].__setitem__("data_offsets", [0, 10 ** 12])),
             mutate(lambda h: h["a.weight"].__setitem__("data_offsets", [100, 50])),
             mutate(lambda h: h["a.weight"].__setitem__("shape", [2 ** 31, 2 ** 31])),
             mutate(lambda h: h["a.weight"].__setitem__("shape", [-1, 16])),
             mutate(lambda h: h["a.weight"].__setitem__("dtype", "F77")),
             mutate(lambda h: h["a.weight"].pop("shape")),
             mutate(lambda h: h.__setitem__("a.weight", "x")),
             mutate(lambda h: h.__setitem__("__metadata__", {"a": 1})),
             # three dimensions whose product wraps a 64-bit size; dimensions and offsets that are not
             # whole numbers, not numbers at all, or beyond every integer type
             mutate(lambda h: h["a.weight"].__setitem__("shape", [2 ** 31 - 1, 2 ** 31 - 1, 2 ** 31 - 1])),
             mutate(lambda h: h["a.weight"].__setitem__("shape", [8.5, 16])),
             mutate(lambda h: h["a.weight"].__setitem__("shape", ["8", 16])),
             mutate(lambda h: h["a.weight"].__setitem__("shape", [1e300, 1])),
             mutate(lambda h: h["a.weight"].__setitem__("data_offsets", [0, 1e300])),
             mutate(lambda h: h["a.weight"].__setitem__("data_offsets", [-512, 0])),
             mutate(lambda h: h["a.weight"].__setitem__("data_offsets", [None, 512]))]

    def raw_header(text, d=data):
        hb = text.encode()
        return struct.pack("<Q", len(hb)) + hb + d
    # numbers std::stod cannot take, and nesting far beyond a header's three levels
    cases += [raw_header('{"t":{"dtype":"F32","shape":[-],"data_offsets":[0,4]}}'),
              raw_header('{"t":{"dtype":"F32","shape":[1e99999],"data_offsets":[0,4]}}'),
              raw_header('{"t":{"dtype":"F32","shape":[+.e],"data_offsets":[0,4]}}'),
              raw_header("[" * 200000), raw_header('{"a":' * 50000)]
    rnd = random.Random(1)
    for _ in range(200):
        b = bytearray(raw)
        for _ in range(rnd.randint(1, 6)):
            b[rnd.randrange(0, 8 + hl)] = rnd.randrange(256)
        cases.append(bytes(b))
    cases += [raw[:rnd.randrange(0, len(raw))] for _ in range(40)]
    bad = tmp_path / "case.safetensors"
    for i, blob in enumerate(cases):
        bad.write_bytes(blob)
        p = subprocess.run([os.path.join(BIN, "st_roundtrip"), "copy", str(bad), str(tmp_path / "o")],
                           capture_output=True)
        assert p.returncode in (0, 1), (i, p.returncode, p.stderr[-300:])


# --------------------------------------------------------------------------- GPU
@pytest.mark.gpu
@pytest.mark.parametrize("out_f,in_f,bs,batch", [(64, 512, 256, 3), (48, 384, 128, 1)])
def test_cpp_api_against_oracle(tmp_path, oracle, out_f, in_f, bs, batch):
    o = oracle
    w = o.lcg_matrix(out_f, in_f, 42) * np.float32(0.05)
    x = o.lcg_matrix(batch, in_f, 99)
    src = str(tmp_path / "inputs.safetensors")
    save_file({"w": w, "x": x}, src, metadata={"block_size": str(bs)})
    assert "cpp api ok" in _run("test_cpp_api", src, str(tmp_path))
    res = load_file(str(tmp_path / "results.safetensors"))

    cb = o.generate_codebook(4)
    for tag, shared in (("dual.", False), ("shared.", True)):
        qw = o.quantize_weight(w, cb, cb, 4, 4, bs, shared)
        assert np.array_equal(res[tag + "packed_primary"], qw.packed_primary)
        assert np.array_equal(res[tag + "packed_residual"], qw.packed_residual)
        assert np.array_equal(res[tag + "norms"], qw.norms)
        assert np.array_equal(res[tag + "seeds"], qw.seeds)
        w_ref = o.dequantize_weight_cpu(qw, cb, cb, bs)
        assert np.array_equal(res[tag + "w"], w_ref)                       # bit-exact
        y_ref = o.matmul_xwT(x, w_ref, acc_double=True)
        rel = np.linalg.norm(res[tag + "y"] - y_ref) / np.linalg.norm(y_ref)
        assert rel < 1e-3, rel                                              # fp32 activations
        xb = o.bf16_bits_to_f32(o.f32_to_bf16_bits(x))
        yb_ref = o.matmul_xwT(xb, w_ref, acc_double=True)
        rel = np.linalg.norm(res[tag + "y_bf16_in"] - yb_ref) / np.linalg.norm(yb_ref)
        assert rel < 1e-3, rel                                              # bf16 activations: batch 1 exact fp32 kernel,
                                                                            # more rows the fp16-weight MFMA kernels
        rel = np.linalg.norm(res[tag + "y_f16"].astype(np.float32) - y_ref) / np.linalg.norm(y_ref)
        assert rel < 2e-3, rel                                              # half-precision in (rounds x itself) and out

    rot = o.wht_forward(w, 0x1234, bs)
    assert np.array_equal(res["rotated"], rot)
    assert np.array_equal(res["unrotated"], o.wht_inverse(rot, 0x1234, bs))
    idx = o.quantize(x.reshape(-1), cb)
    assert np.array_equal(res["x_indices"], idx)
    assert np.array_equal(res["x_centroids"], o.dequantize(idx, cb))
    samples = rot.reshape(-1) * (np.float32(1.0) / w.reshape(-1)[0])
    fit = o.generate_codebook_from_data(samples, 4)
    assert np.array_equal(res["fit_centroids"], fit.centroids)

    # The TQ8 file through a stock reader (reference tests/unit/test_serialization.cpp:120-160).
    tq = load_file(str(tmp_path / "model.safetensors"))
    md = _metadata(str(tmp_path / "model.safetensors"))
    assert md == {"quantization_method": "turboquant", "tq_version": "1", "tq_primary_bits": "4",
                  "tq_residual_bits": "4", "tq_total_bits": "8", "tq_per_layer_codebooks": "true"}
    for layer, tag in (("model.dual_proj", "dual."), ("model.shared_proj", "shared.")):
        assert tq[layer + ".packed_primary"].dtype == np.uint8
        assert tq[layer + ".packed_primary"].shape == (out_f, in_f // 2)
        assert np.array_equal(tq[layer + ".packed_residual"], res[tag + "packed_residual"])
        assert tq[layer + ".norms"].dtype == np.float32 and tq[layer + ".norms"].shape == (out_f,)
        assert tq[layer + ".seeds"].dtype == np.uint32 and tq[layer + ".seeds"].shape == (3,)
    assert np.array_equal(tq["tq_codebook_primary"], cb.centroids)
    assert np.array_equal(tq["tq_codebook_residual"], cb.centroids)
    assert np.array_equal(tq["model.dual_proj.codebook_primary"], cb.centroids)
    assert "model.shared_proj.codebook_primary" not in tq


def _bf16_bits(a):
    return a.view(np.uint16) if a.dtype != np.uint16 else a


@pytest.mark.gpu
@pytest.mark.parametrize("passthrough_dtype", [None, np.float16])
def test_tq_model_dequant_directory(tmp_path, oracle, passthrough_dtype):
    """tq_model_dequant (reference src/turboquant_c_dequant.cpp:20-191) on a directory written
    with the stock safetensors package: TQ8 shard with per-layer codebooks, passthrough shard,
    a non-TQ shard, config.json carrying quantization_config."""
    o = oracle
    pkg = entry.load_package()
    L = pkg.lib()
    src, dst = tmp_path / "tq8", tmp_path / "out"
    src.mkdir()
    cb = o.generate_codebook(4)
    tensors, expect = {}, {}
    for i, (out_f, in_f, bs, shared) in enumerate([(32, 256, 128, True), (16, 512, 512, False)]):
        w = o.lcg_matrix(out_f, in_f, 7 + i) * np.float32(0.03)
        name = f"model.layers.{i}.mlp.up_proj"
        cbp, cbr = (o.fit_layer_codebooks(w, bs) if i == 0 else (cb, cb))
        qw = o.quantize_weight(w, cbp, cbr, 4, 4, bs, shared)
        tensors[name + ".packed_primary"] = qw.packed_primary
        tensors[name + ".packed_residual"] = qw.packed_residual
        tensors[name + ".norms"] = qw.norms
        tensors[name + ".seeds"] = qw.seeds
        if i == 0:
            tensors[name + ".codebook_primary"] = cbp.centroids
            tensors[name + ".codebook_residual"] = cbr.centroids
        expect[name + ".weight"] = o.dequantize_weight_cpu(qw, cbp, cbr, bs)
    tensors["tq_codebook_primary"] = cb.centroids
    tensors["tq_codebook_residual"] = cb.centroids
    save_file(tensors, str(src / "model.safetensors"),
              metadata={"quantization_method": "turboquant", "tq_version": "1", "tq_primary_bits": "4",
                        "tq_residual_bits": "4", "tq_total_bits": "8", "tq_per_layer_codebooks": "true"})
    if passthrough_dtype is not None:
        save_file({"model.norm.weight": np.linspace(-1, 1, 8).astype(passthrough_dtype)},
                  str(src / "model_passthrough.safetensors"))
    plain = {"embed": np.arange(12, dtype=np.float32).reshape(3, 4)}
    save_file(plain, str(src / "extra.safetensors"))
    config = {"model_type": "test", "hidden_size": 64,
              "quantization_config": {"quantization_method": "turboquant", "nested": {"a": 1}, "tq_total_bits": 8}}
    (src / "config.json").write_text(json.dumps(config, indent=2))
    (src / "tokenizer.json").write_text("{}")

    L.tq_model_dequant.restype = ctypes.c_int
    L.tq_model_dequant.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
    assert L.tq_model_dequant(str(src).encode(), str(dst).encode()) == 0

    cfg = json.loads((dst / "config.json").read_text())
    assert cfg == {"model_type": "test", "hidden_size": 64}
    assert (dst / "tokenizer.json").read_text() == "{}"
    assert np.array_equal(load_file(str(dst / "extra.safetensors"))["embed"], plain["embed"])
    assert not (dst / "model_passthrough.safetensors").exists()

    with safe_open(str(dst / "model.safetensors"), framework="np") as f:
        names = set(f.keys())
    want = set(expect) | ({"model.norm.weight"} if passthrough_dtype is not None else set())
    assert names == want
    if passthrough_dtype is None:
        # bf16 output: read the raw bits (numpy has no bf16) and compare with the oracle's
        # fp32 weight rounded to nearest-even.
        import torch
        from safetensors.torch import load_file as load_torch
        got = load_torch(str(dst / "model.safetensors"))
        for k, w_ref in expect.items():
            assert got[k].dtype == torch.bfloat16 and tuple(got[k].shape) == w_ref.shape
            bits = got[k].view(torch.int16).numpy().view(np.uint16)
            assert np.array_equal(bits, o.f32_to_bf16_bits(w_ref)), k
    else:
        got = load_file(str(dst / "model.safetensors"))
        for k, w_ref in expect.items():
            assert got[k].dtype == np.float16
            assert np.array_equal(got[k], w_ref.astype(np.float16)), k
        assert np.array_equal(got["model.norm.weight"], np.linspace(-1, 1, 8).astype(np.float16))


# --------------------------------------------------------------------------- command-line tools
CLI = os.path.join(entry.ROOT, "turboquant-mlx-core_amd", "bin")


def test_cli_usage_and_version():
    """tq-convert / tq-dequant-model (reference tools/): argument handling needs no GPU."""
    for exe in ("tq-convert", "tq-dequant-model"):
        assert os.path.exists(os.path.join(CLI, exe)), "build first (python __graft_entry__.py)"
    p = subprocess.run([os.path.join(CLI, "tq-convert"), "--version"], capture_output=True, text=True)
    assert p.returncode == 0 and p.stdout.startswith("tq-convert ")
    p = subprocess.run([os.path.join(CLI, "tq-convert")], capture_output=True, text=True)
    assert p.returncode == 1 and "Usage: tq-convert --model" in p.stdout
    p = subprocess.run([os.path.join(CLI, "tq-convert"), "--bits", "4"], capture_output=True, text=True)
    assert p.returncode == 1 and "--model is required" in p.stderr
    p = subprocess.run([os.path.join(CLI, "tq-dequant-model"), "only-one-argument"], capture_output=True, text=True)
    assert p.returncode == 1 and "Usage:" in p.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("per_layer,shared", [(True, True), (False, False)])
def test_cli_convert_then_dequant_model_directory(tmp_path, oracle, per_layer, shared):
    """tq-convert on a small HuggingFace-style directory written with the `safetensors` package,
    then tq-dequant-model on its output.  Checked: which tensors are quantized (2-D "*.weight"
    outside the sensitive first / last layer), the TQ8 tensor names, shapes, dtypes and metadata,
    the block size chosen per layer, config.json, the pass-through shard, that the packed bytes
    are the ones the CPU oracle's quantizer produces from the same weight and codebooks, and that
    the round trip returns every tensor (quantized ones within the 8-bit quantization error)."""
    rng = np.random.default_rng(7)
    src = tmp_path / "model"
    src.mkdir()
    (src / "config.json").write_text(json.dumps({"model_type": "toy", "num_hidden_layers": 4}, indent=2))
    (src / "tokenizer.txt").write_text("not a tensor file")
    tensors = {"model.embed_tokens.weight": (rng.standard_normal((96, 64)) * 0.05).astype(np.float16),
               "lm_head.weight": (rng.standard_normal((96, 64)) * 0.05).astype(np.float32),
               "model.norm.weight": np.ones(64, np.float32),
               # a width that is not a multiple of 32 (blocks of 16 columns) is quantized like any other; an odd
               # width cannot share bytes between column pairs and is left as it is
               "model.layers.1.mlp.narrow.weight": (rng.standard_normal((8, 48)) * 0.05).astype(np.float32),
               "model.layers.2.mlp.odd.weight": (rng.standard_normal((8, 45)) * 0.05).astype(np.float32)}
    for n in range(4):
        tensors[f"model.layers.{n}.self_attn.q_proj.weight"] = (rng.standard_normal((64, 64)) * 0.05).astype(np.float32)
        tensors[f"model.layers.{n}.mlp.up_proj.weight"] = (rng.standard_normal((160, 1536)) * 0.02).astype(np.float16)
        tensors[f"model.layers.{n}.self_attn.q_proj.bias"] = rng.standard_normal(64).astype(np.float32)
        tensors[f"model.layers.{n}.input_layernorm.weight"] = np.ones(64, np.float32)
    save_file(tensors, str(src / "model.safetensors"))

    out = tmp_path / "model-tq"
    args = [os.path.join(CLI, "tq-convert"), "--model", str(src), "--output", str(out), "--sensitive-layers", "1"]
    if per_layer:
        args.append("--per-layer-codebooks")
    if shared:
        args.append("--shared-rotation")
    p = subprocess.run(args, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "Sensitive layers: 4 weights kept at fp16, 7 weights quantized" in p.stdout
    assert "model.layers.2.mlp.odd.weight [8, 45] left unquantized" in p.stderr
    assert "narrow" not in p.stderr

    cfg = json.loads((out / "config.json").read_text())
    assert cfg["model_type"] == "toy"
    assert cfg["quantization_config"] == {"quantization_method": "turboquant", "tq_version": "1", "bits": 4,
                                          "residual_bits": 4, "block_size": 512, "shared_rotation": shared,
                                          "sensitive_layers_start": 1, "sensitive_layers_end": 1}
    assert (out / "tokenizer.txt").read_text() == "not a tensor file"

    meta = _metadata(str(out / "model.safetensors"))
    assert meta["quantization_method"] == "turboquant" and meta["tq_version"] == "1"
    assert meta["tq_primary_bits"] == "4" and meta["tq_residual_bits"] == "4" and meta["tq_total_bits"] == "8"
    assert (meta.get("tq_per_layer_codebooks") == "true") == per_layer
    tq_t = load_file(str(out / "model.safetensors"))
    pt = load_file(str(out / "model_passthrough.safetensors"))
    quantized = ["model.embed_tokens", "lm_head", "model.layers.1.mlp.narrow"] + \
                [f"model.layers.{n}.{m}" for n in (1, 2) for m in ("self_attn.q_proj", "mlp.up_proj")]
    assert sorted(k[:-len(".packed_primary")] for k in tq_t if k.endswith(".packed_primary")) == sorted(quantized)
    for name in quantized:
        w = tensors[name + ".weight"].astype(np.float32)
        o_f, i_f = w.shape
        bs = {1536: 512, 64: 64, 48: 16}[i_f]                       # largest power of two <= 512 dividing the width
        assert tq_t[name + ".packed_primary"].shape == (o_f, i_f // 2) and tq_t[name + ".packed_primary"].dtype == np.uint8
        assert tq_t[name + ".packed_residual"].shape == (o_f, i_f // 2)
        assert tq_t[name + ".norms"].shape == (o_f,) and tq_t[name + ".norms"].dtype == np.float32
        seeds = tq_t[name + ".seeds"]
        assert seeds.dtype == np.uint32 and seeds.shape == (3,) and seeds[2] == bs
        assert (seeds[1] == 0) == shared
        assert (name + ".codebook_primary" in tq_t) == per_layer
        # the same weight through the CPU oracle's quantizer with the codebooks of the file
        cbp = oracle.Codebook(tq_t[name + ".codebook_primary"] if per_layer else tq_t["tq_codebook_primary"], 4)
        cbr = oracle.Codebook(tq_t[name + ".codebook_residual"] if per_layer else tq_t["tq_codebook_residual"], 4)
        qw = oracle.quantize_weight(w, cbp, cbr, 4, 4, bs, shared)
        assert np.array_equal(qw.seeds, seeds)
        same = np.mean(qw.packed_primary == tq_t[name + ".packed_primary"])
        assert same > 0.999                                          # boundary ties may round differently on the GPU
        assert np.allclose(qw.norms, tq_t[name + ".norms"], rtol=1e-4)
    # pass-through: 1-D tensors, biases, the sensitive layers 0 and 3, the weight the quantizer cannot take
    kept = [k for k in tensors if k not in {q + ".weight" for q in quantized}]
    assert sorted(pt) == sorted(kept)
    for k in kept:
        assert pt[k].dtype == tensors[k].dtype and np.array_equal(pt[k], tensors[k])

    deq = tmp_path / "model-deq"
    p = subprocess.run([os.path.join(CLI, "tq-dequant-model"), str(out), str(deq)], capture_output=True, text=True,
                       timeout=600)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "quantization_config" not in json.loads((deq / "config.json").read_text())
    back = {}
    for f in os.listdir(deq):
        if f.endswith(".safetensors"):
            back.update(load_file(str(deq / f)))
    assert sorted(back) == sorted(tensors)
    for k, v in tensors.items():
        got = back[k].astype(np.float32)
        if k[:-len(".weight")] in quantized:
            rel = np.linalg.norm(got - v.astype(np.float32)) / np.linalg.norm(v.astype(np.float32))
            assert rel < 0.15, (k, rel)                              # the bound of the reference's own round-trip tests
        else:
            assert np.array_equal(got, v.astype(np.float32))


@pytest.mark.gpu
def test_cli_convert_five_bit_default_output_runs_forward(tmp_path, oracle):
    """`tq-convert --bits 5` with its defaults writes a 5-bit primary plane (one index per byte) and a 4-bit
    residual with its own rotation.  Such a file loads, dequantises to the oracle's bits and runs forward,
    one row and several, through the same entry points as a 4-bit file."""
    import __graft_entry__ as entry
    tq = entry.load_package()
    rng = np.random.default_rng(11)
    src = tmp_path / "model"
    src.mkdir()
    (src / "config.json").write_text(json.dumps({"model_type": "toy", "num_hidden_layers": 1}))
    w = (rng.standard_normal((96, 1024)) * 0.03).astype(np.float32)
    save_file({"model.layers.0.mlp.up_proj.weight": w, "model.norm.weight": np.ones(64, np.float32)},
              str(src / "model.safetensors"))
    out = tmp_path / "model-tq5"
    p = subprocess.run([os.path.join(CLI, "tq-convert"), "--model", str(src), "--output", str(out), "--bits", "5"],
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stdout + p.stderr
    meta = _metadata(str(out / "model.safetensors"))
    assert meta["tq_primary_bits"] == "5" and meta["tq_residual_bits"] == "4"
    t = load_file(str(out / "model.safetensors"))
    name = "model.layers.0.mlp.up_proj"
    pp, pr = t[name + ".packed_primary"], t[name + ".packed_residual"]
    assert pp.shape == (96, 1024) and pr.shape == (96, 512) and int(pp.max()) < 32
    seeds = t[name + ".seeds"]
    assert seeds[1] != 0 and seeds[2] == 512                           # own residual rotation, block 512
    cbp, cbr = oracle.Codebook(t["tq_codebook_primary"], 5), oracle.Codebook(t["tq_codebook_residual"], 4)
    assert len(cbp.centroids) == 32 and len(cbr.centroids) == 16
    qw = oracle.QuantizedWeight(pp, pr, t[name + ".norms"], seeds)
    w_ref = oracle.dequantize_weight_cpu(qw, cbp, cbr, 512)
    assert np.linalg.norm(w_ref - w) / np.linalg.norm(w) < 0.15       # the bound of the reference's own round-trip tests
    layer = tq.TurboQuantLinear(1024, 96, qw, cbp, cbr, 512)
    assert layer.mode() == "dual_5bit"
    assert np.array_equal(layer.dequantize(), w_ref)
    for batch in (1, 6, 20):
        x = rng.standard_normal((batch, 1024)).astype(np.float32)
        y = layer.forward(x)
        ref = oracle.matmul_xwT(x, w_ref, acc_double=True)
        assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 1e-3
        xb = oracle.f32_to_bf16_bits(x)
        yb = layer.forward(xb, tq.BF16, tq.F32)
        refb = oracle.matmul_xwT(oracle.bf16_bits_to_f32(xb), w_ref, acc_double=True)
        assert np.linalg.norm(yb - refb) / np.linalg.norm(refb) < 1e-3
    layer.close()
