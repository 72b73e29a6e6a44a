"""The safetensors reader and load_with_cast (ug_amd/csrc/host/ug/safetensors.cpp, after
ug-core/src/safetensors.rs) on the CPU oracle device, where every conversion runs on the host.
Files come from two independent writers: the `safetensors` package and ug_amd/st_writer.py."""
import os
import struct

import numpy as np
import pytest

from ug_amd import st_writer as st_files
import ug_amd
from ug_amd import rng

DT = {"BF16": ug_amd.BF16, "F16": ug_amd.F16, "F32": ug_amd.F32, "I32": ug_amd.I32, "I64": ug_amd.I64}


def sample_values(n):
    """Floats that exercise rounding, saturation and the specials."""
    x = (rng.normal(3, n) * np.float32(300.0)).astype(np.float32)
    x[:12] = [0.0, -0.0, 1.0, -1.0, 0.5, 1.00390625, 65504.0, 70000.0, 3e9, -3e9, np.inf, -np.inf]
    x[12] = np.nan
    x[13:16] = [1e-8, 6.1e-5, 5.9e-8]   # underflow / f16 subnormals
    return x


def np_from_f32(x, dt):
    """numpy statement of half::{bf16,f16}::from_f32 and Rust's `as` for f32 -> integer."""
    if dt == "F32":
        return x.copy()
    if dt == "BF16":
        out = rng.to_bf16_bits(x)
        nan = np.isnan(x)
        out[nan] = ((x.view(np.uint32)[nan] >> 16) | 0x40).astype(np.uint16)
        return out
    if dt == "F16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16)
    info = np.iinfo(np.int32 if dt == "I32" else np.int64)
    t = np.trunc(np.nan_to_num(x.astype(np.float64), nan=0.0, posinf=np.inf, neginf=-np.inf))
    t = np.clip(t, float(info.min), float(info.max))
    out = np.empty(x.shape, info.dtype)
    big = t >= float(info.max)
    out[big] = info.max
    out[~big] = t[~big].astype(info.dtype)
    return out


def np_to_f32(raw, dt):
    if dt == "BF16":
        return rng.from_bf16_bits(raw)
    return raw.astype(np.float32)


def expected(raw, src, dst):
    if src == dst:
        return raw
    if src == "I32" and dst == "I64":
        return raw.astype(np.int64)
    if src == "I64" and dst == "I32":
        return raw.astype(np.int64).astype(np.int32)    # wraps
    return np_from_f32(np_to_f32(raw, src), dst)


def raw_of(x, dt):
    if dt in ("I32", "I64"):
        v = np.clip(np.nan_to_num(x, nan=0.0, posinf=7.0, neginf=-7.0).astype(np.float64) * 1000.0, -2e9, 2e9)
        v[:4] = [2**31 - 1, -2**31, 16777217, -16777217]      # not representable in f32
        if dt == "I64":
            v = v.astype(np.int64)
            v[4:7] = [2**40 + 1, -2**40 - 1, 2**31]            # beyond i32
            return v
        return v.astype(np.int32)
    return np_from_f32(x, dt)


def bits(a):
    return a.view(np.uint16) if a.dtype == np.float16 else a


@pytest.fixture(scope="module")
def st_file(tmp_path_factory):
    x = sample_values(1000)
    path = str(tmp_path_factory.mktemp("st") / "all_dtypes.safetensors")
    tensors = [(f"t.{dt.lower()}", dt, (10, 100), raw_of(x, dt)) for dt in DT]
    tensors.insert(2, ("odd", "F32", (3,), np.array([1, 2, 3], np.float32)))   # shifts later tensors off 8-byte alignment
    tensors.append(("bytes", "U8", (5,), np.arange(5, dtype=np.uint8)))
    tensors.append(("empty", "F32", (0, 4), np.zeros(0, np.float32)))
    st_files.write_safetensors(path, tensors, metadata={"format": "pt"}, pad_header_to=1)
    return path, {name: (dt, shape, arr) for name, dt, shape, arr in tensors}


def test_header_and_listing(st_file):
    path, tensors = st_file
    st = ug_amd.Safetensors(path)
    listed = st.tensors()
    assert [t[0] for t in listed] == list(tensors)
    for name, dt, shape, nbytes in listed:
        assert (dt, tuple(shape)) == (tensors[name][0], tuple(tensors[name][1]))
        assert nbytes == tensors[name][2].nbytes


@pytest.mark.parametrize("src", list(DT))
def test_load_keeps_the_stored_dtype(cpu, st_file, src):
    path, tensors = st_file
    st = ug_amd.Safetensors(path)
    lb = st.load(f"t.{src.lower()}", cpu)
    assert lb.dtype == DT[src] and lb.dims() == [10, 100]
    np.testing.assert_array_equal(bits(lb.data_vec()), bits(tensors[f"t.{src.lower()}"][2]).ravel())


@pytest.mark.parametrize("dst", list(DT))
@pytest.mark.parametrize("src", list(DT))
def test_load_with_cast_on_the_host(cpu, st_file, src, dst):
    path, tensors = st_file
    st = ug_amd.Safetensors(path)
    name = f"t.{src.lower()}"
    if dst == "I64" and src in ("BF16", "F16"):
        # safetensors.rs:161-165,187-191 collect `as i32` values for an I64 slice: the upload fails
        with pytest.raises(ug_amd.UgError, match="dtype mismatch"):
            st.load(name, cpu, DT[dst])
        return
    lb = st.load(name, cpu, DT[dst])
    assert lb.dtype == DT[dst] and not st.last_cast_on_device
    want = expected(tensors[name][2], src, dst)
    got = lb.data_vec()
    if dst == "F32":
        np.testing.assert_array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))
    elif dst == "F16":
        w = want.view(np.uint16) if want.dtype == np.float16 else want
        g = got.view(np.uint16) if got.dtype == np.float16 else got
        nan = np.isnan(np_to_f32(tensors[name][2], src)) if src != "F16" else np.isnan(tensors[name][2])
        np.testing.assert_array_equal(g[~nan], w[~nan])
        assert np.all((g[nan] & 0x7c00) == 0x7c00) and np.all((g[nan] & 0x03ff) != 0)
    else:
        np.testing.assert_array_equal(got, want)


def test_against_the_safetensors_package(cpu, tmp_path):
    """A file written by the reference implementation of the format, and one of ours read by it."""
    st_np = pytest.importorskip("safetensors.numpy")
    data = {"a": rng.normal(5, 24).reshape(2, 3, 4), "b": np.arange(7, dtype=np.int64), "c": rng.normal(6, 8).astype(np.float16)}
    theirs = str(tmp_path / "theirs.safetensors")
    st_np.save_file(data, theirs, metadata={"k": "v"})
    st = ug_amd.Safetensors(theirs)
    for name, arr in data.items():
        lb = st.load(name, cpu)
        assert lb.dims() == list(arr.shape)
        np.testing.assert_array_equal(bits(lb.data_vec()), bits(arr).ravel())
    ours = str(tmp_path / "ours.safetensors")
    st_files.write_safetensors(ours, [(k, {"float32": "F32", "int64": "I64", "float16": "F16"}[str(v.dtype)], v.shape, v) for k, v in data.items()])
    back = st_np.load_file(ours)
    for name, arr in data.items():
        np.testing.assert_array_equal(back[name], arr)


def test_multi_routes_to_the_last_file(cpu, tmp_path):
    p1, p2 = str(tmp_path / "1.safetensors"), str(tmp_path / "2.safetensors")
    st_files.write_safetensors(p1, [("x", "F32", (2,), np.array([1, 2], np.float32)), ("only1", "I32", (1,), np.array([5], np.int32))])
    st_files.write_safetensors(p2, [("x", "F32", (2,), np.array([3, 4], np.float32))])
    st = ug_amd.Safetensors([p1, p2])
    assert st.load("x", cpu).data_vec().tolist() == [3.0, 4.0]
    assert st.load("only1", cpu).data_vec().tolist() == [5]
    with pytest.raises(ug_amd.UgError, match="cannot find tensor nope"):
        st.load("nope", cpu)


def test_errors(cpu, st_file, tmp_path):
    path, _ = st_file
    st = ug_amd.Safetensors(path)
    with pytest.raises(ug_amd.UgError, match="unsupported dtype for bytes: U8"):
        st.load("bytes", cpu)
    with pytest.raises(ug_amd.UgError, match="cannot find tensor missing"):
        st.load("missing", cpu)
    assert st.load("empty", cpu).dims() == [0, 4]
    assert st.load("empty", cpu, ug_amd.BF16).dtype == ug_amd.BF16
    with pytest.raises(ug_amd.UgError, match="No such file"):
        ug_amd.Safetensors(str(tmp_path / "absent.safetensors"))

    def broken(name, payload):
        p = str(tmp_path / name)
        with open(p, "wb") as f:
            f.write(payload)
        return p

    with pytest.raises(ug_amd.UgError, match="too small"):
        ug_amd.Safetensors(broken("short", b"abc"))
    with pytest.raises(ug_amd.UgError, match="header length"):
        ug_amd.Safetensors(broken("len", struct.pack("<Q", 1000) + b"{}"))
    with pytest.raises(ug_amd.UgError, match="invalid safetensors header"):
        ug_amd.Safetensors(broken("json", struct.pack("<Q", 4) + b"{,,}"))
    h = b'{"x":{"dtype":"F32","shape":[4],"data_offsets":[0,8]}}'
    with pytest.raises(ug_amd.UgError, match="shape and data_offsets disagree"):
        ug_amd.Safetensors(broken("size", struct.pack("<Q", len(h)) + h + b"\0" * 8))
    h = b'{"x":{"dtype":"F32","shape":[2],"data_offsets":[8,16]}}'
    with pytest.raises(ug_amd.UgError, match="do not tile"):
        ug_amd.Safetensors(broken("hole", struct.pack("<Q", len(h)) + h + b"\0" * 16))
    h = b'{"x":{"dtype":"F32","shape":[2],"data_offsets":[0,8]}}'
    with pytest.raises(ug_amd.UgError, match="longer than the tensors"):
        ug_amd.Safetensors(broken("tail", struct.pack("<Q", len(h)) + h + b"\0" * 12))


def test_llama_from_a_bf16_checkpoint_matches_rounded_synthetic_weights(cpu, cpu_ops, tmp_path):
    """A bf16 checkpoint of the synthetic weights, loaded with cast to f32, is the round_bf16 model."""
    import ctypes as C
    cfg = ug_amd.LlamaConfig(hidden_size=128, intermediate_size=320, max_position_embeddings=64, num_attention_heads=4, num_key_value_heads=2,
                             num_hidden_layers=2, vocab_size=512)
    h, isz, kv = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim * cfg.num_key_value_heads
    shapes = {"model.embed_tokens.weight": (cfg.vocab_size, h), "model.norm.weight": (h,)}
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        shapes.update({p + ".input_layernorm.weight": (h,), p + ".post_attention_layernorm.weight": (h,), p + ".mlp.gate_proj.weight": (isz, h),
                       p + ".mlp.up_proj.weight": (isz, h), p + ".mlp.down_proj.weight": (h, isz), p + ".self_attn.q_proj.weight": (h, h),
                       p + ".self_attn.k_proj.weight": (kv, h), p + ".self_attn.v_proj.weight": (kv, h), p + ".self_attn.o_proj.weight": (h, h)})
    tensors = []
    for name, shape in shapes.items():
        n = int(np.prod(shape))
        w = np.zeros(n, np.float32)
        assert ug_amd.host_lib().ugh_synthetic_weights(C.c_uint64(9), C.c_float(0.3), 0, name.encode(), C.c_size_t(n), w.ctypes.data_as(C.c_void_p)) == 0
        tensors.append((name, "BF16", shape, rng.to_bf16_bits(w)))
    path = str(tmp_path / "tiny_llama_bf16.safetensors")
    st_files.write_safetensors(path, tensors)
    prompt = rng.token_ids(10, 12, cfg.vocab_size)
    ids_file, st_file_ = ug_amd.LlamaModel.from_safetensors(cpu, cpu_ops, cfg, path, custom_softmax=True).generate(prompt, 6)
    ids_syn, st_syn = ug_amd.LlamaModel(cpu, cpu_ops, cfg, True, seed=9, std=0.3, round_bf16=True).generate(prompt, 6)
    assert ids_file.tolist() == ids_syn.tolist()
    np.testing.assert_array_equal(st_file_["margins"], st_syn["margins"])
