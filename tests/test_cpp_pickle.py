"""The C++ checkpoint reader (adrastea_amd/host/pickle.hpp, mirror of adrastea_models/src/
pickle.rs:33-338) against torch's own loader on checkpoints written here with torch.save:
names, dtypes, shapes, strides and the exact bytes of every tensor, the `_metadata` skip, the
nested-dict path, shared storages with offsets, non-contiguous strides, a Hugging Face style
sharded directory, and the error cases the reference names."""
import json
import os
import subprocess

import pytest
import torch

from adrastea_amd import build

DT = {torch.float16: ("f16", 2), torch.float32: ("f32", 4), torch.int64: ("i64", 8)}


def fnv1a64(b: bytes) -> int:
    h = 1469598103934665603
    for x in b:
        h = ((h ^ x) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def run(*args):
    r = subprocess.run([build.build_host_test(), *args], capture_output=True, text=True, timeout=60)
    return r.returncode, r.stdout


def expected_line(name, t):
    """What the reader must report for tensor t, derived from torch's view of it: the bytes of
    its storage from the storage offset to the last addressed element (pickle.rs:155-168)."""
    code, el = DT[t.dtype]
    largest = sum((d - 1) * s for d, s in zip(t.shape, t.stride()))
    raw = bytes(t.untyped_storage())
    lo = t.storage_offset() * el
    data = raw[lo:lo + (largest + 1) * el]
    dims = " ".join(str(d) for d in t.shape)
    strides = " ".join(str(s) for s in t.stride())
    return f"{name} {code} {t.dim()} {dims} {strides}", len(data), f"{fnv1a64(data):016x}"


def check(stdout, tensors):
    lines = [l for l in stdout.strip().splitlines() if l]
    assert len(lines) == len(tensors)
    for line, name in zip(lines, sorted(tensors)):        # the reference's BTreeMap order
        head, length, digest = expected_line(name, tensors[name])
        parts = line.split()
        assert " ".join(parts[:-3]) == head, line
        assert int(parts[-2]) - int(parts[-3]) == length, line
        assert parts[-1] == digest, line


def make_state():
    g = torch.Generator().manual_seed(3)
    base = torch.randn(6, 10, generator=g).half()
    return {
        "tok_embeddings.weight": torch.randn(12, 8, generator=g).half(),
        "layers.0.attention.wq.weight": torch.randn(8, 8, generator=g),
        "transposed": torch.randn(5, 7, generator=g).half().t(),         # strides (1, 7)
        "view_with_offset": base[2:5, 3:9],                               # offset 23, strides (10, 1)
        "same_storage_other_view": base[0],
        "steps": torch.arange(4, dtype=torch.int64),
        "vector": torch.randn(33, generator=g).half(),
    }


def test_reader_matches_torch_loader(tmp_path):
    state = make_state()
    path = str(tmp_path / "consolidated.00.pth")
    torch.save(state, path)
    rc, out = run("pickle", path)
    assert rc == 0, out
    back = torch.load(path, weights_only=True)
    check(out, back)
    for k in state:                                       # and torch read back what was written
        assert torch.equal(state[k], back[k])


def test_state_dict_with_metadata_and_nested_path(tmp_path):
    lin = torch.nn.Linear(5, 3).half()
    sd = lin.state_dict()                                  # an OrderedDict carrying _metadata
    path = str(tmp_path / "model.pt")
    torch.save({"model": sd, "epoch": 3, "lr": 0.25, "tag": "x"}, path)
    rc, out = run("pickle", path, "model")
    assert rc == 0, out
    check(out, torch.load(path, weights_only=True)["model"])
    rc, out = run("pickle", path, "missing")
    assert rc == 2 and "key not found" in out
    rc, out = run("pickle", path)                          # the top level holds non-tensors
    assert rc == 2 and "is not a tensor" in out


def test_sharded_huggingface_directory(tmp_path):
    g = torch.Generator().manual_seed(5)
    a = {"model.embed.weight": torch.randn(9, 4, generator=g).half(),
         "model.layers.0.w": torch.randn(4, 4, generator=g).half()}
    b = {"model.layers.1.w": torch.randn(4, 4, generator=g).half(),
         "lm_head.weight": torch.randn(9, 4, generator=g).half()}
    torch.save(a, str(tmp_path / "pytorch_model-00001-of-00002.bin"))
    torch.save(b, str(tmp_path / "pytorch_model-00002-of-00002.bin"))
    index = {"metadata": {"total_size": 1}, "weight_map": {
        **{k: "pytorch_model-00001-of-00002.bin" for k in a},
        **{k: "pytorch_model-00002-of-00002.bin" for k in b}}}
    (tmp_path / "pytorch_model.bin.index.json").write_text(json.dumps(index, indent=2))
    names = sorted({**a, **b})
    rc, out = run("sharded", str(tmp_path), *names)
    assert rc == 0, out
    lines = out.strip().splitlines()
    assert lines[0] == "shards 2"
    check("\n".join(lines[1:]), {**a, **b})
    rc, out = run("sharded", str(tmp_path), "nope")
    assert rc == 2 and "not found" in out


def test_rejects_what_the_reference_rejects(tmp_path):
    # compressed members (pickle.rs:240-242)
    import zipfile
    p = str(tmp_path / "compressed.pt")
    with zipfile.ZipFile(p, "w", zipfile.ZIP_DEFLATED) as z:
        z.writestr("archive/data.pkl", b"\x80\x02}q\x00." * 50)
    rc, out = run("pickle", p)
    assert rc == 2 and "compressed" in out
    # unsupported dtype (pickle.rs:147-152)
    p = str(tmp_path / "bf16.pt")
    torch.save({"w": torch.zeros(2, 2, dtype=torch.bfloat16)}, p)
    rc, out = run("pickle", p)
    assert rc == 2 and "unsupported dtype" in out
    # not an archive at all, and an archive without data.pkl
    p = str(tmp_path / "junk.pt")
    open(p, "wb").write(b"not a zip" * 10)
    rc, out = run("pickle", p)
    assert rc == 2 and "ERROR" in out
    p = str(tmp_path / "empty.zip")
    with zipfile.ZipFile(p, "w") as z:
        z.writestr("other.txt", b"hello")
    rc, out = run("pickle", p)
    assert rc == 2 and "data.pkl not found" in out


@pytest.mark.gpu
def test_checkpoint_to_u8_on_the_device(tmp_path):
    """zip/pickle -> [N, K] fp16 on the device -> adr_quantize_absmax_u8 -> (u8, scales), then
    dequantised again: every weight within half a quantisation step of the file's value, plus
    the two fp16 roundings of the format: of the scale (absmax / scale may exceed 127.5 by
    127.5 * 2^-11 before it is clamped) and of the dequantised number (half an fp16 step at up
    to 127.5 scales: 127.5 * 2^-11 again)."""
    assert os.path.exists(build.HOST_TEST_BIN)
    g = torch.Generator().manual_seed(9)
    path = str(tmp_path / "layer.pth")
    torch.save({"w": (torch.randn(256, 1024, generator=g) * 0.05).half()}, path)
    r = subprocess.run([build.HOST_TEST_BIN, "quantize", path, "w", "32"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    fields = r.stdout.split()
    assert fields[:4] == ["rows", "256", "cols", "1024"]
    assert float(fields[-1]) <= 0.5 + 2 * 127.5 * 2.0 ** -11 + 1e-3


def _zip64_archive(members, cd_off_delta=0, rec_off=None, lho=None, usize=None, extra_len=24,
                   extra_fields=3):
    """A zip archive with EVERY size and offset moved into zip64 records (legal for any size).
    The keyword arguments falsify single fields, for the hostile-archive tests."""
    import struct
    import zipfile
    blob, central = b"", b""
    for name, data in members:
        nb = name.encode()
        off = len(blob)
        # local header: sizes 0xFFFFFFFF + zip64 extra (uncompressed, compressed)
        extra = struct.pack("<HHQQ", 1, 16, len(data), len(data))
        blob += struct.pack("<IHHHHHIIIHH", 0x04034b50, 45, 0, 0, 0, 0, zipfile.crc32(data),
                            0xFFFFFFFF, 0xFFFFFFFF, len(nb), len(extra)) + nb + extra + data
        fields = [len(data) if usize is None else usize, len(data), off if lho is None else lho]
        cextra = struct.pack("<HH", 1, extra_len) + b"".join(struct.pack("<Q", f)
                                                              for f in fields[:extra_fields])
        central += struct.pack("<IHHHHHHIIIHHHHHII", 0x02014b50, 45, 45, 0, 0, 0, 0,
                               zipfile.crc32(data), 0xFFFFFFFF, 0xFFFFFFFF, len(nb), len(cextra),
                               0, 0, 0, 0, 0xFFFFFFFF) + nb + cextra
    cd_off = len(blob)
    real_rec = cd_off + len(central)
    rec = struct.pack("<IQHHIIQQQQ", 0x06064b50, 44, 45, 45, 0, 0, len(members), len(members),
                      len(central), (cd_off + cd_off_delta) & 0xFFFFFFFFFFFFFFFF)
    loc = struct.pack("<IIQI", 0x07064b50, 0, real_rec if rec_off is None else rec_off, 1)
    eocd = struct.pack("<IHHHHIIH", 0x06054b50, 0, 0, 0xFFFF, 0xFFFF, 0xFFFFFFFF, 0xFFFFFFFF, 0)
    return blob + central + rec + loc + eocd


def _members_of(path):
    import zipfile
    with zipfile.ZipFile(path) as z:
        return [(i.filename, z.read(i.filename)) for i in z.infolist()]


def test_zip64_records(tmp_path):
    """Archives beyond 4 GiB carry their sizes and offsets in zip64 records.  A small archive is
    rewritten here with every size and offset moved into those records, so the reader's zip64
    branch is exercised without a 4 GiB file."""
    import zipfile
    state = {"w": torch.arange(24, dtype=torch.float32).reshape(4, 6).half(),
             "b": torch.arange(5, dtype=torch.int64)}
    src = str(tmp_path / "small.pt")
    torch.save(state, src)
    dst = str(tmp_path / "zip64.pt")
    open(dst, "wb").write(_zip64_archive(_members_of(src)))
    with zipfile.ZipFile(dst) as z:                        # Python's reader accepts it too
        assert z.testzip() is None
    rc, out = run("pickle", dst)
    assert rc == 0, out
    lines = out.strip().splitlines()
    ref_rc, ref_out = run("pickle", src)
    # same tensors and bytes as the plain archive (file offsets differ)
    strip = lambda ls: [" ".join(l.split()[:-3]) + " " + l.split()[-1] for l in ls]
    assert ref_rc == 0 and strip(lines) == strip(ref_out.strip().splitlines())
    check(out, state)


@pytest.mark.parametrize("knob", [
    dict(cd_off_delta=-(1 << 20)),                 # directory offset wraps to just below 2^64
    dict(cd_off_delta=1 << 40),                    # ... or lies far beyond the file
    dict(rec_off=(1 << 64) - 40),                  # zip64 record offset + 56 wraps
    dict(lho=(1 << 64) - 16),                      # local header offset + 30 wraps
    dict(usize=(1 << 64) - 8),                     # member size: start + size wraps
    dict(usize=1 << 50),                           # ... or simply runs past the end
    dict(extra_len=24, extra_fields=1),            # zip64 extra field shorter than it claims
    dict(extra_len=8, extra_fields=3),             # ... and fields beyond the declared length
], ids=lambda k: "_".join(k))
def test_hostile_zip_fields_are_rejected_not_followed(tmp_path, knob):
    """Offsets and sizes come from the file: a crafted value must fail the range check (also
    where a sum of two such values would wrap around 2^64), never be used as an address."""
    src = str(tmp_path / "small.pt")
    torch.save({"w": torch.arange(24, dtype=torch.float32).reshape(4, 6).half()}, src)
    dst = str(tmp_path / "hostile.pt")
    open(dst, "wb").write(_zip64_archive(_members_of(src), **knob))
    rc, out = run("pickle", dst)
    assert rc == 2 and "ERROR" in out, (rc, out)


@pytest.mark.parametrize("dim0", [1 << 62, (1 << 64) // 6 + 2, 1 << 40])
def test_tensor_span_overflow_is_rejected(tmp_path, dim0):
    """A shape whose byte span wraps around 2^64 (or merely exceeds its storage) must not pass
    the span check with a small wrapped value."""
    import zipfile
    src = str(tmp_path / "small.pt")
    torch.save({"w": torch.arange(24, dtype=torch.float32).reshape(4, 6).half()}, src)
    members = _members_of(src)
    patched = []
    for name, data in members:
        if name.endswith("data.pkl"):
            old = b"K\x04K\x06\x86"                     # the shape tuple (4, 6)
            assert data.count(old) == 1
            data = data.replace(old, b"\x8a\x09" + dim0.to_bytes(9, "little")[:9] + b"K\x06\x86"
                                if dim0 >= 1 << 63 else
                                b"\x8a\x08" + dim0.to_bytes(8, "little") + b"K\x06\x86")
        patched.append((name, data))
    dst = str(tmp_path / "span.pt")
    with zipfile.ZipFile(dst, "w", zipfile.ZIP_STORED) as z:
        for name, data in patched:
            z.writestr(name, data)
    rc, out = run("pickle", dst)
    assert rc == 2 and "ERROR" in out, (rc, out)


# ---- LLaMA tensor names and the Hugging Face query/key row order (llama.rs:70-243) ---------------

LLAMA = dict(dim=16, n_heads=2, hidden=24, vocab=11, layers=2)


def _meta_llama_state():
    g = torch.Generator().manual_seed(17)
    r = lambda *s: torch.randn(*s, generator=g).half()
    d, hid, v = LLAMA["dim"], LLAMA["hidden"], LLAMA["vocab"]
    st = {"tok_embeddings.weight": r(v, d), "norm.weight": r(d), "output.weight": r(v, d)}
    for l in range(LLAMA["layers"]):
        st.update({f"layers.{l}.attention_norm.weight": r(d), f"layers.{l}.ffn_norm.weight": r(d),
                   f"layers.{l}.attention.wq.weight": r(d, d), f"layers.{l}.attention.wk.weight": r(d, d),
                   f"layers.{l}.attention.wv.weight": r(d, d), f"layers.{l}.attention.wo.weight": r(d, d),
                   f"layers.{l}.feed_forward.w1.weight": r(hid, d), f"layers.{l}.feed_forward.w2.weight": r(d, hid),
                   f"layers.{l}.feed_forward.w3.weight": r(hid, d)})
    return st


def _address_order(layers):
    """(Meta name, Hugging Face name) in the order the C++ driver walks the addresses."""
    out = [("tok_embeddings.weight", "model.embed_tokens.weight")]
    for l in range(layers):
        m, h = f"layers.{l}.", f"model.layers.{l}."
        out += [(m + "attention_norm.weight", h + "input_layernorm.weight"),
                (m + "attention.wq.weight", h + "self_attn.q_proj.weight"),
                (m + "attention.wk.weight", h + "self_attn.k_proj.weight"),
                (m + "attention.wv.weight", h + "self_attn.v_proj.weight"),
                (m + "attention.wo.weight", h + "self_attn.o_proj.weight"),
                (m + "ffn_norm.weight", h + "post_attention_layernorm.weight"),
                (m + "feed_forward.w1.weight", h + "mlp.gate_proj.weight"),
                (m + "feed_forward.w3.weight", h + "mlp.up_proj.weight"),
                (m + "feed_forward.w2.weight", h + "mlp.down_proj.weight")]
    return out + [("norm.weight", "model.norm.weight"), ("output.weight", "lm_head.weight")]


def _check_loaded(stdout, names, state):
    lines = stdout.strip().splitlines()
    assert len(lines) == len(names)
    for line, (name, key) in zip(lines, names):
        t = state[key].contiguous()
        parts = line.split()
        dims = [str(x) for x in t.shape]
        assert parts[0] == name and parts[1] == "f16" and parts[2] == str(t.dim()), line
        assert parts[3:3 + t.dim()] == dims, line
        raw = t.numpy().tobytes()
        assert int(parts[-2]) == len(raw) and parts[-1] == f"{fnv1a64(raw):016x}", line


def test_meta_llama_loader_names(tmp_path):
    st = _meta_llama_state()
    path = str(tmp_path / "consolidated.00.pth")
    torch.save(st, path)
    rc, out = run("llama-meta", path, str(LLAMA["layers"]))
    assert rc == 0, out
    order = _address_order(LLAMA["layers"])
    _check_loaded(out, [(m, m) for m, _ in order], st)
    rc, out = run("llama-meta", path, str(LLAMA["layers"] + 1))       # a layer the file lacks
    assert rc == 2 and "layers.2.attention_norm.weight not found" in out


def test_huggingface_llama_loader_restores_meta_row_order(tmp_path):
    """A Hugging Face style checkpoint made from Meta-layout weights the way the transformers
    conversion script makes it (query/key rows of each head de-interleaved: view(n_heads,
    head/2, 2, dim).transpose(1, 2)), split over two shards, one key projection stored
    transposed (non-unit column stride): the loader must hand back Meta's weights bit for bit
    under the Hugging Face names, as contiguous [dim, dim] matrices for q and k."""
    st = _meta_llama_state()
    d, h = LLAMA["dim"], LLAMA["n_heads"]
    permute = lambda w: w.view(h, d // h // 2, 2, d).transpose(1, 2).reshape(d, d)
    order = _address_order(LLAMA["layers"])
    hf = {}
    for m, name in order:
        w = st[m]
        if name.endswith(("q_proj.weight", "k_proj.weight")):
            w = permute(w).contiguous()
            assert not torch.equal(w, st[m])
        hf[name] = w
    odd = "model.layers.1.self_attn.k_proj.weight"
    hf[odd] = hf[odd].t().contiguous().t()                            # strides (1, dim)
    assert hf[odd].stride() == (1, d)
    names = sorted(hf)
    shards = {"pytorch_model-00001-of-00002.bin": names[:len(names) // 2],
              "pytorch_model-00002-of-00002.bin": names[len(names) // 2:]}
    for f, ks in shards.items():
        torch.save({k: hf[k] for k in ks}, str(tmp_path / f))
    index = {"metadata": {}, "weight_map": {k: f for f, ks in shards.items() for k in ks}}
    (tmp_path / "pytorch_model.bin.index.json").write_text(json.dumps(index))
    rc, out = run("llama-hf", str(tmp_path), str(LLAMA["layers"]), str(d), str(h))
    assert rc == 0, out
    meta_under_hf_names = {name: st[m] for m, name in order}
    _check_loaded(out, [(name, name) for _, name in order], meta_under_hf_names)
    # every q/k line reports the contiguous layout, whatever the file had
    for line in out.strip().splitlines():
        if "q_proj" in line or "k_proj" in line:
            assert line.split()[3:7] == [str(d), str(d), str(d), "1"], line
    # the head split must divide
    rc, out = run("llama-hf", str(tmp_path), "1", str(d), "3")
    assert rc == 2 and "multiple of 2 * n_heads" in out
    rc, out = run("llama-hf", str(tmp_path), "1", "32", "2")          # wrong dim for the file
    assert rc == 2 and "not [dim, dim]" in out
