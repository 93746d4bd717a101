"""CHR0 container: the specification's byte-level example, the reader's refusals
(docs/spec/chr0.md appendix B), and the way from a file to the decoder's weight seats."""

from __future__ import annotations

import json
import os
import struct

import numpy as np
import pytest
import torch

from deepfold_amd import chr0

# docs/spec/chr0.md section 2.4: the header of the three-tensor toy model, byte for byte
# (tests/golden/chr0_toy_header.json, no trailing newline)
GOLDEN_JSON = open(os.path.join(os.path.dirname(__file__), "golden", "chr0_toy_header.json"),
                   encoding="utf-8").read()


def toy_entries(seed=0):
    rng = np.random.default_rng(seed)

    def blob(n):
        return rng.integers(0, 256, n, dtype=np.uint8).tobytes()

    return [
        chr0.TensorEntry("model.layers.0.self_attn.q_proj", "nf4", (64, 64), {"data": blob(2048), "scale": blob(128)}),
        chr0.TensorEntry("model.layers.0.mlp.down_proj", "nf4", (32, 128), {"data": blob(2048), "scale": blob(128)}),
        chr0.TensorEntry("model.norm", "bf16", (64,), {"data": blob(128)}),
    ]


ROOT = dict(arch="toy", hidden_size=64, intermediate_size=128, num_layers=1, vocab_size=0)


@pytest.fixture()
def toy(tmp_path):
    path = tmp_path / "toy.chr"
    entries = toy_entries()
    size = chr0.write_chr(path, entries, **ROOT)
    return path, entries, size


def test_writer_reproduces_the_specification_example(toy):
    path, _, size = toy
    raw = path.read_bytes()
    assert len(GOLDEN_JSON) == 516 and size == 5056 == len(raw)
    assert raw[:8] == bytes.fromhex("0402000000000000")
    assert raw[8:524].decode() == GOLDEN_JSON
    assert raw[524:576] == bytes(52)
    assert not (tmp_path_part := path.with_suffix(".chr.part")).exists(), tmp_path_part


def test_reader_describes_the_example(toy):
    path, entries, size = toy
    h = chr0.load_header(path)
    assert (h.header_nbytes, h.payload_start, h.file_size) == (516, 576, size)
    assert (h.arch, h.hidden_size, h.intermediate_size, h.num_layers, h.vocab_size) == ("toy", 64, 128, 1, 0)
    q = h.tensor("model.layers.0.self_attn.q_proj")
    assert (q.kind, q.codec, q.layer, q.M, q.K, q.K_pad, q.n_groups) == ("q", "nf4", 0, 64, 64, 64, 1)
    assert (q.blobs["data"].start, q.blobs["data"].end, q.blobs["scale"].nbytes) == (576, 2624, 128)
    n = h.tensor("model.norm")
    assert n.layer is None and n.codec == "bf16" and n.blobs["data"].nbytes == 128
    assert list(chr0.iter_linears(h)) == ["model.layers.0.self_attn.q_proj", "model.layers.0.mlp.down_proj"]
    assert chr0.quantized_codec(h) == "nf4"
    assert "model.norm" in h and "nope" not in h
    with pytest.raises(chr0.TensorNotFoundError):
        h.tensor("model.layers.0.self_attn.q_proj.weight")  # no .weight alias
    raw = path.read_bytes()
    for e in entries:
        for key, blob in e.blobs.items():
            b = h.tensor(e.name).blobs[key]
            assert raw[b.start:b.end] == blob


def test_materialize_returns_the_file_bytes(toy):
    path, entries, _ = toy
    m = chr0.materialize_nf4(path, "model.layers.0.mlp.down_proj", "cpu")
    assert (m.M, m.K, m.K_pad, m.n_groups, m.nbytes) == (32, 128, 128, 2, 2048 + 128)
    assert m.packed.dtype == torch.uint8 and tuple(m.packed.shape) == (32, 64)
    assert m.scale.dtype == torch.float16 and tuple(m.scale.shape) == (32, 2)
    assert m.packed.numpy().tobytes() == entries[1].blobs["data"]
    assert m.scale.view(torch.int16).numpy().tobytes() == entries[1].blobs["scale"]
    before = path.read_bytes()
    chr0.read_bf16(path, "model.norm", "cpu")
    assert path.read_bytes() == before
    with pytest.raises(chr0.CodecError):
        chr0.materialize_nf4(path, "model.norm", "cpu")
    with pytest.raises(chr0.CodecError):
        chr0.read_bf16(path, "model.layers.0.mlp.down_proj", "cpu")


def test_k65_pads_to_128(tmp_path):
    e = [chr0.TensorEntry("model.layers.0.mlp.up_proj", "nf4", (3, 65), {"data": bytes(3 * 64), "scale": bytes(12)})]
    path = tmp_path / "pad.chr"
    chr0.write_chr(path, e, **ROOT)
    t = chr0.load_header(path).tensor("model.layers.0.mlp.up_proj")
    assert (t.K, t.K_pad, t.n_groups, t.shape) == (65, 128, 2, (3, 65))
    assert chr0.blob_sizes("nf4", (3, 70)) == {"data": 192, "scale": 12}     # section 7.4
    assert chr0.blob_sizes("vq", (3, 70)) == {"codebook": 8192, "index": 54}
    assert [chr0.align64(x) for x in (0, 1, 64, 524, 582)] == [0, 64, 64, 576, 640]


def test_names_and_kinds():
    assert chr0.chr_name("model.layers.0.mlp.up_proj.weight") == "model.layers.0.mlp.up_proj"
    assert chr0.chr_name("foo.weight.weight") == "foo.weight"
    assert chr0.chr_name("foo.weight_scale") == "foo.weight_scale"
    want = {"a.q_proj": "q", "a.q_proj.bias": "q", "a.q_norm": "norm", "attention.wqkv": "qkv",
            "attention.wo": "o", "experts.3.w1": "gate", "experts.3.w3": "up", "experts.3.w2": "down",
            "model.embed_tokens": "embed", "wte": "embed", "lm_head": "lm_head", "model.norm": "norm",
            "x.my_rmsnorm_2": "norm", "rotary_emb.inv_freq": "other", "mlp.gate": "other"}
    for name, kind in want.items():
        assert chr0.kind_of(name) == kind, name


# ---- refusals -------------------------------------------------------------------------

def rebuild(path, mutate, *, file_pad=0):
    """Rewrite the toy file with ``mutate`` applied to its header object; blobs keep their
    place as long as the header does not outgrow its 568 bytes."""
    raw = path.read_bytes()
    obj = json.loads(raw[8:524])
    mutate(obj)
    text = json.dumps(obj, separators=(",", ":")).encode()
    assert 8 + len(text) <= 576
    out = struct.pack("<Q", len(text)) + text + bytes(576 - 8 - len(text)) + raw[576:] + bytes(file_pad)
    path.write_bytes(out)
    return path


def q_of(obj):
    return obj["tensors"]["model.layers.0.self_attn.q_proj"]


@pytest.mark.parametrize("size", [0, 3, 7])
def test_short_files(tmp_path, size):
    p = tmp_path / "short.chr"
    p.write_bytes(bytes(size))
    with pytest.raises(chr0.TruncatedError):
        chr0.load_header(p)


def test_length_word_lies(toy, tmp_path):
    path, _, _ = toy
    raw = path.read_bytes()
    for n in (0, 1, len(raw), 100_000_001):
        p = tmp_path / f"n{n}.chr"
        p.write_bytes(struct.pack("<Q", n) + raw[8:])
        with pytest.raises(chr0.HeaderError):
            chr0.load_header(p)
    for n in (515, 517):  # cuts the object / runs into the padding
        p = tmp_path / f"n{n}.chr"
        p.write_bytes(struct.pack("<Q", n) + raw[8:])
        with pytest.raises(chr0.HeaderError):
            chr0.load_header(p)


@pytest.mark.parametrize("body", [b"\xef\xbb\xbf{}", b"[1,2]", b"{}{}", b'{"a":1}\x00', b"{\xff}", b"nul"])
def test_broken_json(tmp_path, body):
    p = tmp_path / "bad.chr"
    p.write_bytes(struct.pack("<Q", len(body)) + body + bytes(128))
    with pytest.raises(chr0.HeaderError):
        chr0.load_header(p)


MUTATIONS = [
    (lambda o: o.update(magic="chr0"), chr0.HeaderError),
    (lambda o: o.update(version=2), chr0.HeaderError),
    (lambda o: o.update(version=True), chr0.HeaderError),
    (lambda o: o.update(hidden_size="64"), chr0.HeaderError),
    (lambda o: o.update(hidden_size=0), chr0.HeaderError),
    (lambda o: o.update(arch=""), chr0.HeaderError),
    (lambda o: o["tile"].update(row=32), chr0.HeaderError),
    (lambda o: o.update(tensors={}), chr0.HeaderError),
    (lambda o: o.update(extra=1), chr0.HeaderError),
    (lambda o: o.pop("vocab_size"), chr0.HeaderError),
    (lambda o: q_of(o).update(codec="bf16", **{"data": [576, 576 + 8192]}), chr0.CodecError),   # bf16 keeps group_size
    (lambda o: o["tensors"]["model.norm"].update(codec="nf4", group_size=64, scale=[5120, 5122]), chr0.CodecError),
    (lambda o: q_of(o).update(data=[576, 2625]), chr0.SizeMismatchError),
    (lambda o: q_of(o).update(data=[575, 2623]), chr0.AlignmentError),
    (lambda o: q_of(o).update(data=[2752, 4800]), chr0.OverlapError),
    (lambda o: q_of(o).pop("layer"), chr0.HeaderError),
    (lambda o: q_of(o).update(layer=1), chr0.HeaderError),
    (lambda o: o["tensors"]["model.norm"].update(layer=0), chr0.HeaderError),
    (lambda o: q_of(o).update(group_size=32), chr0.GroupSizeError),
    (lambda o: q_of(o).update(kind="query"), chr0.HeaderError),
    (lambda o: q_of(o).update(codec="fp8"), chr0.CodecError),
    (lambda o: q_of(o).update(zero=[8192, 8320]), chr0.CodecError),
    (lambda o: q_of(o).update(shape=[64, 64, 1]), chr0.HeaderError),
    (lambda o: q_of(o).update(shape=[64, 0]), chr0.HeaderError),
    (lambda o: q_of(o).pop("scale"), chr0.CodecError),
    (lambda o: q_of(o).update(data=[0, 2048]), chr0.OverlapError),   # inside the header
]


@pytest.mark.parametrize("case", range(len(MUTATIONS)))
def test_header_refusals(toy, case):
    path, _, _ = toy
    mutate, error = MUTATIONS[case]
    with pytest.raises(error):
        chr0.load_header(rebuild(path, mutate))


def test_mixed_codecs_are_refused(tmp_path):
    def vq(o):
        q_of(o).clear()
        q_of(o).update(layer=0, kind="q", codec="vq", shape=[64, 64], group_size=8, n_codebooks=2,
                       codebook_bits=8, codebook=[5120, 5120 + 8192], index=[13312, 13312 + 1024])
    path = tmp_path / "mix.chr"
    chr0.write_chr(path, toy_entries(), **ROOT)
    with pytest.raises(chr0.CodecError):
        chr0.load_header(rebuild(path, vq, file_pad=16384))


def test_float_and_duplicate_offsets_are_refused(toy, tmp_path):
    path, _, _ = toy
    raw = path.read_bytes()
    for old, new in ((b'"data":[576,2624]', b'"data":[576.0,2624]'), (b'"data":[576,2624]', b'"data":[576,2.6e3]'),
                     (b'"vocab_size":0', b'"vocab_size":0,"vocab_size":0'), (b'"hidden_size":64', b'"hidden_size":NaN')):
        text = raw[8:524].replace(old, new)
        p = tmp_path / "f.chr"
        p.write_bytes(struct.pack("<Q", len(text)) + text + bytes(576 - 8 - len(text)) + raw[576:])
        with pytest.raises(chr0.HeaderError):
            chr0.load_header(p)


def test_truncated_payload(toy):
    path, _, size = toy
    raw = path.read_bytes()
    path.write_bytes(raw[:4000])  # the header is whole, down_proj's bytes are not
    with pytest.raises(chr0.TruncatedError):
        chr0.load_header(path)
    # a header that validated earlier does not protect a later short read
    path.write_bytes(raw)
    h = chr0.load_header(path)
    path.write_bytes(raw[:4000])
    with pytest.raises(chr0.TruncatedError):
        chr0.materialize_nf4(path, "model.layers.0.mlp.down_proj", "cpu", header=h)
    path.write_bytes(raw + bytes(100))  # bytes after the last blob are ignored
    assert chr0.load_header(path).file_size == size + 100


def test_writer_refusals(tmp_path):
    p = tmp_path / "w.chr"
    e = toy_entries()
    with pytest.raises(chr0.Chr0Error):
        chr0.write_chr(p, [], **ROOT)
    with pytest.raises(chr0.Chr0Error):
        chr0.write_chr(p, [e[0], e[0]], **ROOT)
    with pytest.raises(chr0.Chr0Error):
        chr0.write_chr(p, [chr0.TensorEntry("model.norm", "nf4", (64, 64), e[0].blobs)], **ROOT)
    with pytest.raises(chr0.Chr0Error):
        chr0.write_chr(p, [chr0.TensorEntry("a.q_proj", "nf4", (64, 64), {"data": bytes(5), "scale": bytes(128)})], **ROOT)
    with pytest.raises(chr0.Chr0Error):
        chr0.write_chr(p, [chr0.TensorEntry("a.q_proj", "nf4", (64, 64), {"data": bytes(2048)})], **ROOT)
    assert not p.exists() and not (tmp_path / "w.chr.part").exists()


# ---- from a file to the decoder (GPU) ---------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("family", ["llama", "internlm"])
def test_decoder_from_a_chr_file_equals_the_synthetic_model(tmp_path, family):
    from deepfold_amd import decodev2 as dv2
    from deepfold_amd.decodev2.synth import build
    from oracle import step_oracle as so

    spec = dv2.TINY_LLAMA if family == "llama" else dv2.TINY_INTERNLM
    print("chr decoder", spec.name, flush=True)
    model = build(spec, 3, packed_embed=True)
    path = tmp_path / "tiny.chr"
    size = dv2.write_synth_chr(model, path)
    hdr = chr0.load_header(path)
    assert hdr.file_size == size and hdr.num_layers == spec.n_layers and hdr.arch == spec.family
    m = chr0.materialize_nf4(path, "lm_head", "cuda", header=hdr)
    assert m.packed.is_cuda and m.packed.cpu().numpy().tobytes() == np.ascontiguousarray(model.lm_head.packed).tobytes()
    prompt = [4, 5, 6, 7, 1, 2]
    want = so.greedy_ids(model, prompt, 8)
    outs = []
    for weights in (dv2.DeviceWeights.from_synth(model, "cuda"), dv2.weights_from_chr(path, spec)):
        state = dv2.DecodeState.allocate(spec, device="cuda")
        outs.append(dv2.generate(state, weights, prompt, 8))
    assert outs[0] == outs[1] == want
    with pytest.raises(ValueError):
        dv2.weights_from_chr(path, dv2.MEDIUM_LLAMA)
    with pytest.raises(ValueError):
        dv2.write_synth_chr(build(spec, 3), tmp_path / "dense.chr")
