"""The code-free reader of TorchScript archives (rwkvstic_amd/archive.py) on an archive that carries the reference's
attribute tree as the reference's modules hold it (plain tensor attributes: they are not in state_dict()).  No
export of the reference itself exists here, so agreement with a real .rwkv file stays untested (parity unpinned)."""
import pickle
import zipfile

import pytest
import torch

from oracle import rwkv_oracle as O
from rwkvstic_amd import archive, synth

from archive_standins import write_archive


@pytest.fixture(scope="module")
def saved(tmp_path_factory):
    sd = synth.make_state_dict(layers=2, C=64, V=300, seed=14, ln="random")
    path = str(tmp_path_factory.mktemp("arc") / "model.rwkv")
    write_archive(sd, path)
    return sd, path


def test_reader_returns_the_reference_attribute_tree(saved):
    sd, path = saved
    tree = archive.read_archive_tensors(path)
    assert tree["emptyState"].shape == (2, 5, 64) and tree["emptyState"].dtype == torch.float64
    assert float(tree["emptyState"][1, 4, 3]) == -1e30
    assert torch.equal(tree["emb.w"], sd["emb.weight"])
    assert torch.equal(tree["ln_in.weight"], sd["blocks.0.ln0.weight"].double())
    assert torch.equal(tree["blocks.1.ln2.bias"], sd["blocks.1.ln2.bias"].double())
    names = {"blocks.1.att.weights.0.": ("att.key", "att.value", "att.receptance"), "blocks.1.attout.weights.0.": ("att.output",),
             "blocks.0.ffnkey.weights.0.": ("ffn.key",), "blocks.0.ffnvalue.weights.0.": ("ffn.value",),
             "blocks.1.ffnreceptance.weights.0.": ("ffn.receptance",)}
    for prefix, keys in names.items():
        for suffix, key in zip(("", "1", "2"), keys):
            c, r, o = O.quantize_matrix(sd[f"blocks.{prefix.split('.')[1]}.{key}.weight"].float())
            assert torch.equal(tree[prefix + "weight" + suffix], c) and tree[prefix + "weight" + suffix].dtype == torch.uint8
            assert torch.equal(tree[prefix + "range" + suffix], r) and torch.equal(tree[prefix + "offset" + suffix], o)
    c, r, o = O.quantize_matrix(sd["head.weight"].float())
    assert torch.equal(tree["head.weights.0.weight"], c) and torch.equal(tree["head.weights.0.offset"], o)
    assert tree["blocks.0.attmix"].shape == (3, 1, 64) and tree["blocks.1.ffnmix"].shape == (2, 1, 64)
    assert torch.equal(tree["blocks.0.attmix"][1, 0], sd["blocks.0.att.time_mix_v"].reshape(-1).double())
    assert torch.equal(tree["blocks.1.time_decay"], sd["blocks.1.att.time_decay"].double().exp().neg())
    # what torch.jit.load would give for the same file (this test's own archive): the plain attributes are not in
    # its state_dict, the reader still finds them, with the same values
    loaded = torch.jit.load(path, map_location="cpu")
    assert "head.weights.0.weight" not in loaded.state_dict()
    assert torch.equal(getattr(loaded.head.weights, "0").weight, tree["head.weights.0.weight"])
    assert torch.equal(getattr(getattr(loaded.blocks, "1").att.weights, "0").range2, tree["blocks.1.att.weights.0.range2"])


def test_reader_keeps_non_tensor_attributes_inert(saved):
    _, path = saved
    root = archive.read_archive_object(path)
    assert isinstance(root, archive.ScriptObject) and root.qualified_name.startswith("__torch__.")
    mm = root.head.weights.__dict__["0"]
    assert mm.M == 64 and mm.N == 300 and mm.device == "cpu" and mm.stream is False
    assert root.ln_in.device == "cpu"                     # a torch.device attribute comes back as its name


def test_reader_refuses_anything_but_tensor_data(tmp_path, saved):
    """A data.pkl that names an ordinary Python callable is refused, not resolved."""
    _, path = saved
    evil = str(tmp_path / "evil.rwkv")
    with zipfile.ZipFile(path) as src, zipfile.ZipFile(evil, "w") as dst:
        for item in src.infolist():
            data = src.read(item.filename)
            if item.filename.endswith("/data.pkl"):
                data = pickle.dumps(print)                # GLOBAL builtins.print
            dst.writestr(item, data)
    with pytest.raises(pickle.UnpicklingError, match="builtins"):
        archive.read_archive_tensors(evil)
    with pytest.raises(ValueError):
        plain = str(tmp_path / "plain.zip")
        with zipfile.ZipFile(plain, "w") as z:
            z.writestr("readme.txt", "x")
        archive.read_archive_tensors(plain)
