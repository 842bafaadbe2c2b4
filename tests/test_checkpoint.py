"""Hash-weight checkpoint handling (spotlight/modifier.py:62-76, train_results/convert.py:13-32),
host only."""
import pytest
import torch

from spotlight_amd.modifier import assign_checkpoint, merge_layer_files, read_checkpoint, write_checkpoint


def _layers(n_layers=3, heads=4):
    g = torch.Generator().manual_seed(0)
    mk = lambda *s: torch.nn.Parameter(torch.randn(*s, generator=g))
    return [[mk(1, heads, 128, 256), mk(1, heads, 1, 256), mk(1, heads, 256, 128), mk(1, heads, 1, 128)]
            for _ in range(n_layers)]


def test_round_trip_keeps_order_shapes_and_values(tmp_path):
    layers = _layers()
    flat = [p for ps in layers for p in ps]
    path = str(tmp_path / "a.pth")
    write_checkpoint(flat, path)
    ck = read_checkpoint(path)
    assert [tuple(t.shape) for t in ck] == [tuple(p.shape) for p in flat]
    target = _layers()
    for ps in target:
        for p in ps:
            p.data.zero_()
    assign_checkpoint(target, [0], ck)
    assert all(torch.equal(a, b) for a, b in zip([p for ps in target for p in ps], flat))


def test_training_layout_skips_dense_layers_and_casts_dtype():
    src = _layers()
    target = [[torch.nn.Parameter(torch.zeros_like(p, dtype=torch.bfloat16)) for p in ps] for ps in _layers()]
    ck = [p.detach() for i, ps in enumerate(src) if i != 1 for p in ps]      # layer 1 is dense: left out
    assign_checkpoint(target, [1], ck)
    assert all(p.dtype == torch.bfloat16 for ps in target for p in ps)
    assert torch.equal(target[0][0], src[0][0].to(torch.bfloat16)) and torch.equal(target[2][3], src[2][3].to(torch.bfloat16))
    assert float(target[1][0].detach().abs().sum()) == 0.0


def test_wrong_length_or_shape_is_an_error():
    target = _layers()
    flat = [p.detach() for ps in _layers() for p in ps]
    with pytest.raises(ValueError):
        assign_checkpoint(target, [0], flat[:5])
    flat[2] = flat[2][..., :64]
    before = target[0][0].detach().clone()
    with pytest.raises(ValueError):
        assign_checkpoint(target, [0], flat)
    assert torch.equal(target[0][0], before)          # nothing was assigned


def test_merge_layer_files_orders_by_layer_and_flattens(tmp_path):
    a, b, c = torch.full((2,), 1.0), torch.full((2,), 2.0), torch.full((2,), 3.0)
    torch.save([b, c], str(tmp_path / "2.pth"))
    torch.save(a, str(tmp_path / "0.pth"))
    (tmp_path / "notes.txt").write_text("ignored")
    out = merge_layer_files(str(tmp_path), num_layers=4)
    assert [float(t[0]) for t in out] == [1.0, 2.0, 3.0]
    with pytest.raises(ValueError):
        merge_layer_files(str(tmp_path), num_layers=2)


def test_only_lists_of_tensors_load(tmp_path):
    path = str(tmp_path / "d.pth")
    torch.save({"a": torch.zeros(1)}, path)
    with pytest.raises(ValueError):
        read_checkpoint(path)
