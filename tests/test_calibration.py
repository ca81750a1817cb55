"""Calibration artefact format and the two rules behind its entries (no GPU needed)."""
import math

import pytest
import torch

from arcquant_amd import calibration as cal


def test_reorder_index_sorts_ascending_and_is_stable():
    stat = torch.tensor([3.0, 0.5, 3.0, 9.0, 0.5])
    idx = cal.reorder_index_from_stat(stat)
    assert idx.tolist() == [1, 4, 0, 2, 3]            # outliers last, ties in original order
    assert cal.is_permutation(idx)
    assert not cal.is_permutation(torch.tensor([0, 0, 1]))
    assert not cal.is_permutation(torch.tensor([0.0, 1.0]))


def brute_select_num(keys, gran=64):
    K = len(keys[0])
    cnt = 0
    for row in keys:
        thr = max(row) * 0.125
        cnt += sum(1 for v in row if v > thr)
    return min(math.ceil(K * (cnt / (len(keys) * K)) / gran) * gran, K)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_select_num_matches_loop(seed):
    g = torch.Generator().manual_seed(seed)
    keys = torch.randn(7, 256, generator=g)
    keys[:, :5] *= 30
    want = brute_select_num(keys.tolist())
    assert cal.select_num_from_activations(keys) == want
    assert cal.select_num_from_activations(keys.view(1, 7, 256)) == want


def test_select_num_closed_forms():
    K = 256
    # one dominant channel: only it exceeds max/8 -> 1/K of the values -> one granule of 64
    keys = torch.ones(10, K)
    keys[:, 17] = 100.0
    assert cal.select_num_from_activations(keys) == 64
    # all equal and positive: every value exceeds an eighth of the max -> capped at K
    assert cal.select_num_from_activations(torch.ones(4, K)) == K
    # all negative: the signed max is negative, max/8 is ABOVE the max -> nothing selected
    assert cal.select_num_from_activations(-torch.ones(4, K) - torch.rand(4, K)) == 0
    # 100 of 256 channels large in every token -> ceil(100/64)*64
    keys = torch.full((3, K), 0.01)
    keys[:, :100] = 5.0
    assert cal.select_num_from_activations(keys) == 128
    assert cal.average_bits(4096, 256) == pytest.approx(4.5 * 4352 / 4096)


def test_round_trip_in_the_reference_file_format(tmp_path):
    names = [cal.NAME_TEMPLATE.format(0, "self_attn", "q_proj"), cal.NAME_TEMPLATE.format(0, "mlp", "down_proj")]
    assert names[0] == "layers.0.self_attn.q_proj.input"           # model/qLlamaLayer.py:237-241
    idx = {names[0]: torch.randperm(128), names[1]: torch.randperm(512)}
    sel = {names[0]: 64, names[1]: 128}
    cal.save_reorder_index(tmp_path / "ri.pt", idx)
    cal.save_select_num(tmp_path / "sn.pt", sel)
    idx2, sel2 = cal.load_reorder_index(tmp_path / "ri.pt"), cal.load_select_num(tmp_path / "sn.pt")
    assert sel2 == sel and all(torch.equal(idx[k], idx2[k]) for k in idx)
    # a plain torch.save of the same dicts (what the reference writes, reorder_indices.py:92-95) loads too
    torch.save(idx, tmp_path / "ref.pt")
    assert set(cal.load_reorder_index(tmp_path / "ref.pt")) == set(idx)
    torch.save({names[0]: torch.tensor([0, 0, 1])}, tmp_path / "bad.pt")
    with pytest.raises(ValueError):
        cal.load_reorder_index(tmp_path / "bad.pt")
    with pytest.raises(ValueError):
        cal.save_reorder_index(tmp_path / "bad2.pt", {names[0]: torch.tensor([2, 2, 0])})
    assert cal.kernel_index(idx[names[0]], device="cpu").dtype == torch.int16
