"""The tuning driver's optional recorded inputs (reference python/tests/attntuner_demo.py:38-43: q.pt, k.pt, v.pt, mask.pt
under --input_path, a singleton dimension dropped, the leading corner of the stored tensors used)."""
import pytest
import torch

from attention_autotuner_amd.benchmarks import tune


def test_recorded_inputs_replace_the_synthetic_tensors(tmp_path):
    g = torch.Generator().manual_seed(0)
    stored_q = torch.randn(3, 1, 4, 96, 64, generator=g)              # [B, 1, H, S, d] as the reference's files have it, fp32
    stored_k = torch.randn(3, 4, 128, 64, generator=g).half()
    stored_mask = torch.randn(4, 96, 128, generator=g).half()
    torch.save(stored_q, tmp_path / "q.pt")
    torch.save(stored_k, tmp_path / "k.pt")
    torch.save(stored_mask, tmp_path / "mask.pt")
    arrays = tune.make_tensors("ret", 2, 4, 64, 128, 64, 64, "cpu")
    synthetic_v = arrays[2].clone()
    out = tune.load_inputs(arrays, "ret", str(tmp_path), "cpu")
    assert out[0].shape == (2, 4, 64, 64) and out[0].dtype == torch.float16
    assert torch.equal(out[0], stored_q.squeeze(1)[:2, :4, :64, :64].half())      # singleton dropped, corner taken, cast
    assert torch.equal(out[1], stored_k[:2, :4, :128, :64])
    assert torch.equal(out[2], synthetic_v)                                          # no v.pt: the synthetic tensor stays
    assert torch.equal(out[3], stored_mask[:4, :64, :128])
    assert all(t.is_contiguous() for t in out[:4])


def test_recorded_inputs_must_cover_the_problem_and_are_loaded_as_plain_tensors(tmp_path):
    torch.save(torch.zeros(1, 2, 32, 64), tmp_path / "q.pt")                         # fewer rows than the problem has
    arrays = tune.make_tensors("attn", 1, 2, 64, 64, 64, 64, "cpu")
    with pytest.raises(ValueError, match="does not cover"):
        tune.load_inputs(arrays, "attn", str(tmp_path), "cpu")
    torch.save({"not": "a tensor", "fn": print}, tmp_path / "k.pt")                  # anything but plain data is refused by the loader
    (tmp_path / "q.pt").unlink()
    with pytest.raises(Exception):
        tune.load_inputs(tune.make_tensors("attn", 1, 2, 64, 64, 64, 64, "cpu"), "attn", str(tmp_path), "cpu")
