"""gla_jax_amd.selfcheck, the counterpart of the reference's `python gla.py` (gla.py:1275-1499): the three public
methods against each other on one seeded input, all seven results per pair."""
import io

import pytest
import torch

from gla_jax_amd import selfcheck as sc


def test_compare_reports_what_the_reference_prints():
    a = torch.tensor([1.0, 2.0, -3.0])
    b = torch.tensor([1.0, 2.5, -3.0])
    c = sc.compare(a, b)
    assert not c["allclose"] and c["max_abs"] == 0.5
    assert abs(c["rel_l2"] - 0.5 / 14 ** 0.5) < 1e-6
    assert sc.compare(a, a.clone()) == {"allclose": True, "max_abs": 0.0, "rel_l2": 0.0}


def test_cli_needs_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(SystemExit, match="GPU"):
        sc.main(["--seq-len", "64"])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,l2,reverse", [(torch.bfloat16, 1e-2, False), (torch.float32, 1e-5, False),
                                             (torch.bfloat16, 1e-2, True)])
def test_three_way_selfcheck_small_shape(dtype, l2, reverse):
    buf = io.StringIO()
    rep = sc.selfcheck(batch=2, seq_len=256, key_dim=256, head_dim=64, dtype=dtype, reverse=reverse, time_it=False,
                       gate_shift=3.0, seed=3, out=buf)
    text = buf.getvalue()
    assert set(rep["methods"]) == set(sc.METHODS)
    assert all("non_finite" not in e and e["first_call_s"] > 0 for e in rep["methods"].values())
    want = 1 if reverse else 3          # chunk_gla has no reverse argument: its pairs are skipped then
    assert len(rep["pairs"]) == want and text.count("Verifying") == want
    for pair, res in rep["pairs"].items():
        assert tuple(res) == sc.RESULTS, pair
        for key, c in res.items():
            assert c["rel_l2"] <= l2, f"{pair} {key}: relative L2 difference {c['rel_l2']:.3e}"
    if dtype == torch.bfloat16:
        assert "do not match" in text and "Max abs error" in text and "Rel error" in text


@pytest.mark.gpu
def test_cli_times_first_call_and_steady_state(capsys):
    sc.main(["--batch", "1", "--seq-len", "128", "--key-dim", "128", "--head-dim", "64", "--methods",
             "chunk_gla,recurrent_gla", "--json"])
    out = capsys.readouterr().out
    assert "First call" in out and "Iterations:" in out and "Time:" in out
    assert "Verifying chunk_gla and recurrent_gla" in out
    rep = __import__("json").loads(out.strip().splitlines()[-1])
    assert rep["methods"]["chunk_gla"]["time_ms"] > 0 and rep["methods"]["chunk_gla"]["iterations"] >= 1
