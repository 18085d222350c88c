"""The per-shape GEMM selection shipped for gfx950: it loads, it changes which library kernel serves a listed shape and
nothing else (same products to bf16 rounding), and it can be switched off again."""
import pytest
import torch

from maltos_amd.gemm_tuning import TUNED_FILE, tuned_gemms_off, use_tuned_gemms

pytestmark = pytest.mark.gpu


@pytest.fixture
def tuned():
    n = use_tuned_gemms()
    yield n
    tuned_gemms_off()


def test_shipped_selection_loads_and_keeps_the_products(dev, tuned):
    if tuned == 0:
        pytest.skip("the shipped selection was recorded with other GEMM library versions; torch refused it")
    listed = [line.split(",") for line in TUNED_FILE.read_text().splitlines() if line.startswith("Gemm")]
    assert tuned >= len(listed) and torch.cuda.tunable.is_enabled() and not torch.cuda.tunable.tuning_is_enabled()
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(16384, 512, generator=gen).bfloat16().to(dev)
    for out_features in (1536, 2752, 512):   # q/k/v, gate/up, o_proj of LLaMA-50M: all listed as tn_<out>_16384_512
        assert any(f"tn_{out_features}_16384_512_" in row[1] for row in listed)
        w = (torch.randn(out_features, 512, generator=gen) * 0.05).bfloat16().to(dev)
        got = torch.nn.functional.linear(x, w)
        tuned_gemms_off()
        want = torch.nn.functional.linear(x, w)
        use_tuned_gemms()
        exact = x.float() @ w.float().t()
        # either kernel rounds the fp32 sums once to bf16
        for y in (got, want):
            assert ((y.float() - exact).abs() <= 2.0 ** -8 * exact.abs() + 1e-3).all()


@pytest.mark.filterwarnings("ignore:Failed validator")   # torch says why it refuses the second file
def test_missing_or_foreign_file_changes_nothing(dev, tmp_path):
    assert use_tuned_gemms(tmp_path / "absent.csv") == 0 and not torch.cuda.tunable.is_enabled()
    foreign = tmp_path / "foreign.csv"
    lines = TUNED_FILE.read_text().splitlines()
    foreign.write_text("\n".join("Validator,HIPBLASLT_VERSION,0-other" if l.startswith("Validator,HIPBLASLT_VERSION") else l
                                 for l in lines) + "\n")
    assert use_tuned_gemms(foreign) == 0 and not torch.cuda.tunable.is_enabled()
