"""The GPU facade on the layer orderings and propagation states of
tests/golden/variants.npz (compiled reference): normalization after the
activation, dropout on the normalized values, and the UPDATE_BATCH_NORM pass."""
import pytest

from helpers import RTOL_REDUCED as TR
from test_oracle_variants import build_variant_model, check_variant, load_variants_golden, variant_cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model_factory(pkg):
    from deep_learning_amd.model import Model
    lib = pkg.load_library()
    made = []

    def make(widths):
        m = Model(lib, widths)
        made.append(m)
        return m

    yield make
    for m in made:
        m.close()


@pytest.mark.parametrize("name", list(variant_cases()))
def test_gpu_variants_against_golden(model_factory, name):
    g = load_variants_golden()
    M = build_variant_model(model_factory, g, name, 0)
    check_variant(M, g, name, 0, TR, lambda m: m.get_moving())
