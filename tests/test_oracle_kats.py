"""The oracle against every known-answer vector the reference's own tests hold."""
import pytest

from programs import KATS, check_golden


@pytest.mark.parametrize("name", sorted(KATS))
def test_oracle_reproduces_reference_kat(name, oracle_device):
    out = KATS[name](oracle_device)
    check_golden(name, out)
