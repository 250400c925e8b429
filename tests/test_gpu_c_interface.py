"""tests/cpp/capi_tests.c on the device: the C interface selects the MI355X target by the
reference's name for it ("gpu"), compiles, runs, saves and loads there."""
import pytest

from test_c_interface import run_capi_tests

pytestmark = pytest.mark.gpu


def test_c_program_on_the_device(tmp_path):
    run_capi_tests("gpu", tmp_path)
