"""The upstream-harness compatibility helpers that need no GPU."""
import importlib

import pytest


@pytest.fixture(scope="module")
def harness(pkg):
    return importlib.import_module("amd-developer-challenge-2025_amd.harness")


def test_parse_tests_file_format(harness):
    text = """
    m: 1024; n: 576 ; k: 7168; seed: 12346
    # a comment
    m: 6144; n: 4096; k: 512 ; seed: 45245   # trailing
    """
    assert harness.parse_tests(text) == [{"m": 1024, "n": 576, "k": 7168, "seed": 12346},
                                         {"m": 6144, "n": 4096, "k": 512, "seed": 45245}]
    with pytest.raises(ValueError):
        harness.parse_tests("m: 1; n: 2; k: x; seed: 3")
    with pytest.raises(ValueError):
        harness.parse_tests("m: 1; n: 2; k: 128")


def test_leaderboard_shapes(harness, pkg):
    shapes = harness.LEADERBOARD_SHAPES
    assert len(shapes) == 18
    assert {s["m"] for s in shapes} == {1024, 6144}
    assert all(s["k"] % 128 == 0 and s["n"] % 16 == 0 for s in shapes)
    # every one of them is planned onto a tiled MFMA kernel, none onto the scalar fallback
    for s in shapes:
        assert pkg.plan(s["m"], s["n"], s["k"]).variant != 1


def test_main_usage_errors_need_no_gpu(harness, tmp_path, capsys):
    """The command line of the two upstream modes: bad usage is reported before anything touches the GPU."""
    f = tmp_path / "tests"
    f.write_text("m: 64; n: 128; k: 256; seed: 1\n")
    assert harness.main([]) == 2
    assert harness.main(["rank", str(f)]) == 2
    assert harness.main(["test", str(f)]) == 2                    # test mode without a checker: nothing to compare with
    assert "checker" in capsys.readouterr().err
