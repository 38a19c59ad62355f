"""`python -m sphericart_amd.tune`, the settled measurement of planner settings behind the tables of
csrc/sphx_plan_shapes.hpp: its arguments (no GPU), and one small run on the device."""

import pytest

from gpu_utils import announce
from sphericart_amd import tune


def test_shapes_and_settings_are_parsed_or_refused():
    assert tune.parse_shape("f32:10:gradients:solid") == ("f32", 10, "gradients", "solid", 616016)
    assert tune.parse_shape("f64:19:hessians:spherical:3000") == ("f64", 19, "hessians", "spherical", 3000)
    for bad in ("f16:3:values:solid", "f32:3:laplacians:solid", "f32:3:values", "f32:3:values:round"):
        with pytest.raises(ValueError):
            tune.parse_shape(bad)
    assert tune.parse_values("-1,-1 1,3", 2) == [(-1, -1), (1, 3)]
    with pytest.raises(ValueError, match="2 switches"):
        tune.parse_values("1 0,2", 2)


@pytest.mark.gpu
def test_a_small_run_times_every_setting_and_leaves_no_switch_set(library, capsys):
    announce("tune, small run")
    status = tune.main(["--switch", "SPHX_WAVE_PRIORITIES,SPHX_SEQUENCE_WAVES", "--values", "-1,-1 1,3",
                        "--shapes", "f32:10:gradients:spherical:20000", "--settle", "0.02", "--launches", "5",
                        "--turns", "2"])
    out = capsys.readouterr().out
    assert status == 0 and "\nf32:10:gradients:spherical:20000 " in out and "best" in out
    import ctypes

    text = ctypes.create_string_buffer(512)
    assert library.sphx_describe_plan(600000, 10, 1, 0, 1, text, len(text)) == 0
    assert text.value.decode().endswith("workgroups]"), "the planner's own choice again: no priority at this shape"
    with pytest.raises(ValueError, match="unknown switch"):
        tune.main(["--switch", "SPHX_NO_SUCH", "--values", "1", "--shapes", "f32:8:values:solid:1000",
                   "--settle", "0", "--launches", "1", "--turns", "1"])
