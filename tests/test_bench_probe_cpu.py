"""The benchmark's probe library (libq4probe.so, csrc/bench/q4_probe.hip): it loads, exports what
bench.py binds and validates its arguments on the host (nothing is launched here).  It is not part
of the product library: libq4linear.so must not export the probes."""
import ctypes

import bench


def test_probe_library_is_separate_from_the_product(pkg):
    lib = pkg._lib.load()
    for name in ("q4_probe_read", "q4_probe_lds"):
        assert not hasattr(lib, name), f"{name} is exported by the product library"
    probe = bench.load_probe_lib()
    for name in ("q4_probe_read", "q4_probe_lds", "q4_probe_last_error"):
        assert hasattr(probe, name)


def test_probe_read_rejects_shapes_that_do_not_divide():
    lib = bench.load_probe_lib()
    bad = -1
    buf, sink = 0x1000, 0x2000
    nbytes = 4096 * 4096 // 2
    assert lib.q4_probe_read(buf, nbytes, 0, 0, 256, 256, 4, 1, None, None) == bad      # no sink
    assert lib.q4_probe_read(buf, nbytes, 0, 0, 256, 100, 4, 1, sink, None) == bad      # not whole waves
    assert lib.q4_probe_read(buf, nbytes, 0, 0, 256, 256, 3, 1, sink, None) == bad      # unroll
    assert lib.q4_probe_read(buf, 4096, 0, 0, 256, 256, 4, 1, sink, None) == bad        # less than a round
    assert lib.q4_probe_read(buf, nbytes, 1, 4096, 100, 256, 4, 1, sink, None) == bad   # grid vs column tiles
    assert lib.q4_probe_read(buf, nbytes, 1, 4096, 64 * 3, 256, 4, 1, sink, None) == bad  # steps do not divide
    assert lib.q4_probe_read(buf, nbytes, 1, 1000, 64, 256, 4, 1, sink, None) == bad    # n_words % 64
    assert lib.q4_probe_read(buf, nbytes, 1, 4096, 64, 192, 4, 2, sink, None) == bad    # three waves, two column waves
    assert lib.q4_probe_read(buf, nbytes, 7, 0, 256, 256, 4, 1, sink, None) == bad      # pattern
    assert b"q4_probe_read" in lib.q4_probe_last_error()


def test_probe_lds_rejects_missing_arguments():
    lib = bench.load_probe_lib()
    bad = -1
    assert lib.q4_probe_lds(None, 10, 256, 0x2000, None) == bad    # no lane map
    assert lib.q4_probe_lds(0x1000, 10, 256, None, None) == bad    # no sink
    assert lib.q4_probe_lds(0x1000, 0, 256, 0x2000, None) == bad   # no iterations
    assert lib.q4_probe_lds(0x1000, 10, 0, 0x2000, None) == bad    # no workgroups
    assert b"q4_probe_lds" in lib.q4_probe_last_error()


def test_read_floor_grids_include_the_gate_up_launch():
    """224 workgroups of 512 threads with two column waves: the decode kernel's own gate_up grid."""
    grids = bench.read_floor_configs(4096, 28672)
    assert any(wgs == 224 and threads == 512 and wcol == 2 for wgs, threads, _, wcol in grids)
