"""Host-side checks that need no GPU: the shared library loads and exports what include/mctsnc_hip.h declares, the
ctypes mirrors of the C structs have the C layout, configuration errors come back as error codes with a message,
and the Python class mirrors the reference's constructor behaviour."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mctsnc_hip.h")


@pytest.fixture(scope="module")
def L():
    from mcts_numba_cuda_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):
        build.build()
    return _lib.lib()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mctsnc_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(L):
    names = declared_functions()
    assert {"mctsnc_create", "mctsnc_init_device", "mctsnc_run", "mctsnc_run_batch", "mctsnc_read", "mctsnc_read_size",
            "mctsnc_reseed", "mctsnc_destroy", "mctsnc_last_error", "mctsnc_set_stage_timing"} <= set(names)
    for name in names:
        assert hasattr(L, name), name


def test_ctypes_structs_match_c_layout(tmp_path):
    from mcts_numba_cuda_amd import _lib
    src = tmp_path / "probe.c"
    fields_cfg = [f[0] for f in _lib.Config._fields_]
    fields_res = [f[0] for f in _lib.Result._fields_]
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void) {",
             'printf("%zu %zu\\n", sizeof(mctsnc_config), sizeof(mctsnc_result));']
    for f in fields_cfg:
        lines.append(f'printf("%zu\\n", offsetof(mctsnc_config, {f}));')
    for f in fields_res:
        lines.append(f'printf("%zu\\n", offsetof(mctsnc_result, {f}));')
    lines.append("return 0; }")
    src.write_text("\n".join(lines))
    exe = tmp_path / "probe"
    subprocess.check_call(["gcc", "-std=c99", "-o", str(exe), str(src)])
    out = subprocess.check_output([str(exe)]).decode().split()
    assert int(out[0]) == ctypes.sizeof(_lib.Config) and int(out[1]) == ctypes.sizeof(_lib.Result)
    offs = [int(x) for x in out[2:]]
    mine = [getattr(_lib.Config, f).offset for f in fields_cfg] + [getattr(_lib.Result, f).offset for f in fields_res]
    assert offs == mine


def test_configuration_errors_are_reported(L):
    from mcts_numba_cuda_amd import _lib
    good = dict(game=0, board_m=6, board_n=7, extra_info_memory=7, max_actions=7, n_trees=4, n_playouts=256, variant=3, ucb_c=2.0,
                seed=0, max_tree_size=1000, device=0)
    bad_cases = [dict(game=7), dict(board_n=9), dict(board_m=9), dict(board_m=14, board_n=4, max_actions=4), dict(max_actions=6), dict(n_playouts=100), dict(n_playouts=1024),
                 dict(n_trees=0), dict(variant=4), dict(ucb_c=-1.0), dict(max_tree_size=0), dict(max_tree_size=2**24 + 1),
                 dict(extra_info_memory=3)]
    for bad in bad_cases:
        cfg = _lib.Config(**{**good, **bad})
        h = ctypes.c_void_p()
        rc = L.mctsnc_create(ctypes.byref(cfg), ctypes.byref(h))
        assert rc == -1, bad
        assert len(L.mctsnc_last_error()) > 10
    cfg = _lib.Config(**good)
    h = ctypes.c_void_p()
    assert L.mctsnc_create(ctypes.byref(cfg), ctypes.byref(h)) == 0
    res = _lib.Result()
    board = np.zeros(42, np.int8)
    rc = L.mctsnc_run(h, board.ctypes.data, None, 0, 1, 10.0, 1.0, float("inf"), ctypes.byref(res))
    assert rc == -3  # run before init_device
    assert b"init_device" in L.mctsnc_last_error()
    assert L.mctsnc_read_size(h, 0, 0) == -3
    L.mctsnc_destroy(h)


def test_class_mirrors_reference_constructor(capsys):
    from mcts_numba_cuda_amd import MCTSNC
    e = MCTSNC((6, 7), 7, 7, search_time_limit=5.0, n_trees=4, n_playouts=256, variant="acp_prodigal")
    assert str(e) == ("MCTSNC(search_time_limit=5.0, search_steps_limit=inf, n_trees=4, n_playouts=256, variant='acp_prodigal', "
                      "device_memory=2.0, ucb_c=2.0, seed: 0)")
    assert repr(e).endswith("state_board_shape=(6, 7), state_extra_info_memory=7, state_max_actions=7)")
    assert e._per_state_memory() == (95, 5651185)
    assert MCTSNC.VARIANTS == ["ocp_thrifty", "ocp_prodigal", "acp_thrifty", "acp_prodigal"]
    assert (MCTSNC.DEFAULT_N_TREES, MCTSNC.DEFAULT_N_PLAYOUTS, MCTSNC.MAX_TREE_SIZE, MCTSNC.MAX_TREE_DEPTH) == (8, 128, 2**24, 2048)
    capsys.readouterr()
    e = MCTSNC((6, 7), 7, 7, n_playouts=100, variant="nonsense", n_trees=1000, ucb_c=-3.0, search_time_limit=-1.0)
    out = capsys.readouterr().out
    assert "is not a power of 2; changed to default: 128" in out
    assert "invalid variant: 'nonsense' changed to default: 'acp_prodigal'" in out
    assert "invalid param n_trees: 1000 changed to default: 8" in out
    assert "invalid param ucb_c" in out and "invalid param search_time_limit" in out
    assert (e.n_playouts, e.variant, e.n_trees, e.ucb_c, e.search_time_limit) == (128, "acp_prodigal", 8, 2.0, 5.0)
    g = MCTSNC((15, 15), 0, 225, verbose_info=False)
    assert g.game == "gomoku" and g.state_extra_info_memory == 1 and g._per_state_memory()[0] == 1144
    with pytest.raises(SystemExit):
        MCTSNC((33, 7), 7, 7)
    with pytest.raises(RuntimeError):
        e.run(np.zeros((6, 7), np.int8), np.zeros(7, np.int8), 1)


def test_replay_helpers_reconstruct_positions(archives):
    import replay
    key = replay.find_archive(archives, "mcts_5_inf_vanilla", "mctsnc_5_inf_4_256_acp_prodigal")
    game = archives[key]["games"][0]
    pos = replay.C4Position()
    for ev in game["events"]:
        if ev["type"] == "move":
            pos.play(ev["action"])
    from helpers import c4_has_four
    assert game["outcome"] == "WHITE WINS" and c4_has_four(pos.board, -1) and not c4_has_four(pos.board, 1)


def test_puct_library_exports_every_declared_symbol(tmp_path):
    """libpuct_hip.so loads without a GPU and exports what include/puct_select.h declares, including the two symbols
    the reference's binding resolves by name (src/puct/puct_gpu_v3_cpp.py:88-113); the header is valid C."""
    from mcts_numba_cuda_amd import build, puct
    if not os.path.exists(puct.LIB_PATH):
        build.build(only=build.PUCT_LIB)
    lib = puct._lib()
    header = os.path.join(ROOT, "include", "puct_select.h")
    text = re.sub(r"/\*.*?\*/", "", open(header).read(), flags=re.S)
    names = sorted(set(re.findall(r"\b(puct_[a-z_]+)\s*\(", text)))
    assert {"puct_select_winner_recalc_launch", "puct_cpp_cuda_error_string", "puct_edge_backup_launch",
            "puct_node_backup_launch", "puct_node_select_preclaim_launch",
            "puct_node_select_winner_recalc_launch"} == set(names)
    for name in names:
        assert hasattr(lib, name), name
    src = tmp_path / "probe.c"
    src.write_text(f'#include "{header}"\nint main(void) {{ return PUCT_SELECT_BUSY == 4 ? 0 : 1; }}\n')
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-c", "-o", str(tmp_path / "probe.o"), str(src)])
    assert (puct.PACKED_KIND_SHIFT, puct.PACKED_SLOT_SHIFT, puct.PACKED_REASON_SHIFT) == (22, 14, 25)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it says so and exits with an error instead of printing a figure."""
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)
    assert not r.stdout.strip().startswith("{")


def test_board_shapes_beyond_the_engine_get_a_reference_style_message(capsys):
    """The reference's caps (32 x 32 cells, 512 actions, src/mctsnc.py:180-197) admit drop-game boards this engine's
    bitboard kernels do not take (placement games are taken up to those caps); the class says so in the reference's
    message style before it raises, without touching the device."""
    from mcts_numba_cuda_amd import MCTSNC
    for kw, part in ((dict(state_board_shape=(6, 10), state_extra_info_memory=10, state_max_actions=10), "columns <= 8"),
                     (dict(state_board_shape=(14, 4), state_extra_info_memory=4, state_max_actions=4), "rows <= 13")):
        e = MCTSNC(verbose_info=False, **kw)
        with pytest.raises(ValueError):
            e.init_device_side_arrays()
        out = capsys.readouterr().out
        assert out.startswith("[MCTSNC._init_device_side_arrays(): exiting due to state board shape") and part in out
