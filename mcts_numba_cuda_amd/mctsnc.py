"""``MCTSNC`` for AMD MI355X: the reference's class interface (src/mctsnc.py:174-563) on top of libmctsnc_hip.so.

The constructor arguments, ``init_device_side_arrays()``, ``run(root_board, root_extra_info, root_turn,
forced_search_steps_limit)``, the attributes read by ``game_runner.py`` / ``main.py`` (``actions_info``,
``performance_info``, ``best_*``, ``steps``, ``time_*``, ``max_tree_size``), ``__str__`` and ``_json_dump`` follow
the reference, so an instance can stand where the numba.cuda one stood.  The search itself (selection, expansion,
playouts, backup) runs inside one persistent HIP kernel; this module only validates, marshals and reports.
"""
import atexit
import ctypes
import json
import sys
import time
import weakref

import numpy as np
from numpy import inf

from . import _lib
from .utils import dict_to_str

__version__ = "1.0.2"


class MCTSNC:
    """Monte Carlo Tree Search with many concurrent trees and playouts on one MI355X (four algorithmic variants)."""

    # constants (src/mctsnc.py:180-197)
    VARIANTS = ["ocp_thrifty", "ocp_prodigal", "acp_thrifty", "acp_prodigal"]
    DEFAULT_SEARCH_TIME_LIMIT = 5.0
    DEFAULT_SEARCH_STEPS_LIMIT = np.inf
    DEFAULT_N_TREES = 8
    DEFAULT_N_PLAYOUTS = 128
    DEFAULT_VARIANT = VARIANTS[-1]
    DEFAULT_DEVICE_MEMORY = 2.0
    DEFAULT_UCB_C = 2.0
    DEFAULT_SEED = 0
    DEFAULT_VERBOSE_DEBUG = False
    DEFAULT_VERBOSE_INFO = True
    MAX_STATE_BOARD_SHAPE = (32, 32)
    MAX_STATE_EXTRA_INFO_MEMORY = 4096
    MAX_STATE_MAX_ACTIONS = 512
    MAX_TREE_SIZE = 2**24
    MAX_N_TREES = 512
    MAX_N_PLAYOUTS = 512
    MAX_TREE_DEPTH = 2048
    GAMES = {"c4": _lib.GAME_C4, "gomoku": _lib.GAME_GOMOKU}

    def __init__(self, state_board_shape, state_extra_info_memory, state_max_actions,
                 search_time_limit=DEFAULT_SEARCH_TIME_LIMIT, search_steps_limit=DEFAULT_SEARCH_STEPS_LIMIT,
                 n_trees=DEFAULT_N_TREES, n_playouts=DEFAULT_N_PLAYOUTS, variant=DEFAULT_VARIANT, device_memory=DEFAULT_DEVICE_MEMORY,
                 ucb_c=DEFAULT_UCB_C, seed=DEFAULT_SEED,
                 verbose_debug=DEFAULT_VERBOSE_DEBUG, verbose_info=DEFAULT_VERBOSE_INFO,
                 action_index_to_name_function=None, game=None, device=0):
        """Arguments as in the reference (src/mctsnc.py:199-276).  Two additions: ``game`` ("c4" / "gomoku"; the
        reference picks the game by editing its mechanics module, here it is inferred from the state geometry when
        omitted) and ``device`` (HIP device ordinal)."""
        self._set_cuda_constants()
        self.state_board_shape = tuple(int(x) for x in state_board_shape)
        if self.state_board_shape[0] > self.MAX_STATE_BOARD_SHAPE[0] or self.state_board_shape[1] > self.MAX_STATE_BOARD_SHAPE[1]:
            sys.exit("[MCTSNC.__init__(): exiting due to allowed state board shape exceeded]")
        self.state_extra_info_memory = max(int(state_extra_info_memory), 1)
        if self.state_extra_info_memory > self.MAX_STATE_EXTRA_INFO_MEMORY:
            sys.exit("[MCTSNC.__init__(): exiting due to allowed state extra info memory exceeded]")
        self.state_max_actions = int(state_max_actions)
        if self.state_max_actions > self.MAX_STATE_MAX_ACTIONS:
            sys.exit("[MCTSNC.__init__(): exiting due to allowed state max actions memory exceeded]")
        if self.state_max_actions > self.cuda_tpb_default:
            sys.exit("[MCTSNC.__init__(): exiting due to state max actions exceeding half of cuda default tpb]")
        self.search_time_limit = search_time_limit
        self._validate_param("search_time_limit", float, True, 0.0, False, np.inf, self.DEFAULT_SEARCH_TIME_LIMIT)
        self.search_steps_limit = float(search_steps_limit)
        self._validate_param("search_steps_limit", float, True, 0.0, False, np.inf, self.DEFAULT_SEARCH_STEPS_LIMIT)
        self.n_trees = n_trees
        self._validate_param("n_trees", int, False, 1, False, self.MAX_N_TREES, self.DEFAULT_N_TREES)
        if n_playouts < 1 or 2**np.round(np.log2(n_playouts)) != n_playouts:
            invalid_n_playouts = n_playouts
            n_playouts = self.DEFAULT_N_PLAYOUTS
            print(f"[n_playouts: {invalid_n_playouts} is not a power of 2; changed to default: {n_playouts}]")
        self.n_playouts = n_playouts
        self._validate_param("n_playouts", int, False, 1, False, self.MAX_N_PLAYOUTS, self.DEFAULT_N_PLAYOUTS)
        if variant not in self.VARIANTS:
            invalid_variant = variant
            variant = self.DEFAULT_VARIANT
            print(f"[invalid variant: '{invalid_variant}' changed to default: '{variant}'; possible variants: {self.VARIANTS}]")
        self.variant = variant
        self.ucb_c = ucb_c
        self._validate_param("ucb_c", float, False, 0.0, False, np.inf, self.DEFAULT_UCB_C)
        self.device_memory = device_memory * 1024**3  # GiB to bytes
        self._validate_param("device_memory", float, True, 0.0, False, np.inf, self.DEFAULT_DEVICE_MEMORY)
        self.seed = seed
        self.verbose_debug = verbose_debug
        self._validate_param("verbose_debug", bool, False, False, False, True, self.DEFAULT_VERBOSE_DEBUG)
        self.verbose_info = verbose_info
        self._validate_param("verbose_info", bool, False, False, False, True, self.DEFAULT_VERBOSE_INFO)
        self.action_index_to_name_function = action_index_to_name_function
        if game is None:
            m, n = self.state_board_shape
            game = "c4" if self.state_max_actions == n and self.state_max_actions != m * n else "gomoku"
        if game not in self.GAMES:
            raise ValueError(f"unknown game '{game}'; known: {sorted(self.GAMES)}")
        self.game = game
        self.device = int(device)
        self._engine = None
        self.max_tree_size = None
        self._actions_info = None
        self._performance_info = None
        self._result = None
        self.best_action = self.best_win_flag = self.best_n = self.best_n_wins = self.best_q = None
        self.steps = 0
        self.time_total = self.time_loop = self.time_reduce_over_trees = self.time_reduce_over_actions = 0.0
        self.time_select = self.time_expand = self.time_playout = self.time_backup = 0.0

    def __del__(self):
        # Engines still alive when the interpreter shuts down were already closed by the exit hook below; during
        # finalisation itself nothing is released any more (the HIP runtime may be tearing down at that point).
        if not sys.is_finalizing():
            self._release()

    def close(self):
        """Frees the engine's device memory, stream and events now.  The instance can be initialised again with
        init_device_side_arrays().  Also available as a context manager: ``with MCTSNC(...) as ai: ...``."""
        self._release()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False

    def _release(self):
        eng = getattr(self, "_engine", None)
        if eng:
            self._engine = None
            _lib.lib().mctsnc_destroy(eng)

    def _set_cuda_constants(self):
        """The reference asks numba for MAX_THREADS_PER_BLOCK // 2 (src/mctsnc.py:278-281); 512 on every device it
        was run on, and the value fixes the RNG stream layout, so it is a constant here."""
        self.cuda_available = True
        self.cuda_tpb_default = 512

    def _validate_param(self, name, ptype, leq, low, geq, high, default):
        """Range and type check with fallback to the default, as src/mctsnc.py:283-296."""
        value = getattr(self, name)
        try:
            invalid = value <= low if leq else value < low
            if not invalid:
                invalid = value >= high if geq else value > high
        except TypeError:
            invalid = True
        if not invalid:
            invalid = not isinstance(value, ptype)
        if invalid:
            correct_range_str = ("(" if leq else "[") + f"{low}, {high}" + (")" if geq else "]")
            setattr(self, name, default)
            print(f"[invalid param {name}: {value} changed to default: {default}; correct range: {correct_range_str}, correct type: {ptype}]")

    def __str__(self):
        return f"MCTSNC(search_time_limit={self.search_time_limit}, search_steps_limit={self.search_steps_limit}, n_trees={self.n_trees}, n_playouts={self.n_playouts}, variant='{self.variant}', device_memory={np.round(self.device_memory / 1024**3, 2)}, ucb_c={self.ucb_c}, seed: {self.seed})"

    def __repr__(self):
        repr_str = f"{str(self)}, "
        repr_str += f"state_board_shape={self.state_board_shape}, state_extra_info_memory={self.state_extra_info_memory}, state_max_actions={self.state_max_actions})"
        return repr_str

    # ------------------------------------------------------------------------------------------------------------
    def _per_state_memory(self):
        """Node-pool sizing of the reference (src/mctsnc.py:350-358); returns (per_state_memory, max_tree_size)."""
        per_state_additional_memory = 2 + 1 + 2 * 1 + 1 + 2 * 4
        per_tree_additional_memory = 4 + 4 + 2 * (self.state_max_actions + 2) + 4 * 2 + 4 * (self.MAX_TREE_DEPTH + 2)
        if "acp" in self.variant:
            per_tree_additional_memory += 4 * self.state_max_actions * 2
        per_state_memory = int(np.prod(self.state_board_shape)) + self.state_extra_info_memory + 4 * (1 + self.state_max_actions) + per_state_additional_memory
        max_tree_size = (int(self.device_memory) - self.n_trees * per_tree_additional_memory) // (per_state_memory * self.n_trees)
        return per_state_memory, min(max_tree_size, self.MAX_TREE_SIZE)

    def _engine_shape_limit(self):
        """What of the engine's shape limits (narrower than the reference's MAX_STATE_BOARD_SHAPE / MAX_STATE_MAX_ACTIONS)
        the configured board exceeds, or None."""
        m, n = int(self.state_board_shape[0]), int(self.state_board_shape[1])
        if self.game == "gomoku":
            if m > 32 or n > 32 or m * n > 512:     # (the reference's own caps; it reports them itself before this is reached)
                return "placement games are held on boards with sides up to 32 and up to 512 cells"
        elif (m + 1) * n > 64 or n > 8 or m > 13:
            return "drop games are held in 64-bit column bitboards: (rows + 1) * columns <= 64, columns <= 8, rows <= 13"
        return None

    def init_device_side_arrays(self):
        """Allocates the node pools in HBM and seeds the random streams (src/mctsnc.py:318-407).  ``device_memory``
        fixes the number of nodes per tree exactly as in the reference; a node record here is one 128-byte line, so
        the bytes actually held differ from the reference's accounting."""
        if self.verbose_info:
            print(f"[MCTSNC._init_device_side_arrays()... for {self}]")
        t1_dev_arrays = time.time()
        per_state_memory, self.max_tree_size = self._per_state_memory()
        if self.max_tree_size < 1:
            raise ValueError("device_memory too small for a single node per tree")
        limit = self._engine_shape_limit()
        if limit:
            # in the style of the reference's own cap messages (src/mctsnc.py:240-249); its caps (32 x 32 cells, 512
            # actions) are wider than what this engine's kernels take
            message = f"[MCTSNC._init_device_side_arrays(): exiting due to state board shape {tuple(self.state_board_shape)} beyond this engine's {self.game} kernels: {limit}]"
            print(message)
            raise ValueError(message)
        L = _lib.lib()
        self._release()
        cfg = _lib.Config(game=self.GAMES[self.game], board_m=self.state_board_shape[0], board_n=self.state_board_shape[1],
                          extra_info_memory=self.state_extra_info_memory, max_actions=self.state_max_actions,
                          n_trees=int(self.n_trees), n_playouts=int(self.n_playouts), variant=self.VARIANTS.index(self.variant),
                          ucb_c=float(self.ucb_c), seed=int(self.seed), max_tree_size=int(self.max_tree_size), device=self.device)
        handle = ctypes.c_void_p()
        _lib.check(L.mctsnc_create(ctypes.byref(cfg), ctypes.byref(handle)))
        self._engine = handle
        _LIVE.add(self)
        try:
            _lib.check(L.mctsnc_init_device(self._engine))
        except Exception:
            self._release()
            raise
        t2_dev_arrays = time.time()
        if self.verbose_info:
            print(f"[MCTSNC._init_device_side_arrays() done; time: {t2_dev_arrays - t1_dev_arrays} s, per_state_memory: {per_state_memory} B,  calculated max_tree_size: {self.max_tree_size}]")

    def reseed(self):
        """Restarts the random streams from ``seed`` (what a freshly constructed and initialised instance holds)."""
        self._require_engine()
        _lib.check(_lib.lib().mctsnc_reseed(self._engine))

    def set_option(self, name, value):
        """How the search is laid out on the device, and test hooks (``mctsnc_set_option`` of include/mctsnc_hip.h:
        "agent_fences", "solo_trees", "solo_threads", "team_pool", "team_pool_threads", "prep_levels", "plain_launch",
        "probe_steps", "spin_limit"); results do not depend on any of them.  ``run_batch`` takes those of its first engine."""
        self._require_engine()
        if name not in _lib.OPTIONS:
            raise ValueError(f"unknown option {name!r}; known: {sorted(_lib.OPTIONS)}")
        _lib.check(_lib.lib().mctsnc_set_option(self._engine, _lib.OPTIONS[name], int(value)))

    def _require_engine(self):
        if not self._engine:
            raise RuntimeError("init_device_side_arrays() must be called before run()")

    def run(self, root_board, root_extra_info, root_turn, forced_search_steps_limit=np.inf):
        """Runs the search from the given root (src/mctsnc.py:409-434) and returns the best action."""
        print(f"MCTSNC RUN... [{self}]")
        self._require_engine()
        board = np.ascontiguousarray(root_board, dtype=np.int8)
        if board.shape != self.state_board_shape:
            raise ValueError(f"root_board shape {board.shape} differs from state_board_shape {self.state_board_shape}")
        if root_extra_info is None:
            extra = np.zeros(1, dtype=np.int8)  # fake extra info array (src/mctsnc.py:1090-1091)
        else:
            extra = np.ascontiguousarray(root_extra_info, dtype=np.int8).reshape(-1)
        res = _lib.Result()
        _lib.check(_lib.lib().mctsnc_run(self._engine, board.ctypes.data, extra.ctypes.data, extra.size, int(root_turn),
                                         float(self.search_steps_limit), float(self.search_time_limit), float(forced_search_steps_limit),
                                         ctypes.byref(res)))
        self._absorb_result(res, int(root_turn))
        if self.verbose_info:
            print(f"[actions info:\n{dict_to_str(self.actions_info)}]")
            print(f"[performance info:\n{dict_to_str(self.performance_info)}]")
        best_action_label = str(self.best_action)
        if self.action_index_to_name_function is not None:
            best_action_label += f" ({self.action_index_to_name_function(self.best_action)})"
        print(f"MCTSNC RUN DONE. [time: {self.time_total} s; best action: {best_action_label}, best win_flag: {self.best_win_flag}, best n: {self.best_n}, best n_wins: {self.best_n_wins}, best q: {self.best_q}]")
        return self.best_action

    def _absorb_result(self, res, root_turn):
        self._result = res
        self._root_turn = root_turn
        self.steps = int(res.steps)
        self.best_action = np.int16(res.best_action)
        self.best_win_flag = bool(res.best_win_flag)
        self.best_n = np.int64(res.best_n)
        self.best_n_wins = np.int64(res.best_n_wins)
        self.best_q = float(self.best_n_wins / self.best_n) if self.best_n > 0 else np.nan
        self.time_total = res.time_total
        self.time_loop = res.time_loop
        self.time_device_loop = res.time_device_loop
        self.time_reduce_over_trees = res.time_reduce
        self.time_reduce_over_actions = 0.0  # both reductions are one pass here
        self.time_select, self.time_expand = res.time_select, res.time_expand
        self.time_playout, self.time_backup = res.time_playout, res.time_backup
        self.time_exchange = res.time_exchange
        # the root tables and the two dictionaries are built when first read (a pass over hundreds of engines would
        # otherwise spend milliseconds on dictionaries nobody looks at)
        self._tables = None
        self._actions_info = None
        self._performance_info = None

    def _decode_tables(self):
        if self._tables is None:
            res, A = self._result, self.state_max_actions
            self._tables = (np.array(res.root_actions_expanded[:A + 2], dtype=np.int16), np.array(res.root_ns[:A], dtype=np.int64),
                            np.array(res.actions_ns[:A], dtype=np.int64), np.array(res.actions_ns_wins[:A], dtype=np.int64),
                            np.array(res.actions_win_flags[:A], dtype=bool))
        return self._tables

    _root_actions_expanded = property(lambda self: self._decode_tables()[0])
    _root_ns = property(lambda self: self._decode_tables()[1])
    _actions_ns = property(lambda self: self._decode_tables()[2])
    _actions_ns_wins = property(lambda self: self._decode_tables()[3])
    _actions_win_flags = property(lambda self: self._decode_tables()[4])

    @property
    def actions_info(self):
        """Root action table of the last search (src/mctsnc.py:496-563); None before the first."""
        if self._actions_info is None and self._result is not None:
            if "thrifty" in self.variant:
                self._make_actions_info_thrifty()
            else:
                self._make_actions_info_prodigal()
        return self._actions_info

    @actions_info.setter
    def actions_info(self, value):
        self._actions_info = value

    @property
    def performance_info(self):
        """Performance dictionary of the last search (src/mctsnc.py:448-494); None before the first."""
        if self._performance_info is None and self._result is not None:
            self._make_performance_info()
        return self._performance_info

    @performance_info.setter
    def performance_info(self, value):
        self._performance_info = value

    def _entry(self, i, a):
        entry = {}
        entry["name"] = self.action_index_to_name_function(a) if self.action_index_to_name_function else str(a)
        entry["n_root"] = int(self._root_ns[i])
        entry["win_flag"] = bool(self._actions_win_flags[i])
        entry["n"] = int(self._actions_ns[i])
        entry["n_wins"] = int(self._actions_ns_wins[i])
        # plain Python floats, so that the table prints as the reference's does whatever the numpy version
        entry["q"] = entry["n_wins"] / entry["n"] if entry["n"] > 0 else np.nan
        entry["ucb"] = float(entry["q"] + self.ucb_c * np.sqrt(np.log(entry["n_root"]) / entry["n"])) if entry["n"] > 0 else np.inf
        return entry

    def _make_actions_info_thrifty(self):
        """Root action table with thrifty indexing (src/mctsnc.py:496-529)."""
        actions_info = {}
        best_entry = None
        n_root_actions = int(self._root_actions_expanded[-1])
        for i in range(n_root_actions):
            a = self._root_actions_expanded[i]
            entry = self._entry(i, a)
            actions_info[a] = entry
            if a == self.best_action:
                best_entry = {"index": int(a), **entry}
        actions_info["best"] = best_entry
        self.actions_info = actions_info
        return actions_info

    def _make_actions_info_prodigal(self):
        """Root action table with prodigal indexing (src/mctsnc.py:531-563)."""
        actions_info = {}
        best_entry = None
        for i in range(self.state_max_actions):
            if self._root_ns[i] == 0:
                continue
            a = i
            entry = self._entry(i, a)
            actions_info[a] = entry
            if a == self.best_action:
                best_entry = {"index": int(a), **entry}
        actions_info["best"] = best_entry
        self.actions_info = actions_info
        return actions_info

    def _make_performance_info(self):
        """Performance dictionary with the reference's keys (src/mctsnc.py:448-494).  The four stages run fused in one
        kernel; their per-step means come from device clock readings taken between the stages by one workgroup of
        tree 0 (the backup figure includes the wait for the tree's other workgroups)."""
        res = self._result
        performance_info = {}
        performance_info["steps"] = int(self.steps)
        performance_info["steps_per_second"] = self.steps / self.time_total
        positive = self._root_ns[self._root_ns > 0]
        playouts = int(positive[0]) if positive.size else 0
        performance_info["playouts"] = playouts
        performance_info["playouts_per_second"] = playouts / self.time_total
        ms_factor = 10.0**3
        times_info = {}
        times_info["total"] = ms_factor * self.time_total
        times_info["loop"] = ms_factor * self.time_loop
        times_info["reduce_over_trees"] = ms_factor * self.time_reduce_over_trees
        times_info["reduce_over_actions"] = ms_factor * self.time_reduce_over_actions
        steps = max(self.steps, 1)
        times_info["mean_loop"] = times_info["loop"] / steps
        times_info["mean_select"] = ms_factor * self.time_select / steps
        times_info["mean_expand"] = ms_factor * self.time_expand / steps
        times_info["mean_playout"] = ms_factor * self.time_playout / steps
        times_info["mean_backup"] = ms_factor * self.time_backup / steps
        times_info["mean_exchange"] = ms_factor * self.time_exchange / steps  # part of mean_backup
        times_info["device_loop"] = ms_factor * self.time_device_loop
        performance_info["times_[ms]"] = times_info
        trees_info = {}
        trees_info["count"] = int(self.n_trees)
        trees_info["mean_depth"] = int(res.depth_sum) / int(res.size_sum)
        trees_info["max_depth"] = int(res.max_depth)
        trees_info["mean_size"] = int(res.size_sum) / self.n_trees
        trees_info["max_size"] = int(res.max_size)
        performance_info["trees"] = trees_info
        performance_info["playout_plies"] = int(res.playout_plies)
        self.performance_info = performance_info
        return performance_info

    # ------------------------------------------------------------------------------------------------------------
    def read_array(self, name, tree=0):
        """Copies one array of the last run back in the reference's layout (see include/mctsnc_hip.h, MCTSNC_ARR_*)."""
        self._require_engine()
        L = _lib.lib()
        aid, dtype = _lib.ARRAYS[name]
        nbytes = L.mctsnc_read_size(self._engine, aid, tree)
        if nbytes < 0:
            _lib.check(int(nbytes))
        buf = np.empty(nbytes // np.dtype(dtype).itemsize, dtype=dtype)
        if nbytes:
            _lib.check(L.mctsnc_read(self._engine, aid, tree, buf.ctypes.data, buf.nbytes))
        A = self.state_max_actions
        m, n = self.state_board_shape
        shapes = {"trees": (-1, 1 + A), "boards": (-1, m, n), "extra_infos": (-1, self.state_extra_info_memory),
                  "playout_outcomes_children": (A, 2), "rng_playout": (-1, 2), "rng_expand": (-1, 2)}
        return buf.reshape(shapes[name]) if name in shapes else buf

    def _json_dump(self, fname):
        """Dumps the trees of the last run to a json file with the reference's keys (src/mctsnc.py:2377-2462).  Child
        slots of never-expanded nodes hold -1 (the reference leaves them uninitialised)."""
        if self.verbose_info:
            print(f"JSON DUMP... [to file: {fname}]")
        t1 = time.time()
        d = {}
        d["n_trees"] = self.n_trees
        d["n_playouts"] = self.n_playouts
        d["variant"] = self.variant
        d["search_time_limit"] = self.search_time_limit if self.search_time_limit < np.inf else "inf"
        d["search_steps_limit"] = self.search_steps_limit if self.search_steps_limit < np.inf else "inf"
        d["ucb_c"] = self.ucb_c
        d["seed"] = self.seed
        d["device_memory"] = self.device_memory
        T, A = self.n_trees, self.state_max_actions
        per_tree = {k: [self.read_array(k, t) for t in range(T)] for k in ["trees", "depths", "turns", "ns", "ns_wins"]}
        sizes = np.array([a.shape[0] for a in per_tree["depths"]], dtype=np.int32)
        size_max = int(sizes.max())
        depth_max = max(int(a.max()) for a in per_tree["depths"])

        def padded(key, fill, trailing=()):
            out = np.full((T, size_max) + trailing, fill, dtype=per_tree[key][0].dtype)
            for t in range(T):
                out[t, :sizes[t]] = per_tree[key][t]
            return out

        paths = np.zeros((T, depth_max + 2), dtype=np.int32)
        for t in range(T):
            p = self.read_array("selected_path", t)
            paths[t, :p.size] = p[:depth_max + 1]
            paths[t, -1] = p.size
        d["trees"] = padded("trees", -1, (1 + A,)).tolist()
        d["trees_sizes"] = sizes.tolist()
        d["trees_depths"] = padded("depths", 0).tolist()
        d["trees_turns"] = padded("turns", 0).tolist()
        d["trees_ns"] = padded("ns", 0).tolist()
        d["trees_ns_wins"] = padded("ns_wins", 0).tolist()
        d["trees_nodes_selected"] = [int(self.read_array("node_selected", t)[0]) for t in range(T)]
        d["trees_selected_paths"] = paths.tolist()
        d["trees_actions_expanded"] = [self.read_array("actions_expanded", t).tolist() for t in range(T)]
        d["trees_playout_outcomes"] = [self.read_array("playout_outcomes", t).tolist() for t in range(T)]
        if "acp" in self.variant:
            d["trees_playout_outcomes_children"] = [self.read_array("playout_outcomes_children", t).tolist() for t in range(T)]
        try:
            with open(fname, "w+") as f:
                json.dump(d, f, indent=2)
        except IOError:
            sys.exit(f"[error occurred when trying to dump MCTSNC as json to file: {fname}]")
        t2 = time.time()
        if self.verbose_info:
            print(f"JSON DUMP DONE. [time: {t2 - t1} s]")


_LIVE = weakref.WeakSet()   # instances that hold a device-side engine


@atexit.register
def _close_all_engines():
    """Interpreter exit: every engine still alive gives its device memory, stream and events back while the HIP
    runtime is still fully up (Python's exit hooks run before the C runtime's), instead of from a destructor that
    may run after the runtime's own teardown has begun."""
    for e in list(_LIVE):
        try:
            e._release()
        except Exception:
            pass


def run_batch(engines, root_boards, root_extra_infos, root_turns, forced_search_steps_limit=np.inf, allocate=True):
    """Runs one search on each of several identically configured, initialised ``MCTSNC`` instances concurrently in
    one device pass (no counterpart in the reference).  Every instance ends in the state a separate ``run`` call
    would have left it in.  Returns the list of best actions.  ``allocate=False`` goes through the entry point that
    takes its per-call device buffers from the library's static scratch instead of allocating them (for callers that
    must not allocate device memory while running; batches beyond the scratch size are rejected)."""
    n = len(engines)
    e0 = engines[0]
    for e in engines:
        e._require_engine()
    boards = np.ascontiguousarray(np.stack([np.asarray(b, dtype=np.int8) for b in root_boards]))
    if root_extra_infos is None or root_extra_infos[0] is None:
        extras = np.zeros((n, 1), dtype=np.int8)
    else:
        extras = np.ascontiguousarray(np.stack([np.asarray(x, dtype=np.int8).reshape(-1) for x in root_extra_infos]))
    turns = np.ascontiguousarray(np.asarray(root_turns, dtype=np.int32))
    handles = (ctypes.c_void_p * n)(*[e._engine for e in engines])
    results = (_lib.Result * n)()
    entry = _lib.lib().mctsnc_run_batch if allocate else _lib.lib().mctsnc_run_batch_noalloc
    _lib.check(entry(handles, n, boards.ctypes.data, extras.ctypes.data, extras.shape[1], turns.ctypes.data,
                     float(e0.search_steps_limit), float(e0.search_time_limit), float(forced_search_steps_limit), results))
    for e, r, t in zip(engines, results, turns):
        e._absorb_result(r, int(t))
    return [e.best_action for e in engines]
