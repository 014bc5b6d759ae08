"""Host-side game-state base class and the single-threaded CPU MCTS the reference plays its GPU searches against:
the interface of src/mcts.py (``State`` :29-319, ``MCTS`` :321-629) without numba, so that the reference's callers
(src/game_runner.py, src/main.py) find the same names, arguments, attributes and printed lines.

The random choices (child picked after an expansion, playout moves) go through numpy's legacy global generator,
seeded in the constructor exactly as the reference does, so a search consumes the same stream as the reference's and
ends with the same statistics."""
import time

import numpy as np

from .utils import dict_to_str


class State:
    """A position of a two-player game; subclass it (see c4.C4, gomoku.Gomoku) and implement ``take_action_job``,
    ``compute_outcome_job``, ``take_random_action_playout``, ``__str__``, ``class_repr`` for CPU searches and
    ``get_board``, ``get_extra_info``, ``get_board_shape``, ``get_extra_info_memory``, ``get_max_actions`` for
    ``MCTSNC`` searches (src/mcts.py:39-46)."""

    def __init__(self, parent=None):
        self.win_flag = False
        self.n = 0
        self.n_wins = 0
        self.parent = parent
        self.children = {}
        self.outcome_computed = False
        self.outcome = None   # None while the game goes on, else -1 / 0 / +1
        self.turn = 1 if parent is None else parent.turn
        self.last_action_index = None

    def __str__(self):
        pass

    @staticmethod
    def class_repr():
        pass

    # ---- tree statistics (src/mcts.py:89-110) ----
    def _subtree_size(self):
        return 1 + sum(child._subtree_size() for child in self.children.values())

    def _subtree_max_depth(self):
        return max((1 + child._subtree_max_depth() for child in self.children.values()), default=0)

    def _subtree_depths(self, d=0, depths=[]):
        depths.append(d)
        for child in self.children.values():
            child._subtree_depths(d + 1, depths)
        return depths

    def get_turn(self):
        return self.turn

    def take_action(self, action_index):
        """The child reached by `action_index`: the existing one, or a new one built by ``take_action_job``; None when
        the action is illegal (src/mcts.py:122-145)."""
        known = self.children.get(action_index)
        if known is not None:
            return known
        child = type(self)(self)
        if not child.take_action_job(action_index):
            return None
        child.last_action_index = action_index
        self.children[action_index] = child
        return child

    def take_action_job(self, action_index):
        pass

    def compute_outcome(self):
        """Memoised outcome; a state whose previous mover has just won gets its ``win_flag`` set (src/mcts.py:164-184)."""
        if self.outcome_computed:
            return self.outcome
        if self.last_action_index is None:
            return None
        self.outcome = self.compute_outcome_job()
        self.outcome_computed = True
        if self.outcome == -self.turn:
            self.win_flag = True
        return self.outcome

    def compute_outcome_job(self):
        pass

    def get_board(self):
        pass

    def get_extra_info(self):
        return None

    def expand(self):
        """Creates all children of a non-terminal state that has none (src/mcts.py:229-235)."""
        if not self.children and self.compute_outcome() is None:
            for action_index in range(type(self).get_max_actions()):
                self.take_action(action_index)

    def take_random_action_playout(self):
        pass

    @staticmethod
    def action_name_to_index(action_name):
        pass

    @staticmethod
    def action_index_to_name(action_index):
        pass

    @staticmethod
    def get_board_shape():
        pass

    @staticmethod
    def get_extra_info_memory():
        pass

    @staticmethod
    def get_max_actions():
        pass


class MCTS:
    """Standard single-threaded Monte Carlo Tree Search on the host (src/mcts.py:321-629)."""

    DEFAULT_SEARCH_TIME_LIMIT = 5.0
    DEFAULT_SEARCH_STEPS_LIMIT = np.inf
    DEFAULT_VANILLA = True
    DEFAULT_UCB_C = 2.0
    DEFAULT_SEED = 0
    DEFAULT_VERBOSE_DEBUG = False
    DEFAULT_VERBOSE_INFO = True

    def __init__(self, search_time_limit=DEFAULT_SEARCH_TIME_LIMIT, search_steps_limit=DEFAULT_SEARCH_STEPS_LIMIT,
                 vanilla=DEFAULT_VANILLA, ucb_c=DEFAULT_UCB_C, seed=DEFAULT_SEED, verbose_debug=DEFAULT_VERBOSE_DEBUG,
                 verbose_info=DEFAULT_VERBOSE_INFO):
        self.search_time_limit = search_time_limit
        self.search_steps_limit = search_steps_limit
        self.vanilla = vanilla
        self.ucb_c = ucb_c
        self.seed = seed
        np.random.seed(self.seed)
        self.verbose_debug = verbose_debug
        self.verbose_info = verbose_info

    def __str__(self):
        return (f"MCTS(search_time_limit={self.search_time_limit}, search_steps_limit={self.search_steps_limit}, "
                f"vanilla={self.vanilla}, ucb_c={self.ucb_c}, seed: {self.seed})")

    def __repr__(self):
        return self.__str__()

    def _make_performance_info(self):
        ms = 1e3
        times = {"total": ms * self.time_total, "loop": ms * self.time_loop,
                 "reduce_over_actions": ms * self.time_reduce_over_actions}
        times["mean_loop"] = times["loop"] / self.steps
        for stage in ("select", "expand", "playout", "backup"):
            times["mean_" + stage] = ms * getattr(self, "time_" + stage) / self.steps
        tree = {"initial_n_root": self.initial_n_root, "initial_mean_depth": self.initial_mean_depth,
                "initial_max_depth": self.initial_max_depth, "initial_size": self.initial_size, "n_root": self.root.n,
                "mean_depth": np.mean(self.root._subtree_depths(0, [])), "max_depth": self.root._subtree_max_depth(),
                "size": self.root._subtree_size()}
        self.performance_info = {"steps": self.steps, "steps_per_second": self.steps / self.time_total,
                                 "playouts": self.root.n, "playouts_per_second": self.root.n / self.time_total,
                                 "times_[ms]": times, "tree": tree}
        return self.performance_info

    def _make_actions_info(self, children, best_action_entry=False):
        info = {}
        for key, child in children.items():
            n_root, n, n_wins = child.parent.n, child.n, child.n_wins
            q = n_wins / n if n > 0 else 0.0
            ucb = q + self.ucb_c * np.sqrt(np.log(n_root) / n) if n > 0 else np.inf
            info[key] = {"name": type(child).action_index_to_name(key), "n_root": n_root, "win_flag": child.win_flag,
                         "n": n, "n_wins": n_wins, "q": n_wins / n if n > 0 else np.nan, "ucb": ucb}
        if best_action_entry:
            best_key = self._best_action(children, info)
            info["best"] = {"index": best_key, **info[best_key]}
        self.actions_info = info
        return info

    def _best_action_ucb(self, children, actions_info):
        best_key, best_ucb = None, -1.0
        for key in children:
            if actions_info[key]["ucb"] > best_ucb:
                best_key, best_ucb = key, actions_info[key]["ucb"]
        return best_key

    def _best_action(self, root_children, root_actions_info):
        """Final decision: win flag first, then visits, then wins (src/mcts.py:456-480)."""
        self.best_action, self.best_win_flag, self.best_n, self.best_n_wins = None, False, -1, -1
        for key in root_children:
            entry = root_actions_info[key]
            candidate = (entry["win_flag"], entry["n"], entry["n_wins"])
            if candidate > (self.best_win_flag, self.best_n, self.best_n_wins):
                self.best_win_flag, self.best_n, self.best_n_wins = candidate
                self.best_action = key
        self.best_q = self.best_n_wins / self.best_n if self.best_n > 0 else np.nan
        return self.best_action

    def run(self, root, forced_search_steps_limit=np.inf):
        """Searches from `root` within the budget (`forced_search_steps_limit` overrides both limits) and returns the
        best action (src/mcts.py:482-588)."""
        print("MCTS RUN...")
        t_start = time.time()
        self.root = root
        root.parent = None
        if self.vanilla:
            root.n = 0
            root.children = {}
        if self.verbose_info:
            self.initial_n_root = root.n
            self.initial_mean_depth = np.mean(root._subtree_depths(0, []))
            self.initial_max_depth = root._subtree_max_depth()
            self.initial_size = root._subtree_size()
        self.time_select = self.time_expand = self.time_playout = self.time_backup = 0.0
        self.steps = 0
        stages = (("select", self._select), ("expand", self._expand))
        t_loop = time.time()
        while True:
            now = time.time()
            if forced_search_steps_limit < np.inf:
                if self.steps >= forced_search_steps_limit:
                    break
            elif self.steps >= self.search_steps_limit or now - t_loop >= self.search_time_limit:
                break
            state = root
            for name, stage in stages:
                state = self._timed(name, stage, state)
            playout_root = state
            state = self._timed("playout", self._playout, state)
            self._timed("backup", lambda s: self._backup(s, playout_root), state)
            self.steps += 1
        self.time_loop = time.time() - t_loop

        t_reduce = time.time()
        if self.verbose_debug:
            print("[MCTS._reduce_over_actions()...]")
        self._reduce_over_actions()
        best_action_label = f"{self.best_action} ({type(root).action_index_to_name(self.best_action)})"
        self.time_reduce_over_actions = time.time() - t_reduce
        if self.verbose_debug:
            print(f"[MCTS._reduce_over_actions() done; time: {self.time_reduce_over_actions} s]")
        self.time_total = time.time() - t_start
        if self.verbose_info:
            print(f"[actions info:\n{dict_to_str(self.root_actions_info)}]")
            print(f"[performance info:\n{dict_to_str(self._make_performance_info())}]")
        print(f"MCTS RUN DONE. [time: {self.time_total} s; best action: {best_action_label}, best win_flag: "
              f"{self.best_win_flag}, best n: {self.best_n}, best n_wins: {self.best_n_wins}, best q: {self.best_q}]")
        return self.best_action

    def _timed(self, name, stage, state):
        if self.verbose_debug:
            print(f"[MCTS._{name}()...]")
        t = time.time()
        result = stage(state)
        dt = time.time() - t
        if self.verbose_debug:
            print(f"[MCTS._{name}() done; time: {dt} s]")
        setattr(self, "time_" + name, getattr(self, "time_" + name) + dt)
        return result

    def _select(self, state):
        while state.children:
            info = self._make_actions_info(state.children)
            state = state.children[self._best_action_ucb(state.children, info)]
        return state

    def _expand(self, state):
        state.expand()
        if state.children:
            state = state.children[np.random.choice(list(state.children.keys()))]
        return state

    def _playout(self, state):
        while state.compute_outcome() is None:
            state = state.take_random_action_playout()
        return state

    def _backup(self, state, playout_root):
        outcome = state.compute_outcome()
        playout_root.children = {}   # the playout branch is dropped
        state = playout_root
        while state:
            state.n += 1
            if state.turn == -outcome:
                state.n_wins += 1
            state = state.parent

    def _reduce_over_actions(self):
        self.root_actions_info = self._make_actions_info(self.root.children, best_action_entry=True)
