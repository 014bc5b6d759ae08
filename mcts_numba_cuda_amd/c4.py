"""Connect 4 positions for the host side (interface of src/c4.py:10-314, without numba)."""
import numpy as np

from .mcts import State

_DIRECTIONS = ((1, 0), (0, 1), (1, -1), (1, 1))


class C4(State):
    M = 6
    N = 7
    SYMBOLS = ["○", ".", "●"]

    def __init__(self, parent=None):
        super().__init__(parent)
        if self.parent:
            self.board = np.copy(self.parent.board)
            self.column_fills = np.copy(self.parent.column_fills)
        else:
            self.board = np.zeros((C4.M, C4.N), dtype=np.int8)
            self.column_fills = np.zeros(C4.N, dtype=np.int8)

    @staticmethod
    def class_repr():
        return f"{C4.__name__}_{C4.M}x{C4.N}"

    def __str__(self):
        rows = ["|" + "".join(C4.SYMBOLS[self.board[i, j] + 1] + "|" for j in range(C4.N)) for i in range(C4.M)]
        return "\n".join(rows) + "\n " + "".join(f"{j} " for j in range(C4.N))

    def take_action_job(self, action_index):
        """Drops a disc of the player to move into column `action_index`; False when the column is full."""
        j = action_index
        if self.column_fills[j] == C4.M:
            return False
        self.board[C4.M - 1 - self.column_fills[j], j] = self.turn
        self.column_fills[j] += 1
        self.turn *= -1
        return True

    def compute_outcome_job(self):
        """The last mover wins with at least four in a row through the last disc (three more within three cells on both
        sides, src/c4.py:166-218); 0 when the board is full; None while the game goes on."""
        j = self.last_action_index
        i = C4.M - self.column_fills[j]
        token = -self.turn
        board = self.board
        for di, dj in _DIRECTIONS:
            total = 0
            for sign in (-1, 1):
                for k in range(1, 4):
                    r, c = i + sign * k * di, j + sign * k * dj
                    if r < 0 or r >= C4.M or c < 0 or c >= C4.N or board[r, c] != token:
                        break
                    total += 1
            if total >= 3:
                return token
        if np.sum(board == 0) == 0:
            return 0
        return None

    def take_random_action_playout(self):
        return self.take_action(np.random.choice(np.where(self.column_fills < C4.M)[0]))

    def get_board(self):
        return self.board

    def get_extra_info(self):
        return self.column_fills

    @staticmethod
    def action_name_to_index(action_name):
        return int(action_name)

    @staticmethod
    def action_index_to_name(action_index):
        return str(action_index)

    @staticmethod
    def get_board_shape():
        return (C4.M, C4.N)

    @staticmethod
    def get_extra_info_memory():
        return C4.N

    @staticmethod
    def get_max_actions():
        return C4.N
