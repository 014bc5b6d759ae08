"""Gomoku positions for the host side (interface of src/gomoku.py:10-306, without numba)."""
import numpy as np

from .mcts import State

_DIRECTIONS = ((1, 0), (0, 1), (1, -1), (1, 1))


class Gomoku(State):
    M = 15
    N = 15
    SYMBOLS = ["○", "+", "●"]

    def __init__(self, parent=None):
        super().__init__(parent)
        if self.parent:
            self.board = np.copy(self.parent.board)
        else:
            self.board = np.zeros((Gomoku.M, Gomoku.N), dtype=np.int8)

    @staticmethod
    def class_repr():
        return f"{Gomoku.__name__}_{Gomoku.M}x{Gomoku.N}"

    def __str__(self):
        letters = "  " + "".join(chr(j + ord("A")) for j in range(Gomoku.N))
        rows = [str(i).rjust(2) + "".join(Gomoku.SYMBOLS[self.board[i - 1, j] + 1] for j in range(Gomoku.N)) + str(i).ljust(2)
                for i in range(Gomoku.M, 0, -1)]
        return letters + "\n" + "\n".join(rows) + "\n" + letters

    def take_action_job(self, action_index):
        """Places a stone of the player to move on crossing `action_index` (row-major); False when occupied or off the
        board."""
        i, j = action_index // Gomoku.N, action_index % Gomoku.N
        if i < 0 or i >= Gomoku.M or j < 0 or j >= Gomoku.N or self.board[i, j] != 0:
            return False
        self.board[i, j] = self.turn
        self.turn *= -1
        return True

    def compute_outcome_job(self):
        """The last mover wins with exactly five in a row through the last stone (a longer row does not count,
        src/gomoku.py:163-215); 0 when the board is full; None while the game goes on."""
        i, j = self.last_action_index // Gomoku.N, self.last_action_index % Gomoku.N
        token = -self.turn
        board = self.board
        for di, dj in _DIRECTIONS:
            total = 0
            for sign in (-1, 1):
                for k in range(1, 6):
                    r, c = i + sign * k * di, j + sign * k * dj
                    if r < 0 or r >= Gomoku.M or c < 0 or c >= Gomoku.N or board[r, c] != token:
                        break
                    total += 1
            if total == 4:
                return token
        if np.sum(board == 0) == 0:
            return 0
        return None

    def take_random_action_playout(self):
        return self.take_action(np.random.choice(np.where(np.ravel(self.board) == 0)[0]))

    def get_board(self):
        return self.board

    def get_extra_info(self):
        return None

    @staticmethod
    def action_name_to_index(action_name):
        j = ord(action_name.upper()[0]) - ord("A")
        i = int(action_name[1:]) - 1
        return i * Gomoku.N + j

    @staticmethod
    def action_index_to_name(action_index):
        return f"{chr(ord('A') + action_index % Gomoku.N)}{action_index // Gomoku.N + 1}"

    @staticmethod
    def get_board_shape():
        return (Gomoku.M, Gomoku.N)

    @staticmethod
    def get_extra_info_memory():
        return 0

    @staticmethod
    def get_max_actions():
        return Gomoku.M * Gomoku.N
