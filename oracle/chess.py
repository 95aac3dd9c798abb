"""ctypes front end of the C chess/encoder checker (oracle/chess.c).

TEST INFRASTRUCTURE: imported only by tests, the smoke check and the CPU
baseline leg of the benchmark.  Never imported by the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_chess.so")

STARTPOS_FEN = "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq - 0 1"

# pblczero.NetworkFormat.InputFormat (proto/net.proto:277-286)
INPUT_CLASSICAL_112_PLANE = 1
INPUT_112_WITH_CASTLING_PLANE = 2
INPUT_112_WITH_CANONICALIZATION = 3
INPUT_112_WITH_CANONICALIZATION_HECTOPLIES = 4
INPUT_112_WITH_CANONICALIZATION_V2 = 5
# FillEmptyHistory (src/neural/encoder.h:43)
FILL_NO, FILL_FEN_ONLY, FILL_ALWAYS = 0, 1, 2
# BoardTransform (src/utils/bititer.h:55-63)
NO_TRANSFORM, FLIP_TRANSFORM, MIRROR_TRANSFORM, TRANSPOSE_TRANSFORM = 0, 1, 2, 4


def build():
    subprocess.check_call(["make", "-C", _HERE, "liboracle_chess.so"],
                          stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    lib.orc_sizeof_board.restype = C.c_int
    lib.orc_board_from_fen.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_int), C.POINTER(C.c_int)]
    lib.orc_board_from_fen.restype = C.c_int
    lib.orc_perft.argtypes = [C.c_void_p, C.c_int]
    lib.orc_perft.restype = C.c_uint64
    lib.orc_gen_legal.argtypes = [C.c_void_p, C.POINTER(C.c_uint16)]
    lib.orc_gen_legal.restype = C.c_int
    lib.orc_parse_move.argtypes = [C.c_void_p, C.c_char_p]
    lib.orc_parse_move.restype = C.c_uint16
    lib.orc_move_to_uci.argtypes = [C.c_uint16, C.c_int, C.c_char_p]
    lib.orc_history_new.restype = C.c_void_p
    lib.orc_history_free.argtypes = [C.c_void_p]
    lib.orc_history_len.argtypes = [C.c_void_p]
    lib.orc_history_len.restype = C.c_int
    lib.orc_history_at.argtypes = [C.c_void_p, C.c_int]
    lib.orc_history_at.restype = C.c_void_p
    lib.orc_history_last_board.argtypes = [C.c_void_p]
    lib.orc_history_last_board.restype = C.c_void_p
    lib.orc_history_reset_fen.argtypes = [C.c_void_p, C.c_char_p]
    lib.orc_history_reset_fen.restype = C.c_int
    lib.orc_history_append.argtypes = [C.c_void_p, C.c_uint16]
    lib.orc_history_did_repeat_since_zeroing.argtypes = [C.c_void_p]
    lib.orc_history_did_repeat_since_zeroing.restype = C.c_int
    lib.orc_encode_position.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int,
                                        C.c_void_p, C.c_void_p, C.POINTER(C.c_int)]
    lib.orc_encode_position.restype = C.c_int
    lib.orc_move_to_nn_index.argtypes = [C.c_uint16, C.c_int]
    lib.orc_move_to_nn_index.restype = C.c_int
    lib.orc_move_str.argtypes = [C.c_int]
    lib.orc_move_str.restype = C.c_char_p
    lib.orc_random_playout.argtypes = [C.c_void_p, C.POINTER(C.c_uint64), C.c_char_p, C.c_int]
    lib.orc_random_playout.restype = C.c_int
    lib.orc_choose_transform.argtypes = [C.c_void_p]
    lib.orc_choose_transform.restype = C.c_int
    for name in ("orc_reverse_bits_in_bytes", "orc_reverse_bytes_in_bytes",
                 "orc_transpose_bits_in_bytes"):
        getattr(lib, name).argtypes = [C.c_uint64]
        getattr(lib, name).restype = C.c_uint64
    return lib


lib = _load()


class _PositionView(C.Structure):
    _fields_ = [("ours", C.c_uint64), ("theirs", C.c_uint64), ("rooks", C.c_uint64),
                ("bishops", C.c_uint64), ("pawns", C.c_uint64),
                ("our_king", C.c_uint8), ("their_king", C.c_uint8), ("castle", C.c_uint8),
                ("our_qrook", C.c_uint8), ("their_qrook", C.c_uint8),
                ("our_krook", C.c_uint8), ("their_krook", C.c_uint8), ("flipped", C.c_uint8),
                ("rule50", C.c_int), ("repetitions", C.c_int), ("cycle", C.c_int),
                ("ply", C.c_int)]


def perft(fen, depth):
    buf = C.create_string_buffer(lib.orc_sizeof_board())
    rc = lib.orc_board_from_fen(buf, fen.encode(), None, None)
    if rc:
        raise ValueError("bad fen (%d): %s" % (rc, fen))
    return lib.orc_perft(buf, depth)


class History:
    """Mirror of lczero::PositionHistory for the parts the encoder needs."""

    def __init__(self, fen=STARTPOS_FEN):
        self._h = lib.orc_history_new()
        rc = lib.orc_history_reset_fen(self._h, fen.encode())
        if rc:
            raise ValueError("bad fen (%d): %s" % (rc, fen))

    def __del__(self):
        if getattr(self, "_h", None):
            lib.orc_history_free(self._h)
            self._h = None

    def __len__(self):
        return lib.orc_history_len(self._h)

    def position(self, idx):
        if idx < 0:
            idx += len(self)
        p = _PositionView.from_address(lib.orc_history_at(self._h, idx))
        return p

    def black_to_move(self):
        return bool(self.position(-1).flipped)

    def parse_move(self, uci):
        m = lib.orc_parse_move(lib.orc_history_last_board(self._h), uci.encode())
        if m == 0xffff:
            raise ValueError("bad move " + uci)
        return m

    def append_uci(self, uci):
        lib.orc_history_append(self._h, self.parse_move(uci))

    def append(self, move):
        lib.orc_history_append(self._h, move)

    def legal_moves(self):
        arr = (C.c_uint16 * 256)()
        n = lib.orc_gen_legal(lib.orc_history_last_board(self._h), arr)
        return [arr[i] for i in range(n)]

    def did_repeat_since_last_zeroing_move(self):
        return bool(lib.orc_history_did_repeat_since_zeroing(self._h))

    def choose_transform(self):
        return lib.orc_choose_transform(lib.orc_history_last_board(self._h))

    def encode(self, input_format=INPUT_CLASSICAL_112_PLANE, history_planes=8,
               fill=FILL_FEN_ONLY):
        """Returns (masks u64[112], values f32[112], transform)."""
        masks = np.zeros(112, dtype=np.uint64)
        values = np.zeros(112, dtype=np.float32)
        t = C.c_int(0)
        rc = lib.orc_encode_position(self._h, input_format, history_planes, fill,
                                     masks.ctypes.data, values.ctypes.data, C.byref(t))
        if rc:
            raise ValueError("Unsupported input plane encoding %d" % input_format)
        return masks, values, t.value

    def random_playout(self, rng_state):
        """Replaces this history by a seeded random game; returns (uci, state)."""
        st = C.c_uint64(rng_state)
        buf = C.create_string_buffer(1024)
        lib.orc_random_playout(self._h, C.byref(st), buf, 1024)
        return buf.value.decode(), st.value


def move_to_uci(move, black_to_move):
    buf = C.create_string_buffer(6)
    lib.orc_move_to_uci(move, int(black_to_move), buf)
    return buf.value.decode()


def move_to_nn_index(move, transform=0):
    return lib.orc_move_to_nn_index(move, transform)


def move_strs():
    return [lib.orc_move_str(i).decode() for i in range(1858)]


def random_positions(n, seed, input_format=INPUT_CLASSICAL_112_PLANE, fill=FILL_FEN_ONLY):
    """n seeded random-playout positions.

    Returns dict(masks u64[n,112], values f32[n,112], uci list[str],
    legal list of int arrays (policy indices of the legal moves)).
    """
    masks = np.zeros((n, 112), dtype=np.uint64)
    values = np.zeros((n, 112), dtype=np.float32)
    ucis, legal = [], []
    state = seed
    h = History()
    for i in range(n):
        uci, state = h.random_playout(state)
        m, v, t = h.encode(input_format, 8, fill)
        masks[i], values[i] = m, v
        ucis.append(uci)
        legal.append(np.array(sorted(move_to_nn_index(mv, t) for mv in h.legal_moves()),
                              dtype=np.int32))
    return dict(masks=masks, values=values, uci=ucis, legal=legal)
