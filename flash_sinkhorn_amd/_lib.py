"""ctypes binding of ``libflash_sinkhorn_hip.so`` (C ABI in include/flash_sinkhorn_hip.h).

The shared object is built in-tree by ``flash_sinkhorn_amd/csrc/Makefile``.  There
is no fallback: if it is missing, every kernel entry point raises.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("FLASH_SINKHORN_HIP_LIB", os.path.join(_HERE, "libflash_sinkhorn_hip.so"))
CSRC_DIR = os.path.join(_HERE, "csrc")

FS_FLAG_EXP2 = 1
FS_FLAG_REDUCED_OPERANDS = 2
FS_FLAG_FP32_MFMA = 4
FS_FLAG_OPERANDS_PREPARED = 16
FS_FLAG_NO_TILE_SKIP = 32
FS_FLAG_COARSE_TEST = 64
FS_FLAG_COARSE_AUTO = 128
FS_FLAG_START_PLAIN = 256
FS_FLAG_NO_SWEEP = 512
# Every call runs on the two-plane fp16 operands (fp32-grade accuracy, the fastest mode here),
# whatever allow_tf32 says: permission to reduce precision is not an obligation.
# STRICT_OPERANDS (or env FLASH_SINKHORN_STRICT_OPERANDS) = "fp32_mfma" makes allow_tf32=False
# mean fp32 operands on the fp32 MFMA instruction instead.
STRICT_OPERANDS = os.environ.get("FLASH_SINKHORN_STRICT_OPERANDS", "fp16x2")
OP_LSE, OP_SYMMETRIC_STEP, OP_GRAD, OP_APPLY_VEC, OP_APPLY_MAT, OP_MAT5, OP_C_TRANSFORM = range(7)

# d <= 128 log-sum-exp kernel: leave out the exponentials of logits tiles that lie 2^40 below
# the running row maxima (no effect on fp32 sums); False computes every exponential.
TILE_SKIP = os.environ.get("FLASH_SINKHORN_TILE_SKIP", "1") != "0"
# Two-sided steps on prepared planes compute both sides' sums from one sweep over the logits
# once the potentials move little from step to step (FS_FLAG_NO_SWEEP switches that off)
SWEEP = os.environ.get("FLASH_SINKHORN_SWEEP", "1") != "0"
_lib: Optional[ctypes.CDLL] = None

_P = ctypes.c_void_p
_I = ctypes.c_int64
_F = ctypes.c_float
_U = ctypes.c_uint32
_Z = ctypes.c_size_t
_TAIL = [_U, _P, _Z, _P]  # flags, workspace, workspace_bytes, stream

_SIGNATURES = {
    "fs_version": (ctypes.c_int, []),
    "fs_error_string": (ctypes.c_char_p, [ctypes.c_int]),
    "fs_workspace_bytes": (_Z, [ctypes.c_int, _I, _I, _I]),
    "fs_prepare_operands": (ctypes.c_int, [_P] * 2 + [_I] * 3 + _TAIL),
    "fs_variant_state_offset": (_Z, [_P] * 2 + [_I] * 3 + [_U]),
    "fs_best_keys_offset": (_Z, [_P] * 2 + [_I] * 3 + [_U, ctypes.c_int]),
    "fs_lse": (ctypes.c_int, [_P] * 4 + [_I] * 3 + [_F] * 3 + _TAIL),
    "fs_lse_fused": (ctypes.c_int, [_P] * 5 + [_I] * 3 + [_F] * 3 + _TAIL),
    "fs_symmetric_step": (ctypes.c_int, [_P] * 10 + [_I] * 3 + [_F] * 5 + _TAIL),
    "fs_symmetric_step_noalloc": (ctypes.c_int, [_P] * 10 + [_I] * 3 + [_F] * 5 + [_U, _P]),
    "fs_symmetric_steps": (ctypes.c_int, [_P] * 12 + [_I] * 3 + [_P] * 4 + [ctypes.c_int, _F] + _TAIL),
    "fs_schur_matvec": (ctypes.c_int, [_P] * 11 + [_I] * 3 + [_F, _F] + _TAIL),
    "fs_cg_init": (ctypes.c_int, [_P] * 5 + [_I, _F, _F, _P]),
    "fs_cg_update": (ctypes.c_int, [_P] * 5 + [_I, _P]),
    "fs_self_pair_steps": (ctypes.c_int, [_P] * 12 + [_I] * 3 + [_P] * 5 + [ctypes.c_int, _F] + _TAIL),
    "fs_grad": (ctypes.c_int, [_P] * 13 + [_I] * 3 + [_F] * 2 + _TAIL),
    "fs_grad_seeded": (ctypes.c_int, [_P] * 13 + [_I] * 3 + [_F] * 2 + [_P] * 2 + _TAIL),
    "fs_apply_vec": (ctypes.c_int, [_P] * 8 + [_I] * 3 + [_F] * 2 + [ctypes.c_int] + _TAIL),
    "fs_apply_mat": (ctypes.c_int, [_P] * 9 + [_I] * 4 + [_F] * 2 + [ctypes.c_int] + _TAIL),
    "fs_mat5": (ctypes.c_int, [_P] * 8 + [_I] * 3 + [_F] * 2 + _TAIL),
    "fs_c_transform": (ctypes.c_int, [_P] * 5 + [_I] * 3 + [_F] + _TAIL),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def build(verbose: bool = False, force: bool = False) -> str:
    """Compile every HIP source for gfx950 (hipcc cross-compiles without a GPU); with
    ``force`` also the ones whose objects are up to date."""
    cmd = ["make", "-C", CSRC_DIR, "-j8"] + (["-B"] if force else [])
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("building libflash_sinkhorn_hip.so failed:\n" + res.stdout[-4000:]
                           + res.stderr[-8000:])
    if verbose:
        print(res.stdout[-2000:])
    return LIB_PATH


def lib() -> ctypes.CDLL:
    """Load the shared object once; raise loudly when it is not there."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
                "(flash_sinkhorn_amd has no non-HIP code path).")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = lib().fs_error_string(code).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {code})")


def ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def stream_of(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def workspace(op: int, n: int, m: int, d: int, device) -> Optional[torch.Tensor]:
    nbytes = int(lib().fs_workspace_bytes(op, n, m, d))
    if nbytes == 0:
        return None
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def flags(use_exp2: bool, allow_tf32: bool) -> int:
    f = FS_FLAG_EXP2 if use_exp2 else 0
    if not TILE_SKIP:
        f |= FS_FLAG_NO_TILE_SKIP
    if not SWEEP:
        f |= FS_FLAG_NO_SWEEP
    if STRICT_OPERANDS not in _STRICT_FLAGS:
        raise ValueError(f"STRICT_OPERANDS must be one of {sorted(_STRICT_FLAGS)}")
    if allow_tf32:
        return f | FS_FLAG_REDUCED_OPERANDS  # accepted by the library, same kernels as the default
    return f | _STRICT_FLAGS[STRICT_OPERANDS]


_STRICT_FLAGS = {"fp16x2": 0, "fp32_mfma": FS_FLAG_FP32_MFMA}
# words of the variant-choice state: the permission for the one-sweep step (kSelSweep) and the
# count of such steps that were redone (kSelSweepRedone)
_SEL_SWEEP, _SEL_REDONE = 247, 269


class PreparedOperands:
    """16-bit operand planes of (x, y), written once into a workspace that every LSE call
    of a solver loop then shares (``fs_prepare_operands`` + ``FS_FLAG_OPERANDS_PREPARED``).

    x and y must stay alive and unchanged while the object is in use, and the calls must
    run on the stream current at construction.
    """

    def __init__(self, x: torch.Tensor, y: torch.Tensor, flag_bits: int, self_pair: bool = False,
                 start_plain: bool = False):
        n, d = x.shape
        m = y.shape[0]
        L = lib()
        nbytes = max(int(L.fs_workspace_bytes(op, n, m, d))
                     for op in (OP_LSE, OP_SYMMETRIC_STEP))
        if self_pair:  # the two self problems of fs_self_pair_steps share the workspace
            nbytes = max(nbytes, int(L.fs_workspace_bytes(OP_SYMMETRIC_STEP, n, n, d))
                         + int(L.fs_workspace_bytes(OP_SYMMETRIC_STEP, m, m, d)))
        self.ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
        self.nbytes = nbytes
        self.flag_bits = flag_bits
        self.keys = {(x.data_ptr(), n), (y.data_ptr(), m)}
        self.d = d
        self.state_offset = int(L.fs_variant_state_offset(x.data_ptr(), y.data_ptr(), n, m, d,
                                                          flag_bits))
        self._keys_at = [(int(L.fs_best_keys_offset(x.data_ptr(), y.data_ptr(), n, m, d, flag_bits, w)),
                          rows) for w, rows in ((0, n), (1, m))]
        # start_plain: with the kernel variant left to the device, the first steps run the plain
        # kernel (a schedule that begins at a large eps begins on a flat plan)
        check(L.fs_prepare_operands(x.data_ptr(), y.data_ptr(), n, m, d,
                                    flag_bits | (FS_FLAG_START_PLAIN if start_plain else 0),
                                    self.ws.data_ptr(), nbytes, stream_of(x)),
              "fs_prepare_operands")

    def best_keys(self, which: int) -> Optional[torch.Tensor]:
        """View (int32, one entry per row of x for ``which`` = 0, of y for 1) of the keys the
        kernel with the coarse tile test starts its rows from; None when the configuration keeps
        none.  Whatever a caller writes there, results stay exact: a diagnostic and test hook."""
        off, rows = self._keys_at[which]
        if off == 0:
            return None
        return self.ws[off:off + 4 * rows].view(torch.int32)

    def variant_state(self) -> dict:
        """What ``FS_FLAG_COARSE_AUTO`` has done on these planes so far (reads the device: a
        diagnostic, not part of any solve): which variant the steps now run, and how many
        32 x 32 logits tiles of the coarse variant ended at its test."""
        if self.state_offset == 0:
            return {"plain_selected": True, "decisions": 0, "tiles_ended": 0, "tiles_tested": 0,
                    "tiles_skipped": 0, "sweep_next": False, "sweep_redone": 0}
        w = self.ws[self.state_offset:self.state_offset + 4 * _SEL_REDONE + 4].cpu().view(torch.int32).tolist()
        u = [v & 0xFFFFFFFF for v in w]
        # sweep_next: the next two-sided step may take both sides' sums from one sweep over the
        # logits; sweep_redone: how many such steps the two-sided kernel had to redo so far
        return {"plain_selected": u[0] != 0, "decisions": u[1],
                "tiles_ended": u[2] | (u[3] << 32), "tiles_tested": u[4] | (u[5] << 32),
                "tiles_skipped": u[6] | (u[7] << 32), "sweep_next": u[_SEL_SWEEP] != 0,
                "sweep_redone": u[_SEL_REDONE]}

    def serves(self, x: torch.Tensor, y: torch.Tensor, flag_bits: int) -> bool:
        # the workspace layout depends on the set of matrices, so the call must name the same set
        # (the permission bit and the choice of kernels for a two-sided step do not change the planes)
        same = ~(FS_FLAG_REDUCED_OPERANDS | FS_FLAG_NO_SWEEP)
        return ((flag_bits & same) == (self.flag_bits & same) and x.shape[1] == self.d
                and {(x.data_ptr(), x.shape[0]), (y.data_ptr(), y.shape[0])} == self.keys)


def coarse_flag(coarse) -> int:
    """Flag bits for the ``coarse`` argument of the step launchers: False, True or "auto"."""
    if coarse == "auto":
        return FS_FLAG_COARSE_AUTO
    return FS_FLAG_COARSE_TEST if coarse else 0


def lse_workspace(op: int, x: torch.Tensor, y: torch.Tensor, flag_bits: int,
                  prepared: Optional[PreparedOperands]):
    """(workspace pointer, bytes, flags, keep-alive) for an LSE-type call."""
    if prepared is not None and prepared.serves(x, y, flag_bits):
        return (prepared.ws.data_ptr(), prepared.nbytes,
                flag_bits | FS_FLAG_OPERANDS_PREPARED, prepared.ws)
    ws = workspace(op, x.shape[0], y.shape[0], x.shape[1], x.device)
    return ptr(ws), 0 if ws is None else ws.numel(), flag_bits, ws
