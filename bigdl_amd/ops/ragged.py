"""Operations of the ragged engine (``bigdl_amd/models/ragged_engine.py``) over a flat batch of token rows.

Two implementations of one interface:

* ``HipOps``: the gfx950 kernels of ``libbigdl_ragged.so`` (``bigdl_amd/csrc/ragged``), loaded with ctypes and launched
  on PyTorch's current stream.  The library is small and separate from ``libbigdl_hip.so`` so that a checkout without
  built files compiles only what this engine needs (a handful of translation units, side by side) the first time it is used.
* ``TorchOps``: the same operations as unfused PyTorch statements, sequence by sequence.  It exists for host-side tests
  of the engine's bookkeeping (pages, slots, portions) and is only ever chosen for tensors on the CPU; on a GPU the
  kernels run or the call raises.

Activations (``act``) are bfloat16 or float32; residual stream, norms, rotary angles, attention scores, gates and
recurrent state are float32 in both.
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess
import sys
from pathlib import Path

import torch
import torch.nn.functional as F

PAGE = 64
_PKG = Path(__file__).resolve().parent.parent
_SRC = _PKG / "csrc" / "ragged"
_LIB_PATH = Path(os.environ.get("BIGDL_RAGGED_LIB") or _PKG / "lib" / "libbigdl_ragged.so")
_LIB = None
_DT = {torch.bfloat16: 1, torch.float32: 2}

HIP_FLAGS = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Wall", "-Wno-unused-function", "-DNDEBUG",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(force: bool = False) -> Path:
    """Compile ``csrc/ragged/*.hip`` into ``lib/libbigdl_ragged.so`` (hipcc cross-compiles gfx950 without a GPU)."""
    srcs = sorted(_SRC.glob("*.hip"))
    deps = srcs + sorted(_SRC.glob("*.h"))
    if not force and _LIB_PATH.exists() and all(p.stat().st_mtime <= _LIB_PATH.stat().st_mtime for p in deps):
        return _LIB_PATH
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _LIB_PATH.parent.mkdir(exist_ok=True)
    tmp = _LIB_PATH.with_suffix(f".{os.getpid()}.tmp")
    # the translation units are compiled side by side (one hipcc each), then linked
    objs = [_LIB_PATH.parent / f".ragged_{os.getpid()}_{p.stem}.o" for p in srcs]
    procs = [(subprocess.Popen([hipcc, *HIP_FLAGS, "-c", "-o", str(o), str(p)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                               text=True), p) for p, o in zip(srcs, objs)]
    failed = []
    for proc, p in procs:
        out, _ = proc.communicate()
        if proc.returncode != 0:
            failed.append(f"{p}:\n{out}")
    try:
        if not failed:
            cmd = [hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", str(tmp), *map(str, objs)]
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                failed.append(" ".join(cmd) + "\n" + r.stdout + r.stderr)
    finally:
        for o in objs:
            if o.exists():
                o.unlink()
    if failed:
        sys.stderr.write("\n".join(failed))
        raise RuntimeError("building libbigdl_ragged.so failed")
    os.replace(tmp, _LIB_PATH)
    return _LIB_PATH


class _Batch(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in ("tok_seq", "tok_pos", "seq_start", "seq_past", "seq_slot", "pages")] + \
               [(n, ctypes.c_int) for n in ("T", "B", "max_pages")]


class _ConvHeadArgs(ctypes.Structure):
    _fields_ = [("P", ctypes.c_void_p), ("ldp", ctypes.c_int64), ("col0", ctypes.c_int), ("cw", ctypes.c_void_p),
                ("taps", ctypes.c_int), ("C", ctypes.c_int), ("ch0", ctypes.c_int), ("state", ctypes.c_void_p),
                ("ngroups", ctypes.c_int), ("gsize", ctypes.c_int), ("normw", ctypes.c_void_p), ("eps", ctypes.c_float),
                ("rot", ctypes.c_int), ("cossin", ctypes.c_void_p), ("out_dense", ctypes.c_void_p),
                ("pages", ctypes.c_void_p), ("rowlen", ctypes.c_int), ("heads", ctypes.c_int), ("norm_n", ctypes.c_int),
                ("rot0", ctypes.c_int), ("interleaved", ctypes.c_int)]


class _AttnArgs(ctypes.Structure):
    _fields_ = [("q", ctypes.c_void_p), ("kpages", ctypes.c_void_p), ("vpages", ctypes.c_void_p), ("out", ctypes.c_void_p),
                ("gate", ctypes.c_void_p), ("ldg", ctypes.c_int64), ("gate0", ctypes.c_int), ("H", ctypes.c_int),
                ("G", ctypes.c_int), ("d", ctypes.c_int), ("vd", ctypes.c_int), ("window", ctypes.c_int),
                ("keep_first", ctypes.c_int), ("scale", ctypes.c_float), ("lam", ctypes.c_float),
                ("out_scale", ctypes.c_float), ("out_norm", ctypes.c_int), ("eps", ctypes.c_float),
                ("rows", ctypes.c_void_p), ("n_rows", ctypes.c_int), ("tiles", ctypes.c_void_p), ("n_tiles", ctypes.c_int),
                ("ldv", ctypes.c_int64), ("sink", ctypes.c_int), ("sink_score", ctypes.c_float), ("chunk", ctypes.c_int),
                ("softcap", ctypes.c_float), ("gate_wide", ctypes.c_int), ("sinks", ctypes.c_void_p),
                ("slopes", ctypes.c_void_p)]


def lib():
    global _LIB
    if _LIB is None:
        if not _LIB_PATH.exists():
            build()
        L = ctypes.CDLL(str(_LIB_PATH))
        vp, i64, ci, cf = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
        L.ragged_sum_group_norm.argtypes = [vp, vp, vp, vp, vp, i64, ci, ci, cf, cf, ci, vp]
        L.ragged_conv_head.argtypes = [_ConvHeadArgs, _Batch, ci, vp]
        L.ragged_conv_state.argtypes = [vp, i64, ci, vp, ci, ci, _Batch, ci, vp]
        L.ragged_clamped_glu.argtypes = [vp, vp, i64, ci, cf, cf, ci, vp]
        L.ragged_hgrn2_gates.argtypes = [vp, i64, ci, ci, vp, vp, vp, vp, i64, ci, ci, vp]
        L.ragged_hgrn2_scan.argtypes = [vp, vp, vp, vp, i64, ci, vp, vp, ci, ci, ci, ci, _Batch, ci, vp]
        L.ragged_post_norm_add.argtypes = [vp, vp, vp, vp, vp, i64, ci, cf, ci, vp]
        L.ragged_mlstm_gates.argtypes = [vp, i64, ci, vp, cf, cf, vp, vp, vp, vp, ci, _Batch, ci, vp]
        L.ragged_mlstm_expand.argtypes = [vp, i64, ci, ci, vp, vp, vp, vp, vp, i64, ci, ci, ci, vp]
        L.ragged_head_norm_gate.argtypes = [vp, vp, vp, i64, ci, vp, i64, ci, ci, cf, ci, vp, cf, cf, ci, vp]
        L.ragged_moe_route.argtypes = [vp, i64, vp, vp, vp, i64, ci, ci, ci, ci, ci, cf, ci, ci, ci, ci, vp]
        L.ragged_embed_rows.argtypes = [vp, vp, vp, vp, cf, vp, i64, ci, ci, vp]
        L.ragged_add_norm.argtypes = [vp, vp, vp, vp, vp, i64, ci, cf, ci, vp]
        L.ragged_act_cols.argtypes = [vp, i64, ci, vp, i64, ci, ci, cf, cf, ci, vp]
        L.ragged_hc_step.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, ci, ci, cf, ci, vp]
        L.ragged_gate_cols.argtypes = [vp, vp, i64, ci, vp, i64, ci, cf, ci, vp]
        L.ragged_delta_gates.argtypes = [vp, i64, ci, ci, ci, vp, vp, vp, cf, cf, vp, vp, vp, vp, vp, i64, ci, ci, ci, vp]
        L.ragged_delta_scan.argtypes = [vp, vp, vp, vp, vp, vp, i64, ci, vp, vp, ci, ci, ci, ci, _Batch, ci, vp]
        L.ragged_delta_chain_ok.argtypes = [ci]
        L.ragged_delta_chain.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, vp]
        L.ragged_glu_pairs.argtypes = [vp, i64, vp, i64, ci, ci, vp]
        L.ragged_relu2.argtypes = [vp, vp, i64, ci, vp]
        L.ragged_moe_combine.argtypes = [vp, vp, vp, vp, vp, i64, ci, ci, ci, vp]
        L.ragged_moe_grouped_ok.argtypes = [ci, ci, ci]
        L.ragged_moe_tile_map.argtypes = [vp, ci, vp, vp, vp, ci, vp]
        L.ragged_moe_grouped_gemm.argtypes = [vp, i64, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
        L.ragged_moe_rows.argtypes = [vp, i64, vp, vp, vp, vp, vp, vp, vp, i64, ci, ci, ci, ci, ci, vp]
        L.ragged_hgrn2_chunk_decay.argtypes = [vp, vp, vp, ci, ci, vp]
        L.ragged_hgrn2_chunk_combine.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, vp]
        L.ragged_row_norm.argtypes = [vp, vp, vp, i64, ci, cf, ci, vp]
        L.ragged_paged_attn.argtypes = [_AttnArgs, _Batch, ci, ci, vp]
        L.ragged_paged_attn_mfma.argtypes = [_AttnArgs, _Batch, ci, vp]
        L.ragged_paged_attn_mfma_ok.argtypes = [ci, ci]
        L.ragged_paged_attn_mfma_wide.argtypes = [_AttnArgs, _Batch, vp]
        L.ragged_paged_attn_mfma_heads.argtypes = [_AttnArgs, _Batch, vp]
        L.ragged_paged_attn_mfma_wide_ok.argtypes = [ci, ci]
        _LIB = L
    return _LIB


class BatchMeta:
    """One step's batch: ``seqs`` is a list of (slot, past, n_new, page ids covering past + n_new tokens)."""

    def __init__(self, seqs, device, max_pages=None, static=False):
        """``static``: the device buffer keeps its address and layout (``max_pages`` fixed) and ``update`` refills it, so
        that a step recorded into a hipGraph reads the next step's batch from the same place."""
        device = torch.device(device)
        self.device = device
        self.B = len(seqs)
        self.T = sum(n for _, _, n, _ in seqs)
        self.max_pages = max_pages or max(1, max(len(pg) for *_, pg in seqs))
        T, B = self.T, self.B
        self._static = static
        self._c = None
        self._split = {}
        self._rot = {}
        self._chunks = {}
        if static:
            size = 2 * T + 3 * B + 1 + B * self.max_pages
            self._host = torch.empty(size, dtype=torch.int32, pin_memory=device.type == "cuda")
            self.buf = torch.empty(size, dtype=torch.int32, device=device)
            self._views()
        self.update(seqs)

    def _views(self):
        T, B, buf = self.T, self.B, self.buf
        o = [0, T, 2 * T, 2 * T + B + 1, 2 * T + 2 * B + 1, 2 * T + 3 * B + 1]
        self.tok_seq, self.tok_pos = buf[o[0]:o[1]], buf[o[1]:o[2]]
        self.seq_start, self.seq_past, self.seq_slot = buf[o[2]:o[3]], buf[o[3]:o[4]], buf[o[4]:o[5]]
        self.pages = buf[o[5]:].view(B, self.max_pages)

    def update(self, seqs):
        """Fill the buffer for this step's sequences (same count and row total as at construction)."""
        self.seqs = seqs
        self.start = [0]
        for _, _, n, _ in seqs:
            self.start.append(self.start[-1] + n)
        if len(seqs) != self.B or self.start[-1] != self.T or max(len(pg) for *_, pg in seqs) > self.max_pages:
            raise ValueError("this batch does not fit the buffer's layout")
        tok_seq, tok_pos = [], []
        for b, (_, past, n, _) in enumerate(seqs):
            tok_seq += [b] * n
            tok_pos += range(past, past + n)
        flat = tok_seq + tok_pos + self.start + [s[1] for s in seqs] + [s[0] for s in seqs]
        for *_, pg in seqs:
            flat += list(pg) + [0] * (self.max_pages - len(pg))
        if self._static:
            self._host.copy_(torch.tensor(flat, dtype=torch.int32))
            self.buf.copy_(self._host, non_blocking=True)
            return
        buf = torch.tensor(flat, dtype=torch.int32)
        if self.device.type == "cuda":
            buf = buf.pin_memory().to(self.device, non_blocking=True)
        self.buf = buf
        self._views()

    def chunks(self, length: int):
        """Every sequence's rows cut into chunks of ``length``: (number of chunks, device int32 arrays
        chunk_start[NC + 1] (token rows), zeros[NC], ones[NC], chunk_id[NC], first_chunk_of_sequence[B + 1]) and the
        host list of each sequence's last chunk."""
        if length not in self._chunks:
            cstart, cfirst, last = [0], [0], []
            for _, _, n, _ in self.seqs:
                for c0 in range(0, n, length):
                    cstart.append(cstart[-1] + min(length, n - c0))
                cfirst.append(len(cstart) - 1)
                last.append(len(cstart) - 2)
            nc = len(cstart) - 1
            flat = cstart + [0] * nc + [1] * nc + list(range(nc)) + cfirst
            buf = torch.tensor(flat, dtype=torch.int32)
            if self.device.type == "cuda":
                buf = buf.pin_memory().to(self.device, non_blocking=True)
            o = [0, nc + 1, 2 * nc + 1, 3 * nc + 1, 4 * nc + 1]
            self._chunks[length] = (nc, buf[o[0]:o[1]], buf[o[1]:o[2]], buf[o[2]:o[3]], buf[o[3]:o[4]], buf[o[4]:], last)
        return self._chunks[length]

    def cossin(self, inv_freq: torch.Tensor, amp: float = 1.0) -> torch.Tensor:
        """[T, rot / 2, 2] float32: ``amp`` times cos and sin of position * frequency for every row, made once per step
        and set of frequencies with the library's full-precision functions (the angle itself is the float32 product)."""
        key = (inv_freq.data_ptr(), float(amp))
        if key not in self._rot:
            ang = self.tok_pos.to(inv_freq.device).float()[:, None] * inv_freq[None]
            tab = torch.stack([ang.cos(), ang.sin()], -1)
            self._rot[key] = (tab * float(amp) if amp != 1.0 else tab).contiguous()
        return self._rot[key]

    def attn_split(self, min_rows: int):
        """Portions of at least ``min_rows`` rows as 64-row tiles [(sequence, first row)] for the matrix-core attention
        kernel, all other token rows as a list for the row-wise kernel: (tiles, n_tiles, rows, n_rows), device int32."""
        if min_rows not in self._split:
            tiles, rows = [], []
            for b, (_, _, n, _) in enumerate(self.seqs):
                if n >= min_rows:
                    tiles += [v for r0 in range(0, n, 64) for v in (b, r0)]
                else:
                    rows += range(self.start[b], self.start[b] + n)
            buf = torch.tensor(tiles + rows + [0], dtype=torch.int32)
            if self.device.type == "cuda":
                buf = buf.pin_memory().to(self.device, non_blocking=True)
            self._split[min_rows] = (buf[:len(tiles)], len(tiles) // 2, buf[len(tiles):len(tiles) + len(rows)], len(rows))
        return self._split[min_rows]

    def c(self):
        if self._c is None:
            self._c = _Batch(self.tok_seq.data_ptr(), self.tok_pos.data_ptr(), self.seq_start.data_ptr(),
                             self.seq_past.data_ptr(), self.seq_slot.data_ptr(), self.pages.data_ptr(), self.T, self.B,
                             self.max_pages)
        return self._c


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ok(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what}: the native launcher rejected the call (code {rc})")


def _f32(*ts):
    for t in ts:
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or t.device.type != "cuda"):
            raise ValueError("expected a contiguous float32 tensor on the HIP device")


def _act(*ts):
    for t in ts:
        if t is not None and (t.dtype not in _DT or t.stride(-1) != 1 or t.device.type != "cuda"):
            raise ValueError("expected a bfloat16 / float32 tensor with contiguous rows on the HIP device")


def _page_check(meta: BatchMeta, pages: torch.Tensor):
    need = max((p for *_, pg in meta.seqs for p in pg), default=0)
    if need >= pages.shape[0] or pages.shape[2] != PAGE or not pages.is_contiguous():
        raise ValueError("page ids outside the pool, or a pool that is not [pages, heads, 64, row]")
    for _, past, n, pg in meta.seqs:
        if len(pg) * PAGE < past + n:
            raise ValueError("a sequence's pages do not cover its tokens")


class HipOps:
    """The kernels.  Every call checks shapes against what the kernel's indexing assumes before it launches."""
    name = "hip"
    mfma = os.environ.get("BIGDL_RAGGED_MFMA", "1") != "0"      # 0: every row through the row-wise attention kernel
    mfma_min_rows = 8
    scan_chunk = 128          # portions of at least twice this many tokens run their recurrence in chunks

    def before_recording(self, meta):
        """Host-built tables a step needs (pinned allocations and copies cannot be recorded into a graph)."""
        meta.attn_split(self.mfma_min_rows)

    def sum_group_norm(self, x, y, w, groups, alpha, eps, act, x_out=None, want_act=True):
        _f32(x, w, x_out)
        _act(y)
        rows, D = x.shape
        if y is not None and (y.shape != x.shape or not y.is_contiguous() or y.dtype != act):
            raise ValueError("y must match x's shape and the activation type")
        if w.numel() != D or D % groups:
            raise ValueError("norm weight / group count do not fit the width")
        xa = torch.empty(rows, D, dtype=act, device=x.device) if want_act else None
        xo = x if x_out is None else x_out
        _ok(lib().ragged_sum_group_norm(x.data_ptr(), None if y is None else y.data_ptr(), w.data_ptr(), xo.data_ptr(),
                                        None if xa is None else xa.data_ptr(), rows, D, groups, alpha, eps, _DT[act],
                                        _stream()), "sum_group_norm")
        return xa

    def conv_head(self, P, col0, meta, *, cw, taps, C, ch0, state, ngroups, gsize, normw, eps, rot, inv_freq,
                  out_dense=None, pages=None, norm_n=None, rot0=0, interleaved=False, rot_amp=1.0):
        _act(P, state, pages)
        _f32(cw, normw, inv_freq, out_dense)
        if P.dim() != 2 or P.shape[0] != meta.T or col0 < 0 or col0 + ngroups * gsize > P.shape[1]:
            raise ValueError("segment outside the projection matrix")
        a = _ConvHeadArgs()
        a.P, a.ldp, a.col0 = P.data_ptr(), P.stride(0), col0
        if cw is not None:
            if cw.shape != (C, taps) or ch0 + ngroups * gsize > C:
                raise ValueError("convolution taps do not cover the segment")
            if taps > 1 and (state.dtype != P.dtype or state.shape[1:] != (taps - 1, C) or not state.is_contiguous()
                             or max(s[0] for s in meta.seqs) >= state.shape[0]):
                raise ValueError("convolution state does not fit")
            a.cw, a.taps, a.C, a.ch0 = cw.data_ptr(), taps, C, ch0
            a.state = None if state is None else state.data_ptr()
        a.ngroups, a.gsize, a.eps = ngroups, gsize, eps
        if normw is not None:
            if normw.numel() != (gsize if norm_n is None else norm_n) or not 0 < normw.numel() <= gsize:
                raise ValueError("norm weight must have the size of the group's normed part")
            a.normw, a.norm_n = normw.data_ptr(), normw.numel()
        if rot:
            if inv_freq.numel() != rot // 2 or rot % 2 or rot0 < 0 or rot0 + rot > gsize:
                raise ValueError("one frequency per rotated pair, pairs inside the group")
            a.rot, a.cossin, a.rot0, a.interleaved = rot, meta.cossin(inv_freq, rot_amp).data_ptr(), rot0, int(bool(interleaved))
        if out_dense is not None:
            if out_dense.shape != (meta.T, ngroups * gsize):
                raise ValueError("dense output shape")
            a.out_dense = out_dense.data_ptr()
        else:
            _page_check(meta, pages)
            heads, rowlen = pages.shape[1], pages.shape[3]
            if pages.dtype != P.dtype or heads * rowlen != ngroups * gsize:
                raise ValueError("cache pages do not fit the segment")
            a.pages, a.rowlen, a.heads = pages.data_ptr(), rowlen, heads
        _ok(lib().ragged_conv_head(a, meta.c(), _DT[P.dtype], _stream()), "conv_head")

    def conv_state(self, P, col0, state, taps, C, meta):
        _act(P, state)
        if P.shape[0] != meta.T or col0 + C > P.shape[1] or state.shape[1:] != (taps - 1, C) or state.dtype != P.dtype \
                or not state.is_contiguous() or max(s[0] for s in meta.seqs) >= state.shape[0]:
            raise ValueError("convolution state does not fit")
        _ok(lib().ragged_conv_state(P.data_ptr(), P.stride(0), col0, state.data_ptr(), taps, C, meta.c(), _DT[P.dtype],
                                    _stream()), "conv_state")

    def clamped_glu(self, GU, limit, slope):
        _act(GU)
        if not GU.is_contiguous() or GU.shape[1] % 2:
            raise ValueError("[gate | up] rows expected")
        rows, F2 = GU.shape
        out = torch.empty(rows, F2 // 2, dtype=GU.dtype, device=GU.device)
        _ok(lib().ragged_clamped_glu(GU.data_ptr(), out.data_ptr(), rows, F2 // 2, limit, slope, _DT[GU.dtype], _stream()),
            "clamped_glu")
        return out

    def hgrn2_gates(self, P, q0, f0, fb, lower, HD):
        _act(P)
        _f32(fb, lower)
        if max(q0, f0) + HD > P.shape[1] or fb.numel() != HD or lower.numel() != HD:
            raise ValueError("gate segments outside the projection matrix")
        rows = P.shape[0]
        qf = torch.empty(rows, HD, dtype=torch.float32, device=P.device)
        ff = torch.empty_like(qf)
        _ok(lib().ragged_hgrn2_gates(P.data_ptr(), P.stride(0), q0, f0, fb.data_ptr(), lower.data_ptr(), qf.data_ptr(),
                                     ff.data_ptr(), rows, HD, _DT[P.dtype], _stream()), "hgrn2_gates")
        return qf, ff

    def hgrn2_scan(self, qf, ff, P, v0, state, H, d, vd, meta, gf=None, ones_col=False):
        """S <- diag(f) S + g v^T, o = S^T q per head; g = 1 - f unless ``gf`` gives it.  ``ones_col``: the last of the
        ``vd`` columns is not in P, its value is the constant 1 (state column n <- f n + g, output column n . q)."""
        _f32(qf, ff, state, gf)
        _act(P)
        oc = int(bool(ones_col))
        if qf.shape != (meta.T, H * d) or ff.shape != qf.shape or v0 + H * (vd - oc) > P.shape[1] or P.shape[0] != meta.T \
                or state.shape[1:] != (H, d, vd) or max(s[0] for s in meta.seqs) >= state.shape[0] \
                or (gf is not None and gf.shape != qf.shape):
            raise ValueError("recurrent state / gates do not fit")
        out = torch.empty(meta.T, H * vd, dtype=torch.float32, device=P.device)
        L, dt, st = lib(), _DT[P.dtype], _stream()
        g = None if gf is None else gf.data_ptr()
        longest = max(n for _, _, n, _ in meta.seqs)
        if longest < 2 * self.scan_chunk:
            _ok(L.ragged_hgrn2_scan(qf.data_ptr(), ff.data_ptr(), g, P.data_ptr(), P.stride(0), v0, state.data_ptr(),
                                    out.data_ptr(), H, d, vd, oc, meta.c(), dt, st), "hgrn2_scan")
            return out
        # long portions: chunks scanned side by side from zero, chunk-start states chained, chunks scanned again from them
        nc, cstart, zeros, ones, cid, cfirst, last = meta.chunks(self._chunk_length(meta, H, d, vd))
        local = torch.empty(nc, H, d, vd, dtype=torch.float32, device=P.device)
        begin = torch.empty_like(local)
        decay = torch.empty(nc, H * d, dtype=torch.float32, device=P.device)

        def chunk_batch(past):
            return _Batch(None, None, cstart.data_ptr(), past.data_ptr(), cid.data_ptr(), None, meta.T, nc, 0)
        _ok(L.ragged_hgrn2_scan(qf.data_ptr(), ff.data_ptr(), g, P.data_ptr(), P.stride(0), v0, local.data_ptr(), out.data_ptr(),
                                H, d, vd, oc, chunk_batch(zeros), dt, st), "hgrn2_scan (chunks from zero)")
        _ok(L.ragged_hgrn2_chunk_decay(ff.data_ptr(), cstart.data_ptr(), decay.data_ptr(), nc, H * d, st), "hgrn2_chunk_decay")
        _ok(L.ragged_hgrn2_chunk_combine(state.data_ptr(), local.data_ptr(), decay.data_ptr(), begin.data_ptr(), cfirst.data_ptr(),
                                         meta.seq_past.data_ptr(), meta.seq_slot.data_ptr(), meta.B, H, d, vd, st),
            "hgrn2_chunk_combine")
        _ok(L.ragged_hgrn2_scan(qf.data_ptr(), ff.data_ptr(), g, P.data_ptr(), P.stride(0), v0, begin.data_ptr(), out.data_ptr(),
                                H, d, vd, oc, chunk_batch(ones), dt, st), "hgrn2_scan (chunks from their start states)")
        slots = torch.tensor([s[0] for s in meta.seqs], dtype=torch.int64, device=P.device)
        state[slots] = begin[torch.tensor(last, dtype=torch.int64, device=P.device)]     # every sequence's end state
        return out

    scan_resident = 512       # workgroups of the scan that run at one time (two per CU)

    def _chunk_length(self, meta, H, d, vd):
        """Tokens per chunk of a long scan: a pass takes (rounds of resident workgroups) x (tokens of a chunk), so the
        length is chosen for the fewest token steps in a row; among equals the longest (fewer chunk states to chain)."""
        R = 1
        while R * 32 < d:
            R *= 2
        blocks = -(-vd // (4 * (64 // R)))                   # column blocks of a head
        best = None
        for length in (256, 224, 192, 160, 128, 96, 64):
            chunks = sum(-(-n // length) for _, _, n, _ in meta.seqs)
            cost = -(-(chunks * H * blocks) // self.scan_resident) * min(length, max(n for _, _, n, _ in meta.seqs))
            if best is None or cost < best[0]:
                best = (cost, length)
        return best[1]

    def row_norm(self, x, w, eps, act):
        _f32(x, w)
        n = x.shape[-1]
        if w is not None and w.numel() != n:
            raise ValueError("norm weight size")
        out = torch.empty(x.shape, dtype=act, device=x.device)
        _ok(lib().ragged_row_norm(x.data_ptr(), None if w is None else w.data_ptr(), out.data_ptr(), x.numel() // n, n, eps,
                                  _DT[act], _stream()), "row_norm")
        return out

    def paged_attn(self, q, kpages, vpages, meta, *, maps, H, G, d, vd, window, keep_first, scale, lam, out_scale, out_norm,
                   eps, gate=None, gate0=0, sink=None, chunk=0, softcap=0.0, gate_wide=False, sinks=None, slopes=None):
        """``vpages`` may be ``kpages`` itself: the values are then the leading ``vd`` channels of the key rows.
        ``chunk`` > 0: a key is visible only inside the query's block of that many positions; ``softcap`` > 0: scores go
        through softcap * tanh(. / softcap); ``gate_wide``: one gate column per output channel instead of one per head;
        ``sinks`` float [H]: every head's own sink score (instead of the one number ``sink``); ``slopes`` float [H]:
        slopes[h] * (i - j) is taken off the scaled score of query i and key j."""
        _f32(q, sinks, slopes)
        if any(t is not None and t.numel() != H for t in (sinks, slopes)):
            raise ValueError("one sink score / one slope per query head")
        _act(kpages, vpages, gate)
        _page_check(meta, kpages)
        _page_check(meta, vpages)
        shared = vpages.data_ptr() == kpages.data_ptr()
        if q.shape != (meta.T, H * maps * d) or kpages.shape[1:] != (G, PAGE, maps * d) or kpages.dtype != vpages.dtype \
                or kpages.shape[0] != vpages.shape[0] or not q.is_contiguous() \
                or (vpages.shape[1:] != (G, PAGE, vd) and not (shared and vd <= maps * d)):
            raise ValueError("queries / cache pages do not fit the head layout")
        out = torch.empty(meta.T, H * vd, dtype=kpages.dtype, device=q.device)
        a = _AttnArgs()
        a.q, a.kpages, a.vpages, a.out = q.data_ptr(), kpages.data_ptr(), vpages.data_ptr(), out.data_ptr()
        if gate is not None:
            if gate.shape[0] != meta.T or gate0 + (H * vd if gate_wide else H) > gate.shape[1] or gate.dtype != kpages.dtype:
                raise ValueError("gate columns outside the projection matrix")
            a.gate, a.ldg, a.gate0, a.gate_wide = gate.data_ptr(), gate.stride(0), gate0, int(bool(gate_wide))
        if chunk < 0 or softcap < 0:
            raise ValueError("block size and score cap cannot be negative")
        a.chunk, a.softcap = int(chunk), float(softcap)
        a.H, a.G, a.d, a.vd, a.window, a.keep_first = H, G, d, vd, window, keep_first
        a.scale, a.lam, a.out_scale, a.out_norm, a.eps = scale, lam, out_scale, int(out_norm), eps
        a.ldv = vpages.shape[3]
        if sink is not None:
            a.sink, a.sink_score = 1, float(sink)
        if sinks is not None:
            a.sink, a.sinks = 1, sinks.data_ptr()
        if slopes is not None:
            a.slopes = slopes.data_ptr()
        if kpages.dtype == torch.bfloat16 and self.mfma and maps == 1 and not lib().ragged_paged_attn_mfma_ok(d, vd) \
                and lib().ragged_paged_attn_mfma_wide_ok(d, vd) and a.ldv % 8 == 0 and not keep_first and not out_norm \
                and gate is None and not chunk and not softcap and sinks is None and slopes is None:
            # rows too wide for the row-wise kernel's lanes: long portions as tiles of 64 rows of one head, single tokens
            # and short portions with 16 heads of a row side by side, both on the matrix cores
            tiles, n_tiles, rows, n_rows = meta.attn_split(self.mfma_min_rows)
            if n_tiles:
                a.tiles, a.n_tiles = tiles.data_ptr(), n_tiles
                _ok(lib().ragged_paged_attn_mfma_wide(a, meta.c(), _stream()), "paged_attn_mfma_wide")
            if n_rows:
                a.rows, a.n_rows = rows.data_ptr(), n_rows
                _ok(lib().ragged_paged_attn_mfma_heads(a, meta.c(), _stream()), "paged_attn_mfma_heads")
            return out
        if kpages.dtype == torch.bfloat16 and self.mfma and lib().ragged_paged_attn_mfma_ok(d, vd) and a.ldv % 8 == 0 \
                and not (gate_wide and (a.ldg % 4 or gate0 % 4)):
            # long portions on the matrix cores, single tokens and short portions row by row
            tiles, n_tiles, rows, n_rows = meta.attn_split(self.mfma_min_rows)
            if n_tiles:
                a.tiles, a.n_tiles = tiles.data_ptr(), n_tiles
                _ok(lib().ragged_paged_attn_mfma(a, meta.c(), maps, _stream()), "paged_attn_mfma")
            if n_rows:
                a.rows, a.n_rows = rows.data_ptr(), n_rows
                _ok(lib().ragged_paged_attn(a, meta.c(), maps, _DT[kpages.dtype], _stream()), "paged_attn")
            return out
        _ok(lib().ragged_paged_attn(a, meta.c(), maps, _DT[kpages.dtype], _stream()), "paged_attn")
        return out

    def post_norm_add(self, x, y, w_post, w_next, eps, act):
        """x <- x + w_post * rmsnorm(y) in place; returns w_next * rmsnorm(x) as ``act`` (None without ``w_next``)."""
        _f32(x, w_post, w_next)
        _act(y)
        rows, D = x.shape
        if y.shape != x.shape or not y.is_contiguous() or y.dtype != act or w_post.numel() != D \
                or (w_next is not None and w_next.numel() != D):
            raise ValueError("sublayer output / norm weights do not fit the stream")
        xa = None if w_next is None else torch.empty(rows, D, dtype=act, device=x.device)
        _ok(lib().ragged_post_norm_add(x.data_ptr(), y.data_ptr(), w_post.data_ptr(), None if w_next is None else w_next.data_ptr(),
                                       None if xa is None else xa.data_ptr(), rows, D, eps, _DT[act], _stream()), "post_norm_add")
        return xa

    def relu2(self, A):
        _act(A)
        if not A.is_contiguous():
            raise ValueError("contiguous activations expected")
        out = torch.empty_like(A)
        if A.numel():
            _ok(lib().ragged_relu2(A.data_ptr(), out.data_ptr(), A.numel(), _DT[A.dtype], _stream()), "relu2")
        return out

    def head_norm_gate(self, o, w, P, g0, H, vd, eps, act, em=None, den_floor=0.0, scale=1.0):
        """each head's rows of ``o`` divided by their root mean square, times ``w``, times sigmoid(gate columns of P), times
        ``scale``.  With ``em`` [T, H]: ``o`` has vd + 1 columns per head and is first divided by max(|last column|, em) +
        den_floor."""
        _f32(o, w, em)
        _act(P)
        T = o.shape[0]
        ldo = vd + (0 if em is None else 1)
        if o.shape != (T, H * ldo) or w.numel() != H * vd or P.shape[0] != T or g0 + H * vd > P.shape[1] or P.dtype != act \
                or (em is not None and em.shape != (T, H)):
            raise ValueError("head outputs / gate columns do not fit")
        out = torch.empty(T, H * vd, dtype=act, device=o.device)
        _ok(lib().ragged_head_norm_gate(o.data_ptr(), w.data_ptr(), P.data_ptr(), P.stride(0), g0, out.data_ptr(), T, H, vd, eps,
                                        ldo, None if em is None else em.data_ptr(), den_floor, float(scale), _DT[act],
                                        _stream()), "head_norm_gate")
        return out

    def mlstm_gates(self, P, i0, gate_bias, cap, m_start, H, mstate, meta):
        """Soft-capped log gates of this step's rows (columns i0 .. of P: input gates, then forget gates) and the running
        maximum m carried in ``mstate`` [slots, H]; returns the decay a, the input weight b and e^-m, float [T, H] each."""
        _act(P)
        _f32(gate_bias, mstate)
        if P.shape[0] != meta.T or i0 + 2 * H > P.shape[1] or gate_bias.numel() != 2 * H or mstate.shape[1] != H \
                or max(s[0] for s in meta.seqs) >= mstate.shape[0]:
            raise ValueError("gate columns / state slots do not fit")
        a = torch.empty(meta.T, H, dtype=torch.float32, device=P.device)
        b, em = torch.empty_like(a), torch.empty_like(a)
        _ok(lib().ragged_mlstm_gates(P.data_ptr(), P.stride(0), i0, gate_bias.data_ptr(), cap, m_start, mstate.data_ptr(),
                                     a.data_ptr(), b.data_ptr(), em.data_ptr(), H, meta.c(), _DT[P.dtype], _stream()), "mlstm_gates")
        return a, b, em

    def mlstm_expand(self, P, q0, k0, a, b, H, d):
        """The matrix scan's arrays: q dim^-1/2, the decay repeated over the rows, b k; float [T, H d] each."""
        _act(P)
        _f32(a, b)
        T = P.shape[0]
        if max(q0, k0) + H * d > P.shape[1] or a.shape != (T, H) or b.shape != (T, H):
            raise ValueError("query / key columns do not fit")
        qf = torch.empty(T, H * d, dtype=torch.float32, device=P.device)
        ff, gf = torch.empty_like(qf), torch.empty_like(qf)
        _ok(lib().ragged_mlstm_expand(P.data_ptr(), P.stride(0), q0, k0, a.data_ptr(), b.data_ptr(), qf.data_ptr(), ff.data_ptr(),
                                      gf.data_ptr(), T, H, d, _DT[P.dtype], _stream()), "mlstm_expand")
        return qf, ff, gf

    def moe_route(self, xa, w_router, groups, keep, top, scale, score="softmax", group_top=1, renorm=False):
        """``score``: "softmax" over all experts or "sigmoid" per expert; a group is worth the sum of its ``group_top``
        best scores; ``renorm``: the chosen scores are divided by their sum (+ 1e-20) before ``scale``."""
        _act(xa)
        _f32(w_router)
        T, D = xa.shape
        E = w_router.shape[0]
        if w_router.shape[1] != D:
            raise ValueError("router rows do not fit the stream")
        idx = torch.empty(T, top, dtype=torch.int32, device=xa.device)
        wts = torch.empty(T, top, dtype=torch.float32, device=xa.device)
        _ok(lib().ragged_moe_route(xa.data_ptr(), xa.stride(0), w_router.data_ptr(), idx.data_ptr(), wts.data_ptr(), T, D, E, groups,
                                   keep, top, scale, {"softmax": 0, "sigmoid": 1}[score], int(group_top), int(bool(renorm)),
                                   _DT[xa.dtype], _stream()), "moe_route")
        return idx, wts

    def moe_sorted(self, xa, idx, wts, w_up, w_dn, base, gated=False):
        """The experts of long bfloat16 portions without a word to the host: (row, choice) pairs sorted by expert, every
        expert's run cut into 64-row tiles on the device, one grouped matrix-core product for all up projections (relu^2,
        or with ``gated`` silu(gate) * up over neighbouring weight rows, on the way out) and one for all down projections,
        then every row's weighted sum.  None when the sizes are not served (the caller then runs the experts one by one)."""
        T, D = xa.shape
        E, wrows, top = w_up.shape[0], w_up.shape[1], idx.shape[1]
        ff = wrows // 2 if gated else wrows
        L = lib()
        if xa.dtype != torch.bfloat16 or not (L.ragged_moe_grouped_ok(wrows, D, E) and L.ragged_moe_grouped_ok(D, ff, E)) \
                or xa.stride(0) % 8 or w_up.shape != (E, wrows, D) or w_dn.shape != (E, D, ff) or not w_up.is_contiguous() \
                or not w_dn.is_contiguous() or w_up.dtype != xa.dtype or w_dn.dtype != xa.dtype:
            return None
        _act(xa, w_up, w_dn, base)
        M = T * top
        order = idx.view(-1).sort(stable=True)
        pair = order.indices                                    # pair t * top + j at every sorted place
        seg = torch.zeros(E + 1, dtype=torch.int32, device=xa.device)
        seg[1:] = torch.bincount(order.values, minlength=E).cumsum(0)
        src = (pair // top).to(torch.int32)
        place = torch.empty(M, dtype=torch.int32, device=xa.device)
        place[pair] = torch.arange(M, dtype=torch.int32, device=xa.device)
        max_tiles = M // 64 + E
        tiles = torch.empty(2 * max_tiles + 1, dtype=torch.int32, device=xa.device)
        te, tr, nt = tiles[:max_tiles], tiles[max_tiles:2 * max_tiles], tiles[2 * max_tiles:]
        st = _stream()
        _ok(L.ragged_moe_tile_map(seg.data_ptr(), E, te.data_ptr(), tr.data_ptr(), nt.data_ptr(), max_tiles, st), "moe_tile_map")
        A = torch.empty(M, ff, dtype=xa.dtype, device=xa.device)
        ys = torch.empty(M, D, dtype=xa.dtype, device=xa.device)
        _ok(L.ragged_moe_grouped_gemm(xa.data_ptr(), xa.stride(0), src.data_ptr(), w_up.data_ptr(), A.data_ptr(), seg.data_ptr(),
                                      te.data_ptr(), tr.data_ptr(), nt.data_ptr(), max_tiles, wrows, D, E, 2 if gated else 1, st),
            "moe_grouped_gemm (up)")
        _ok(L.ragged_moe_grouped_gemm(A.data_ptr(), ff, None, w_dn.data_ptr(), ys.data_ptr(), seg.data_ptr(), te.data_ptr(),
                                      tr.data_ptr(), nt.data_ptr(), max_tiles, D, ff, E, 0, st), "moe_grouped_gemm (down)")
        return self.moe_combine(ys, place.view(T, top), wts, base)

    def moe_combine(self, ys, place, wts, base):
        """y[t] = base[t] + sum_j wts[t, j] * ys[place[t, j]]"""
        _act(ys, base)
        _f32(wts)
        T, top = place.shape
        D = ys.shape[1]
        if ys.shape[0] != T * top or not ys.is_contiguous() or place.dtype != torch.int32 or not place.is_contiguous() \
                or wts.shape != (T, top) or (base is not None and (base.shape != (T, D) or base.dtype != ys.dtype
                                                                   or not base.is_contiguous())):
            raise ValueError("expert outputs / places do not fit")
        y = torch.empty(T, D, dtype=ys.dtype, device=ys.device)
        _ok(lib().ragged_moe_combine(ys.data_ptr(), place.data_ptr(), wts.data_ptr(), None if base is None else base.data_ptr(),
                                     y.data_ptr(), T, D, top, _DT[ys.dtype], _stream()), "moe_combine")
        return y

    def moe_rows(self, xa, idx, wts, w_up, w_dn, base, gated=False):
        """y = base + sum over a row's chosen experts of weight * W_down relu(W_up x)^2, every pair served on its own.
        ``gated``: w_up holds (gate, up) rows next to each other and the inner activation is silu(gate) * up."""
        _act(xa, w_up, w_dn, base)
        _f32(wts)
        T, D = xa.shape
        E, top = w_up.shape[0], idx.shape[1]
        ff = w_up.shape[1] // 2 if gated else w_up.shape[1]
        if w_up.shape != (E, 2 * ff if gated else ff, D) or w_dn.shape != (E, D, ff) or not w_up.is_contiguous() or not w_dn.is_contiguous() \
                or w_up.dtype != xa.dtype or w_dn.dtype != xa.dtype or idx.shape != (T, top) or wts.shape != (T, top) \
                or idx.dtype != torch.int32 or not idx.is_contiguous() \
                or (base is not None and (base.shape != (T, D) or base.dtype != xa.dtype or not base.is_contiguous())):
            raise ValueError("expert weights / choices do not fit")
        A = torch.empty(T * top, ff, dtype=xa.dtype, device=xa.device)
        y = torch.empty(T, D, dtype=xa.dtype, device=xa.device)
        _ok(lib().ragged_moe_rows(xa.data_ptr(), xa.stride(0), idx.data_ptr(), wts.data_ptr(), w_up.data_ptr(), w_dn.data_ptr(),
                                  None if base is None else base.data_ptr(), A.data_ptr(), y.data_ptr(), T, D, ff, top,
                                  int(bool(gated)), _DT[xa.dtype], _stream()), "moe_rows")
        return y

    def embed_rows(self, ids, table, ids2=None, table2=None, scale=1.0):
        """float32 [T, width]: scale * table[ids] (+ table2[ids2]), summed in float."""
        _act(table, table2)
        T, D = ids.numel(), table.shape[1]
        for i, t in ((ids, table), (ids2, table2)):
            if t is not None and (i is None or i.dtype != torch.int64 or not i.is_contiguous() or i.numel() != T
                                  or not t.is_contiguous() or t.shape[1] != D or t.dtype != table.dtype or i.device != t.device):
                raise ValueError("row ids / embedding tables do not fit")
        x = torch.empty(T, D, dtype=torch.float32, device=table.device)
        _ok(lib().ragged_embed_rows(ids.data_ptr(), table.data_ptr(), None if table2 is None else ids2.data_ptr(),
                                    None if table2 is None else table2.data_ptr(), scale, x.data_ptr(), T, D, _DT[table.dtype],
                                    _stream()), "embed_rows")
        return x

    def add_norm(self, x, y1, y2, w_next, eps, act):
        """x <- x + y1 (+ y2) in place on the float32 stream; returns w_next * rmsnorm(x) as ``act`` (None without
        ``w_next``).  Without y1 it is a plain norm of the stream."""
        _f32(x, w_next)
        _act(y1, y2)
        rows, D = x.shape
        for y in (y1, y2):
            if y is not None and (y.shape != x.shape or not y.is_contiguous() or y.dtype != act):
                raise ValueError("sublayer outputs must match the stream's shape and the activation type")
        if (y2 is not None and y1 is None) or (w_next is not None and w_next.numel() != D) or not x.is_contiguous():
            raise ValueError("norm weight / operands do not fit the stream")
        xa = None if w_next is None else torch.empty(rows, D, dtype=act, device=x.device)
        _ok(lib().ragged_add_norm(x.data_ptr(), None if y1 is None else y1.data_ptr(), None if y2 is None else y2.data_ptr(),
                                  None if w_next is None else w_next.data_ptr(), None if xa is None else xa.data_ptr(), rows, D, eps,
                                  _DT[act], _stream()), "add_norm")
        return xa

    _ACT_KINDS = {"gelu_erf": 0, "gelu_tanh": 1, "relu2": 2, "xielu": 3, "tanh": 4}

    def act_cols(self, P, col0, n, kind, params=(0.0, 0.0)):
        """act(P[:, col0 : col0 + n]) as a contiguous [rows, n] matrix; kind: gelu_erf, gelu_tanh, relu2, tanh, or xielu with
        ``params`` = (a, b) >= 0: a z^2 + z / 2 right of zero, (1/2 + b)(e^z - 1 - z) + z / 2 left of it."""
        _act(P)
        if P.dim() != 2 or col0 < 0 or col0 + n > P.shape[1]:
            raise ValueError("columns outside the matrix")
        out = torch.empty(P.shape[0], n, dtype=P.dtype, device=P.device)
        _ok(lib().ragged_act_cols(P.data_ptr(), P.stride(0), col0, out.data_ptr(), P.shape[0], n, self._ACT_KINDS[kind], float(params[0]),
                                  float(params[1]), _DT[P.dtype], _stream()), "act_cols")
        return out

    def glu_pairs(self, P):
        """silu(P[:, 0::2]) * P[:, 1::2]: inner channels that come as neighbouring (gate, up) pairs."""
        _act(P)
        if P.dim() != 2 or P.shape[1] % 2:
            raise ValueError("(gate, up) pairs expected")
        out = torch.empty(P.shape[0], P.shape[1] // 2, dtype=P.dtype, device=P.device)
        if out.numel():
            _ok(lib().ragged_glu_pairs(P.data_ptr(), P.stride(0), out.data_ptr(), P.shape[0], P.shape[1] // 2, _DT[P.dtype], _stream()),
                "glu_pairs")
        return out


    def hc_step(self, X, y, prev, nxt, w_next, eps, act, want_u=False):
        """The stream in S copies, X float [rows, S, D], between two sublayers.  ``prev`` / ``nxt``: float [2 S + S S] =
        [read-out weights | write-back weights | mixing matrix (from, to)] of the sublayer that produced ``y`` and of the
        one that reads next.  With ``y``: X[t] <- sum_s mix[s, t] X[s] + out[t] y in place.  With ``nxt``: u = sum_s in[s] X[s];
        returns (w_next * rmsnorm(u) as ``act`` or None, u as float if ``want_u`` else None)."""
        _f32(X, prev, nxt, w_next)
        _act(y)
        rows, S, D = X.shape
        if S > 8 or (y is not None and (prev is None or y.shape != (rows, D) or not y.is_contiguous() or y.dtype != act)) \
                or any(c is not None and c.numel() != 2 * S + S * S for c in (prev, nxt)) \
                or (w_next is not None and (nxt is None or w_next.numel() != D)) or (want_u and nxt is None):
            raise ValueError("stream copies / coefficients / sublayer output do not fit")
        xa = None if w_next is None else torch.empty(rows, D, dtype=act, device=X.device)
        u = torch.empty(rows, D, dtype=torch.float32, device=X.device) if want_u else None
        _ok(lib().ragged_hc_step(X.data_ptr(), None if y is None else y.data_ptr(), None if prev is None else prev.data_ptr(),
                                 None if nxt is None else nxt.data_ptr(), None if w_next is None else w_next.data_ptr(),
                                 None if xa is None else xa.data_ptr(), None if u is None else u.data_ptr(), rows, S, D, eps,
                                 _DT[act], _stream()), "hc_step")
        return xa, u

    def gate_cols(self, o, P, g0, act, scale=1.0):
        """scale * o * sigmoid(P[:, g0 : g0 + n]) for float head outputs o [rows, n], rounded once to ``act``"""
        _f32(o)
        _act(P)
        rows, n = o.shape
        if P.shape[0] != rows or g0 < 0 or g0 + n > P.shape[1] or P.dtype != act:
            raise ValueError("gate columns outside the projection matrix")
        out = torch.empty(rows, n, dtype=act, device=o.device)
        _ok(lib().ragged_gate_cols(o.data_ptr(), P.data_ptr(), P.stride(0), g0, out.data_ptr(), rows, n, float(scale), _DT[act],
                                   _stream()), "gate_cols")
        return out

    def delta_gates(self, P, r0, k0, a0, wl, w0, ab, rate, tiny, H, d):
        """The delta-rule scan's arrays, float [T, H d] each: r, decay exp(-rate sigmoid(wl + w0)), unit key n = k / sqrt(|k|^2
        + tiny) per head, removal sigmoid(a + ab) * n, and k.  r, k and the removal logits are columns of P; ``wl`` [T, H d]
        float are the decay logits."""
        _act(P)
        _f32(wl, w0, ab)
        T, HD = P.shape[0], H * d
        if max(r0, k0, a0) + HD > P.shape[1] or wl.shape != (T, HD) or w0.numel() != HD or ab.numel() != HD:
            raise ValueError("delta-rule columns / biases do not fit")
        outs = [torch.empty(T, HD, dtype=torch.float32, device=P.device) for _ in range(5)]
        _ok(lib().ragged_delta_gates(P.data_ptr(), P.stride(0), r0, k0, a0, wl.data_ptr(), w0.data_ptr(), ab.data_ptr(), float(rate),
                                     float(tiny), *[t.data_ptr() for t in outs], T, H, d, _DT[P.dtype], _stream()), "delta_gates")
        return outs

    delta_chunked_from = 192  # portions of at least this many tokens run the delta rule in chunks
    delta_chain = True        # False: the walk over a sequence's chunks as library products (what very tall states get)

    def _delta_chunk_length(self, meta, H, d, vd):
        """Tokens per chunk of a long delta-rule scan: three passes of (rounds of resident workgroups) x (chunk tokens) token
        steps in a row, plus the walk over a sequence's chunks (about two token steps per chunk)."""
        R = 1
        while R * 32 < d:
            R *= 2
        best = None
        for length in (128, 96, 64, 48, 32):
            chunks = [-(-n // length) for _, _, n, _ in meta.seqs]
            cols = 64 // R                                   # columns of a wavefront; a workgroup is two or four of them
            blocks = -(-max(vd, d) // ((2 if max(vd, d) <= 2 * cols else 4) * cols))
            cost = 3 * -(-(sum(chunks) * H * blocks) // self.scan_resident) * length + 2 * max(chunks)
            if best is None or cost < best[0]:
                best = (cost, length)
        return best[1]

    def delta_scan(self, arrays, P, v0, state, H, d, vd, meta):
        """S <- diag(w) S - b (n^T S) + k v^T, o = S^T r per head over this step's rows; ``arrays`` = (r, w, n, b, k) from
        ``delta_gates``, v = columns v0 .. of P, ``state`` float [slots, H, d, vd].  Returns o float [T, H vd]."""
        _f32(state, *arrays)
        _act(P)
        if any(a.shape != (meta.T, H * d) for a in arrays) or v0 + H * vd > P.shape[1] or P.shape[0] != meta.T \
                or state.shape[1:] != (H, d, vd) or max(s[0] for s in meta.seqs) >= state.shape[0]:
            raise ValueError("recurrent state / scan arrays do not fit")
        out = torch.empty(meta.T, H * vd, dtype=torch.float32, device=P.device)
        L, dt, st = lib(), _DT[P.dtype], _stream()
        ptrs = [a.data_ptr() for a in arrays]
        longest = max(n for _, _, n, _ in meta.seqs)
        if longest < self.delta_chunked_from:
            _ok(L.ragged_delta_scan(*ptrs, P.data_ptr(), P.stride(0), v0, state.data_ptr(), out.data_ptr(), H, d, vd, 1, meta.c(),
                                    dt, st), "delta_scan")
            return out
        # Long portions: chunks side by side.  A chunk maps its start state linearly, S_end = A S_start + L: L is the chunk
        # scanned from zero, A (d x d per head) the chunk scanned without inputs from the identity.  The chunk-start states
        # follow one after the other from those, and the chunks are scanned again from them for the outputs.
        nc, cstart, zeros, ones, cid, cfirst, last = meta.chunks(self._delta_chunk_length(meta, H, d, vd))
        local = torch.empty(nc, H, d, vd, dtype=torch.float32, device=P.device)
        trans = torch.eye(d, dtype=torch.float32, device=P.device).repeat(nc, H, 1, 1)
        begin = torch.empty_like(local)

        def chunk_batch(past):
            return _Batch(None, None, cstart.data_ptr(), past.data_ptr(), cid.data_ptr(), None, meta.T, nc, 0)
        _ok(L.ragged_delta_scan(*ptrs, P.data_ptr(), P.stride(0), v0, local.data_ptr(), None, H, d, vd, 1, chunk_batch(zeros), dt, st),
            "delta_scan (chunks from zero)")
        _ok(L.ragged_delta_scan(*ptrs, None, 0, 0, trans.data_ptr(), None, H, d, d, 0, chunk_batch(ones), dt, st),
            "delta_scan (transition matrices)")
        if self.delta_chain and L.ragged_delta_chain_ok(d):
            _ok(L.ragged_delta_chain(state.data_ptr(), local.data_ptr(), trans.data_ptr(), begin.data_ptr(), cfirst.data_ptr(),
                                     meta.seq_past.data_ptr(), meta.seq_slot.data_ptr(), meta.B, H, d, vd, st), "delta_chain")
        else:                                                # very tall states: the same walk as library products
            first = [0]
            for _, _, n, _ in meta.seqs:
                first.append(last[len(first) - 1] + 1)
            slots = torch.tensor([s[0] for s in meta.seqs], dtype=torch.int64, device=P.device)
            fresh = torch.tensor([s[1] == 0 for s in meta.seqs], device=P.device)
            S = torch.where(fresh[:, None, None, None], torch.zeros((), device=P.device), state[slots])      # [B, H, d, vd]
            for j in range(max(first[b + 1] - first[b] for b in range(meta.B))):     # the j-th chunk of every sequence that has one
                bs = [b for b in range(meta.B) if first[b + 1] - first[b] > j]
                cs = torch.tensor([first[b] + j for b in bs], dtype=torch.int64, device=P.device)
                bi = torch.tensor(bs, dtype=torch.int64, device=P.device)
                begin[cs] = S[bi]
                S[bi] = torch.matmul(trans[cs], S[bi]) + local[cs]
            state[slots] = S
        _ok(L.ragged_delta_scan(*ptrs, P.data_ptr(), P.stride(0), v0, begin.data_ptr(), out.data_ptr(), H, d, vd, 1,
                                chunk_batch(ones), dt, st), "delta_scan (chunks from their start states)")
        return out


class TorchOps:
    """The same interface as unfused PyTorch statements (host-side tests of the engine's bookkeeping)."""
    name = "torch"

    def sum_group_norm(self, x, y, w, groups, alpha, eps, act, x_out=None, want_act=True):
        v = alpha * x if y is None else alpha * x + y.float()
        g = v.view(v.shape[0], groups, -1)
        g = g / torch.sqrt(g.pow(2).mean(-1, keepdim=True) + eps)
        v = g.reshape(v.shape) * w
        (x if x_out is None else x_out).copy_(v)
        return v.to(act) if want_act else None

    def _segment(self, P, col0, meta, cw, taps, C, ch0, state, width):
        """convolved (or plain) float rows of a segment"""
        u = P[:, col0:col0 + width].float()
        if cw is None:
            return u
        out = torch.empty_like(u)
        wseg = cw[ch0:ch0 + width]
        for b, (slot, past, n, _) in enumerate(meta.seqs):
            s0 = meta.start[b]
            hist = state[slot, :, ch0:ch0 + width].float() if taps > 1 else u[:0]
            if past < taps - 1:
                hist = hist.clone()
                hist[: taps - 1 - past] = 0
            full = torch.cat([hist, u[s0:s0 + n]], 0)
            acc = torch.zeros(n, width, dtype=torch.float32, device=P.device)
            for j in range(taps):
                acc += wseg[:, j] * full[j:j + n]
            out[s0:s0 + n] = acc
        return out

    def conv_head(self, P, col0, meta, *, cw, taps, C, ch0, state, ngroups, gsize, normw, eps, rot, inv_freq,
                  out_dense=None, pages=None, norm_n=None, rot0=0, interleaved=False, rot_amp=1.0):
        width = ngroups * gsize
        v = self._segment(P, col0, meta, cw, taps, C, ch0, state, width).view(meta.T, ngroups, gsize)
        if normw is not None:
            nn = gsize if norm_n is None else norm_n
            u = v[..., :nn]
            v = torch.cat([u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps) * normw, v[..., nn:]], -1)
        if rot:
            half = rot // 2
            ang = meta.tok_pos.to(P.device).float()[:, None] * inv_freq[None]
            c, s = ang.cos()[:, None, :] * rot_amp, ang.sin()[:, None, :] * rot_amp
            if interleaved:
                a, b2 = v[..., rot0:rot0 + rot:2], v[..., rot0 + 1:rot0 + rot:2]
                turned = torch.stack([a * c - b2 * s, b2 * c + a * s], -1).flatten(-2)
            else:
                a, b2 = v[..., rot0:rot0 + half], v[..., rot0 + half:rot0 + rot]
                turned = torch.cat([a * c - b2 * s, b2 * c + a * s], -1)
            v = torch.cat([v[..., :rot0], turned, v[..., rot0 + rot:]], -1)
        v = v.reshape(meta.T, width)
        if out_dense is not None:
            out_dense.copy_(v)
            return
        heads, rowlen = pages.shape[1], pages.shape[3]
        v = v.view(meta.T, heads, rowlen).to(pages.dtype)
        for b, (slot, past, n, pg) in enumerate(meta.seqs):
            for i in range(n):
                pos = past + i
                pages[pg[pos // PAGE], :, pos % PAGE] = v[meta.start[b] + i]

    def conv_state(self, P, col0, state, taps, C, meta):
        keep = taps - 1
        for b, (slot, past, n, _) in enumerate(meta.seqs):
            old = state[slot].clone()
            if past < keep:
                old[: keep - past] = 0
            full = torch.cat([old, P[meta.start[b]:meta.start[b] + n, col0:col0 + C]], 0)
            state[slot] = full[-keep:]

    def clamped_glu(self, GU, limit, slope):
        f = GU.shape[1] // 2
        g = GU[:, :f].float().clamp(max=limit)
        u = GU[:, f:].float().clamp(-limit, limit)
        return (g * torch.sigmoid(slope * g) * (u + 1)).to(GU.dtype)

    def hgrn2_gates(self, P, q0, f0, fb, lower, HD):
        q = P[:, q0:q0 + HD].float()
        f = lower + (1 - lower) * torch.sigmoid(P[:, f0:f0 + HD].float() + fb)
        return q * torch.sigmoid(q), f

    def hgrn2_scan(self, qf, ff, P, v0, state, H, d, vd, meta, gf=None, ones_col=False):
        out = torch.empty(meta.T, H * vd, dtype=torch.float32, device=P.device)
        pv = vd - int(bool(ones_col))
        for b, (slot, past, n, _) in enumerate(meta.seqs):
            S = state[slot].clone() if past > 0 else torch.zeros_like(state[slot])
            for i in range(n):
                t = meta.start[b] + i
                f = ff[t].view(H, d, 1)
                v = P[t, v0:v0 + H * pv].float().view(H, 1, pv)
                if ones_col:
                    v = torch.cat([v, torch.ones(H, 1, 1)], -1)
                S = f * S + (1 - f if gf is None else gf[t].view(H, d, 1)) * v
                out[t] = (S * qf[t].view(H, d, 1)).sum(1).reshape(-1)
            state[slot] = S
        return out

    def row_norm(self, x, w, eps, act):
        v = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        return (v if w is None else v * w).to(act)

    def paged_attn(self, q, kpages, vpages, meta, *, maps, H, G, d, vd, window, keep_first, scale, lam, out_scale, out_norm,
                   eps, gate=None, gate0=0, sink=None, chunk=0, softcap=0.0, gate_wide=False, sinks=None, slopes=None):
        out = torch.empty(meta.T, H * vd, dtype=torch.float32, device=q.device)
        q = q.view(meta.T, H, maps, d)
        for b, (slot, past, n, pg) in enumerate(meta.seqs):
            L = past + n
            idx = torch.tensor(pg, dtype=torch.long, device=q.device)
            k = kpages[idx].float().permute(1, 0, 2, 3).reshape(G, -1, maps, d)[:, :L]       # [G, L, maps, d]
            v = vpages[idx][..., :vd].float().permute(1, 0, 2, 3).reshape(G, -1, vd)[:, :L]
            i = torch.arange(past, L, device=q.device)[:, None]
            j = torch.arange(L, device=q.device)[None]
            vis = j <= i
            if window > 0:
                vis &= (i - j < window) | (j < keep_first)
            if chunk > 0:
                vis &= (i // chunk) == (j // chunk)
            qs = q[meta.start[b]:meta.start[b] + n]
            rep = H // G
            o = None
            for mp in range(maps):
                s = torch.einsum("thd,hld->htl", qs[:, :, mp], k[:, :, mp].repeat_interleave(rep, 0)) * scale
                if slopes is not None:
                    s = s - slopes.view(H, 1, 1) * (i - j).float()
                if softcap > 0:
                    s = softcap * torch.tanh(s / softcap)
                s = s.masked_fill(~vis, float("-inf"))
                if sink is None and sinks is None:
                    w = torch.softmax(s, -1)
                else:                                     # one more score in the normaliser, no value behind it
                    sk = sinks.view(H, 1, 1) if sinks is not None else torch.full((H, 1, 1), float(sink))
                    top = torch.maximum(s.max(-1, keepdim=True).values, sk)
                    w = torch.exp(s - top)
                    w = w / (w.sum(-1, keepdim=True) + torch.exp(sk - top))
                a = w @ v.repeat_interleave(rep, 0)       # [H, n, vd]
                o = a if mp == 0 else o - lam * a
            o = o.permute(1, 0, 2)
            if out_norm:
                o = o / torch.sqrt(o.pow(2).mean(-1, keepdim=True) + eps)
            out[meta.start[b]:meta.start[b] + n] = (o * out_scale).reshape(n, H * vd)
        if gate is not None and gate_wide:
            out = out * torch.sigmoid(gate[:, gate0:gate0 + H * vd].float())
        elif gate is not None:
            out = (out.view(meta.T, H, vd) * torch.sigmoid(gate[:, gate0:gate0 + H].float())[:, :, None]).view(meta.T, H * vd)
        return out.to(kpages.dtype)

    def post_norm_add(self, x, y, w_post, w_next, eps, act):
        v = y.float()
        x += v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w_post
        if w_next is None:
            return None
        return (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w_next).to(act)

    def relu2(self, A):
        return torch.relu(A.float()).pow(2).to(A.dtype)

    def head_norm_gate(self, o, w, P, g0, H, vd, eps, act, em=None, den_floor=0.0, scale=1.0):
        v = o.view(o.shape[0], H, -1)
        if em is not None:
            v = v[..., :vd] / (torch.maximum(v[..., vd].abs(), em) + den_floor)[..., None]
        v = (v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)).reshape(-1, H * vd)
        return (v * w * scale * torch.sigmoid(P[:, g0:g0 + H * vd].float())).to(act)

    def mlstm_gates(self, P, i0, gate_bias, cap, m_start, H, mstate, meta):
        li = cap * torch.tanh((P[:, i0:i0 + H].float() + gate_bias[:H]) / cap)
        lf = F.logsigmoid(cap * torch.tanh((P[:, i0 + H:i0 + 2 * H].float() + gate_bias[H:]) / cap))
        a, b, em = torch.empty_like(li), torch.empty_like(li), torch.empty_like(li)
        for s, (slot, past, n, _) in enumerate(meta.seqs):
            m = mstate[slot].clone() if past > 0 else torch.full((H,), float(m_start))
            for i in range(n):
                t = meta.start[s] + i
                m2 = torch.maximum(lf[t] + m, li[t])
                a[t], b[t], em[t] = torch.exp(lf[t] + m - m2), torch.exp(li[t] - m2), torch.exp(-m2)
                m = m2
            mstate[slot] = m
        return a, b, em

    def mlstm_expand(self, P, q0, k0, a, b, H, d):
        T = P.shape[0]
        q = P[:, q0:q0 + H * d].float() * d ** -0.5
        k = P[:, k0:k0 + H * d].float().view(T, H, d)
        return q, a[:, :, None].expand(T, H, d).reshape(T, -1).contiguous(), (b[:, :, None] * k).reshape(T, -1)

    def moe_route(self, xa, w_router, groups, keep, top, scale, score="softmax", group_top=1, renorm=False):
        z = xa.float() @ w_router.t()
        s = torch.sigmoid(z) if score == "sigmoid" else torch.softmax(z, -1)
        E = s.shape[1]
        best = s.view(-1, groups, E // groups).topk(min(group_top, E // groups), -1).values.sum(-1)
        kept = torch.zeros_like(best, dtype=torch.bool)
        kept.scatter_(1, best.topk(keep, -1).indices, True)
        idx = s.masked_fill(~kept.repeat_interleave(E // groups, 1), -1.0).topk(top, -1).indices
        w = s.gather(1, idx)
        if renorm:
            w = w / (w.sum(-1, keepdim=True) + 1e-20)
        return idx.to(torch.int32), w * scale

    def moe_sorted(self, xa, idx, wts, w_up, w_dn, base, gated=False):
        return None                                             # (the host statements run the experts one by one)

    def moe_combine(self, ys, place, wts, base):
        y = torch.zeros(place.shape[0], ys.shape[1]) if base is None else base.float().clone()
        for j in range(place.shape[1]):
            y += wts[:, j, None] * ys[place[:, j].long()].float()
        return y.to(ys.dtype)

    def moe_rows(self, xa, idx, wts, w_up, w_dn, base, gated=False):
        y = torch.zeros(xa.shape[0], w_dn.shape[1]) if base is None else base.float().clone()
        for t in range(xa.shape[0]):
            for j in range(idx.shape[1]):
                e = int(idx[t, j])
                a = w_up[e].float() @ xa[t].float()
                a = (F.silu(a[0::2]) * a[1::2] if gated else torch.relu(a).pow(2)).to(xa.dtype)
                y[t] += wts[t, j] * (w_dn[e].float() @ a.float())
        return y.to(xa.dtype)

    def embed_rows(self, ids, table, ids2=None, table2=None, scale=1.0):
        x = table[ids].float() * scale
        return x if table2 is None else x + table2[ids2].float()

    def add_norm(self, x, y1, y2, w_next, eps, act):
        if y1 is not None:
            x += y1.float() if y2 is None else y1.float() + y2.float()
        if w_next is None:
            return None
        return (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w_next).to(act)

    def act_cols(self, P, col0, n, kind, params=(0.0, 0.0)):
        z = P[:, col0:col0 + n].float()
        if kind == "gelu_erf":
            v = 0.5 * z * (1.0 + torch.erf(z * 0.7071067811865476))
        elif kind == "gelu_tanh":
            v = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        elif kind == "tanh":
            v = torch.tanh(z)
        elif kind == "xielu":
            v = torch.where(z > 0, params[0] * z * z + 0.5 * z, (0.5 + params[1]) * (torch.expm1(z.clamp(max=0.0)) - z) + 0.5 * z)
        else:
            v = torch.relu(z).pow(2)
        return v.to(P.dtype)

    def glu_pairs(self, P):
        return (F.silu(P[:, 0::2].float()) * P[:, 1::2].float()).to(P.dtype)

    def hc_step(self, X, y, prev, nxt, w_next, eps, act, want_u=False):
        S = X.shape[1]
        if y is not None:
            out, mix = prev[S:2 * S], prev[2 * S:].view(S, S)
            X.copy_(torch.einsum("st,rsd->rtd", mix, X) + out[None, :, None] * y.float()[:, None, :])
        if nxt is None:
            return None, None
        u = torch.einsum("s,rsd->rd", nxt[:S], X)
        xa = None if w_next is None else (u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w_next).to(act)
        return xa, (u if want_u else None)

    def gate_cols(self, o, P, g0, act, scale=1.0):
        return (scale * o * torch.sigmoid(P[:, g0:g0 + o.shape[1]].float())).to(act)

    def delta_gates(self, P, r0, k0, a0, wl, w0, ab, rate, tiny, H, d):
        T, HD = P.shape[0], H * d
        k = P[:, k0:k0 + HD].float()
        n = (k.view(T, H, d) / torch.sqrt(k.view(T, H, d).pow(2).sum(-1, keepdim=True) + tiny)).reshape(T, HD)
        return [P[:, r0:r0 + HD].float(), torch.exp(-rate * torch.sigmoid(wl + w0)), n,
                torch.sigmoid(P[:, a0:a0 + HD].float() + ab) * n, k]

    def delta_scan(self, arrays, P, v0, state, H, d, vd, meta):
        rf, wf, nf, bf, kf = arrays
        out = torch.empty(meta.T, H * vd, dtype=torch.float32, device=P.device)
        for b, (slot, past, n, _) in enumerate(meta.seqs):
            S = state[slot].clone() if past > 0 else torch.zeros_like(state[slot])
            for i in range(n):
                t = meta.start[b] + i
                v = P[t, v0:v0 + H * vd].float().view(H, 1, vd)
                dot = (nf[t].view(H, d, 1) * S).sum(1, keepdim=True)
                S = wf[t].view(H, d, 1) * S - bf[t].view(H, d, 1) * dot + kf[t].view(H, d, 1) * v
                out[t] = (S * rf[t].view(H, d, 1)).sum(1).reshape(-1)
            state[slot] = S
        return out


def ops_for(device) -> object:
    """The kernels for a GPU, the PyTorch statements for the CPU.  A GPU never gets the latter."""
    device = torch.device(device)
    if device.type == "cuda":
        lib()
        return HipOps()
    return TorchOps()
