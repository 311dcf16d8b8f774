"""The HIP kernel library behind the parts: thin, checking wrappers over its C entry points.

Every function takes torch tensors on the GPU, checks shape, dtype and layout on the host (a kernel is never
launched on operands it does not fit), and enqueues on torch's current stream.  There is no CPU path: without
a GPU or a compiled library, loading fails with an error.
"""
import ctypes

import torch

from . import build as _build

_c = ctypes
_P, _I, _L, _F = _c.c_void_p, _c.c_int, _c.c_long, _c.c_float

_CORE_SIGS = {
    "tp_embed_rows": [_P, _P, _I, _F, _P, _I, _I, _I, _P],
    "tp_rms_norm": [_P, _I, _P, _F, _P, _I, _I, _I, _I, _P],
    "tp_add_rms_norm": [_P, _P, _I, _I, _L, _P, _F, _P, _F, _P, _I, _I, _I, _I, _P],
    "tp_scale_rows": [_P, _L, _F, _P],
    "tp_causal_conv": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
    "tp_latent_prepare": [_P, _L, _I, _I, _I, _I, _I, _I, _P, _F, _P, _I, _P, _P, _P, _P, _I, _P, _I, _I, _P, _P, _I, _P, _L, _P],
    "tp_head_linear": [_P, _L, _L, _P, _P, _L, _L, _I, _I, _I, _I, _I, _I, _P],
    "tp_route_top": [_P, _I, _I, _I, _I, _I, _P, _P, _P],
    "tp_expert_ffn_workspace_bytes": [_I, _I, _I, _I, _I, _I],
    "tp_expert_ffn": [_P, _I, _I, _I, _P, _P, _I, _I, _I, _P, _P, _F, _F, _F, _I, _P, _L, _P, _I, _P],
    "tp_conv_act": [_P, _L, _I, _P, _P, _P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _I, _P],
    "tp_ssd_scan_workspace_bytes": [_I, _I, _I, _I, _I, _I],
    "tp_ssd_scan": [_P, _L, _P, _L, _P, _L, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _L, _P],
    "tp_pair_norm_mean": [_P, _P, _I, _P, _P, _F, _P, _I, _I, _P],
    "tp_mul_sigmoid": [_P, _L, _P, _L, _I, _I, _I, _P],
    "tp_gather_rows": [_P, _P, _P, _I, _I, _I, _P],
    "tp_sum_slices": [_P, _I, _L, _P, _I, _L, _P],
    "tp_rope_kv_write": [_P, _L, _P, _L, _P, _L, _I, _I, _I, _I, _I, _P, _I, _P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _P],
    "tp_kv_write": [_P, _L, _P, _L, _I, _I, _I, _I, _P, _P, _P, _P, _I, _P, _P, _I, _I, _P],
    "tp_gated_act": [_P, _P, _I, _I, _I, _I, _F, _F, _P],
    "tp_linear": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _F, _F, _P, _L, _I, _I, _P],
    "tp_shift_mix": [_P, _I, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P],
    "tp_bias_act": [_P, _I, _P, _P, _I, _I, _I, _I, _I, _P],
    "tp_mul_sigmoid_heads": [_P, _L, _I, _P, _L, _I, _I, _I, _I, _P],
    "tp_qkv_prepare": [_P, _L, _I, _P, _I, _I, _I, _I, _I, _P, _I, _I, _F, _P, _P, _P, _P, _I, _P],
    "tp_pool_write": [_P, _L, _P, _L, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _P, _P, _I, _P],
    "tp_attn_pooled": [_P, _L, _P, _L, _P, _L, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _P, _I, _P, _P, _I,
                       _F, _F, _I, _I, _P, _P],
    "tp_talk_mix": [_P, _P, _P, _I, _I, _I, _I, _I, _P],
    "tp_unary_tanh": [_P, _I, _L, _P],
    "tp_weighted_sum": [_P, _F, _P, _F, _I, _P, _L, _P],
    "tp_head_norm_gate": [_P, _P, _P, _L, _I, _F, _P, _I, _I, _I, _I, _I, _P],
    "tp_time_mix_scan": [_P, _L, _P, _L, _P, _L, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _P],
    "tp_matrix_memory_scan": [_P, _L, _P, _L, _P, _L, _I, _P, _F, _F, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _P],
    "tp_time_mix_scan_workspace_floats": [_I, _I, _I, _I],
    "tp_matrix_memory_scan_workspace_floats": [_I, _I, _I, _I, _I],
    "tp_linear_workspace_bytes": [_I, _I, _I, _I, _I, _I, _I, _I, _I],
    "tp_attn_simple_prefill": [_P, _L, _P, _L, _P, _L, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _I, _P, _P, _P, _P],
    "tp_attn_simple_decode": [_P, _L, _I, _I, _I, _I, _I, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _I, _P, _P, _P, _P],
    "tp_argmax": [_P, _I, _I, _P, _P, _P],
    "tp_argmax_workspace_bytes": [_I, _I],
    "tp_repetition_penalty": [_P, _I, _I, _P, _I, _F, _P],
    "tp_recent_push": [_P, _P, _P, _I, _I, _P],
    "tp_add_bias": [_P, _I, _P, _I, _I, _P],
    "tp_sample": [_P, _I, _I, _F, _I, _F, _P, _P, _P, _P],
    "tp_sample_workspace_bytes": [_I, _I],
    "tp_probe_stream": [_P, _L, _P, _I, _P],
    "tp_probe_mfma": [_I, _I, _I, _P, _P, _P],
}
_ATTN_SIGS = {
    "tp_attn_prefill": [_P, _L, _P, _L, _P, _L, _I, _I, _I, _P, _I, _I, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _I, _P, _P, _P, _I, _P],
    "tp_attn_decode": [_P, _L, _I, _I, _I, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _I, _P, _P, _P, _P, _I, _P],
    "tp_attn_decode_shared": [_P, _L, _I, _I, _I, _I, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _P, _P, _I, _P],
    "tp_attn_decode_workspace_floats": [_I, _I, _I],
    "tp_attn_pooled_tile": [_P, _L, _P, _L, _P, _L, _I, _I, _I, _I, _P, _P, _P, _I, _P, _P, _I, _I, _P, _I, _P, _P, _I, _F, _F, _I, _I, _P, _P],
    "tp_attn_decode_fused": [_P, _I, _I, _L, _L, _P, _I, _I, _I, _I, _I, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _P, _P, _I, _P],
}

EPI_NONE, EPI_SOFTCAP, EPI_GATED = 0, 1, 2
ROPE_PAIRINGS = {"halves": 0, "neighbours": 1}          # the kernel library's TP_ROPE_* enumerators
GATE_ACTIVATIONS = {"gelu_tanh": 0, "silu": 1, "relu": 2, "quick_gelu": 3}       # what a gated product's epilogue can apply to the gate
HEAD_GATES = {"sigmoid": 0, "silu": 1}               # what `head_norm_gate` multiplies a normed head by: act(g)
ROUTE_SCORES = {"softmax": 0, "sigmoid": 1}          # how a router's logits become scores
CONV_ACTIVATIONS = {None: 0, "silu": 1}
BIAS_ACTIVATIONS = {None: 0, "gelu_erf": 1}          # what `bias_act` applies after the bias
GATE_GROUP = 16


class KernelError(RuntimeError):
    """A kernel refused its operands, or the library could not be loaded."""


class SplitRows:
    """Rows of a product still in K slices: fp32 [slices, M, N], to be added in slice order by the kernel that
    consumes them (`add_rms_norm`), which saves a launch and a rounding.  `HipOps.rows()` adds them otherwise."""

    def __init__(self, slices):
        self.slices = slices
        self.shape = tuple(slices.shape[1:])
        self.dtype = torch.float32


def _code(dtype):
    if dtype == torch.float32:
        return 0
    if dtype == torch.bfloat16:
        return 1
    raise KernelError(f"dtype {dtype} is not supported by the kernels (float32 or bfloat16)")


def _bind(lib, sigs):
    lib.tp_last_error.restype = _c.c_char_p
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = _c.c_long if name.endswith(("_bytes", "_floats", "_elems")) else _I


class HipOps:
    SplitRows = SplitRows

    def __init__(self, device):
        if device.type != "cuda" or not torch.cuda.is_available():
            raise KernelError(
                "the HIP kernels need an AMD GPU: no CPU path exists (device %s, torch.cuda.is_available() = %s)"
                % (device, torch.cuda.is_available()))
        self.device = device
        try:
            path = _build.build_core()
            self.lib = _c.CDLL(path)
        except (OSError, _build.BuildError) as e:
            raise KernelError(f"the HIP kernel library could not be built or loaded: {e}") from None
        _bind(self.lib, _CORE_SIGS)
        self._attn = {}
        self._sample_ws = {}
        from .. import flags
        plain = flags.force_plain()
        self.force_linear = 1 if plain else 0   # 1 plain, 2 skinny, 3 tiled (6: its wide tile, 7: its 128 x 96 tile, 8, 9: loads into LDS, 128 x 128 and 128 x 96; 10, 11: 64 x 32 and 64 x 64 tiles, two k steps ahead), 4 multiply-adds (1-2 rows), 5 blocks of 8 rows of W
        self.force_plain_attention = plain
        self._timed = None                      # with TRAPETUM_AMD_PROFILE=1: [(entry point, start event, end event)] not yet summed
        self._profile_totals = {}               # entry point -> (milliseconds, calls)
        if flags.profile():
            import atexit
            self._timed = []
            atexit.register(self.profile_report)

    # ---- helpers -----------------------------------------------------------------------------------
    def _stream(self):
        return torch.cuda.current_stream(self.device).cuda_stream

    def _call(self, lib, name, *args):
        if self._timed is not None:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            rc = getattr(lib, name)(*args)
            b.record()
            self._timed.append((name, a, b))
            if len(self._timed) >= self.PROFILE_FOLD:
                self._fold_profile()            # so that a long run holds a bounded number of events
        else:
            rc = getattr(lib, name)(*args)
        if rc != 0:
            raise KernelError(lib.tp_last_error().decode())

    PROFILE_FOLD = 4096                         # timed calls kept as events before they are summed

    def _fold_profile(self):
        """Sum the timed calls so far into the totals per entry point and let go of their events."""
        if not self._timed:
            return
        self._timed[-1][2].synchronize()
        for name, a, b in self._timed:
            ms, n = self._profile_totals.get(name, (0.0, 0))
            self._profile_totals[name] = (ms + a.elapsed_time(b), n + 1)
        self._timed = []

    def profile_report(self, file=None):
        """The time of the calls so far per entry point, most expensive first (TRAPETUM_AMD_PROFILE=1); forgets them."""
        import sys
        if self._timed is None:
            return
        self._fold_profile()
        total, self._profile_totals = self._profile_totals, {}
        if not total:
            return
        out = file or sys.stderr
        for name, (ms, n) in sorted(total.items(), key=lambda kv: -kv[1][0]):
            print(f"[profile] op={name} calls={n} total_ms={ms:.3f} mean_us={1e3 * ms / n:.2f}", file=out, flush=True)

    def _dev(self, *tensors):
        for t in tensors:
            if t is not None and t.device != self.device and not (t.device.type == "cuda" and t.device.index == (self.device.index or 0)):
                raise KernelError(f"tensor on {t.device}, the kernels run on {self.device}")

    @staticmethod
    def _rows(t, what):
        """2-D, unit stride along the row; returns the row stride in elements."""
        if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
            raise KernelError(f"{what}: expected rows with contiguous elements, found shape {tuple(t.shape)} strides {t.stride()}")
        return t.stride(0)

    def attn_lib(self, head_dim, wide=False):
        key = (head_dim, bool(wide))
        if key not in self._attn:
            try:
                lib = _c.CDLL(_build.build_attention(head_dim, wide=wide))
            except (OSError, _build.BuildError) as e:
                raise KernelError(f"the attention kernels for head_dim {head_dim} could not be built or loaded: {e}") from None
            _bind(lib, _ATTN_SIGS)
            self._attn[key] = lib
        return self._attn[key]

    # ---- weights layout ----------------------------------------------------------------------------
    def pack_gate_up(self, w_gate, w_up):
        """[2 * ceil16(I), K]: 16 rows of gate, the 16 rows of up of the same units, and so on; zero rows pad."""
        i, k = w_gate.shape
        ip = -(-i // GATE_GROUP) * GATE_GROUP
        out = torch.zeros((2, ip, k), dtype=w_gate.dtype, device=w_gate.device)
        out[0, :i] = w_gate
        out[1, :i] = w_up
        return out.reshape(2, ip // GATE_GROUP, GATE_GROUP, k).transpose(0, 1).reshape(2 * ip, k).contiguous()

    # ---- row-wise kernels ----------------------------------------------------------------------------
    def embed_rows(self, tokens, table, scale):
        self._dev(tokens, table)
        if tokens.dtype != torch.int32 or tokens.dim() != 1 or not tokens.is_contiguous():
            raise KernelError("embed_rows: tokens must be a contiguous int32 vector")
        if not table.is_contiguous() or table.dim() != 2:
            raise KernelError("embed_rows: the table must be a contiguous matrix")
        m, (v, d) = tokens.numel(), table.shape
        out = torch.empty((m, d), dtype=torch.float32, device=self.device)
        self._call(self.lib, "tp_embed_rows", tokens.data_ptr(), table.data_ptr(), _code(table.dtype), float(scale),
                   out.data_ptr(), m, d, v, self._stream())
        return out

    def rms_norm(self, x, gain, eps, out_dtype, groups=1):
        """groups: the row is cut into that many equal consecutive parts, each over its own root mean square."""
        self._dev(x, gain)
        if not x.is_contiguous() or x.dim() != 2:
            raise KernelError("rms_norm: rows must be a contiguous matrix")
        m, d = x.shape
        if gain.dtype != torch.float32 or gain.numel() != d or not gain.is_contiguous():
            raise KernelError(f"rms_norm: gain must be float32 [{d}]")
        out = torch.empty((m, d), dtype=out_dtype, device=self.device)
        if groups < 1 or d % groups:
            raise KernelError(f"rms_norm: rows of {d} elements cannot be cut into {groups} equal groups")
        self._call(self.lib, "tp_rms_norm", x.data_ptr(), _code(x.dtype), gain.data_ptr(), float(eps), out.data_ptr(),
                   _code(out_dtype), m, d, int(groups), self._stream())
        return out

    def add_rms_norm(self, stream, rows, gain_post, eps_post, gain_next, eps_next, out_dtype, groups=1):
        """stream += post-norm(rows) (or rows); returns next-norm(stream) or None.  rows: a tensor or SplitRows.
        groups: both norms cut the row into that many equal consecutive parts."""
        m, d = stream.shape
        if groups < 1 or d % groups:
            raise KernelError(f"add_rms_norm: rows of {d} elements cannot be cut into {groups} equal groups")
        n_slices, stride = 1, 0
        if isinstance(rows, SplitRows) and d > self.MAX_SLICED_WIDTH:
            rows = self.rows(rows, out_dtype)            # the fused kernel keeps a row in registers: wider rows are added first
        if isinstance(rows, SplitRows):
            n_slices, stride = rows.slices.shape[0], rows.slices.stride(0)
            rows = rows.slices[0]
        self._dev(stream, rows, gain_post, gain_next)
        if stream.dtype != torch.float32 or not stream.is_contiguous():
            raise KernelError("add_rms_norm: the stream must be contiguous float32")
        if tuple(rows.shape) != (m, d) or not rows.is_contiguous():
            raise KernelError(f"add_rms_norm: rows {tuple(rows.shape)} do not match the stream {(m, d)}")
        for g in (gain_post, gain_next):
            if g is not None and (g.dtype != torch.float32 or g.numel() != d or not g.is_contiguous()):
                raise KernelError(f"add_rms_norm: gains must be float32 [{d}]")
        out = torch.empty((m, d), dtype=out_dtype, device=self.device) if gain_next is not None else None
        self._call(self.lib, "tp_add_rms_norm", stream.data_ptr(), rows.data_ptr(), _code(rows.dtype), n_slices, stride,
                   gain_post.data_ptr() if gain_post is not None else None, float(eps_post),
                   gain_next.data_ptr() if gain_next is not None else None, float(eps_next),
                   out.data_ptr() if out is not None else None, _code(out_dtype), m, d, int(groups), self._stream())
        return out

    def scale_rows(self, x, scale):
        """x *= scale, in place (float32)."""
        self._dev(x)
        if x.dtype != torch.float32 or not x.is_contiguous():
            raise KernelError("scale_rows: expected a contiguous float32 tensor")
        self._call(self.lib, "tp_scale_rows", x.data_ptr(), x.numel(), float(scale), self._stream())

    def causal_conv(self, stream, w, state, slot_ids, cu_rows, row_seq, out_dtype, residual=True, one_row_each=False, w_t=None):
        """out[r] = (stream[r]) + sum_j w[:, j] * stream[r - (taps - 1) + j] within each sequence; the rows before the
        step are read from state[slot] (float32 [slots, taps - 1, D], oldest first), which then takes the last
        taps - 1 rows of (state, step).  one_row_each: every sequence brings one row (one launch does both).
        w_t: the taps transposed, contiguous float32 [taps, D], for the kernel that takes four channels a thread."""
        self._dev(stream, w, state, slot_ids, cu_rows, row_seq)
        if stream.dtype != torch.float32 or stream.dim() != 2 or not stream.is_contiguous():
            raise KernelError("causal_conv: the stream must be contiguous float32 [rows, channels]")
        m, d = stream.shape
        if w.dtype != torch.float32 or w.dim() != 2 or w.shape[0] != d or not w.is_contiguous():
            raise KernelError(f"causal_conv: the taps must be contiguous float32 [{d}, taps]")
        taps, n_seq = w.shape[1], cu_rows.numel() - 1
        for t, n in ((cu_rows, n_seq + 1), (row_seq, m), (slot_ids, n_seq)):
            if t.dtype != torch.int32 or t.numel() != n:
                raise KernelError("causal_conv: cu_rows, row_seq and slot_ids must be int32 of the step's geometry")
        if taps > 1 and (state is None or state.dtype != torch.float32 or state.dim() != 3 or tuple(state.shape[1:]) != (taps - 1, d)
                         or not state.is_contiguous()):
            raise KernelError(f"causal_conv: the state must be contiguous float32 [slots, {taps - 1}, {d}]")
        if w_t is not None and (w_t.dtype != torch.float32 or tuple(w_t.shape) != (taps, d) or not w_t.is_contiguous()):
            raise KernelError(f"causal_conv: the transposed taps must be contiguous float32 [{taps}, {d}]")
        self._dev(w_t)
        out = torch.empty((m, d), dtype=out_dtype, device=self.device)
        self._call(self.lib, "tp_causal_conv", stream.data_ptr(), w.data_ptr(), w_t.data_ptr() if w_t is not None else None,
                   state.data_ptr() if taps > 1 else None,
                   slot_ids.data_ptr(), cu_rows.data_ptr(), row_seq.data_ptr(), out.data_ptr(), _code(out_dtype), m, n_seq, d, taps,
                   1 if residual else 0, 1 if one_row_each else 0, self._stream())
        return out

    # ---- attention through a cached latent ---------------------------------------------------------------------
    def latent_prepare(self, proj, H, dn, dr, R, gain, eps, inv_freq, rot, row_seq, row_pos, new_len, table, pool, rows_cap,
                       own=True, out_dtype=None, tail=None, write=True):
        """proj [M, H (dr + dn) (+ dr + R)]: per head [rotated | unrotated] query parts, then (own) [key part | latent];
        tail: the [key part | latent] as rows of their own [M, dr + R] (then proj holds the queries only).  write False:
        the step's rows are returned and not cached (the caller caches them after its attention has read the cache).
        Returns q [M, H (dr + R)] with every head's first dr elements set (the rotated query part; the rest is left
        for `head_linear`) and, when own, the step's rows [rope(key part) | rmsnorm(latent) * gain] [M, dr + R], which
        are also written into the cache pool [pages, 1, page, dr + R]."""
        self._dev(proj, gain, inv_freq, row_seq, row_pos, new_len, table, pool)
        m = proj.shape[0]
        stride = self._rows(proj, "latent_prepare proj")
        width = H * (dr + dn) + ((dr + R) if own and tail is None else 0)
        tail_stride = 0
        if tail is not None:
            self._dev(tail)
            tail_stride = self._rows(tail, "latent_prepare tail")
            if not own or tuple(tail.shape) != (m, dr + R) or tail.dtype != proj.dtype:
                raise KernelError(f"latent_prepare: the key part and latent as rows of their own must be [{m}, {dr + R}] of {proj.dtype}")
        if proj.shape[1] != width or (out_dtype is not None and out_dtype != proj.dtype):
            raise KernelError(f"latent_prepare: rows of {proj.shape[1]} columns, this geometry needs {width} of the output's dtype")
        if rot and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rot // 2):
            raise KernelError(f"latent_prepare: a rotation over {rot} needs float32 inv_freq [{rot // 2}]")
        for t in (row_seq, row_pos):
            if t.dtype != torch.int32 or t.numel() != m:
                raise KernelError("latent_prepare: row_seq and row_pos must be int32, one entry per row")
        q = torch.empty((m, H * (dr + R)), dtype=proj.dtype, device=self.device)
        mine = None
        page = table_w = 1
        if own:
            if gain is None or gain.dtype != torch.float32 or gain.numel() != R or not gain.is_contiguous():
                raise KernelError(f"latent_prepare: the latent's gain must be contiguous float32 [{R}]")
            self._check_pools("latent_prepare", proj.dtype, new_len.numel(), 1, dr + R, new_len, table, pool, pool)
            page, table_w = pool.shape[2], table.shape[1]
            mine = torch.empty((m, dr + R), dtype=proj.dtype, device=self.device)
        self._call(self.lib, "tp_latent_prepare", proj.data_ptr(), stride, _code(proj.dtype), m, H, dn, dr, R,
                   gain.data_ptr() if own else None, float(eps), inv_freq.data_ptr() if rot else None, int(rot),
                   row_seq.data_ptr(), row_pos.data_ptr(), new_len.data_ptr(), table.data_ptr() if own and write else None, table_w,
                   pool.data_ptr() if own and write else None, page, rows_cap if own and write else 0, q.data_ptr(),
                   mine.data_ptr() if own else None, 1 if own else 0, tail.data_ptr() if tail is not None else None, tail_stride,
                   self._stream())
        return q, mine

    def head_linear(self, x, w, out=None):
        """out[m, h, :] = w[h] @ x[m, h, :].  x: a view [M, H, K] of wider rows (a head's elements contiguous), w
        contiguous [H, N, K]; out: a view [M, H, N] to fill, or None for a new contiguous tensor."""
        self._dev(x, w, out)
        if x.dim() != 3 or w.dim() != 3 or w.shape[0] != x.shape[1] or w.shape[2] != x.shape[2] or not w.is_contiguous() or x.dtype != w.dtype:
            raise KernelError(f"head_linear: rows {tuple(x.shape)} and matrices {tuple(w.shape)} do not fit, or differ in dtype")
        m, H, K = x.shape
        N = w.shape[1]
        if out is None:
            out = torch.empty((m, H, N), dtype=x.dtype, device=self.device)
        if out.dim() != 3 or tuple(out.shape) != (m, H, N) or out.dtype != x.dtype:
            raise KernelError(f"head_linear: the output must be {(m, H, N)} of {x.dtype}")
        for t, what in ((x, "rows"), (out, "output")):
            if t.shape[2] > 1 and t.stride(2) != 1:
                raise KernelError(f"head_linear: a head's elements must be contiguous in the {what}")
        self._call(self.lib, "tp_head_linear", x.data_ptr(), x.stride(0), x.stride(1), w.data_ptr(), out.data_ptr(),
                   out.stride(0), out.stride(1), _code(x.dtype), m, H, N, K, 1 if self.force_linear == 1 else 0, self._stream())
        return out

    # ---- mixture of experts ------------------------------------------------------------------------------------
    def route_top(self, logits, top, renormalize=False, score="softmax"):
        """Scores: softmax over all experts, or the sigmoid of each logit; the `top` largest scores (ties: the smaller
        index): int32 [M, top], float32 [M, top]."""
        if score not in ROUTE_SCORES:
            raise KernelError(f"route_top: score '{score}' has no kernel ({', '.join(ROUTE_SCORES)})")
        self._dev(logits)
        if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
            raise KernelError("route_top: router logits must be contiguous float32 [rows, experts]")
        m, e = logits.shape
        if not 0 < top <= e:
            raise KernelError(f"route_top: {top} of {e} experts cannot be chosen")
        chosen = torch.empty((m, top), dtype=torch.int32, device=self.device)
        weight = torch.empty((m, top), dtype=torch.float32, device=self.device)
        self._call(self.lib, "tp_route_top", logits.data_ptr(), m, e, int(top), 1 if renormalize else 0, ROUTE_SCORES[score], chosen.data_ptr(),
                   weight.data_ptr(), self._stream())
        return chosen, weight

    def expert_ffn(self, x, chosen, weights, w_gate_up, w_down, limit, alpha, shift, weight_input=False, out=None):
        """float32 [M, D]: sum over a row's chosen experts of weight * W_down,e (g' sigmoid(alpha g') (u' + shift)), with
        g' = min(W_gate,e x, limit), u' = clamp(W_up,e x, -limit, limit).  w_gate_up [E, 2 F, D] (gate rows, then up
        rows), w_down [E, D, F].  limit None: no clamp.  weight_input: the weight multiplies the expert's input instead,
        expert(weight * x), and the outputs are summed as they are.  out: a contiguous float32 [M, D] to fill."""
        limit = float("inf") if limit is None else limit
        self._dev(x, chosen, weights, w_gate_up, w_down)
        if x.dim() != 2 or not x.is_contiguous() or x.dtype != w_gate_up.dtype or x.dtype != w_down.dtype:
            raise KernelError("expert_ffn: rows and matrices must be contiguous and of one dtype")
        m, d = x.shape
        if w_gate_up.dim() != 3 or w_down.dim() != 3 or not w_gate_up.is_contiguous() or not w_down.is_contiguous():
            raise KernelError("expert_ffn: the experts' matrices must be contiguous [experts, rows, columns]")
        e, f2, _ = w_gate_up.shape
        f = f2 // 2
        if f2 % 2 or w_gate_up.shape[2] != d or tuple(w_down.shape) != (e, d, f):
            raise KernelError(f"expert_ffn: matrices {tuple(w_gate_up.shape)} and {tuple(w_down.shape)} do not fit rows of {d}")
        top = chosen.shape[1]
        if chosen.dtype != torch.int32 or tuple(chosen.shape) != (m, top) or weights.dtype != torch.float32 or tuple(weights.shape) != (m, top) \
                or not chosen.is_contiguous() or not weights.is_contiguous():
            raise KernelError("expert_ffn: the choice must be int32 [rows, top] with float32 weights of the same shape")
        nbytes = self.lib.tp_expert_ffn_workspace_bytes(_code(x.dtype), m, top, e, f, d)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        if out is None:
            out = torch.empty((m, d), dtype=torch.float32, device=self.device)
        elif out.dtype != torch.float32 or tuple(out.shape) != (m, d) or not out.is_contiguous():
            raise KernelError(f"expert_ffn: the output must be contiguous float32 {(m, d)}")
        self._dev(out)
        self._call(self.lib, "tp_expert_ffn", x.data_ptr(), _code(x.dtype), m, d, chosen.data_ptr(), weights.data_ptr(), top, e, f,
                   w_gate_up.data_ptr(), w_down.data_ptr(), float(limit), float(alpha), float(shift), 1 if weight_input else 0,
                   ws.data_ptr(), nbytes,
                   out.data_ptr(), 1 if self.force_linear == 1 else 0, self._stream())
        return out

    # ---- a state-space mixer; two mixers side by side ------------------------------------------------------------------
    def conv_act(self, x, w_t, bias, state, slot_ids, cu_rows, row_seq, activation=None, one_row_each=False):
        """out[r] = act(bias + sum_j w_t[j] * x[r - (taps - 1) + j]) within each sequence, on a view x [M, C] of wider rows;
        the rows before the step are read from state[slot] (float32 [slots, taps - 1, C], oldest first), which then takes
        the last taps - 1 rows of (state, step).  w_t: float32 [taps, C].  Returns a contiguous [M, C] of x's dtype."""
        if activation not in CONV_ACTIVATIONS:
            raise KernelError(f"conv_act: activation '{activation}' has no kernel")
        self._dev(x, w_t, bias, state, slot_ids, cu_rows, row_seq)
        stride = self._rows(x, "conv_act rows")
        m, c = x.shape
        if w_t.dtype != torch.float32 or w_t.dim() != 2 or w_t.shape[1] != c or not w_t.is_contiguous():
            raise KernelError(f"conv_act: the taps must be contiguous float32 [taps, {c}]")
        taps, n_seq = w_t.shape[0], cu_rows.numel() - 1
        if bias is not None and (bias.dtype != torch.float32 or bias.numel() != c or not bias.is_contiguous()):
            raise KernelError(f"conv_act: the bias must be contiguous float32 [{c}]")
        for t, n in ((cu_rows, n_seq + 1), (row_seq, m), (slot_ids, n_seq)):
            if t.dtype != torch.int32 or t.numel() != n:
                raise KernelError("conv_act: cu_rows, row_seq and slot_ids must be int32 of the step's geometry")
        if taps > 1 and (state is None or state.dtype != torch.float32 or state.dim() != 3 or tuple(state.shape[1:]) != (taps - 1, c)
                         or not state.is_contiguous()):
            raise KernelError(f"conv_act: the state must be contiguous float32 [slots, {taps - 1}, {c}]")
        out = torch.empty((m, c), dtype=x.dtype, device=self.device)
        self._call(self.lib, "tp_conv_act", x.data_ptr(), stride, _code(x.dtype), w_t.data_ptr(), bias.data_ptr() if bias is not None else None,
                   state.data_ptr() if taps > 1 else None, slot_ids.data_ptr(), cu_rows.data_ptr(), row_seq.data_ptr(), out.data_ptr(), c,
                   _code(out.dtype), m, n_seq, c, taps, CONV_ACTIVATIONS[activation], 1 if one_row_each else 0, self._stream())
        return out

    SSD_CHUNK = 64                 # rows of a piece when a long scan is cut into pieces that run side by side

    def ssd_scan(self, xbc, z, dt, dt_bias, a_log, skip, state, slot_ids, cu_rows, max_count, heads, groups, n_state, head_dim):
        """The recurrence of a state-space mixer over the step's rows, sequence by sequence, from state[slot] (float32
        [slots, heads, n_state, head_dim]), which it leaves updated:
            S <- exp(-exp(a_log) d) S + d B x^T,  y = (S^T C + skip x) * silu(z),  d = softplus(dt + dt_bias)
        xbc [M, heads head_dim + 2 groups n_state] = [x | B | C]; z [M, heads head_dim] and dt [M, heads] may be views of
        wider rows.  Returns y float32 [M, heads head_dim]."""
        self._dev(xbc, z, dt, dt_bias, a_log, skip, state, slot_ids, cu_rows)
        m = xbc.shape[0]
        inner = heads * head_dim
        xs, zs, ds = self._rows(xbc, "ssd_scan xbc"), self._rows(z, "ssd_scan z"), self._rows(dt, "ssd_scan dt")
        if xbc.shape[1] != inner + 2 * groups * n_state or tuple(z.shape) != (m, inner) or tuple(dt.shape) != (m, heads):
            raise KernelError(f"ssd_scan: rows {tuple(xbc.shape)}, gates {tuple(z.shape)} and steps {tuple(dt.shape)} do not fit "
                              f"{heads} heads of {head_dim}, {groups} groups and a state of {n_state}")
        if not (xbc.dtype == z.dtype == dt.dtype):
            raise KernelError("ssd_scan: rows, gates and steps share one dtype")
        if heads % groups:
            raise KernelError(f"ssd_scan: {heads} heads are no multiple of {groups} groups")
        for t in (dt_bias, a_log, skip):
            if t.dtype != torch.float32 or t.numel() != heads or not t.is_contiguous():
                raise KernelError(f"ssd_scan: dt_bias, a_log and skip must be contiguous float32 [{heads}]")
        n_seq = cu_rows.numel() - 1
        if slot_ids.dtype != torch.int32 or slot_ids.numel() != n_seq or cu_rows.dtype != torch.int32:
            raise KernelError("ssd_scan: slot_ids and cu_rows must be int32 of the step's geometry")
        if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (heads, n_state, head_dim) or not state.is_contiguous():
            raise KernelError(f"ssd_scan: the state must be contiguous float32 [slots, {heads}, {n_state}, {head_dim}]")
        y = torch.empty((m, inner), dtype=torch.float32, device=self.device)
        # pieces enough to give the GPU some four thousand waves, of at least SSD_CHUNK rows each
        waves = n_seq * heads * -(-head_dim // 64)
        chunk = max(self.SSD_CHUNK, -(-int(max_count) // max(1, 4096 // waves)))
        chunk = -(-chunk // 16) * 16
        nbytes = self.lib.tp_ssd_scan_workspace_bytes(n_seq, int(max_count), heads, n_state, head_dim, chunk)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device) if nbytes else None
        self._call(self.lib, "tp_ssd_scan", xbc.data_ptr(), xs, z.data_ptr(), zs, dt.data_ptr(), ds, _code(xbc.dtype), dt_bias.data_ptr(),
                   a_log.data_ptr(), skip.data_ptr(), state.data_ptr(), slot_ids.data_ptr(), cu_rows.data_ptr(), y.data_ptr(), n_seq,
                   int(max_count), heads, groups, n_state, head_dim, chunk, ws.data_ptr() if ws is not None else None, nbytes, self._stream())
        return y

    # ---- mixers that carry a matrix per head from token to token --------------------------------------------------------
    def _geometry(self, what, m, slot_ids, cu_rows, row_seq=None):
        n_seq = cu_rows.numel() - 1
        for t, n in ((cu_rows, n_seq + 1), (slot_ids, n_seq)) + (((row_seq, m),) if row_seq is not None else ()):
            if t.dtype != torch.int32 or t.numel() != n:
                raise KernelError(f"{what}: cu_rows, row_seq and slot_ids must be int32 of the step's geometry")
        return n_seq

    def shift_mix(self, x, mu, state, slot_ids, cu_rows, row_seq, one_row_each=False, out_dtype=None):
        """out[s, r] = x[r] + (x[r - 1] - x[r]) * mu[s] within each sequence; the row before a sequence's first row of
        the step is state[slot] (float32 [slots, D]), which then takes the sequence's last row.  mu float32 [S, D];
        returns [S, M, D] of x's dtype, or of out_dtype (float32 rows may give bfloat16 mixes)."""
        self._dev(x, mu, state, slot_ids, cu_rows, row_seq)
        if x.dim() != 2 or not x.is_contiguous():
            raise KernelError("shift_mix: rows must be a contiguous matrix")
        m, d = x.shape
        if mu.dtype != torch.float32 or mu.dim() != 2 or mu.shape[1] != d or not mu.is_contiguous():
            raise KernelError(f"shift_mix: the mixing vectors must be contiguous float32 [mixes, {d}]")
        if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] != d or not state.is_contiguous():
            raise KernelError(f"shift_mix: the state must be contiguous float32 [slots, {d}]")
        n_seq = self._geometry("shift_mix", m, slot_ids, cu_rows, row_seq)
        out = torch.empty((mu.shape[0], m, d), dtype=out_dtype or x.dtype, device=self.device)
        self._call(self.lib, "tp_shift_mix", x.data_ptr(), _code(x.dtype), mu.data_ptr(), mu.shape[0], state.data_ptr(), slot_ids.data_ptr(),
                   cu_rows.data_ptr(), row_seq.data_ptr(), out.data_ptr(), _code(out.dtype), m, n_seq, d, 1 if one_row_each else 0, self._stream())
        return out

    def unary_(self, x, name):
        """In place on a contiguous tensor: x <- tanh(x)."""
        if name != "tanh":
            raise KernelError(f"unary_: '{name}' has no kernel (tanh)")
        self._dev(x)
        if not x.is_contiguous():
            raise KernelError("unary_: expected a contiguous tensor")
        self._call(self.lib, "tp_unary_tanh", x.data_ptr(), _code(x.dtype), x.numel(), self._stream())
        return x

    def weighted_sum(self, a, wa, b, wb):
        """float32: wa * a + wb * b, for two contiguous tensors of one shape and dtype."""
        self._dev(a, b)
        if a.shape != b.shape or a.dtype != b.dtype or not a.is_contiguous() or not b.is_contiguous():
            raise KernelError("weighted_sum: two contiguous tensors of one shape and dtype")
        out = torch.empty(a.shape, dtype=torch.float32, device=self.device)
        self._call(self.lib, "tp_weighted_sum", a.data_ptr(), float(wa), b.data_ptr(), float(wb), _code(a.dtype), out.data_ptr(), a.numel(), self._stream())
        return out

    def head_norm_gate(self, y, gain, g, eps, heads, activation, out_dtype):
        """Every head's part of a row of y (float32 [M, D]) over its root mean square, times gain (float32 [D]), times
        act(g) with act one of HEAD_GATES; g [M, D] of the output's dtype, possibly a view of wider rows."""
        if activation not in HEAD_GATES:
            raise KernelError(f"head_norm_gate: gate '{activation}' has no kernel ({', '.join(HEAD_GATES)})")
        self._dev(y, gain, g)
        if y.dtype != torch.float32 or y.dim() != 2 or not y.is_contiguous():
            raise KernelError("head_norm_gate: rows must be a contiguous float32 matrix")
        m, d = y.shape
        if heads < 1 or d % heads:
            raise KernelError(f"head_norm_gate: rows of {d} elements are not {heads} equal heads")
        if gain.dtype != torch.float32 or gain.numel() != d or not gain.is_contiguous():
            raise KernelError(f"head_norm_gate: the gain must be contiguous float32 [{d}]")
        gs = self._rows(g, "head_norm_gate gates")
        if tuple(g.shape) != (m, d) or g.dtype != out_dtype:
            raise KernelError(f"head_norm_gate: gates must be {(m, d)} of the output's dtype {out_dtype}")
        out = torch.empty((m, d), dtype=out_dtype, device=self.device)
        self._call(self.lib, "tp_head_norm_gate", y.data_ptr(), gain.data_ptr(), g.data_ptr(), gs, _code(g.dtype), float(eps), out.data_ptr(),
                   _code(out_dtype), m, heads, d // heads, HEAD_GATES[activation], self._stream())
        return out

    MAX_SCAN_DIM = 256             # key rows a lane of a scan keeps of its column, and columns of a block

    def time_mix_scan(self, r, k, v, log_rate, w0, bonus, state, slot_ids, cu_rows, max_count, heads, dim, chunk=None):
        """o = (S + diag(bonus) k v^T)^T r, then S <- diag(w) S + k v^T with w = exp(-exp(log_rate + w0)), row after row
        of every sequence from state[slot] (float32 [slots, heads, dim, dim]: key row, value column), which is left
        updated.  r, k, v [M, heads dim], possibly views of wider rows; log_rate float32 [M, heads dim]; w0 float32
        [heads dim]; bonus float32 [heads, dim].  Returns float32 [M, heads dim].  chunk: rows of a chunk (0: whole
        sequences; None: `scan_chunks` decides by max_count, which no sequence's rows may exceed)."""
        self._dev(r, k, v, log_rate, w0, bonus, state, slot_ids, cu_rows)
        m, inner = r.shape[0], heads * dim
        rs, ks, vs = self._rows(r, "time_mix_scan r"), self._rows(k, "time_mix_scan k"), self._rows(v, "time_mix_scan v")
        if any(tuple(t.shape) != (m, inner) for t in (r, k, v)) or not (r.dtype == k.dtype == v.dtype):
            raise KernelError(f"time_mix_scan: r, k and v must be {(m, inner)} of one dtype")
        if dim > self.MAX_SCAN_DIM:
            raise KernelError(f"time_mix_scan: heads of {dim} channels exceed {self.MAX_SCAN_DIM}")
        if log_rate.dtype != torch.float32 or tuple(log_rate.shape) != (m, inner) or not log_rate.is_contiguous():
            raise KernelError(f"time_mix_scan: the decays' logarithms must be contiguous float32 {(m, inner)}")
        for t in (w0, bonus):
            if t.dtype != torch.float32 or t.numel() != inner or not t.is_contiguous():
                raise KernelError(f"time_mix_scan: w0 and the bonus must be contiguous float32 of {inner} elements")
        if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (heads, dim, dim) or not state.is_contiguous():
            raise KernelError(f"time_mix_scan: the state must be contiguous float32 [slots, {heads}, {dim}, {dim}]")
        n_seq = self._geometry("time_mix_scan", m, slot_ids, cu_rows)
        y = torch.empty((m, inner), dtype=torch.float32, device=self.device)
        chunk, n_chunks = self.scan_chunks(max_count) if chunk is None else (int(chunk), -(-int(max_count) // int(chunk)) if chunk else 0)
        ws = None
        if chunk:
            ws = torch.empty(self.lib.tp_time_mix_scan_workspace_floats(n_seq, n_chunks, heads, dim), dtype=torch.float32, device=self.device)
        self._call(self.lib, "tp_time_mix_scan", r.data_ptr(), rs, k.data_ptr(), ks, v.data_ptr(), vs, _code(r.dtype), log_rate.data_ptr(),
                   w0.data_ptr(), bonus.data_ptr(), state.data_ptr(), slot_ids.data_ptr(), cu_rows.data_ptr(), y.data_ptr(), n_seq, heads, dim,
                   chunk, n_chunks, ws.data_ptr() if ws is not None else None, self._stream())
        return y

    SCAN_CHUNK_FROM = 96         # rows of the longest sequence from which a scan runs in chunks

    def scan_chunks(self, max_count):
        """(rows of a chunk, chunks that cover the longest sequence) for the two scans of a matrix state; (0, 0): every
        sequence in one piece, row after row.  Chunks of 32 rows give a prompt of a few thousand tokens as many waves
        as the chip has places for; longer ones take longer chunks, so that the states between them stay small."""
        n = int(max_count)
        if n < self.SCAN_CHUNK_FROM:
            return 0, 0
        chunk = 32 if n <= 8192 else 64 if n <= 32768 else 128
        return chunk, -(-n // chunk)

    def matrix_memory_scan(self, q, k, v, gates, cap, q_scale, memory, normalizer, maximum, slot_ids, cu_rows, max_count, heads, dk, dv,
                           chunk=None):
        """gates float32 [M, 2 heads]: the input gates' sums, then the forget gates'.  i = cap tanh(. / cap),
        f = logsigmoid(cap tanh(. / cap)), m' = max(f + m, i), S <- e^(f + m - m') S + e^(i - m') k v^T, n likewise with k,
        o = S^T q' / (max(|n . q'|, e^(-m')) + 1e-6) with q' = q q_scale, row after row of every sequence from the states
        memory [slots, heads, dk, dv], normalizer [slots, heads, dk] and maximum [slots, heads] (float32), which are left
        updated.  q, k [M, heads dk] and v [M, heads dv] may be views of wider rows.  Returns float32 [M, heads dv].
        chunk: as in `time_mix_scan`."""
        self._dev(q, k, v, gates, memory, normalizer, maximum, slot_ids, cu_rows)
        m = q.shape[0]
        qs, ks, vs = self._rows(q, "matrix_memory_scan q"), self._rows(k, "matrix_memory_scan k"), self._rows(v, "matrix_memory_scan v")
        if tuple(q.shape) != (m, heads * dk) or tuple(k.shape) != (m, heads * dk) or tuple(v.shape) != (m, heads * dv) or not (q.dtype == k.dtype == v.dtype):
            raise KernelError(f"matrix_memory_scan: q, k {(m, heads * dk)} and v {(m, heads * dv)} of one dtype")
        if dk > self.MAX_SCAN_DIM or dv > self.MAX_SCAN_DIM:
            raise KernelError(f"matrix_memory_scan: heads of {dk} x {dv} exceed {self.MAX_SCAN_DIM}")
        if gates.dtype != torch.float32 or tuple(gates.shape) != (m, 2 * heads) or not gates.is_contiguous():
            raise KernelError(f"matrix_memory_scan: the gates' sums must be contiguous float32 {(m, 2 * heads)}")
        for t, shape in ((memory, (heads, dk, dv)), (normalizer, (heads, dk)), (maximum, (heads,))):
            if t.dtype != torch.float32 or tuple(t.shape[1:]) != shape or not t.is_contiguous():
                raise KernelError(f"matrix_memory_scan: a state must be contiguous float32 [slots, {', '.join(map(str, shape))}]")
        if not (memory.shape[0] == normalizer.shape[0] == maximum.shape[0]):
            raise KernelError("matrix_memory_scan: the three states must have the same slots")
        if not cap > 0:
            raise KernelError("matrix_memory_scan: the gates' cap must be positive")
        n_seq = self._geometry("matrix_memory_scan", m, slot_ids, cu_rows)
        y = torch.empty((m, heads * dv), dtype=torch.float32, device=self.device)
        chunk, n_chunks = self.scan_chunks(max_count) if chunk is None else (int(chunk), -(-int(max_count) // int(chunk)) if chunk else 0)
        ws = None
        if chunk:
            ws = torch.empty(self.lib.tp_matrix_memory_scan_workspace_floats(n_seq, n_chunks, heads, dk, dv), dtype=torch.float32, device=self.device)
        self._call(self.lib, "tp_matrix_memory_scan", q.data_ptr(), qs, k.data_ptr(), ks, v.data_ptr(), vs, _code(q.dtype), gates.data_ptr(),
                   float(cap), float(q_scale), memory.data_ptr(), normalizer.data_ptr(), maximum.data_ptr(), slot_ids.data_ptr(),
                   cu_rows.data_ptr(), y.data_ptr(), n_seq, heads, dk, dv, chunk, n_chunks, ws.data_ptr() if ws is not None else None,
                   self._stream())
        return y

    def pair_norm_mean(self, a, b, gain_a, gain_b, eps):
        """float32 [M, D]: 0.5 (a / rms(a) * gain_a + b / rms(b) * gain_b), each row over its own root mean square."""
        self._dev(a, b, gain_a, gain_b)
        if a.dim() != 2 or a.shape != b.shape or a.dtype != b.dtype or not a.is_contiguous() or not b.is_contiguous():
            raise KernelError("pair_norm_mean: two contiguous matrices of one shape and dtype")
        m, d = a.shape
        for g in (gain_a, gain_b):
            if g.dtype != torch.float32 or g.numel() != d or not g.is_contiguous():
                raise KernelError(f"pair_norm_mean: gains must be contiguous float32 [{d}]")
        out = torch.empty((m, d), dtype=torch.float32, device=self.device)
        self._call(self.lib, "tp_pair_norm_mean", a.data_ptr(), b.data_ptr(), _code(a.dtype), gain_a.data_ptr(), gain_b.data_ptr(), float(eps),
                   out.data_ptr(), m, d, self._stream())
        return out

    def mul_sigmoid(self, x, g):
        """x *= sigmoid(g), in place; both [M, C] of one dtype, possibly views of wider rows."""
        self._dev(x, g)
        xs, gs = self._rows(x, "mul_sigmoid rows"), self._rows(g, "mul_sigmoid gates")
        if x.shape != g.shape or x.dtype != g.dtype:
            raise KernelError("mul_sigmoid: rows and gates of one shape and dtype")
        self._call(self.lib, "tp_mul_sigmoid", x.data_ptr(), xs, g.data_ptr(), gs, _code(x.dtype), x.shape[0], x.shape[1], self._stream())
        return x

    def mul_sigmoid_heads(self, x, g, heads):
        """x[r, h, :] *= sigmoid(g[r, h]), in place: x [M, heads * per] (a view of wider rows may do), g [M, heads]."""
        self._dev(x, g)
        xs, gs = self._rows(x, "mul_sigmoid_heads rows"), self._rows(g, "mul_sigmoid_heads gates")
        if g.shape != (x.shape[0], heads) or x.shape[1] % heads:
            raise KernelError(f"mul_sigmoid_heads: rows {tuple(x.shape)} and gates {tuple(g.shape)} do not fit {heads} heads")
        self._call(self.lib, "tp_mul_sigmoid_heads", x.data_ptr(), xs, _code(x.dtype), g.data_ptr(), gs, _code(g.dtype), x.shape[0], heads,
                   x.shape[1] // heads, self._stream())
        return x

    def bias_act(self, rows, bias, activation, out_dtype, pad=0):
        """act(rows + bias) in float32, rounded once to out_dtype: rows [M, N] float32 or bfloat16, bias float32 [N] or None;
        activation: one of BIAS_ACTIVATIONS.  pad: the output has that many more columns, a one and then zeros (the product
        that follows then carries its own bias as a column of its matrix)."""
        if activation not in BIAS_ACTIVATIONS:
            raise KernelError(f"bias_act: activation '{activation}' has no kernel ({', '.join(str(a) for a in BIAS_ACTIVATIONS)})")
        self._dev(rows, bias)
        if rows.dim() != 2 or not rows.is_contiguous():
            raise KernelError("bias_act: rows must be a contiguous matrix")
        m, n = rows.shape
        if bias is not None and (bias.dtype != torch.float32 or bias.numel() != n or not bias.is_contiguous()):
            raise KernelError(f"bias_act: the bias must be contiguous float32 [{n}]")
        out = torch.empty((m, n + pad), dtype=out_dtype, device=self.device)
        self._call(self.lib, "tp_bias_act", rows.data_ptr(), _code(rows.dtype), bias.data_ptr() if bias is not None else None, out.data_ptr(),
                   _code(out_dtype), m, n, int(pad), BIAS_ACTIVATIONS[activation], self._stream())
        return out

    MAX_SLICED_WIDTH = 8192        # widest row `add_rms_norm` takes in K slices

    def rows(self, rows, dtype):
        """A tensor of `dtype` from what `linear` returned: K slices are added in slice order."""
        if not isinstance(rows, SplitRows):
            return rows
        sl = rows.slices
        self._dev(sl)
        if sl.dtype != torch.float32 or sl.dim() != 3 or not sl.is_contiguous():
            raise KernelError("rows: K slices must be contiguous float32 [slices, rows, columns]")
        out = torch.empty(sl.shape[1:], dtype=dtype, device=self.device)
        self._call(self.lib, "tp_sum_slices", sl.data_ptr(), sl.shape[0], sl.stride(0), out.data_ptr(), _code(dtype),
                   out.numel(), self._stream())
        return out

    def gather_rows(self, x, rows):
        self._dev(x, rows)
        if x.dtype != torch.float32 or not x.is_contiguous() or x.dim() != 2:
            raise KernelError("gather_rows: expected a contiguous float32 matrix")
        if rows.dtype != torch.int32 or not rows.is_contiguous():
            raise KernelError("gather_rows: row indices must be contiguous int32")
        out = torch.empty((rows.numel(), x.shape[1]), dtype=torch.float32, device=self.device)
        self._call(self.lib, "tp_gather_rows", x.data_ptr(), rows.data_ptr(), out.data_ptr(), rows.numel(),
                   x.shape[1], x.shape[0], self._stream())
        return out

    def rope_kv_write(self, q, k, v, H, KV, hd, inv_freq, rotary_dim, row_seq, row_pos, new_len, table,
                      k_pool, v_pool, rows_cap, pairing="halves", write=True):
        """Rotate q and k in place and write k, v into the cache.  write=False: rotate only (a step whose attention
        reads the cache as earlier steps left it caches its rows afterwards, with `kv_write`).
        pairing: one of ROPE_PAIRINGS, which elements of a head turn together."""
        if pairing not in ROPE_PAIRINGS:
            raise KernelError(f"rope_kv_write: pairing '{pairing}' has no kernel ({', '.join(ROPE_PAIRINGS)})")
        self._dev(q, k, v, inv_freq, row_seq, row_pos, new_len, table, k_pool, v_pool)
        m = q.shape[0]
        qs = self._rows(q, "rope_kv_write q")
        if q.shape[1] != H * hd:
            raise KernelError(f"rope_kv_write: q has {q.shape[1]} columns, {H} heads of {hd} need {H * hd}")
        if rotary_dim:
            if inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rotary_dim // 2:
                raise KernelError(f"rope_kv_write: a rotation over {rotary_dim} needs float32 inv_freq [{rotary_dim // 2}]")
        for t, n in ((row_seq, m), (row_pos, m)):
            if t.dtype != torch.int32 or t.numel() != n:
                raise KernelError("rope_kv_write: row_seq and row_pos must be int32, one entry per row")
        kp = vp = ks = vs = 0
        page = table_w = 1
        write = write and k is not None
        if k is not None:
            ks, vs = self._rows(k, "rope_kv_write k"), self._rows(v, "rope_kv_write v")
            if k.shape != (m, KV * hd) or v.shape != (m, KV * hd) or k.dtype != q.dtype or v.dtype != q.dtype:
                raise KernelError("rope_kv_write: k and v must be [rows, kv_heads * head_dim] of q's dtype")
            kp, vp = k.data_ptr(), v.data_ptr()
        if write:
            self._check_pools("rope_kv_write", q.dtype, new_len.numel(), KV, hd, new_len, table, k_pool, v_pool)
            page, table_w = k_pool.shape[2], table.shape[1]
        self._call(self.lib, "tp_rope_kv_write", q.data_ptr(), qs, kp or None, ks, vp or None, vs, _code(q.dtype), m, H, KV, hd,
                   inv_freq.data_ptr() if rotary_dim else None, rotary_dim, row_seq.data_ptr(), row_pos.data_ptr(),
                   new_len.data_ptr(), table.data_ptr() if write else None, table_w,
                   k_pool.data_ptr() if write else None, v_pool.data_ptr() if write else None,
                   page, rows_cap if write else 0, ROPE_PAIRINGS[pairing], self._stream())

    def kv_write(self, k, v, KV, hd, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap):
        """The step's keys (rotated already) and values into the cache: what `rope_kv_write(write=False)` left undone."""
        self._dev(k, v, row_seq, row_pos, new_len, table, k_pool, v_pool)
        m = k.shape[0]
        ks, vs = self._rows(k, "kv_write k"), self._rows(v, "kv_write v")
        if k.shape != (m, KV * hd) or v.shape != (m, KV * hd) or k.dtype != v.dtype:
            raise KernelError("kv_write: k and v must be [rows, kv_heads * head_dim] of one dtype")
        for t in (row_seq, row_pos):
            if t.dtype != torch.int32 or t.numel() != m:
                raise KernelError("kv_write: row_seq and row_pos must be int32, one entry per row")
        self._check_pools("kv_write", k.dtype, new_len.numel(), KV, hd, new_len, table, k_pool, v_pool)
        self._call(self.lib, "tp_kv_write", k.data_ptr(), ks, v.data_ptr(), vs, _code(k.dtype), m, KV, hd, row_seq.data_ptr(),
                   row_pos.data_ptr(), new_len.data_ptr(), table.data_ptr(), table.shape[1], k_pool.data_ptr(),
                   v_pool.data_ptr(), k_pool.shape[2], rows_cap, self._stream())

    # ---- attention over a window and pooled blocks ------------------------------------------------------
    def qkv_prepare(self, x, bias, H, KV, row, dim, inv_freq, rotary_dim, row_pos, unit_eps, out_dtype, pairing="halves"):
        """A step's projected rows [M, (H + 2 KV) row] (or [M, H row] with KV = 0), float32 or out_dtype: bias, rotation of
        every query and key head's first rotary_dim elements by its row's position, then (unit_eps not None) every
        query and key head over the root mean square of its `dim` elements; everything in float32, rounded once.
        Returns q [M, H row], k, v [M, KV row] (None with KV = 0) of out_dtype."""
        self._dev(x, bias, inv_freq, row_pos)
        xs = self._rows(x, "qkv_prepare rows")
        m = x.shape[0]
        if x.shape[1] != (H + 2 * KV) * row:
            raise KernelError(f"qkv_prepare: rows of {x.shape[1]} columns, {H} + 2 x {KV} heads of {row} need {(H + 2 * KV) * row}")
        if bias is not None and (bias.dtype != torch.float32 or bias.numel() != x.shape[1] or not bias.is_contiguous()):
            raise KernelError(f"qkv_prepare: the bias must be contiguous float32 [{x.shape[1]}]")
        if rotary_dim and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rotary_dim // 2):
            raise KernelError(f"qkv_prepare: a rotation over {rotary_dim} needs float32 inv_freq [{rotary_dim // 2}]")
        if row_pos.dtype != torch.int32 or row_pos.numel() != m:
            raise KernelError("qkv_prepare: row_pos must be int32, one entry per row")
        if pairing not in ROPE_PAIRINGS:
            raise KernelError(f"qkv_prepare: pairing '{pairing}' has no kernel")
        q = torch.empty((m, H * row), dtype=out_dtype, device=self.device)
        k = torch.empty((m, KV * row), dtype=out_dtype, device=self.device) if KV else None
        v = torch.empty((m, KV * row), dtype=out_dtype, device=self.device) if KV else None
        self._call(self.lib, "tp_qkv_prepare", x.data_ptr(), xs, _code(x.dtype), bias.data_ptr() if bias is not None else None, m, H, KV, row, dim,
                   inv_freq.data_ptr() if rotary_dim else None, rotary_dim, ROPE_PAIRINGS[pairing],
                   -1.0 if unit_eps is None else float(unit_eps), row_pos.data_ptr(), q.data_ptr(),
                   k.data_ptr() if KV else None, v.data_ptr() if KV else None, _code(out_dtype), self._stream())
        return q, k, v

    def pool_write(self, k, v, KV, row, block, cu_rows, max_count, new_len, slot_ids, sums, table, k_blocks, v_blocks):
        """The mean key and value of every block of `block` positions that the step completes, into the pools
        [pages, KV, page, row] that keep one row per block (found through `table`); sums float32 [slots, 2, KV row]
        carries an unfinished block's sums from step to step."""
        self._dev(k, v, cu_rows, new_len, slot_ids, sums, table, k_blocks, v_blocks)
        ks, vs = self._rows(k, "pool_write k"), self._rows(v, "pool_write v")
        n = new_len.numel()
        if k.shape != v.shape or k.shape[1] != KV * row or k.dtype != v.dtype:
            raise KernelError("pool_write: k and v must be [rows, kv_heads * row] of one dtype")
        for t, cnt in ((cu_rows, n + 1), (new_len, n), (slot_ids, n)):
            if t.dtype != torch.int32 or t.numel() != cnt:
                raise KernelError("pool_write: cu_rows, new_len and slot_ids must be int32 of the step's geometry")
        if sums.dtype != torch.float32 or sums.dim() != 3 or tuple(sums.shape[1:]) != (2, KV * row) or not sums.is_contiguous():
            raise KernelError(f"pool_write: the sums must be contiguous float32 [slots, 2, {KV * row}]")
        for pool in (k_blocks, v_blocks):
            if pool.dim() != 4 or pool.shape[1] != KV or pool.shape[3] != row or pool.dtype != k.dtype or not pool.is_contiguous():
                raise KernelError(f"pool_write: a pool must be contiguous [pages, {KV}, page, {row}] of {k.dtype}")
        if table.dtype != torch.int32 or table.dim() != 2 or table.shape[0] != n or table.stride(1) != 1 or table.stride(0) != table.shape[1]:
            raise KernelError("pool_write: the page table must be contiguous int32 [sequences, pages]")
        self._call(self.lib, "tp_pool_write", k.data_ptr(), ks, v.data_ptr(), vs, _code(k.dtype), n, int(max_count), KV, row, int(block),
                   cu_rows.data_ptr(), new_len.data_ptr(), slot_ids.data_ptr(), sums.data_ptr(), table.data_ptr(), table.shape[1],
                   k_blocks.data_ptr(), v_blocks.data_ptr(), k_blocks.shape[2], self._stream())

    def attention_pooled(self, q, k, v, H, KV, hd, cu_rows, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap,
                         scale, softcap, window, blocks=None, all_values=False, max_count=None):
        """Attention of the step's queries over the positions their window still holds (those before the step read in
        place from the cache, the step's own rows from k and v) and, with blocks = (block size, page table, key pool,
        value pool), over one pooled key and value per block of positions that lies wholly before the window; one
        softmax over both.  Returns float32 [M, H, KV if all_values else 1, hd]: with all_values every query head's
        weights are applied to the values of every kv head (what a mix of the heads' weights needs).  max_count: the most
        rows a sequence brings (a host number; with it bf16 heads of a multiple of 32 elements up to 256 run on the
        matrix cores)."""
        self._dev(q, k, v, cu_rows, row_seq, row_pos, new_len, table, k_pool, v_pool)
        m = q.shape[0]
        qs, ks, vs = self._rows(q, "attention_pooled q"), self._rows(k, "attention_pooled k"), self._rows(v, "attention_pooled v")
        if q.shape[1] != H * hd or k.shape != (m, KV * hd) or v.shape != (m, KV * hd) or k.dtype != q.dtype or v.dtype != q.dtype:
            raise KernelError(f"attention_pooled: q [rows, {H * hd}], k and v [rows, {KV * hd}] of one dtype, found {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
        n = new_len.numel()
        for t, cnt in ((cu_rows, n + 1), (row_seq, m), (row_pos, m)):
            if t.dtype != torch.int32 or t.numel() != cnt:
                raise KernelError("attention_pooled: cu_rows, row_seq and row_pos must be int32 of the step's geometry")
        self._check_pools("attention_pooled", q.dtype, n, KV, hd, new_len, table, k_pool, v_pool)
        page = k_pool.shape[2]
        if blocks is not None:
            block, btable, kb, vb = blocks
            self._dev(btable, kb, vb)
            self._check_pools("attention_pooled (blocks)", q.dtype, n, KV, hd, new_len, btable, kb, vb)
            if kb.shape[2] != page or not window:
                raise KernelError("attention_pooled: the blocks' pools have the cache's page size, and blocks need a window")
        self_out = torch.empty((m, H, KV if all_values else 1, hd), dtype=torch.float32, device=self.device)
        pieces = all(t is None or (t.data_ptr() % 16 == 0) for t in (q, k, v)) and qs % 8 == 0 and ks % 8 == 0 and vs % 8 == 0
        if max_count and not self.force_plain_attention and q.dtype == torch.bfloat16 and hd % 32 == 0 and hd <= 256 and pieces \
                and page & (page - 1) == 0:
            self._call(self.attn_lib(hd), "tp_attn_pooled_tile", q.data_ptr(), qs, k.data_ptr(), ks, v.data_ptr(), vs, n, int(max_count), H, KV,
                       cu_rows.data_ptr(), new_len.data_ptr(), table.data_ptr(), table.shape[1], k_pool.data_ptr(), v_pool.data_ptr(), page,
                       rows_cap or 0, btable.data_ptr() if blocks else None, btable.shape[1] if blocks else 0,
                       kb.data_ptr() if blocks else None, vb.data_ptr() if blocks else None, int(block) if blocks else 0,
                       float(scale), float(softcap or 0.0), int(window or 0), 1 if all_values else 0, self_out.data_ptr(), self._stream())
            return self_out
        self._call(self.lib, "tp_attn_pooled", q.data_ptr(), qs, k.data_ptr(), ks, v.data_ptr(), vs, _code(q.dtype), m, H, KV, hd,
                   cu_rows.data_ptr(), row_seq.data_ptr(), row_pos.data_ptr(), new_len.data_ptr(), table.data_ptr(), table.shape[1],
                   k_pool.data_ptr(), v_pool.data_ptr(), page, rows_cap or 0,
                   btable.data_ptr() if blocks else None, btable.shape[1] if blocks else 0, kb.data_ptr() if blocks else None,
                   vb.data_ptr() if blocks else None, int(block) if blocks else 0,
                   float(scale), float(softcap or 0.0), int(window or 0), 1 if all_values else 0, self_out.data_ptr(), self._stream())
        return self_out

    def talk_mix(self, a, talk, out_dtype):
        """out[r, h] = sum_g talk[h, g] a[r, g, kv(h)]: a float32 [M, H, KV, hd] as `attention_pooled(all_values=True)`
        gives it, talk float32 [H, H]; returns [M, H * hd] of out_dtype."""
        self._dev(a, talk)
        if a.dtype != torch.float32 or a.dim() != 4 or not a.is_contiguous():
            raise KernelError("talk_mix: the heads' outputs must be contiguous float32 [rows, heads, kv heads, head_dim]")
        m, H, KV, hd = a.shape
        if talk.dtype != torch.float32 or tuple(talk.shape) != (H, H) or not talk.is_contiguous():
            raise KernelError(f"talk_mix: the mixing matrix must be contiguous float32 [{H}, {H}]")
        out = torch.empty((m, H * hd), dtype=out_dtype, device=self.device)
        self._call(self.lib, "tp_talk_mix", a.data_ptr(), talk.data_ptr(), out.data_ptr(), _code(out_dtype), m, H, KV, hd, self._stream())
        return out

    # ---- matrix products -----------------------------------------------------------------------------
    def _linear(self, x, w, out_dtype, epilogue, cap, units, defer=False, act=0, out=None, limit=float("inf"), shift=0.0):
        self._dev(x, w)
        if x.dim() != 2 or w.dim() != 2 or not x.is_contiguous() or not w.is_contiguous():
            raise KernelError("linear: rows and matrix must be contiguous 2-D tensors")
        if x.dtype != w.dtype:
            raise KernelError(f"linear: rows are {x.dtype}, the matrix is {w.dtype}")
        m, k = x.shape
        n = w.shape[0]
        if w.shape[1] != k:
            raise KernelError(f"linear: rows have {k} columns, the matrix {w.shape[1]}")
        cols = units if epilogue == EPI_GATED else n
        algo = self.force_linear
        nbytes = self.lib.tp_linear_workspace_bytes(_code(x.dtype), _code(out_dtype), m, n, k, epilogue, units,
                                                    1 if defer else 0, algo)
        if defer and epilogue == EPI_NONE and nbytes and nbytes % (m * n * 4) == 0 and nbytes // (m * n * 4) > 1:
            slices = torch.empty((nbytes // (m * n * 4), m, n), dtype=torch.float32, device=self.device)
            self._call(self.lib, "tp_linear", x.data_ptr(), w.data_ptr(), None, _code(x.dtype), _code(out_dtype),
                       m, n, k, epilogue, float(cap), units, act, float(limit), float(shift), slices.data_ptr(), nbytes, 1, algo, self._stream())
            return SplitRows(slices)
        if out is None:
            out = torch.empty((m, cols), dtype=out_dtype, device=self.device)
        elif out.dtype != out_dtype or tuple(out.shape) != (m, cols) or not out.is_contiguous():
            raise KernelError(f"linear: the output must be contiguous {out_dtype} {(m, cols)}")
        self._dev(out)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device) if nbytes else None
        self._call(self.lib, "tp_linear", x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(x.dtype), _code(out_dtype),
                   m, n, k, epilogue, float(cap), units, act, float(limit), float(shift),
                   ws.data_ptr() if ws is not None else None, nbytes, 0, algo, self._stream())
        return out

    def linear(self, x, w, out_dtype, softcap=None, defer=False, bias=None, out=None):
        """x @ w^T (+ bias).  defer: the caller hands the result to `add_rms_norm` (or through `rows()`), so a product
        computed in K slices may come back as SplitRows.  bias: float32 [rows of w], added by a kernel of its own
        (the products have no bias operand), so a product with a bias is never left in slices.  out: a contiguous
        tensor to fill (a plain product only)."""
        if out is not None:
            if bias is not None or softcap or defer:
                raise KernelError("linear: an output to fill goes with a plain product only")
            return self._linear(x, w, out_dtype, EPI_NONE, 0.0, 0, out=out)
        if bias is not None:
            if softcap:
                raise KernelError("linear: a bias and a cap together have no kernel")
            y = self._linear(x, w, out_dtype, EPI_NONE, 0.0, 0)
            self._dev(bias)
            if bias.dtype != torch.float32 or bias.numel() != y.shape[1] or not bias.is_contiguous():
                raise KernelError(f"linear: the bias must be contiguous float32 [{y.shape[1]}]")
            self._call(self.lib, "tp_add_bias", y.data_ptr(), _code(y.dtype), bias.data_ptr(), y.shape[0], y.shape[1], self._stream())
            return y
        if softcap:
            return self._linear(x, w, out_dtype, EPI_SOFTCAP, softcap, 0)
        return self._linear(x, w, out_dtype, EPI_NONE, 0.0, 0, defer=defer)

    def gated_linear(self, x, w_packed, inter, activation, out_dtype, limit=None, up_shift=0.0):
        """act(g) * (u + up_shift) with g = x @ gate^T and u = x @ up^T over the packed matrix of `pack_gate_up`;
        activation: one of GATE_ACTIVATIONS.  limit: g is cut at it from above and u from both sides, before the
        activation (None: neither is cut)."""
        if activation not in GATE_ACTIVATIONS:
            raise KernelError(f"gated_linear: activation '{activation}' has no kernel ({', '.join(GATE_ACTIVATIONS)})")
        if limit is not None and not limit > 0:
            raise KernelError(f"gated_linear: the sums' limit must be positive, found {limit}")
        return self._linear(x, w_packed, out_dtype, EPI_GATED, 0.0, inter, act=GATE_ACTIVATIONS[activation],
                            limit=float("inf") if limit is None else limit, shift=up_shift)

    # ---- attention -------------------------------------------------------------------------------------
    DECODE_GROUP = 16              # query heads per kv head the matrix-core decode kernel takes

    def _fast_attention(self, dtype, H, KV, hd, decode=True):
        """Whether the matrix-core kernels take this geometry; the kernel of many queries takes any number of query
        heads per kv head, the decode kernel up to DECODE_GROUP."""
        return not self.force_plain_attention and dtype == torch.bfloat16 and hd % 16 == 0 and hd <= 256 and \
            (not decode or H // KV <= self.DECODE_GROUP)

    def attention_prefill(self, q, k, v, H, KV, hd, cu_rows, max_count, scale, softcap, window, out_dtype,
                          row_seq=None, row_pos=None, cached=None, shape=0, wide_weights=False, chunk=0, head_scale=None, sink=None):
        """Causal attention of the step's queries over the step's own rows of keys and values and, with
        `cached` = (new_len, table, k_pool, v_pool, rows_cap), over the positions before them, read in place from the
        cache as earlier steps left it (the step's own rows are not looked for there).  Without `cached` every sequence
        starts at position 0; with it row_pos holds absolute positions, sequence s's first row standing at
        new_len[s] - its count.  shape: the matrix-core kernel's block shape (0: chosen by the size of the step).
        wide_weights: the matrix-core kernel multiplies the values by softmax weights of 16 bits of mantissa (two bf16
        terms) instead of 8; the plain kernel's weights are float32 in any case.
        chunk C: a query at position p sees keys from floor(p / C) C on only.  head_scale, sink: float32 [H], a factor on
        every head's scores and a score without key or value in every head's softmax."""
        self._dev(q, k, v, cu_rows, head_scale, sink)
        self._head_vectors("attention_prefill", H, chunk, head_scale, sink)
        m = q.shape[0]
        qs, ks, vs = self._rows(q, "attention q"), self._rows(k, "attention k"), self._rows(v, "attention v")
        if q.shape[1] != H * hd or k.shape != (m, KV * hd) or v.shape != (m, KV * hd):
            raise KernelError("attention_prefill: q must be [rows, heads * head_dim], k and v [rows, kv_heads * head_dim]")
        if not (q.dtype == k.dtype == v.dtype == out_dtype):
            raise KernelError("attention_prefill: q, k, v and the output share one dtype")
        n_seq = cu_rows.numel() - 1
        new_len = table = k_pool = v_pool = None
        page, rows_cap, table_w = 1, 0, 1
        if cached is not None:
            new_len, table, k_pool, v_pool, rows_cap = cached
            self._dev(new_len, table, k_pool, v_pool)
            self._check_pools("attention_prefill", q.dtype, n_seq, KV, hd, new_len, table, k_pool, v_pool)
            page, table_w, rows_cap = k_pool.shape[2], table.shape[1], rows_cap or 0
        ptr = lambda t: t.data_ptr() if t is not None else None
        out = torch.empty((m, H * hd), dtype=out_dtype, device=self.device)
        if self._fast_attention(q.dtype, H, KV, hd, decode=False) and (cached is None or (page >= 16 and page & (page - 1) == 0)):
            lib = self.attn_lib(hd, wide=wide_weights)
            self._call(lib, "tp_attn_prefill", q.data_ptr(), qs, k.data_ptr(), ks, v.data_ptr(), vs,
                       m, H, KV, cu_rows.data_ptr(), n_seq, int(max_count), ptr(new_len), ptr(table), table_w,
                       ptr(k_pool), ptr(v_pool), page, rows_cap,
                       float(scale), float(softcap), int(window), int(chunk), ptr(head_scale), ptr(sink), out.data_ptr(), int(shape),
                       self._stream())
            return out
        if cached is not None and (row_seq is None or row_pos is None):
            raise KernelError("attention_prefill: cached positions need every row's sequence and position")
        if row_seq is None:
            counts = (cu_rows[1:] - cu_rows[:-1]).long()
            row_seq = torch.repeat_interleave(torch.arange(n_seq, device=self.device, dtype=torch.int32), counts)
            row_pos = (torch.arange(m, device=self.device, dtype=torch.int32) - cu_rows[:-1][row_seq.long()]).to(torch.int32)
        self._call(self.lib, "tp_attn_simple_prefill", q.data_ptr(), qs, k.data_ptr(), ks, v.data_ptr(), vs, _code(q.dtype),
                   m, H, KV, hd, cu_rows.data_ptr(), row_seq.data_ptr(), row_pos.data_ptr(), ptr(new_len), ptr(table), table_w,
                   ptr(k_pool), ptr(v_pool), page, rows_cap, float(scale), float(softcap),
                   int(window), int(chunk), ptr(head_scale), ptr(sink), out.data_ptr(), self._stream())
        return out

    def _head_vectors(self, what, H, chunk, head_scale, sink):
        """Checks a chunk size and the vectors of one number per head; whether any of them is asked for."""
        if chunk < 0:
            raise KernelError(f"{what}: chunks of {chunk} positions")
        for t, name in ((head_scale, "head_scale"), (sink, "sink")):
            if t is not None and (t.dtype != torch.float32 or t.numel() != H or not t.is_contiguous()):
                raise KernelError(f"{what}: {name} must be contiguous float32 [{H}]")
        return bool(chunk) or head_scale is not None or sink is not None

    @staticmethod
    def decode_splits(n, KV, hd, keys):
        """Slices of the keys per (sequence, kv head) in a decode step: enough blocks to keep every CU streaming
        (about 1536; 768 when the pairs alone are many), each with at least one round of 64 keys.  Measured on
        MI355X from 1 to 64 sequences and 500 to 8000 keys this is within 7 % of the best count everywhere; more
        slices cost little (a second launch adds them), fewer cost up to half."""
        pairs = n * KV
        want = -(-(1536 if pairs < 192 else 768) // pairs)
        return max(1, min(want, -(-keys // 64), 128))

    def _check_pools(self, what, dtype, n, KV, hd, new_len, table, k_pool, v_pool):
        if new_len.numel() != n or new_len.dtype != torch.int32:
            raise KernelError(f"{what}: one int32 length per sequence")
        if k_pool.dtype != dtype or k_pool.dim() != 4 or tuple(k_pool.shape[1:]) != (KV, k_pool.shape[2], hd) \
                or v_pool.shape != k_pool.shape or not k_pool.is_contiguous() or not v_pool.is_contiguous():
            raise KernelError(f"{what}: cache pools must be contiguous [pages, kv_heads, page, head_dim] of {dtype}")
        if table.dtype != torch.int32 or table.dim() != 2 or table.shape[0] != n or not table.is_contiguous():
            raise KernelError(f"{what}: the page table must be contiguous int32 [sequences, pages]")

    def attention_decode(self, q, H, KV, hd, new_len, table, k_pool, v_pool, rows_cap, scale, softcap, window,
                         out_dtype, max_keys=None, splits=None, head_groups=None, chunk=0, head_scale=None, sink=None):
        """head_groups: cut the query heads into that many groups (a multiple of KV), each read the pool head
        `group % KV` by a block of its own: for caches whose one kv head serves many heads, where one block would
        otherwise form all their weighted sums.  The plain kernel takes any grouping as it is.
        chunk, head_scale, sink: as in `attention_prefill`."""
        self._dev(q, new_len, table, k_pool, v_pool, head_scale, sink)
        per_head = self._head_vectors("attention_decode", H, chunk, head_scale, sink)
        n = q.shape[0]
        qs = self._rows(q, "attention q")
        if q.shape[1] != H * hd:
            raise KernelError("attention_decode: q must be [sequences, heads * head_dim]")
        self._check_pools("attention_decode", q.dtype, n, KV, hd, new_len, table, k_pool, v_pool)
        out = torch.empty((n, H * hd), dtype=out_dtype, device=self.device)
        page = k_pool.shape[2]
        groups = int(head_groups) if head_groups else KV
        if groups % KV or H % groups:
            raise KernelError(f"attention_decode: {H} heads in {groups} groups on {KV} kv heads")
        if self._fast_attention(q.dtype, H, groups, hd) and page >= 16 and page & (page - 1) == 0 and not (per_head and groups != KV):
            lib = self.attn_lib(hd)
            keys = int(max_keys) if max_keys else k_pool.shape[0] * k_pool.shape[2]
            nsplit = int(splits) if splits else self.decode_splits(n, groups, hd, keys)
            floats = lib.tp_attn_decode_workspace_floats(n, H, nsplit)
            ws = torch.empty(floats, dtype=torch.float32, device=self.device) if floats else None
            if groups != KV:
                self._call(lib, "tp_attn_decode_shared", q.data_ptr(), qs, n, H, groups, KV, new_len.data_ptr(), table.data_ptr(),
                           table.shape[1], k_pool.data_ptr(), v_pool.data_ptr(), k_pool.shape[2], rows_cap, float(scale),
                           float(softcap), int(window), out.data_ptr(), ws.data_ptr() if ws is not None else None, nsplit,
                           self._stream())
                return out
            self._call(lib, "tp_attn_decode", q.data_ptr(), qs, n, H, KV, new_len.data_ptr(), table.data_ptr(),
                       table.shape[1], k_pool.data_ptr(), v_pool.data_ptr(), k_pool.shape[2], rows_cap, float(scale),
                       float(softcap), int(window), int(chunk), head_scale.data_ptr() if head_scale is not None else None,
                       sink.data_ptr() if sink is not None else None, out.data_ptr(), ws.data_ptr() if ws is not None else None, nsplit,
                       self._stream())
            return out
        self._call(self.lib, "tp_attn_simple_decode", q.data_ptr(), qs, _code(q.dtype), n, H, KV, hd, new_len.data_ptr(),
                   table.data_ptr(), table.shape[1], k_pool.data_ptr(), v_pool.data_ptr(), k_pool.shape[2], rows_cap,
                   float(scale), float(softcap), int(window), int(chunk), head_scale.data_ptr() if head_scale is not None else None,
                   sink.data_ptr() if sink is not None else None, out.data_ptr(), self._stream())
        return out

    def fuses_decode_step(self, dtype, H, KV, hd, k_pool):
        """Whether `attention_decode_step` exists for this geometry: the caller then skips `rope_kv_write`."""
        page = k_pool.shape[2]
        return self._fast_attention(dtype, H, KV, hd) and page >= 16 and page & (page - 1) == 0

    def attention_decode_step(self, qkv, H, KV, hd, inv_freq, rotary_dim, new_len, table, k_pool, v_pool, rows_cap,
                              scale, softcap, window, out_dtype, max_keys=None, write_kv=True, splits=None):
        """A decode step's rotation, cache write and attention in one launch.  qkv: each sequence's projections
        [queries | keys | values] (queries only when write_kv is false), a bf16 tensor or what
        `linear(..., defer=True)` returned; sequence i's token has position new_len[i] - 1."""
        split = isinstance(qkv, SplitRows)
        rows = qkv.slices if split else qkv
        self._dev(rows, inv_freq, new_len, table, k_pool, v_pool)
        n, width = rows.shape[-2], rows.shape[-1]
        if width != (H + (2 * KV if write_kv else 0)) * hd:
            raise KernelError(f"attention_decode_step: rows of {width} columns, {H} heads and {KV} kv heads of {hd} need "
                              f"{(H + (2 * KV if write_kv else 0)) * hd}")
        if out_dtype != torch.bfloat16 or not self.fuses_decode_step(out_dtype, H, KV, hd, k_pool):
            raise KernelError("attention_decode_step: no fused kernel for this geometry (see fuses_decode_step)")
        if split:
            if rows.dtype != torch.float32 or not rows.is_contiguous():
                raise KernelError("attention_decode_step: K slices must be contiguous float32")
            n_slices, slice_stride, row_stride = rows.shape[0], rows.shape[1] * rows.shape[2], rows.shape[2]
        else:
            if rows.dim() != 2 or rows.dtype not in (torch.bfloat16, torch.float32):
                raise KernelError("attention_decode_step: projections must be 2-D, bfloat16 or float32")
            n_slices, slice_stride, row_stride = 1, 0, self._rows(rows, "attention_decode_step qkv")
        if rotary_dim and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rotary_dim // 2):
            raise KernelError(f"attention_decode_step: a rotation over {rotary_dim} needs float32 inv_freq [{rotary_dim // 2}]")
        self._check_pools("attention_decode_step", torch.bfloat16, n, KV, hd, new_len, table, k_pool, v_pool)
        lib = self.attn_lib(hd)
        keys = int(max_keys) if max_keys else k_pool.shape[0] * k_pool.shape[2]
        nsplit = int(splits) if splits else self.decode_splits(n, KV, hd, keys)
        floats = lib.tp_attn_decode_workspace_floats(n, H, nsplit)
        ws = torch.empty(floats, dtype=torch.float32, device=self.device) if floats else None
        out = torch.empty((n, H * hd), dtype=out_dtype, device=self.device)
        self._call(lib, "tp_attn_decode_fused", rows.data_ptr(), _code(rows.dtype), n_slices, slice_stride, row_stride,
                   inv_freq.data_ptr() if rotary_dim else None, int(rotary_dim), 1 if write_kv else 0,
                   n, H, KV, new_len.data_ptr(), table.data_ptr(), table.shape[1], k_pool.data_ptr(), v_pool.data_ptr(),
                   k_pool.shape[2], rows_cap, float(scale), float(softcap), int(window), out.data_ptr(),
                   ws.data_ptr() if ws is not None else None, nsplit, self._stream())
        return out

    # ---- token choice -------------------------------------------------------------------------------------
    def argmax(self, logits, out=None):
        """Smallest index of the largest value per row, int32; into `out` if given."""
        self._dev(logits)
        if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
            raise KernelError("argmax: logits must be contiguous float32 [rows, vocab]")
        if out is None:
            out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
        else:
            self._dev(out)
            if out.dtype != torch.int32 or out.shape != (logits.shape[0],) or not out.is_contiguous():
                raise KernelError("argmax: the output must be contiguous int32 [rows]")
        nbytes = self.lib.tp_argmax_workspace_bytes(logits.shape[0], logits.shape[1])
        ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device) if nbytes else None
        self._call(self.lib, "tp_argmax", logits.data_ptr(), logits.shape[0], logits.shape[1], out.data_ptr(),
                   ws.data_ptr() if ws is not None else None, self._stream())
        return out

    def apply_repetition_penalty(self, logits, recent, penalty):
        """In place.  recent: int32 [rows, R], -1 where empty."""
        self._dev(logits, recent)
        if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
            raise KernelError("repetition_penalty: logits must be contiguous float32 [rows, vocab]")
        if recent.dtype != torch.int32 or recent.dim() != 2 or recent.shape[0] != logits.shape[0] or not recent.is_contiguous():
            raise KernelError("repetition_penalty: recent tokens must be contiguous int32 [rows, R]")
        self._call(self.lib, "tp_repetition_penalty", logits.data_ptr(), logits.shape[0], logits.shape[1],
                   recent.data_ptr(), recent.shape[1], float(penalty), self._stream())

    def recent_push(self, tokens, recent, cursor):
        """Row i's token goes into row i of the ring `recent` (int32 [rows, R]) at cursor[i], which moves on by one."""
        self._dev(tokens, recent, cursor)
        n = tokens.numel()
        if tokens.dtype != torch.int32 or not tokens.is_contiguous() or cursor.dtype != torch.int32 or cursor.numel() != n \
                or not cursor.is_contiguous():
            raise KernelError("recent_push: tokens and cursors must be contiguous int32 of one length")
        if recent.dtype != torch.int32 or recent.dim() != 2 or recent.shape[0] != n or not recent.is_contiguous():
            raise KernelError("recent_push: the ring must be contiguous int32 [rows, R]")
        self._call(self.lib, "tp_recent_push", tokens.data_ptr(), recent.data_ptr(), cursor.data_ptr(), n, recent.shape[1],
                   self._stream())

    def sample(self, logits, temperature, top_k, top_p, uniforms, out=None):
        self._dev(logits, uniforms)
        if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
            raise KernelError("sample: logits must be contiguous float32 [rows, vocab]")
        if uniforms.dtype != torch.float32 or uniforms.numel() != logits.shape[0] or not uniforms.is_contiguous():
            raise KernelError("sample: one float32 uniform number per row")
        if out is None:
            out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
        else:
            self._dev(out)
            if out.dtype != torch.int32 or out.shape != (logits.shape[0],) or not out.is_contiguous():
                raise KernelError("sample: the output must be contiguous int32 [rows]")
        # the candidate filter's workspace starts zeroed and every call leaves it zeroed again: kept between calls
        shape = tuple(logits.shape)
        if shape not in self._sample_ws:
            nbytes = self.lib.tp_sample_workspace_bytes(shape[0], shape[1])
            self._sample_ws[shape] = torch.zeros(nbytes, dtype=torch.uint8, device=self.device) if nbytes else None
        ws = self._sample_ws[shape]
        self._call(self.lib, "tp_sample", logits.data_ptr(), shape[0], shape[1], float(temperature),
                   int(top_k), float(top_p), uniforms.data_ptr(), out.data_ptr(), ws.data_ptr() if ws is not None else None,
                   self._stream())
        return out

    # ---- probes: what the GPU gives a kernel at best -----------------------------------------------------------
    def _best_ms(self, launch, repeats):
        launch()
        torch.cuda.synchronize(self.device)
        best = float("inf")
        for _ in range(repeats):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            launch()
            b.record()
            b.synchronize()
            best = min(best, a.elapsed_time(b))
        return best

    def measured_ceilings(self, stream_bytes=4 << 30, repeats=5):
        """(GB/s of a streaming read of device memory, flop/s of a loop of bf16 matrix instructions), each the best
        of a few runs of a probe kernel."""
        cus = torch.cuda.get_device_properties(self.device).multi_processor_count
        sink = torch.zeros(4, dtype=torch.float32, device=self.device)
        buf = torch.empty(stream_bytes, dtype=torch.uint8, device=self.device).fill_(1)
        ms = self._best_ms(lambda: self._call(self.lib, "tp_probe_stream", buf.data_ptr(), stream_bytes, sink.data_ptr(),
                                              cus * 32, self._stream()), repeats)
        gbs = stream_bytes / (ms * 1e-3) / 1e9
        del buf
        best, mhz = 0.0, 0.0
        clocks = torch.zeros(2, dtype=torch.int64, device=self.device)
        for kind in (0, 1):                            # the 16x16x32 and the 32x32x16 form of the instruction
            iters, blocks = 20000, cus * 8
            ms = self._best_ms(lambda: self._call(self.lib, "tp_probe_mfma", kind, iters, blocks, sink.data_ptr(),
                                                  clocks.data_ptr(), self._stream()), repeats)
            flops = blocks * 4 * iters * 131072.0 / (ms * 1e-3)
            if flops > best:
                c = clocks.tolist()
                best, mhz = flops, (100.0 * c[0] / c[1] if c[1] else 0.0)
        self.matrix_clock_mhz = mhz                    # the shader clock while the matrix loop ran
        return gbs, best
