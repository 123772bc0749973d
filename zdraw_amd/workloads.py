"""Seeded synthetic inputs for the five benchmark configurations and the
device-side runner that pushes them through the fused entry point.

Layout contracts follow the reference: activations are token-major
`[segment][token][head][128]`; Klein sequences are text-first
(klein/zflux2.zig:99-102), Z-Image sequences are image-then-caption
(zimage/zunify.zig:31-34). Draw order is Q, K, V from one generator.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from . import hip, host

HEAD_DIM = 128
KLEIN_EPS = 1e-6    # klein/zflux2.zig:70
ZIMAGE_EPS = 1e-5   # zimage/zshape.zig:49 (norm_eps)
ZIMAGE_DIMS = (32, 48, 48)      # zimage/zshape.zig:46
ZIMAGE_LENS = (1536, 512, 512)  # zimage/zshape.zig:47
ZIMAGE_THETA = 256.0


@dataclass
class Workload:
    name: str
    kind: str            # "plain" | "klein" | "zimage"
    batch: int
    heads: int
    tokens: int
    q: np.ndarray        # fp32 draws [B][S][H][128]
    k: np.ndarray
    v: np.ndarray
    txt_len: int = 0
    grid: tuple = (0, 0)
    ref_grid: tuple = (0, 0)
    theta: float = 0.0
    text_lens: tuple | None = None     # ragged text lengths (one per segment) or None
    key_pad: np.ndarray | None = None  # u8 [B][S], 1 = key excluded
    rope_cos: np.ndarray | None = None
    rope_sin: np.ndarray | None = None
    pos: np.ndarray | None = None      # [S][3]
    rope_pairs: np.ndarray | None = None
    rope_bases: tuple = (0, 0, 0)
    extra: dict = field(default_factory=dict)

    @property
    def flops(self) -> float:
        """Algorithmic FLOPs: 4 * D * H * sum_b S_q * S_k(unmasked)."""
        if self.key_pad is None:
            keys = [self.tokens] * self.batch
        else:
            keys = [int((self.key_pad[b] == 0).sum()) for b in range(self.batch)]
        return 4.0 * HEAD_DIM * self.heads * sum(self.tokens * kk for kk in keys)

    @property
    def bytes_bf16(self) -> float:
        """Algorithmic bytes with bf16 activations: Q + K + V read, O written."""
        return 4.0 * self.batch * self.heads * self.tokens * HEAD_DIM * 2


def _draw(seed, batch, tokens, heads):
    rng = np.random.default_rng(seed)
    shape = (batch, tokens, heads, HEAD_DIM)
    q = rng.standard_normal(shape, dtype=np.float32)
    k = rng.standard_normal(shape, dtype=np.float32)
    v = rng.standard_normal(shape, dtype=np.float32)
    return q, k, v


def plumbing(seed=0, heads=2, tokens=256) -> Workload:
    """Config 1: B=1, H=2, S=256, fp32 N(0,1), no mask / norm / rope."""
    q, k, v = _draw(seed, 1, tokens, heads)
    return Workload("plumbing", "plain", 1, heads, tokens, q, k, v)


def klein(seed=0, batch=1, heads=24, grid=(64, 64), ref_grid=(0, 0), txt_len=512, theta=10000.0,
          text_lens=None, name="klein") -> Workload:
    """Configs 2, 3, 5: text tokens then image tokens (then reference-image tokens)."""
    tokens = txt_len + grid[0] * grid[1] + ref_grid[0] * ref_grid[1]
    q, k, v = _draw(seed, batch, tokens, heads)
    cos, sin = host.klein_build_rope_ref(grid[0], grid[1], ref_grid[0], ref_grid[1], theta=theta, txt_len=txt_len)
    w = Workload(name, "klein", batch, heads, tokens, q, k, v, txt_len=txt_len, grid=grid, ref_grid=ref_grid,
                 theta=theta, rope_cos=cos, rope_sin=sin)
    if text_lens is not None:
        assert len(text_lens) == batch and all(0 < n <= txt_len for n in text_lens)
        pad = np.zeros((batch, tokens), np.uint8)
        for b, n in enumerate(text_lens):
            pad[b, n:txt_len] = 1
        w.key_pad = pad
        w.text_lens = tuple(text_lens)
    return w


def zimage(seed=0, heads=30, grid=(64, 64), cap_tokens=512, name="zimage") -> Workload:
    """Config 4: image tokens then caption tokens, 3-axis rope from positions."""
    pos = host.zimage_sequence_positions(grid[0], grid[1], cap_tokens)
    tokens = pos.shape[0]
    q, k, v = _draw(seed, 1, tokens, heads)
    pairs, bases = host.zimage_rope_fill(ZIMAGE_DIMS, ZIMAGE_LENS, ZIMAGE_THETA)
    return Workload(name, "zimage", 1, heads, tokens, q, k, v, grid=grid, theta=ZIMAGE_THETA,
                    pos=pos, rope_pairs=pairs, rope_bases=bases, extra={"cap_tokens": cap_tokens})


def by_name(name: str, seed=0, small=False) -> Workload:
    """The five benchmark configurations; `small` keeps the structure at a size
    a CPU oracle finishes in seconds."""
    if name == "plumbing":
        return plumbing(seed)
    if name == "klein_1024":
        return klein(seed, 1, 24 if not small else 3, (64, 64) if not small else (9, 11),
                     txt_len=512 if not small else 40, name=name)
    if name == "klein_512_x4":
        return klein(seed, 4 if not small else 3, 24 if not small else 2, (32, 32) if not small else (6, 7),
                     txt_len=512 if not small else 24, name=name)
    if name == "zimage_1024":
        return zimage(seed, 30 if not small else 3, (64, 64) if not small else (7, 9),
                      512 if not small else 33, name=name)
    if name == "klein_edit_ragged":
        if small:
            return klein(seed, 2, 2, (6, 7), (6, 7), txt_len=200, text_lens=(13, 150), name=name)
        return klein(seed, 2, 24, (64, 64), (64, 64), txt_len=512, text_lens=(77, 300), name=name)
    raise KeyError(name)


# The reference's attention-scaling measurement (cmd/gemmbench.zig:631-678): heads 30,
# head_dim 128, these token counts; one N(0, 0.01) array serves as q, k and v.
ATTN_SCALE_TOKENS = (4224, 8448, 16896)
ATTN_SCALE_HEADS = 30


def attn_scale_input(tokens, heads=ATTN_SCALE_HEADS, seed=0xA77) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return rng.standard_normal((tokens, heads, HEAD_DIM), dtype=np.float32) * np.float32(0.1)


NAMES = ("plumbing", "klein_1024", "klein_512_x4", "zimage_1024", "klein_edit_ragged")


# ----------------------------------------------------------- device residency
class Resident:
    """A workload's operands uploaded once; `launch()` enqueues one pass of the
    hot path (inputs already in HBM), `run()` also waits and reads O back."""

    def __init__(self, ctx: host.Context, w: Workload, dtype=hip.BF16, k_site=hip.K_IN_TILE_LOAD, bounded=True,
                 staging=0, in_dtype=None):
        """dtype: element type of the output (and of the operands unless in_dtype says otherwise);
        staging: hip.F16 stages the prepared Q and K as IEEE half (needs the pre-pass)."""
        self.ctx, self.w, self.dtype, self.k_site = ctx, w, dtype, k_site
        in_dtype = dtype if in_dtype is None else in_dtype
        conv = {hip.BF16: host.f32_to_bf16_bits, hip.F16: (lambda a: np.ascontiguousarray(a, np.float16)),
                hip.F32: (lambda a: np.ascontiguousarray(a, np.float32))}[in_dtype]
        self.q = ctx.buffer(conv(w.q))
        self.k = ctx.buffer(conv(w.k))
        self.v = ctx.buffer(conv(w.v))
        self.esize = 2 if dtype == hip.BF16 else 4
        n = w.batch * w.tokens * w.heads * HEAD_DIM
        self.o = ctx.buffer(nbytes=n * self.esize)
        ones = np.ones(HEAD_DIM, np.float32)
        self.wq = ctx.buffer(ones)
        self.wk = ctx.buffer(ones)
        self.key_pad = ctx.buffer(w.key_pad) if w.key_pad is not None else None
        self.ext = hip.AttnExt()
        self.ops = hip.QkOperands()
        self.params = hip.AttnParams(w.tokens, w.heads, w.heads, HEAD_DIM, 0, 0)
        hidden = w.heads * HEAD_DIM
        x = self.ext
        for s in (x.q_stride, x.k_stride, x.v_stride, x.out_stride):
            s[0] = w.tokens * hidden if w.batch > 1 else 0
            s[1] = hidden
            s[2] = HEAD_DIM
        x.batch, x.in_dtype, x.out_dtype, x.k_site, x.staging = w.batch, in_dtype, dtype, k_site, staging
        if w.kind == "plain":
            x.qk_mode = hip.QK_NONE
        elif w.kind == "klein":
            x.qk_mode, x.eps = hip.QK_KLEIN, KLEIN_EPS
            self.cos = ctx.buffer(w.rope_cos)
            self.sin = ctx.buffer(w.rope_sin)
            self.ops.q_weight, self.ops.k_weight = self.wq.handle, self.wk.handle
            self.ops.rope_cos, self.ops.rope_sin = self.cos.handle, self.sin.handle
            x.rope_batch_rows = 0  # one table shared by the segments
        else:
            x.qk_mode, x.eps = hip.QK_ZIMAGE, ZIMAGE_EPS
            self.pos = ctx.buffer(np.ascontiguousarray(w.pos, np.uint64))
            self.pairs = ctx.buffer(w.rope_pairs)
            self.ops.q_weight, self.ops.k_weight = self.wq.handle, self.wk.handle
            self.ops.pos, self.ops.rope_pairs = self.pos.handle, self.pairs.handle
            for a in range(3):
                x.zimage_dims[a] = ZIMAGE_DIMS[a]
                x.zimage_base[a] = w.rope_bases[a]
        if w.kind != "plain" and bounded:
            # unit norm weights: the normalised rows have norm sqrt(128), rope rotates
            x.score_bound = host.score_bound(ones, ones)
        if self.key_pad is not None:
            self.ops.key_pad = self.key_pad.handle
            x.mask_batch_bytes = w.tokens

    def launch(self, batch_handle):
        """Enqueue one pass on an open batch; returns the C-ABI return code."""
        import ctypes as C
        return hip.lib().zdraw_hip_run_attention_fused_enc(
            batch_handle, self.q.handle, self.k.handle, self.v.handle, self.o.handle,
            C.byref(self.params), C.byref(self.ext), C.byref(self.ops))

    def run(self) -> np.ndarray:
        """One blocking pass; returns O as fp32 [B][S][H][128]."""
        import ctypes as C
        rc = hip.lib().zdraw_hip_run_attention_fused(
            self.ctx.queue, self.q.handle, self.k.handle, self.v.handle, self.o.handle,
            C.byref(self.params), C.byref(self.ext), C.byref(self.ops))
        if rc != 0:
            raise RuntimeError(f"zdraw_hip_run_attention_fused rc={rc}: {hip.last_error()}")
        return self.read_output()

    def read_output(self) -> np.ndarray:
        w = self.w
        shape = (w.batch, w.tokens, w.heads, HEAD_DIM)
        if self.dtype == hip.BF16:
            return host.bf16_bits_to_f32(self.o.read(np.uint16, shape))
        return self.o.read(np.float32, shape)

    def release(self):
        for name in ("q", "k", "v", "o", "wq", "wk", "key_pad", "cos", "sin", "pos", "pairs"):
            b = getattr(self, name, None)
            if b is not None:
                b.release()
