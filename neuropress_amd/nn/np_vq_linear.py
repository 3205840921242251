"""NPVQLinear: drop-in ``nn.Linear`` replacement with a VQ-compressed weight.

The weight is a packed stream of codebook indices plus a codebook shared
through a :class:`VQProxy`:

    ``W[n, g*VL + v] = centroids[idx[n * n_groups + g], v]``

Same module surface as the reference (neuropress/nn/np_vq_linear.py:399-1517):
``VQProxy``, ``NPVQLinear(proxy, packed_indices, bits, out_features, in_features,
vector_len, backend, bias, column_perm, ...)``, ``from_qtensor_linear``,
``to_qtensor``, ``forward``, ``linearize_vq_weights``.  What differs is what runs
underneath: hand-written gfx950 kernels instead of CUDA/Triton, selected by
token count ``m = x.numel() // in_features``:

====================  ==============================  ==========================
band                  condition                        kernel
====================  ==============================  ==========================
(a) fused GEMV        ``m <= _FUSED_MAX_TOKENS``, or   ``kernels.vq_linear``
                      ``m <= 32`` while x is small
(b) tile-decode GEMM  ``m <= _TILE_MAX_TOKENS``        ``kernels.vq_gemm_tile``
(c) decode + GEMM     otherwise                        ``kernels.vq_dequant`` + ``F.linear``
====================  ==============================  ==========================

The dispatch rule itself is the reference's (np_vq_linear.py:1014-1058); the
thresholds are re-derived for one MI355X and stay overridable through the same
environment variables.  Prefix-coded index formats (tiered / n-tier /
zero-escape) are expanded to the fixed-width stream once, at construction.
"""

from __future__ import annotations

import logging
import os
import weakref

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..qweights import VQScheme, VQWeight, is_vq_weight
from ..transforms.vq_entropy_packing import decode_to_flat
from ..transforms.vq_packing import (
    IndexPacking,
    NTieredIndexPacking,
    TieredIndexPacking,
    ZeroEscapePacking,
)
from .backends import Backend, VQBackend, is_hip_backend_available, tensor_version, tile_band_ok

log = logging.getLogger(__name__)

_unprepared_warned = False


def _warn_unprepared_once() -> None:
    """One WARNING per process when a layer meant for the slice-list GEMV runs without its lists."""
    global _unprepared_warned
    if not _unprepared_warned:
        _unprepared_warned = True
        log.warning(
            "NPVQLinear: a layer with a codebook of more than 4096 rows has no slice lists for its current "
            "buffers (never prepared, or its indices were reloaded): decode steps run the slower fused GEMV.  "
            "Call neuropress_amd.prepare_decode(model) once the model is on its GPU."
        )


def _env_int(names: tuple[str, ...], default: int) -> int:
    for name in names:
        v = os.environ.get(name)
        if v is not None and v.strip():
            return int(v)
    return default


# Token-count bands (tokens = rows of the flattened input), read once at import
# like the reference's (np_vq_linear.py:73-87).  The fused GEMV issues the
# contraction as 16-row MFMA tiles, so 1..16 tokens cost the same: the fused
# band ends at 16 here (2 in the reference, whose GEMV re-reads the weight per token).
_FUSED_MAX_TOKENS: int = _env_int(("NEUROPRESS_VQ_FUSED_MAX_TOKENS",), 16)
# 17..32 tokens: the GEMV reuses every decoded operand for two 16-token tiles.  Each of its
# workgroups reads all of x from L2, so it wins while x is small (tokens x in_features at most
# _FUSED_WIDE_MAX_ACTIVATIONS).  Measured, GEMV vs tile GEMM at 17 / 24 / 32 tokens, bf16:
# 14336 x 4096, 4096-row codebook 12.9 / 14.6 / 16.2 vs 27 us, 65536-row 42 / 44 / 47 vs 46-50 us;
# 4096 x 4096 8.7 / 9.8 / 11.1 vs 16 us; 4096 x 14336 22.4 / 26.4 / 31.2 vs 28 us.  Residual
# layers 35-41 vs 70 us (14336 x 4096) and 41-50 vs 74 us (4096 x 14336): GEMV at any length.
_FUSED_WIDE_MAX_TOKENS: int = _env_int(("NEUROPRESS_VQ_FUSED_WIDE_MAX_TOKENS",), 32)
_FUSED_WIDE_MAX_ACTIVATIONS: int = 1 << 18
_GEMV_KERNEL_MAX_TOKENS: int = 32  # what the GEMV entry points accept (NPAMD_GEMV_MAX_M)

# Decode steps (1-7 tokens) of layers whose codebook is too large to sit in a
# compute unit's LDS next to the GEMV's buffers (more than 4096 rows): the fused
# GEMV then pays one L2 lookup per index (34-35 us on a 14336 x 4096 layer with a
# 65536-row codebook, any token count up to 16), while the slice-list GEMV
# (kernels.vq_linear_sliced) keeps 4096-row codebook slices in LDS: 10.3-10.9 / 14.2 /
# 20.3 / 30.9 us at 1 / 2 / 4 / 7 tokens; an eighth token needs a second pass over the
# entries.  The slice lists are built on the host by prepare_sliced() / prepare_decode(),
# never by forward() (about 26 MB per such layer, on top of the packed stream the other
# bands keep reading).  0 disables the path.
_SLICED_MAX_TOKENS: int = _env_int(("NEUROPRESS_VQ_SLICED_MAX_TOKENS",), 7)
_SLICED_MIN_CENTROIDS: int = 4097
_SLICED_MIN_INDICES: int = _env_int(("NEUROPRESS_VQ_SLICED_MIN_INDICES",), 1 << 20)
# Whether a module that reaches a GPU through .to() / .cuda() / load_state_dict() builds the tensors
# its kernels derive from the buffers there and then (slice lists: a host round trip per layer).
_PREPARE_ON_MOVE: bool = _env_int(("NEUROPRESS_VQ_PREPARE_ON_MOVE",), 1) != 0

# cuda_lut layers: 0 = always decode + GEMM, the reference's default routing.
_LUT_MAX_TOKENS: int = _env_int(("NEUROPRESS_VQ_LUT_MAX_TOKENS",), 0)

# Upper end of the tile-decode GEMM band.  NEUROPRESS_VQ_TRITON_MAX_TOKENS is the
# reference's name for the same knob and is honoured too.  0 disables the band.
# Measured on one MI355X (14336 x 4096 layer): the tile GEMM beats decode + GEMM
# from 17 to about 320 tokens (58 vs 67 us at 64, 74 vs 86 us at 256, 100 vs 96 us
# at 384, 190 vs 101 us at 512, where a second row block re-decodes the weight).
_TILE_MAX_TOKENS: int = _env_int(
    ("NEUROPRESS_VQ_TILE_MAX_TOKENS", "NEUROPRESS_VQ_TRITON_MAX_TOKENS"), 256
)

# Layers whose codebook LDS does not hold (more than 4096 rows of eight) run the 128-column tile GEMM,
# which splits the reduction by itself and stays ahead of decode + GEMM up to a token count that goes
# with the layer's weights (us at 128 / 256 / 384 tokens, tile against decode + GEMM): 14336 x 4096
# 47 / 59 / 73 against 81 / 96 / 101, 4096 x 14336 53 / 67 / 82 against 114 / 103 / 117; 6144 x 4096
# 32 / 41 / 56 against 47 / 61 / 55, 4096 x 4096 28 / 34 / 42 against 40 / 38 / 41, 8192 x 2048 28 / 34 / 46
# against 34 / 40 / 38; 1024 x 4096 18 / 24 / 29 against 20 / 21 / 22, 2048 x 2048 16 / 23 / 28 against 17 / 20 / 20.
_TILE_WIDE_MAX_TOKENS: int = _env_int(("NEUROPRESS_VQ_TILE_WIDE_MAX_TOKENS",), 384)
_TILE_WIDE_MIN_WEIGHTS: int = 1 << 25  # below: 256 tokens
_TILE_WIDE_SMALL_WEIGHTS: int = 1 << 24  # below: 128 tokens
_TILE_WIDE_MID_MAX_TOKENS: int = 256
_TILE_WIDE_SMALL_MAX_TOKENS: int = 128

# The tile GEMM gives each workgroup 64 output columns (and up to 384 rows).  When
# that grid covers less than this fraction of the compute units the kernel splits
# the reduction over up to 16 workgroups per tile (at least 512 input features
# each); a layer that still cannot cover the fraction takes decode + GEMM.
_TILE_MIN_GRID_FRACTION: float = 0.7

# Upper end of the band for layers that need the split.  Measured on one MI355X,
# tile GEMM vs decode + GEMM: 4096 x 14336 layer 51-60 vs 75-113 us up to 128
# tokens and 82 vs 101 us at 256; 4096 x 4096 layer 25-31 vs 30-39 us up to 128
# tokens, 39 vs 36 us at 256.
_TILE_SPLIT_MAX_TOKENS: int = 128
_TILE_SPLIT_LONG_K: int = 8192  # from this many input features on, _TILE_MAX_TOKENS applies
# Layers of at least this many indices time their slice-list GEMV against the fused one when the
# lists are built (NPVQLinear._sliced_token_limit).
_SLICED_TUNE_MIN_INDICES: int = 1 << 20
# Residual layers take the tile band under the same grid rule as plain ones.  Measured, tile
# GEMM vs decode + GEMM, bf16, 33 / 128 / 256 tokens: 14336 x 4096 53 / 56 / 72 against 75 / 76 /
# 92 us; 4096 x 4096 26 / 31 / 40 against 33 / 42 / 41 us; 4096 x 14336 54 / 63 / 84 against
# 78 / 107 / 100 us; 1024 x 4096 (too few column blocks, decode + GEMM by the grid rule) 20 / 22 /
# 27 against 24 / 21 / 22 us.

# Opt-in: when a HIP kernel call fails, warn once and run torch ops instead (the
# reference's behaviour).  Off by default so a missing or broken kernel library
# is an error, not a silent slow path.
_ALLOW_FALLBACK: bool = os.environ.get("NEUROPRESS_ALLOW_KERNEL_FALLBACK", "").strip() in (
    "1", "true", "yes",
)  # fmt: skip

# Backends that run the HIP bands.  The three per-format members name, in the reference, kernels
# that decode a prefix-coded stream inside the GEMV; here such layers are expanded to the fixed-width
# stream at construction, so the members are labels that route like CUDA_WMMA.
_CODED_BACKENDS = frozenset({VQBackend.CUDA_TIERED, VQBackend.CUDA_NTIER, VQBackend.CUDA_ZERO_ESCAPE})
_FUSED_BACKENDS = frozenset({VQBackend.CUDA_WMMA, VQBackend.CUDA_LUT, VQBackend.CUDA}) | _CODED_BACKENDS

# Latched once the tile GEMM fails with fallback allowed, so later calls go
# straight to decode + GEMM (reference: np_vq_linear.py:91-93).
_tile_failed: bool = False

# Index widths the fast kernels stream directly; other widths are widened to
# 16 bits once, on first GPU use.
_FAST_BITS = frozenset({4, 8, 12, 16})


def _fused_max_tokens(backend: VQBackend) -> int:
    """Largest token count for which *backend*'s fused kernel is used."""
    return _LUT_MAX_TOKENS if backend == VQBackend.CUDA_LUT else _FUSED_MAX_TOKENS


def _resolve_vq_backend(
    backend: str | VQBackend | Backend | None,
    use_tiered: bool = False,
    use_ntier: bool = False,
    use_zero_escape: bool = False,
    bits: int = 8,
    out_features: int = 0,
    num_centroids: int = 0,
    vector_len: int = 8,
) -> VQBackend:
    """Resolve a backend alias to a concrete :class:`VQBackend` (never ``AUTO``).

    Signature and alias handling follow the reference
    (neuropress/nn/np_vq_linear.py:101-170): ``None`` / ``"torch"`` ->
    ``DEFAULT``, unknown strings raise ``ValueError``.  ``"auto"`` on a machine
    where the HIP library can run resolves to ``CUDA_WMMA`` -- the three-band
    path -- for every codebook size and vector length: the reference's detours
    (vector_len != 4 -> COMPILE, bits > 12 -> CUDA_LUT) exist because its
    tensor-core kernels are fixed to VL = 4 and a 4096-entry shared-memory
    codebook; the kernels here have neither limit.  Without a GPU ``"auto"``
    resolves to ``COMPILE`` as in the reference.
    """
    if backend is None or backend == "torch":
        return VQBackend.DEFAULT
    if isinstance(backend, (VQBackend, Backend)):
        val = backend.value
    elif isinstance(backend, str):
        val = backend
    else:
        val = str(backend)
    if val != "auto":
        return VQBackend(val)  # raises ValueError for unknown strings
    if not (torch.cuda.is_available() and is_hip_backend_available()):
        return VQBackend.COMPILE
    # Same precedence as the reference (np_vq_linear.py:158-163); all four run the same kernels.
    if use_zero_escape:
        return VQBackend.CUDA_ZERO_ESCAPE
    if use_ntier:
        return VQBackend.CUDA_NTIER
    if use_tiered:
        return VQBackend.CUDA_TIERED
    return VQBackend.CUDA_WMMA


def _vq_dequant_linear(
    x: torch.Tensor,
    packed_indices: torch.Tensor,
    centroids: torch.Tensor,
    bits: int,
    n_vectors: int,
    out_features: int,
    in_features: int,
    bias: torch.Tensor | None,
) -> torch.Tensor:
    """Unpack, gather, ``F.linear`` with torch ops: the specification of the layer.

    Follows neuropress/nn/np_vq_linear.py:178-211.  Runs on whatever device the
    buffers live on; used by the ``default`` / ``compile`` backends.
    """
    indices = IndexPacking.unpack(packed_indices, bits, n_vectors)
    w = centroids[indices].reshape(out_features, in_features)
    return F.linear(x, w.to(x.dtype), bias)


# ---------------------------------------------------------------------------
# VQProxy — shared codebook
# ---------------------------------------------------------------------------


def _versions_of(packed, bias, perm, cent) -> tuple:
    return (
        packed._version,
        cent._version,
        -1 if bias is None else bias._version,
        -1 if perm is None else perm._version,
    )


class VQProxy(nn.Module):
    """Shared VQ codebook holder (reference: neuropress/nn/np_vq_linear.py:399-455).

    Holds ``centroids`` ``[num_centroids, vector_len]`` as a float16 buffer.
    One instance is shared by every :class:`NPVQLinear` of a quantization group
    and is registered on the model root, not on each layer.
    """

    centroids: torch.Tensor

    def __init__(self, centroids: torch.Tensor) -> None:
        super().__init__()
        self.register_buffer("centroids", centroids.to(torch.float16))
        self._cast_cache: dict = {}
        # Layers that read this codebook (weakly held, not copied or pickled with the proxy): told
        # when the codebook moves or is reloaded, because a parent's .to() may move a layer first.
        self._users: weakref.WeakSet = weakref.WeakSet()
        self.register_load_state_dict_post_hook(VQProxy._after_load_state_dict)

    def _bind(self, user: nn.Module) -> None:
        self._users.add(user)

    def _notify_users(self) -> None:
        for user in list(self._users):
            if user.proxy is self or user.residual_proxy is self:
                user._prepare_after_move()

    def _apply(self, fn, recurse: bool = True):
        result = super()._apply(fn, recurse)
        self._cast_cache = {}
        self._notify_users()
        return result

    @staticmethod
    def _after_load_state_dict(module, incompatible_keys) -> None:
        module._cast_cache = {}
        module._notify_users()

    def __getstate__(self):
        state = self.__dict__.copy()
        state.pop("_users", None)
        return state

    def __setstate__(self, state):
        super().__setstate__(state)
        self._users = weakref.WeakSet()

    @property
    def num_centroids(self) -> int:
        return self.centroids.shape[0]

    @property
    def vector_len(self) -> int:
        return self.centroids.shape[1]

    def centroids_as(self, dtype: torch.dtype) -> torch.Tensor:
        """The codebook cast to *dtype*, cached until the buffer moves or changes.

        A bf16 model multiplies by bf16-rounded codebook rows (that is what
        ``W.to(x.dtype)`` means); casting the table once keeps that conversion
        out of the kernels' inner loops.
        """
        c = self.centroids
        if dtype == c.dtype:
            return c
        key = (dtype, c.device, c.data_ptr(), tensor_version(c))
        hit = self._cast_cache.get("entry")
        if hit is None or hit[0] != key:
            hit = (key, c.to(dtype).contiguous())
            self._cast_cache["entry"] = hit
        return hit[1]

    def extra_repr(self) -> str:
        return f"num_centroids={self.num_centroids}, vector_len={self.vector_len}"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise RuntimeError(
            "VQProxy.forward() should not be called.  Access centroids "
            "directly via self.proxy.centroids."
        )


# ---------------------------------------------------------------------------
# NPVQLinear
# ---------------------------------------------------------------------------


class NPVQLinear(nn.Module):
    """Linear layer with a VQ-compressed weight and a shared codebook proxy.

    Constructor arguments up to ``zesc_row_offsets`` are the reference's
    (neuropress/nn/np_vq_linear.py:493-513).  With ``use_tiered`` / ``tier_bits`` /
    ``zero_escape`` the buffer passed as ``packed_indices`` is a prefix-coded one
    (``transforms/vq_entropy_packing.py``): it is expanded once, here, into the
    fixed-width stream all kernels read (``self.packed_indices``, ``self.bits`` wide),
    so these layers run the same three bands as any other; the ``*_row_offsets``
    arguments, which the reference's per-format kernels need, are accepted and
    unused, and :meth:`to_qtensor` packs the indices back.  The
    ``residual_*`` / ``row_*`` arguments add an optional residual codebook and
    a per-output-row fp16 scale and bias on the decoded weight:

        ``W[n, :] = ((Cm[im] + Cr[ir]) * row_scale[n]) + row_bias[n]``

    each operation rounded to fp16 (the benchmark's residual-VQ configuration; not in the reference).
    """

    def __init__(
        self,
        proxy: VQProxy,
        packed_indices: torch.Tensor,
        bits: int,
        out_features: int,
        in_features: int,
        vector_len: int,
        backend: str | VQBackend | None,
        bias: torch.Tensor | None = None,
        column_perm: torch.Tensor | None = None,
        use_tiered: bool = False,
        cold_bits: int = 8,
        hot_row_offsets: torch.Tensor | None = None,
        cold_row_offsets: torch.Tensor | None = None,
        qtensor_meta: dict[str, str] | None = None,
        tier_bits: list[int] | None = None,
        ntier_row_offsets: list[torch.Tensor] | None = None,
        zero_escape: bool = False,
        zesc_row_offsets: list[torch.Tensor] | None = None,
        residual_proxy: VQProxy | None = None,
        packed_residual: torch.Tensor | None = None,
        residual_bits: int = 0,
        row_scale: torch.Tensor | None = None,
        row_bias: torch.Tensor | None = None,
    ) -> None:
        super().__init__()
        if in_features % vector_len:
            raise ValueError(f"in_features={in_features} not divisible by vector_len={vector_len}")
        if proxy.vector_len != vector_len:
            raise ValueError(f"vector_len={vector_len} does not match the codebook ({proxy.vector_len})")
        self._qtensor_meta = qtensor_meta
        self.out_features = out_features
        self.in_features = in_features
        self.vector_len = vector_len
        self.bits = bits
        self.n_vectors = out_features * (in_features // vector_len)
        # Same precedence as the reference's scheme (neuropress/transforms/vq.py:220-247).
        self.zero_escape = bool(zero_escape)
        self.tier_bits = None if zero_escape or tier_bits is None else list(tier_bits)
        self.use_tiered = bool(use_tiered) and not zero_escape and tier_bits is None
        self.cold_bits = cold_bits
        self._hot_bits = TieredIndexPacking.DEFAULT_HOT_BITS
        self._coded_bits = bits
        if self.zero_escape or self.tier_bits is not None or self.use_tiered:
            packed_indices, bits = self._expand_prefix_coded(packed_indices, proxy.num_centroids)
            self.bits = bits
        self.backend = _resolve_vq_backend(
            backend,
            use_tiered=self.use_tiered,
            use_ntier=self.tier_bits is not None,
            use_zero_escape=self.zero_escape,
            bits=bits,
            out_features=out_features,
            num_centroids=proxy.num_centroids,
            vector_len=vector_len,
        )
        need = IndexPacking.packed_nbytes(self.n_vectors, bits)
        if packed_indices.numel() < need:
            raise ValueError(
                f"packed_indices holds {packed_indices.numel()} bytes, {need} needed for "
                f"{self.n_vectors} indices of {bits} bits"
            )

        # The proxy is a plain attribute, not a sub-module: it must not appear
        # once per layer in state_dict (reference: np_vq_linear.py:588-590).
        object.__setattr__(self, "proxy", proxy)
        object.__setattr__(self, "residual_proxy", residual_proxy)
        self._bind_proxies()

        self.register_buffer("packed_indices", packed_indices.contiguous())
        self._register_optional("bias", bias)
        self._register_optional(
            "column_perm", None if column_perm is None else column_perm.to(torch.int64)
        )
        self.residual_bits = residual_bits
        if residual_proxy is not None:
            if packed_residual is None:
                raise ValueError("residual_proxy given without packed_residual")
            if residual_proxy.vector_len != vector_len:
                raise ValueError("residual codebook must have the same vector length")
            self.residual_bits = residual_bits or IndexPacking.bits_for(residual_proxy.num_centroids)
        self._register_optional("packed_residual", packed_residual)
        self._register_optional("row_scale", None if row_scale is None else row_scale.to(torch.float16))
        self._register_optional("row_bias", None if row_bias is None else row_bias.to(torch.float16))
        # Derived, rebuilt on demand: f32 bias for the kernels, widened index stream.
        self._derived: dict = {}
        # Per activation dtype: the decode call with its constant arguments worked out once (see forward).
        self._plans: dict = {}
        # load_state_dict() copies into the buffers in place: what was derived from them is stale.
        self.register_load_state_dict_post_hook(NPVQLinear._after_load_state_dict)

    def _expand_prefix_coded(self, coded: torch.Tensor, num_centroids: int) -> tuple[torch.Tensor, int]:
        """Prefix-coded buffer -> ``(fixed-width stream, its bit width)``.

        The reference keeps such layers in their coded form and decodes prefixes in
        every GEMV (np_vq_linear.py:644-801, kernels/vq_linear_tiered.cu); here the
        coded form is a storage format only.
        """
        self._coded_bits = self.bits  # the width argument as given (the reference's cold-tier width)
        if self.use_tiered:
            _, _, self.cold_bits, self._hot_bits, _ = TieredIndexPacking._parse_header(coded)
        elif self.zero_escape:
            self.cold_bits = ZeroEscapePacking._parse_header(coded)[1]
        idx = decode_to_flat(
            coded, use_tiered=self.use_tiered, tier_bits=self.tier_bits, zero_escape=self.zero_escape
        )
        if idx.numel() != self.n_vectors:
            raise ValueError(
                f"prefix-coded buffer holds {idx.numel()} indices, the layer needs {self.n_vectors}"
            )
        if idx.numel() and int(idx.max().item()) >= num_centroids:
            raise ValueError("prefix-coded buffer names a codebook row past the end of the codebook")
        width = IndexPacking.bits_for(num_centroids)
        if width == 4 and idx.numel() % 2:
            width = 8  # a 4-bit stream needs an even count
        return IndexPacking.pack(idx, width), width

    def _coded_indices(self) -> torch.Tensor:
        """The layer's indices packed back into the prefix-coded format it was built from."""
        idx = IndexPacking.unpack(self.packed_indices.cpu(), self.bits, self.n_vectors)
        if self.zero_escape:
            return ZeroEscapePacking.pack(idx, self.cold_bits)
        if self.tier_bits is not None:
            return NTieredIndexPacking.pack(idx, self.tier_bits)
        return TieredIndexPacking.pack(idx, self.cold_bits, self._hot_bits)

    def _register_optional(self, name: str, t: torch.Tensor | None) -> None:
        if t is not None:
            self.register_buffer(name, t.contiguous())
        else:
            setattr(self, name, None)

    def _bind_proxies(self) -> None:
        for proxy in (self.proxy, self.residual_proxy):
            if proxy is not None:
                proxy._bind(self)

    def _buffer_places(self) -> tuple:
        return tuple((b.device, b.data_ptr(), b.dtype) for b in self._buffers.values() if b is not None)

    def _apply(self, fn, recurse: bool = True):
        """``.to()`` / ``.cuda()`` / ``.half()``: the derived tensors belong to the old buffers.  A move
        is already a heavy host operation, so when the module arrives on a GPU the tensors its
        kernels derive from the buffers -- the slice lists included -- are made here (or, when the
        shared codebook arrives after the layer, by the codebook's own move): ``lower on the CPU ->
        model.to("cuda") -> forward`` reaches the fast decode kernel with no further call, as a
        caller of the reference expects (neuropress/t2n/model_io.py:590-596).
        ``NEUROPRESS_VQ_PREPARE_ON_MOVE=0`` leaves that to :func:`neuropress_amd.prepare_decode`."""
        before = self._buffer_places()
        result = super()._apply(fn, recurse)
        if self._buffer_places() != before:
            self._derived = {}
        self._plans = {}
        self._bind_proxies()  # a copied or unpickled proxy starts with no users
        self._prepare_after_move()
        return result

    def _prepare_after_move(self) -> None:
        if not _PREPARE_ON_MOVE or not self.packed_indices.is_cuda or self.backend not in _FUSED_BACKENDS:
            return
        if torch.cuda.is_current_stream_capturing():
            return
        # The shared codebooks are sub-modules of the model root, not of this layer, and may still be
        # on their way: they call back when they arrive.
        for proxy in (self.proxy, self.residual_proxy):
            if proxy is not None and proxy.centroids.device != self.packed_indices.device:
                return
        try:
            if not self.prepare_sliced():
                self.prepare()
        except RuntimeError as exc:  # no kernel library on this machine: forward will say so
            if not _ALLOW_FALLBACK:
                raise
            self._fallback("prepare", "unprepared kernels", exc)

    @staticmethod
    def _after_load_state_dict(module, incompatible_keys) -> None:
        module._derived = {}
        module._plans = {}
        module._prepare_after_move()

    # ------------------------------------------------------------------
    # Factory / inverse
    # ------------------------------------------------------------------

    @classmethod
    def from_qtensor_linear(
        cls,
        linear: nn.Linear,
        proxy: VQProxy,
        backend: str | VQBackend | None = VQBackend.AUTO,
        residual_proxy: VQProxy | None = None,
    ) -> NPVQLinear:
        """Build from an ``nn.Linear`` whose ``weight`` is a VQ weight.

        Follows neuropress/nn/np_vq_linear.py:831-921.  Raises ``TypeError``
        (message naming ``QTensorTractVQ``, as the reference does) when the
        weight is not vector-quantized.
        """
        weight_q = linear.weight
        if not is_vq_weight(weight_q):
            raise TypeError(
                f"Expected a VQ weight (QTensorTractVQ / VQWeight), got {type(weight_q).__name__!r}."
            )
        qs = weight_q.qscheme
        bias = linear.bias.detach().clone() if linear.bias is not None else None
        perm = getattr(qs, "column_permutation", None)
        res_c = getattr(qs, "residual_centroids", None)
        if res_c is not None and residual_proxy is None:
            residual_proxy = VQProxy(res_c)
        row_scale = getattr(qs, "row_scale", None)
        row_bias = getattr(qs, "row_bias", None)
        return cls(
            proxy=proxy,
            packed_indices=weight_q.u8_blob.detach().clone(),
            bits=qs.is_packed_indices,
            out_features=linear.out_features,
            in_features=linear.in_features,
            vector_len=qs.vector_len,
            backend=backend,
            bias=bias,
            column_perm=perm.detach().clone() if perm is not None else None,
            use_tiered=bool(getattr(qs, "use_tiered", False)),
            tier_bits=getattr(qs, "tier_bits", None),
            zero_escape=bool(getattr(qs, "zero_escape", False)),
            qtensor_meta={"original_shape": tuple(getattr(qs, "original_shape", ()))},
            residual_proxy=residual_proxy,
            packed_residual=getattr(weight_q, "residual_blob", None),
            residual_bits=getattr(qs, "residual_bits", 0),
            row_scale=row_scale,
            row_bias=row_bias,
        )

    def to_qtensor(self) -> VQWeight:
        """Rebuild the VQ weight this module was lowered from (for unlowering / saving).

        Same contract as neuropress/nn/np_vq_linear.py:977-1008: raises
        ``RuntimeError`` when the module was not built by :meth:`from_qtensor_linear`.
        """
        if self._qtensor_meta is None:
            raise RuntimeError(
                "Cannot reconstruct QTensor: no serde metadata stored. "
                "Build via NPVQLinear.from_qtensor_linear() to enable to_qtensor()."
            )
        coded = self.use_tiered or self.tier_bits is not None or self.zero_escape
        scheme = VQScheme(
            centroids=self.proxy.centroids,
            original_shape=(self.out_features, self.in_features),
            is_packed_indices=self._coded_bits if coded else self.bits,
            column_permutation=self.column_perm,
            use_tiered=self.use_tiered,
            tier_bits=self.tier_bits,
            zero_escape=self.zero_escape,
            residual_centroids=None if self.residual_proxy is None else self.residual_proxy.centroids,
            residual_bits=self.residual_bits,
            row_scale=self.row_scale,
            row_bias=self.row_bias,
        )
        blob = self._coded_indices().to(self.packed_indices.device) if coded else self.packed_indices
        return VQWeight(blob, scheme, self.packed_residual)

    # ------------------------------------------------------------------
    # Derived buffers
    # ------------------------------------------------------------------

    @property
    def is_residual(self) -> bool:
        return self.residual_proxy is not None or self.row_scale is not None or self.row_bias is not None

    def _derive(self, name: str, source: torch.Tensor, build):
        """``build()`` cached under *name* until *source* moves, is replaced or is written to.

        Every tensor derived from a buffer (a widened index stream, the slice lists, the fp32
        bias, the int32 permutation) is keyed on the buffer's device, address and version
        counter, so ``load_state_dict`` or an in-place ``copy_`` into the buffer invalidates it.
        Inside a graph capture nothing is stored: a tensor made there lives in the graph's
        private pool and holds data only after a replay, so a later eager call must make its own.
        """
        key = (source.device, source.data_ptr(), tensor_version(source))
        hit = self._derived.get(name)
        if hit is not None and hit[0] == key:
            return hit[1]
        value = build()
        if not (source.is_cuda and torch.cuda.is_current_stream_capturing()):
            self._derived[name] = (key, value)
        return value

    def _derived_hit(self, name: str, source: torch.Tensor):
        """The cached value of :meth:`_derive`, or None when it is missing or stale."""
        hit = self._derived.get(name)
        if hit is not None and hit[0] == (source.device, source.data_ptr(), tensor_version(source)):
            return hit[1]
        return None

    def _bias_f32(self) -> torch.Tensor | None:
        if self.bias is None:
            return None
        return self._derive("bias_f32", self.bias, lambda: self.bias.detach().to(torch.float32).contiguous())

    def _bias_as(self, dtype: torch.dtype) -> torch.Tensor | None:
        """Bias in the activation dtype for the torch GEMM (``F.linear`` wants one dtype)."""
        if self.bias is None or self.bias.dtype == dtype:
            return self.bias
        return self.bias.to(dtype)

    def _kernel_stream(self) -> tuple[torch.Tensor, int]:
        """Index stream and width the fused kernels read.

        Widths outside {4, 8, 12, 16} are widened to a 16-bit stream once per
        device so they take the vectorised index loads (precedent: the
        reference re-lays index streams out at construction, np_vq_linear.py:644-696).
        """
        if self.bits in _FAST_BITS or self.bits > 16:
            return self.packed_indices, self.bits
        from .. import kernels

        wide = self._derive(
            "wide", self.packed_indices,
            lambda: kernels.widen_indices_u16(self.packed_indices, self.n_vectors, self.bits),
        )  # fmt: skip
        return wide, 16

    # ------------------------------------------------------------------
    # Forward
    # ------------------------------------------------------------------

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """Band dispatch by token count (reference: neuropress/nn/np_vq_linear.py:1014-1058)."""
        entry = self._plans.get(x.dtype)
        if entry is not None:
            # A decode call this layer has made before: same buffers, not written to since?  Then the
            # call is issued with its constant arguments as they were worked out then.
            plan, packed, bias, perm, cent, versions = entry
            buffers = self._buffers
            if (
                buffers["packed_indices"] is packed
                and buffers.get("bias") is bias
                and buffers.get("column_perm") is perm
                and self.proxy._buffers["centroids"] is cent
                and (versions is None or versions == _versions_of(packed, bias, perm, cent))
            ):
                y = plan.run(x)
                if y is not None:
                    return y
            else:
                self._plans = {}
        if self.backend in _FUSED_BACKENDS and x.dtype in (torch.float16, torch.bfloat16):
            m = x.numel() // self.in_features
            if m <= min(_SLICED_MAX_TOKENS, _fused_max_tokens(self.backend)) and x.is_cuda:
                sliced = self._sliced_for(m)
                if sliced is not None:
                    return self._forward_sliced(x, sliced)  # applies column_perm inside the kernel
            if self.column_perm is not None and self._perm_fusable(x, m):
                return self._fused(x, tile=False, perm=self._perm_i32(x.device))
        if self.column_perm is not None:
            x = x[..., self.column_perm]
        if self.backend in _FUSED_BACKENDS:
            if x.dtype not in (torch.float16, torch.bfloat16):
                return self._forward_dequant_gemm(x)  # fp32 activations: decode + GEMM
            if x.is_cuda and not self._mfma_layer():
                # Shapes without an MFMA kernel (vector lengths other than 8 and 4, K not a
                # multiple of 64): the element-wise GEMV is slower than decoding once and calling
                # the dense GEMM at every token count (14336 x 4096: 99 us against 57 us at one token).
                return self._forward_dequant_gemm(x)
            m = x.numel() // self.in_features
            if m > self._gemv_max_tokens(m):
                if (
                    self.backend != VQBackend.CUDA_LUT
                    and m <= self._tile_max_tokens()
                    and self._tile_band_ok(x, m)
                ):
                    return self._forward_tile_gemm(x)
                return self._forward_dequant_gemm(x)
        if self.backend == VQBackend.CUDA_LUT:
            return self._forward_cuda_lut(x)
        if self.backend == VQBackend.CUDA_WMMA or self.backend in _CODED_BACKENDS:
            return self._forward_cuda_wmma(x)
        if self.backend == VQBackend.CUDA:
            return self._forward_cuda(x)
        if self.backend == VQBackend.COMPILE:
            return self._forward_compile(x)
        return self._forward_default(x)

    # -- slice-list GEMV ---------------------------------------------------

    def _sliced_eligible(self) -> bool:
        return (
            _SLICED_MAX_TOKENS > 0
            and not self.is_residual
            and self.vector_len == 8
            and self.proxy.num_centroids >= _SLICED_MIN_CENTROIDS
            and self.n_vectors >= _SLICED_MIN_INDICES
        )

    def prepare_sliced(self) -> bool:
        """Build the slice-list form of the indices for the module's current device.

        Host work (the stream is copied to the host, re-laid there and uploaded; then both decode
        GEMVs are timed on the layer's own indices), so it is never done by ``forward``: call it --
        or :func:`neuropress_amd.prepare_decode` for a whole model -- after the module has reached
        its GPU and before the first decode step or graph capture.  Returns False when the layer
        does not use the path.
        """
        if not (self._sliced_eligible() and self.packed_indices.is_cuda):
            return False
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("NPVQLinear.prepare_sliced() copies to the host and back: call it before the capture")
        self._derive("sliced", self.packed_indices, self._build_sliced)
        self.prepare()
        return True

    def prepare(self) -> None:
        """Make every tensor the kernels derive from the module's buffers (widened index stream,
        fp32 bias, int32 permutation, the codebook in the usual activation dtypes) for the current
        device, so that a first call inside a graph capture finds them."""
        if not self.packed_indices.is_cuda:
            return
        self._kernel_stream()
        self._bias_f32()
        if self.column_perm is not None:
            self._perm_i32(self.packed_indices.device)
        for dtype in (torch.float16, torch.bfloat16):
            self.proxy.centroids_as(dtype)
        if self.is_residual:
            self._res_stream()
            self._res_centroids()

    def _build_sliced(self):
        """(slice lists, most tokens for which they beat the fused GEMV on this layer)."""
        from .. import kernels

        sl = kernels.vq_slice_indices(
            self.packed_indices, self.bits, self.out_features, self.in_features,
            self.vector_len, self.proxy.num_centroids,
        )  # fmt: skip
        kernels.sliced_workspace(sl.blob.device, sl.workspace_bytes(_SLICED_MAX_TOKENS))
        return sl, self._sliced_token_limit(sl)

    def _sliced_token_limit(self, sl) -> int:
        """Most tokens for which this layer's slice-list GEMV beats its fused GEMV.

        With indices spread evenly over the codebook the slice lists win up to
        ``_SLICED_MAX_TOKENS`` by a wide margin.  A skewed index distribution (one codebook
        slice holding most of the indices) does two things: the hot slice's workgroups
        carry more of the work, or outnumber the compute units, and the fused GEMV's
        lookups start hitting in L1.  Which one wins then depends on the layer, so every
        layer of the size the path is meant for is timed here, once, when its lists are
        built (by ``prepare_sliced``, never by ``forward``)."""
        if self.n_vectors < _SLICED_TUNE_MIN_INDICES:
            return _SLICED_MAX_TOKENS
        dev = sl.blob.device
        from .. import kernels

        dt = torch.float16
        cb = self.proxy.centroids_as(dt)
        stream, bits = self._kernel_stream()

        def timed(fn) -> float:
            # GPU time, not issue time: eight calls captured in a HIP graph and replayed (launched
            # eagerly, both kernels finish faster than Python can issue them).
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(side):
                fn()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    for _ in range(8):
                        fn()
                graph.replay()
                t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                t0.record()
                for _ in range(3):
                    graph.replay()
                t1.record()
                t1.synchronize()
            torch.cuda.current_stream(dev).wait_stream(side)
            return t0.elapsed_time(t1)

        limit = 0
        try:
            for m in (1, 2, 4, _SLICED_MAX_TOKENS):
                if m > _SLICED_MAX_TOKENS:
                    break
                x = torch.ones(m, self.in_features, dtype=dt, device=dev)
                ws = torch.zeros(sl.workspace_bytes(m) // 4, dtype=torch.float32, device=dev)
                t_sliced = timed(lambda: kernels.vq_linear_sliced(x, sl, cb, workspace=ws))
                t_fused = timed(lambda: kernels.vq_linear(x, stream, cb, bits, self.vector_len, None, self.out_features))
                if t_sliced >= t_fused:
                    break
                limit = m
        except RuntimeError:
            # e.g. another thread of the process is capturing a graph: keep the measured default
            return _SLICED_MAX_TOKENS
        return limit

    def _sliced_for(self, m: int):
        """The slice lists when they exist for the buffer as it is now and win at *m* tokens, else None.

        A lookup only: an eligible layer whose lists were never built (or whose indices were
        reloaded since) runs the fused GEMV, and says so once."""
        hit = self._derived_hit("sliced", self.packed_indices)
        if hit is None:
            if self._sliced_eligible():
                _warn_unprepared_once()
            return None
        sl, limit = hit
        return sl if m <= limit else None

    def _perm_i32(self, device: torch.device) -> torch.Tensor:
        """``column_perm`` as the int32 device tensor the kernels read (cached)."""
        return self._derive(
            "perm_i32", self.column_perm,
            lambda: self.column_perm.to(device=device, dtype=torch.int32).contiguous(),
        )  # fmt: skip

    def _gemv_max_tokens(self, m: int) -> int:
        """End of band (a) for a call of *m* tokens: the fused limit, or 32 while x stays small."""
        limit = _fused_max_tokens(self.backend)
        if limit == 16 and 16 < m <= min(_FUSED_WIDE_MAX_TOKENS, 32):
            if self.is_residual or m * self.in_features <= _FUSED_WIDE_MAX_ACTIVATIONS:
                return 32
            if self._gemv_stages_activations(m) and not self._tile_ahead_from_17():
                return 32
        return limit

    def _tile_ahead_from_17(self) -> bool:
        """Large layers with at least twice as many output as input features and a codebook kept in memory: the
        128-column tile GEMM is level with the staged GEMV at 17 tokens and ahead at 24-32 (tile vs GEMV at
        17 / 24 / 32 tokens: 14336 x 4096 40.3 / 39.0 / 40.4 vs 41.0 / 42.2 / 43.1 us, 11008 x 4096 35.4 / 35.8 / 36.1
        vs 35.6 / 36.9 / 39.2); on 8192 x 8192 they tie, on 4096 x 14336 (44 vs 39-41.5 us) and on small layers
        (4096 x 4096: 20.6-21.3 vs 13.3-14.0) the GEMV stays ahead."""
        return (
            _TILE_MAX_TOKENS > 0
            and self._wide_tile_layer()
            and self.out_features >= 2 * self.in_features
            and self.in_features * self.out_features >= _TILE_WIDE_MIN_WEIGHTS
        )

    def _gemv_stages_activations(self, m: int) -> bool:
        """Layers of one row tile per workgroup whose lookups go to memory run the GEMV that stages
        its activations through LDS, which stays ahead of the tile GEMM at any K (65536-row
        codebook, GEMV vs tile GEMM at 17 / 24 / 32 tokens: 4096 x 14336 39.8 / 39.7 / 42.0 vs
        48.7-49.6 us, 4096 x 8192 24.2 / 24.1 / 24.8 vs 33.8-34.8 us; with a 4096-row table, which
        the GEMV looks up in LDS, it does not: 23.4 / 28.4 / 33.4 vs 24.6-25.8 us)."""
        hit = self._derived.get("stages")
        if hit is None or hit[0] != m:
            from .. import kernels

            rows = max(1, self.proxy.num_centroids * self.vector_len // 8)  # table size in rows of eight
            hit = (m, kernels.gemv_stages_activations(m, self.out_features, self.in_features, rows))
            self._derived["stages"] = hit
        return hit[1]

    def _perm_fusable(self, x: torch.Tensor, m: int) -> bool:
        """Whether the fused GEMV gathers ``x[..., column_perm]`` itself for this call."""
        if not x.is_cuda or self.is_residual or m > min(_fused_max_tokens(self.backend), 16):
            return False
        if self.bits > 16 or not self._mfma_layer():
            return False  # index widths the fused kernel does not stream (codebooks beyond 65536 rows)
        from .. import kernels

        bits = self.bits if self.bits in _FAST_BITS else 16  # as _kernel_stream
        return kernels.vq_linear_perm_supported(
            m, self.out_features, self.in_features, self.proxy.num_centroids, self.vector_len, bits
        )

    def _forward_sliced(self, x: torch.Tensor, sliced) -> torch.Tensor:
        from .. import kernels

        *leading, _ = x.shape
        perm = self._perm_i32(x.device) if self.column_perm is not None else None
        if x.device != self.packed_indices.device:
            raise RuntimeError(f"NPVQLinear: input on {x.device}, weights on {self.packed_indices.device}")
        x2d = x.reshape(-1, self.in_features)
        if x2d.stride(1) != 1:
            x2d = x2d.contiguous()
        try:
            # forward() has checked x's dtype and device; the other tensors come out of this
            # module's caches in the form the kernel reads.
            y = kernels.vq_linear_sliced_checked(
                x2d, sliced, self.proxy.centroids_as(x.dtype), self._bias_f32(), perm
            )
        except RuntimeError as exc:
            self._fallback("vq_linear_sliced", "decode + GEMM", exc)
            if self.column_perm is not None:
                x = x[..., self.column_perm]
            return self._forward_dequant_gemm(x)
        if x.dtype not in self._plans and not torch.cuda.is_current_stream_capturing():
            self._plan_sliced_calls(x.dtype, sliced, perm)
        return y.reshape(*leading, self.out_features)

    def _plan_sliced_calls(self, dtype: torch.dtype, sliced, perm) -> None:
        """Remember how the slice-list call for *dtype* activations was made, with the buffers it was
        made from: forward() reuses it while those are the module's buffers and unwritten."""
        from .. import kernels

        hit = self._derived_hit("sliced", self.packed_indices)
        if hit is None or hit[0] is not sliced:
            return
        packed, bias, column_perm, cent = self.packed_indices, self.bias, self.column_perm, self.proxy.centroids
        plan = kernels.SlicedCallPlan(sliced, self.proxy.centroids_as(dtype), self._bias_f32(), perm, dtype,
                                      min(hit[1], _SLICED_MAX_TOKENS, _fused_max_tokens(self.backend)))  # fmt: skip
        try:
            versions = _versions_of(packed, bias, column_perm, cent)
        except RuntimeError:  # inference tensors count no versions: writes into them go unseen, as for every cache here
            versions = None
        self._plans[dtype] = (plan, packed, bias, column_perm, cent, versions)

    def _mfma_layer(self) -> bool:
        """Whether the MFMA kernels take this layer's shape (vector length 8, K a multiple of 64)."""
        ok = self._derived.get("mfma_layer")
        if ok is None:
            from .. import kernels

            bits = self.bits if (self.bits in _FAST_BITS or self.bits > 16) else 16  # as _kernel_stream
            ok = kernels.vq_fused_supported(self.in_features, self.vector_len, bits)
            self._derived["mfma_layer"] = ok
        return ok

    def _wide_tile_layer(self) -> bool:
        """Whether the tile GEMM of this layer is the 128-column kernel (codebook kept in memory)."""
        return (
            not self.is_residual
            and self.vector_len == 8
            and 12 < self.bits <= 16  # read as a 16-bit stream (see _kernel_stream)
            and self.proxy.num_centroids * self.vector_len * 2 > 65536
        )

    def _tile_max_tokens(self) -> int:
        """Upper end of the tile-decode GEMM band for this layer."""
        if _TILE_MAX_TOKENS > 0 and self._wide_tile_layer():
            weights = self.in_features * self.out_features
            if weights >= _TILE_WIDE_MIN_WEIGHTS:
                return max(_TILE_MAX_TOKENS, _TILE_WIDE_MAX_TOKENS)
            if weights >= _TILE_WIDE_SMALL_WEIGHTS:
                return min(_TILE_WIDE_MAX_TOKENS, _TILE_WIDE_MID_MAX_TOKENS)
            return min(_TILE_WIDE_MAX_TOKENS, _TILE_WIDE_SMALL_MAX_TOKENS)
        return _TILE_MAX_TOKENS

    def _tile_band_ok(self, x: torch.Tensor, m: int) -> bool:
        """True when the tile GEMM's grid (64 columns x up to 384 rows per workgroup,
        times the reduction splits the kernel adds for layers with few output
        features) covers at least ``_TILE_MIN_GRID_FRACTION`` of the compute units."""
        if not x.is_cuda:
            return True
        if not self._mfma_layer():
            return False  # the tile entry point would run its element-wise fallback
        if self._wide_tile_layer():
            return True  # the 128-column kernel fills the GPU by splitting the reduction; its band is a token count
        cus = self._derived.get("cus")
        if cus is None:
            cus = torch.cuda.get_device_properties(x.device).multi_processor_count
            self._derived["cus"] = cus
        return tile_band_ok(
            m, self.out_features, self.in_features, cus,
            _TILE_MIN_GRID_FRACTION, _TILE_SPLIT_MAX_TOKENS, _TILE_SPLIT_LONG_K,
        )  # fmt: skip

    # -- torch-op paths ---------------------------------------------------

    def _dense_weight_torch(self, dtype: torch.dtype) -> torch.Tensor:
        idx = IndexPacking.unpack(self.packed_indices, self.bits, self.n_vectors)
        w = self.proxy.centroids[idx]
        if self.is_residual:
            if self.residual_proxy is not None:
                ir = IndexPacking.unpack(self.packed_residual, self.residual_bits, self.n_vectors)
                w = w + self.residual_proxy.centroids[ir]
            w = w.reshape(self.out_features, self.in_features)
            if self.row_scale is not None:
                w = w * self.row_scale[:, None]
            if self.row_bias is not None:
                w = w + self.row_bias[:, None]
        return w.reshape(self.out_features, self.in_features).to(dtype)

    def _forward_default(self, x: torch.Tensor) -> torch.Tensor:
        """Follows neuropress/nn/np_vq_linear.py:1091-1095."""
        if self.is_residual:
            return F.linear(x, self._dense_weight_torch(x.dtype), self._bias_as(x.dtype))
        return _vq_dequant_linear(
            x, self.packed_indices, self.proxy.centroids, self.bits, self.n_vectors,
            self.out_features, self.in_features, self._bias_as(x.dtype),
        )  # fmt: skip

    def _forward_compile(self, x: torch.Tensor) -> torch.Tensor:
        """The reference compiles the gather path with a tracing compiler
        (np_vq_linear.py:1150-1160); here the same ops run eagerly."""
        return self._forward_default(x)

    # -- HIP paths --------------------------------------------------------

    def _fallback(self, kernel: str, fallback: str, exc: Exception) -> None:
        """Re-raise unless fallbacks were opted into; then warn once per kernel."""
        if not _ALLOW_FALLBACK:
            raise exc
        from .. import kernels

        kernels.warn_kernel_fallback(kernel, fallback, exc)

    def _forward_dequant_gemm(self, x: torch.Tensor) -> torch.Tensor:
        """Band (c): decode the weight in one kernel pass, then a dense GEMM.

        Follows neuropress/nn/np_vq_linear.py:1127-1148.  The decoded ``[N, K]``
        weight is a temporary returned to the allocator after the matmul.
        """
        from .. import kernels

        try:
            if self.is_residual:
                w = kernels.rvq_dequant(
                    self.packed_indices, self.bits, self._res_stream(), self._res_bits(),
                    self.proxy.centroids, self._res_centroids(), self.row_scale, self.row_bias,
                    self.out_features, self.in_features, x.dtype,
                )  # fmt: skip
            else:
                w = kernels.vq_dequant(
                    self.packed_indices, self.proxy.centroids, self.bits,
                    self.out_features, self.in_features, x.dtype,
                )  # fmt: skip
        except RuntimeError as exc:
            self._fallback("vq_dequant", "the gather path", exc)
            return self._forward_compile(x)
        return F.linear(x, w, self._bias_as(x.dtype))

    def _forward_tile_gemm(self, x: torch.Tensor) -> torch.Tensor:
        """Band (b): MFMA GEMM decoding weight tiles in-kernel.

        Takes the place of the reference's Triton band (np_vq_linear.py:1097-1125).
        """
        global _tile_failed
        if _tile_failed or x.dtype not in (torch.bfloat16, torch.float16):
            return self._forward_dequant_gemm(x)
        try:
            y = self._fused(x, tile=True)
        except RuntimeError as exc:
            self._fallback("vq_gemm_tile", "decode + GEMM", exc)
            _tile_failed = True
            return self._forward_dequant_gemm(x)
        return y

    def _res_stream(self) -> torch.Tensor:
        if self.packed_residual is not None:
            return self.packed_residual
        dev = self.packed_indices.device
        return self._derive("zero_res", self.packed_indices, lambda: torch.zeros(self.n_vectors, dtype=torch.uint8, device=dev))

    def _res_bits(self) -> int:
        return self.residual_bits if self.packed_residual is not None else 8

    def _res_centroids(self) -> torch.Tensor:
        if self.residual_proxy is not None:
            return self.residual_proxy.centroids
        dev = self.packed_indices.device
        return self._derive(
            "zero_cb", self.packed_indices, lambda: torch.zeros((1, self.vector_len), dtype=torch.float16, device=dev)
        )

    def _fused(self, x: torch.Tensor, tile: bool, perm: torch.Tensor | None = None) -> torch.Tensor:
        from .. import kernels

        *leading, _ = x.shape
        x2d = x.reshape(-1, self.in_features)
        if self.is_residual:
            y = kernels.rvq_linear(
                x2d, self.packed_indices, self.bits, self._res_stream(), self._res_bits(),
                self.proxy.centroids, self._res_centroids(), self.row_scale, self.row_bias,
                self.out_features, self._bias_f32(), tile=tile,
            )  # fmt: skip
        else:
            stream, bits = self._kernel_stream()
            cb = self.proxy.centroids_as(x.dtype)
            fn = kernels.vq_gemm_tile if tile else kernels.vq_linear
            if tile:
                y = fn(x2d, stream, cb, bits, self.out_features, self._bias_f32())
            else:
                y = fn(x2d, stream, cb, bits, self.vector_len, self._bias_f32(), self.out_features,
                       column_perm=perm)  # fmt: skip
        return y.reshape(*leading, self.out_features)

    def _forward_cuda(self, x: torch.Tensor) -> torch.Tensor:
        """Band (a) (reference: np_vq_linear.py:1173-1187).  Above the kernel's
        32-token limit (reachable only with a raised threshold) the tile GEMM runs."""
        m = x.numel() // self.in_features
        return self._fused(x, tile=m > _GEMV_KERNEL_MAX_TOKENS)

    def _forward_cuda_wmma(self, x: torch.Tensor) -> torch.Tensor:
        """GEMV / GEMM by token count (reference: np_vq_linear.py:1250-1267)."""
        m = x.numel() // self.in_features
        return self._fused(x, tile=m > _GEMV_KERNEL_MAX_TOKENS)

    def _forward_cuda_lut(self, x: torch.Tensor) -> torch.Tensor:
        """Reached only when ``_LUT_MAX_TOKENS`` was raised above 0.

        The reference's LUT kernel (np_vq_linear.py:1192-1248) builds an
        ``[M, n_groups, NC]`` table, which for the codebooks it is chosen for is
        larger than the weight and loses at every M (np_vq_linear.py:75-79);
        it is not rebuilt.  The same result is produced by the fused kernels.
        """
        m = x.numel() // self.in_features
        return self._fused(x, tile=m > _GEMV_KERNEL_MAX_TOKENS)

    # ------------------------------------------------------------------

    def extra_repr(self) -> str:
        perm_str = ", perm=True" if self.column_perm is not None else ""
        res_str = ", residual=True" if self.is_residual else ""
        if self.zero_escape:
            tiered_str = ", zero_escape=True"
        elif self.tier_bits is not None:
            tiered_str = f", ntier={self.tier_bits}"
        elif self.use_tiered:
            tiered_str = f", tiered=True(cold={self.cold_bits})"
        else:
            tiered_str = ""
        return (
            f"in={self.in_features}, out={self.out_features}, "
            f"vector_len={self.vector_len}, "
            f"num_centroids={self.proxy.num_centroids}, "
            f"bits={self.bits}, backend={self.backend.value}"
            f"{perm_str}{tiered_str}{res_str}"
        )


# ---------------------------------------------------------------------------
# Model-level transform
# ---------------------------------------------------------------------------


def linearize_vq_weights(
    model: nn.Module,
    backend: str | VQBackend | None = VQBackend.AUTO,
) -> nn.Module:
    """Replace every ``nn.Linear`` carrying a VQ weight with an :class:`NPVQLinear`.

    Follows neuropress/nn/np_vq_linear.py:1432-1517: layers whose codebook is
    the same tensor object share one :class:`VQProxy`; each unique proxy is
    registered on the model root as ``_vq_proxy_<i>`` (residual codebooks as
    ``_vq_res_proxy_<i>``).  The model is mutated in place and returned.
    """
    proxy_cache: dict[int, VQProxy] = {}
    res_cache: dict[int, VQProxy] = {}
    replacements: list[tuple[str, NPVQLinear]] = []

    for name, module in model.named_modules():
        if not isinstance(module, nn.Linear) or not is_vq_weight(module.weight):
            continue
        qs = module.weight.qscheme
        cid = id(qs.centroids)
        if cid not in proxy_cache:
            proxy_cache[cid] = VQProxy(qs.centroids)
        res_proxy = None
        res_c = getattr(qs, "residual_centroids", None)
        if res_c is not None:
            if id(res_c) not in res_cache:
                res_cache[id(res_c)] = VQProxy(res_c)
            res_proxy = res_cache[id(res_c)]
        try:
            layer = NPVQLinear.from_qtensor_linear(module, proxy_cache[cid], backend, res_proxy)
        except (TypeError, ValueError, NotImplementedError) as exc:
            log.warning("linearize_vq_weights: skipping %s — %s", name, exc)
            continue
        replacements.append((name, layer))

    if not replacements:
        log.info("linearize_vq_weights: no VQ-weight linear layers found.")
        return model

    for i, proxy in enumerate(proxy_cache.values()):
        model.add_module(f"_vq_proxy_{i}", proxy)
    for i, proxy in enumerate(res_cache.values()):
        model.add_module(f"_vq_res_proxy_{i}", proxy)

    for name, layer in replacements:
        if "." in name:
            parent_name, attr = name.rsplit(".", 1)
            parent = model.get_submodule(parent_name)
        else:
            parent, attr = model, name
        setattr(parent, attr, layer)

    counts: dict[str, int] = {}
    for _, layer in replacements:
        counts[layer.backend.value] = counts.get(layer.backend.value, 0) + 1
    summary = ", ".join(f"{v}x{k}" for k, v in sorted(counts.items()))
    log.info(
        "linearize_vq_weights: replaced %d layer(s) [%s], %d unique proxy/ies",
        len(replacements),
        summary,
        len(proxy_cache),
    )
    return model
