"""The product kernel backend: hand-written HIP for gfx950 behind a C interface.

Each call checks shapes and dtypes on the host, launches on torch's current
stream and raises with the library's message if the library refuses. torch is
the allocator and nothing else here. A missing library is compiled at first use;
if that fails the call fails: there is no other path.
"""
import ctypes
from typing import Dict, Optional

import numpy as np
import torch

from . import build
from .attention_plan import QUERY_TILE
from .. import debug

_F32, _BF16 = 0, 1
_ACT = {None: 0, "none": 0, "relu": 1, "gelu": 2, "gelu_new": 3}
_LIBS: Dict[str, ctypes.CDLL] = {}

_c_void_p, _c_int, _c_float, _c_ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong

_SIGNATURES = {
    "elementwise": {
        "tnx_gather_rows": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_void_p],
        "tnx_copy_ints": [_c_void_p, _c_void_p, _c_int, _c_void_p],
        "tnx_device_pointer": [_c_void_p, _c_void_p],
        "tnx_add_positions": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
                              _c_int, _c_int, _c_int, _c_void_p],
        "tnx_cast": [_c_void_p, _c_int, _c_void_p, _c_int, _c_ll, _c_void_p],
        "tnx_epilogue": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_layernorm": [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                          _c_int, _c_void_p],
    },
    "gemm": {
        "tnx_gemm_f32": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                         _c_int, _c_void_p],
        "tnx_gemm_bf16": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                          _c_int, _c_int, _c_int, _c_void_p],
        "tnx_gemm_bf16_qkv": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
                              _c_void_p, _c_void_p, _c_void_p, _c_float, _c_int, _c_int, _c_int, _c_int, _c_int,
                              _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
        "tnx_gemm_skinny_tiles_per_block": [_c_int, _c_int],
        "tnx_gemm_bf16_mid": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                              _c_int, _c_void_p, ctypes.c_size_t, _c_int, _c_int, _c_void_p],
        "tnx_gemm_library": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                             _c_int, _c_void_p, ctypes.c_size_t, _c_void_p, ctypes.c_size_t, _c_int, _c_void_p],
        "tnx_gemm_bf16_normed": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_int,
                                 _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_gemm_bf16_qkv_normed": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int,
                                     _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_int, _c_int,
                                     _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                                     _c_int, _c_void_p],
    },
    "attention": {
        "tnx_qkv_write": [_c_void_p, _c_int, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                          _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p,
                          _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_int,
                          _c_void_p],
        "tnx_attention_any": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                              _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_attention_prefill": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                                  _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                                  _c_int, _c_int, _c_int, _c_void_p],
        "tnx_attention_decode": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                                 _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                                 _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_void_p],
        "tnx_attention_decode_static": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                        _c_int, _c_int, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                                        _c_int, _c_int, _c_void_p, _c_void_p],
    },
    "sampling": {
        "tnx_ban_tokens": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
        "tnx_ban_pairs": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_argmax": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
        "tnx_store_tokens": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p,
                             _c_void_p],
        "tnx_sample": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                       _c_int, _c_void_p],
    },
    "probe": {
        "tnx_probe_stream_read": [_c_void_p, ctypes.c_size_t, _c_void_p, _c_int, _c_void_p],
        "tnx_probe_mfma_loop": [_c_int, _c_int, _c_void_p, _c_void_p],
    },
}


def register_signatures(module: str, signatures: Dict[str, list]) -> None:
    """The C entry points (name -> ctypes argument types, all returning int) of a kernel module registered
    with `build.register_module`."""
    _SIGNATURES.setdefault(module, {}).update(signatures)


class PreparedWeight:
    """A `[out, in]` matrix as the kernels want it: the tensor itself, and beside it (bfloat16, `out` a
    multiple of 16, `in` of 128) a copy in the order the few-rows kernel streams it,
    `[out/16][in/128][4][16][4][8]`: each block then reads one contiguous run of memory. The copy doubles
    the memory of the matrices; it is what decoding reads, the plain tensor is what prompts read."""

    __slots__ = ("tensor", "tiles", "folded", "inner")

    def __init__(self, tensor: torch.Tensor, tiles: Optional[torch.Tensor], inner: Optional[int] = None):
        self.tensor, self.tiles = tensor, tiles
        self.folded: Optional["FoldedNorm"] = None
        # the matrix's own inner size where `tensor` carries columns of zeros after it (bfloat16 rows are
        # read 16 bytes at a time: an inner size that is no multiple of 8 is filled up once, here, and the
        # rows that meet it are filled up as they come)
        self.inner = tensor.shape[1] if inner is None else inner

    @property
    def shape(self):
        return torch.Size((self.tensor.shape[0], self.inner))

    @property
    def dtype(self):
        return self.tensor.dtype


class FoldedNorm:
    """A matrix with the LayerNorm in front of it folded in, for the few-rows kernel: `tiles` is
    W diag(gamma) in tile order, `c` its row sums (of the rounded values, which are what is multiplied),
    `d` = W beta; `key` names the norm's tensors it was made from."""

    __slots__ = ("tiles", "c", "d", "key", "_with_bias")

    def __init__(self, tiles, c, d, key):
        self.tiles, self.c, self.d, self.key = tiles, c, d, key
        self._with_bias = {}

    def d_with(self, bias):
        """`d + bias`: what a plain product of the folded copy with rows that are normalised but not yet
        scaled adds (made once a bias vector)."""
        if bias is None:
            return self.d
        k = bias.data_ptr()
        if k not in self._with_bias:
            self._with_bias[k] = (self.d + bias).contiguous()
        return self._with_bias[k]


class DeferredNorm:
    """The input of a LayerNorm whose output only a matrix product reads: the product of few rows applies the
    norm itself (`HipOps.linear`, `HipOps.qkv_project`); whoever else gets one calls `materialize()`."""

    __slots__ = ("ops", "x", "weight", "bias", "eps", "dtype", "center")

    def __init__(self, ops, x, weight, bias, eps, dtype, center=True):
        self.ops, self.x, self.weight, self.bias, self.eps, self.dtype = ops, x, weight, bias, eps, dtype
        self.center = center

    @property
    def shape(self):
        return self.x.shape

    @property
    def key(self):
        return (self.weight.data_ptr() if self.weight is not None else 0,
                self.bias.data_ptr() if self.bias is not None else 0, bool(self.center))

    def materialize(self):
        return self.ops.layernorm(self.x, self.weight, self.bias, self.eps, self.dtype, False, True, self.center)[1]

    def normalised(self):
        """`(x - mean) rstd` alone, for a product with a folded copy."""
        return self.ops.layernorm(self.x, None, None, self.eps, self.dtype, False, True, self.center)[1]


def tile_order(w: torch.Tensor) -> torch.Tensor:
    """`w[n, k]` -> `[n/16][k/128][s][r][g][e]` with n = 16*nt + r and k = 128*kt + 32*s + 8*g + e."""
    n, k = w.shape
    return w.view(n // 16, 16, k // 128, 4, 4, 8).permute(0, 2, 3, 1, 4, 5).contiguous()


def library(module: str) -> ctypes.CDLL:
    """The compiled library of a kernel module, compiled now if it is not there."""
    lib = _LIBS.get(module)
    if lib is None:
        path = build.find_library(module) or build.compile_module(module)
        lib = ctypes.CDLL(path)
        lib.tnx_last_error.restype = ctypes.c_char_p
        for name, argtypes in _SIGNATURES[module].items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _c_int
        _LIBS[module] = lib
    return lib


def loaded_libraries() -> Dict[str, str]:
    return {m: lib._name for m, lib in _LIBS.items()}


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise TypeError(f"the kernels take float32 and bfloat16, not {dtype}")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _want(t: torch.Tensor, name: str, dtype=None, shape=None):
    if not t.is_cuda:
        raise ValueError(f"{name} must be on the GPU")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    return t


class HipOps:
    name = "hip"

    def __init__(self, dtype: torch.dtype, device="cuda:0"):
        self.dtype = dtype
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise RuntimeError("the HIP kernels need a GPU; none is visible to torch")
        _code(dtype)
        self.compute_units = torch.cuda.get_device_properties(self.device).multi_processor_count
        self._bias_copies = {}
        self._later = []
        self._tiles_per_block = {}
        self._landing, self._landing_turn = [None, None], 0
        self._ints, self._ints_done, self._ints_turn = [None, None], [None, None], 0

    def _call(self, module: str, fn: str, *args, work=None):
        """`work` = (what, bytes, flops) names the launch for a kernel timer: what it is (its sizes), what it has
        to read and write once, and its multiply-adds times two."""
        lib = library(module)
        timer = debug.timer()
        end = None
        if timer is not None:
            end = timer.start(fn, 0, 0) if work is None else timer.start(f"{fn} {work[0]}", work[1], work[2])
        rc = getattr(lib, fn)(*args)
        if end is not None:
            end.record()
        if rc != 0:
            raise RuntimeError(f"{fn}: {lib.tnx_last_error().decode()}")

    def call(self, module: str, fn: str, *args) -> None:
        """An entry point of any registered kernel module (also one a part brought itself); `stream()` and
        `pointer()` give what such entry points take."""
        self._call(module, fn, *args)

    stream = staticmethod(_stream)
    pointer = staticmethod(_ptr)

    @staticmethod
    def _product_work(m, n, k, item=2, x_item=2, out_item=2, residual=False):
        """What a product out[m, n] = x[m, k] w[n, k]^T is for a kernel timer: its sizes, the bytes it has to move
        (the matrix, the rows, the result, the residual) and its flops."""
        return (f"{m}x{n}x{k}", n * k * item + m * k * x_item + m * n * (out_item + (4 if residual else 0)), 2.0 * m * n * k)

    @staticmethod
    def _attention_work(ctx, which, num_heads, num_kv_heads, head_size, window, item):
        """The same for the attention of a step's decoding runs (`which` "decode": bytes of the keys and values
        they read) or of its longer runs ("prompt": flops of scores and weighted values under the causal mask)."""
        lens, cached = ctx.run_lens_host.astype(np.float64), ctx.cached_lens_host.astype(np.float64)
        pick = lens == 1 if which == "decode" else lens > 1
        seen = cached[pick] + (lens[pick] + 1) / 2                     # keys a query of the run sees on average
        if window:
            seen = np.minimum(seen, window)
        keys = float((lens[pick] * seen).sum())
        nbytes = float((np.minimum(cached[pick] + lens[pick], window or 1e18)).sum()) * 2 * num_kv_heads * head_size * item
        return (f"{which} {int(pick.sum())} runs", nbytes, 4.0 * num_heads * head_size * keys)

    # ---------------------------------------------------------------- input end

    def gather_rows(self, x, rows, indirect=None):
        """`x[rows]`; a row number -1 - k stands for `indirect[k]` (int32, on the device)."""
        _want(x, "x")
        _want(rows, "rows", torch.int32)
        if x.dim() != 2:
            raise ValueError("gather_rows takes a matrix")
        if indirect is not None:
            _want(indirect, "indirect rows", torch.int32)
        out = torch.empty(rows.numel(), x.shape[1], dtype=x.dtype, device=x.device)
        self._call("elementwise", "tnx_gather_rows", _ptr(x), _ptr(rows), _ptr(out), rows.numel(),
                   x.shape[1] * x.element_size(), x.shape[0], _ptr(indirect),
                   indirect.numel() if indirect is not None else 0, _stream())
        return out

    def embed(self, token_ids, table, dtype=None, kept_tokens=None):
        """Rows of the token table; an id -1 - k is the token kept in `kept_tokens[k]`."""
        return self.gather_rows(table, token_ids, kept_tokens)

    def pinned_ints(self, n: int):
        """`n` int32 in pinned host memory, and the address under which kernels reach them."""
        host = torch.empty(n, dtype=torch.int32, pin_memory=True)
        address = ctypes.c_void_p()
        self._call("elementwise", "tnx_device_pointer", ctypes.c_void_p(host.data_ptr()), ctypes.byref(address))
        return host, address

    def copy_ints(self, dst, pinned, n=None) -> None:
        """`dst[:n] = host[:n]` for what `pinned_ints` returned, by a kernel on the current stream."""
        host, address = pinned
        n = host.numel() if n is None else n
        _want(dst, "dst", torch.int32)
        if n > host.numel() or n > dst.numel():
            raise ValueError(f"copy_ints: {n} integers from {host.numel()} into {dst.numel()}")
        self._call("elementwise", "tnx_copy_ints", address, _ptr(dst), n, _stream())

    def send_ints(self, flat):
        """A host array of int32 as a device tensor, through pinned memory and a copy kernel (two buffers
        in turn; one is written again only when the copy that read it has run)."""
        n = flat.size
        self._ints_turn ^= 1
        i = self._ints_turn
        if self._ints_done[i] is not None:
            self._ints_done[i].synchronize()   # also before a buffer is replaced: its copy may still read it
        if self._ints[i] is None or self._ints[i][0].numel() < n:
            self._ints[i] = self.pinned_ints(max(2 * n, 1024))
        self._ints[i][0].numpy()[:n] = flat
        dst = torch.empty(n, dtype=torch.int32, device=self.device)
        self.copy_ints(dst, self._ints[i], n)
        if self._ints_done[i] is None:
            self._ints_done[i] = torch.cuda.Event()
        self._ints_done[i].record()
        return dst

    def send_tokens(self, tokens, kept, ctx):
        """Leave the chosen tokens for the next step (`kept[slot]`, see `store_tokens`) and write them into
        pinned host memory by the same kernel. Returns what `receive_tokens` takes."""
        n = tokens.numel()
        self._landing_turn ^= 1
        pinned = self._landing[self._landing_turn]
        if pinned is None or pinned[0].numel() < n:
            pinned = self._landing[self._landing_turn] = self.pinned_ints(max(2 * n, 256))
        self.store_tokens(kept, tokens, ctx, pinned[1])
        landed = torch.cuda.Event()
        landed.record()
        return pinned[0], n, landed

    def receive_tokens(self, sent):
        host, n, landed = sent
        landed.synchronize()
        return host[:n].tolist()

    def store_tokens(self, kept, tokens, ctx, landing=None):
        """`kept[slot]` = the token chosen for the request in that slot; `tokens[i]` belongs to the
        request of the step's i-th wanted row. `landing`: an address in pinned host memory that gets
        the tokens too."""
        _want(kept, "kept tokens", torch.int32)
        _want(tokens, "tokens", torch.int32, (ctx.logits_rows.numel(),))
        self._call("sampling", "tnx_store_tokens", _ptr(tokens), _ptr(ctx.logits_rows), _ptr(ctx.token_request),
                   _ptr(ctx.slots), tokens.numel(), _ptr(kept), kept.numel(), landing, _stream())

    def add_positions(self, src, positions, table, offset, dtype, want_compute):
        _want(src, "src")
        t, width = src.shape
        _want(positions, "positions", torch.int32, (t,))
        _want(table, "position table")
        if table.shape[1] != width:
            raise ValueError(f"position table is {table.shape[1]} wide, the tokens {width}")
        out = torch.empty(t, width, dtype=torch.float32, device=src.device)
        cd = torch.empty(t, width, dtype=dtype, device=src.device) if want_compute and dtype != torch.float32 else None
        self._call("elementwise", "tnx_add_positions", _ptr(src), _code(src.dtype), _ptr(positions), _ptr(table),
                   _code(table.dtype), table.shape[0], offset, _ptr(out), _ptr(cd), _code(dtype), t, width, _stream())
        return out, ((cd if cd is not None else out) if want_compute else None)

    def to_stream(self, src, dtype, want_compute):
        _want(src, "src")
        t, width = src.shape
        out = torch.empty(t, width, dtype=torch.float32, device=src.device)
        cd = torch.empty(t, width, dtype=dtype, device=src.device) if want_compute and dtype != torch.float32 else None
        self._call("elementwise", "tnx_add_positions", _ptr(src), _code(src.dtype), None, None, 0, 0, 0, _ptr(out),
                   _ptr(cd), _code(dtype), t, width, _stream())
        return out, ((cd if cd is not None else out) if want_compute else None)

    def cast(self, x, dtype):
        _want(x, "x")
        if x.dtype == dtype:
            return x
        out = torch.empty_like(x, dtype=dtype)
        self._call("elementwise", "tnx_cast", _ptr(x), _code(x.dtype), _ptr(out), _code(dtype), x.numel(), _stream())
        return out

    # ---------------------------------------------------------------- norms

    def layernorm(self, x, weight, bias, eps, dtype, want_f32, want_compute, center=True):
        """`center=False`: the norm that only scales, x / sqrt(mean(x^2) + eps) (times weight, plus bias)."""
        _want(x, "x", torch.float32)
        t, width = x.shape
        if weight is not None:
            _want(weight, "norm weight", torch.float32, (width,))
        if bias is not None:
            _want(bias, "norm bias", torch.float32, (width,))
        same = dtype == torch.float32
        out_f32 = torch.empty_like(x) if (want_f32 or (want_compute and same)) else None
        out_cd = torch.empty(t, width, dtype=dtype, device=x.device) if (want_compute and not same) else None
        self._call("elementwise", "tnx_layernorm", _ptr(x), _ptr(weight), _ptr(bias), float(eps), _ptr(out_f32),
                   _ptr(out_cd), _code(dtype), t, width, int(bool(center)), _stream())
        return (out_f32 if want_f32 else None), ((out_f32 if same else out_cd) if want_compute else None)

    # Steps of few rows: a LayerNorm that only a matrix product reads is done by that product (`fold_norm`,
    # `layernorm_deferred`). Up to `fuse_norm_rows` rows the few-rows kernel reads the float32 rows itself
    # (measured at 4,096 -> 12,288: 23.0 us against 24.4 for norm and product at 8 rows, but 25.8 against 25.2 at
    # 16 and twice the time at 32: every block reads all rows, and these are float32); beyond that, as far as
    # the few-rows kernel goes, the norm's kernel normalises and the folded copy does the rest.
    # Where the blocks take one tile of weight rows each (what `tnx_gemm_skinny_tiles_per_block` says), every
    # 32 bytes of weight come with 64 of float32 rows and the norm's own kernel is the cheaper way again
    # (9,216 -> 27,648 at 8 rows: 120 us against 10 + 91). And where the blocks between them read more than
    # `fuse_norm_bytes` of rows: 4,096 -> 16,384, 512 blocks of two tiles, is 0.3 to 0.6 us quicker with the norm
    # inside up to 4 rows, as quick at 6 (50 MB of rows) and 0.8 us slower at 8 (28.1 against 27.3 us), while
    # 4,096 -> 12,288, 256 blocks of three, stays 0.6 us quicker at 8 rows (34 MB); 9,216 -> 36,864 at 8 rows
    # (226 MB): 111.1 us against 106.3.
    fuse_norm = True
    fuse_norm_rows = 8
    fuse_norm_bytes = 40 << 20

    def _norm_in_the_product(self, m, n, k) -> bool:
        if m > self.fuse_norm_rows:
            return False
        key = (m, n)
        if key not in self._tiles_per_block:
            self._tiles_per_block[key] = library("gemm").tnx_gemm_skinny_tiles_per_block(m, n)
        tiles = self._tiles_per_block[key]
        blocks = -(-(n // 16) // tiles)
        return tiles >= 2 and blocks * m * k * 4 <= self.fuse_norm_bytes
    few_rows = 32           # the few-rows kernel takes up to this many rows

    def fold_norm(self, w, weight, bias, center=True) -> bool:
        """Called once when a layer has its tensors, for a matrix `w` that reads a LayerNorm's output and
        nothing else does: keeps, in the place of its tile-ordered copy, the copy with the norm's weight
        folded in and the two vectors that go with it (see `FoldedNorm`). False if this matrix has no such
        copy (then the norm stays a kernel of its own)."""
        if not (self.fuse_norm and self.dtype == torch.bfloat16 and isinstance(w, PreparedWeight)
                and w.tiles is not None and w.tensor.dtype == torch.bfloat16):
            return False
        full = w.tensor.float()
        scaled = (full * weight.float()[None, :] if weight is not None else full).to(torch.bfloat16)
        c = scaled.float().sum(dim=1).contiguous()
        d = (full @ bias.float() if bias is not None else torch.zeros_like(c)).contiguous()
        key = (weight.data_ptr() if weight is not None else 0, bias.data_ptr() if bias is not None else 0, bool(center))
        w.folded = FoldedNorm(tile_order(scaled), c, d, key)
        w.tiles = None          # the few-rows steps read the folded copy; the memory stays what it was
        return True

    def layernorm_deferred(self, x, weight, bias, eps, dtype, center=True):
        """The compute-dtype output of the norm, or, in steps of few rows, a `DeferredNorm`."""
        if self.fuse_norm and dtype == torch.bfloat16 and self.dtype == torch.bfloat16 \
                and x.shape[0] <= self.few_rows and x.shape[1] % 128 == 0 and not debug.tapping():
            return DeferredNorm(self, x, weight, bias, eps, dtype, center)
        return self.layernorm(x, weight, bias, eps, dtype, False, True, center)[1]

    def _folded_for(self, h, w):
        """The folded copy of `w` that fits the deferred norm `h`, or None."""
        if isinstance(w, PreparedWeight) and w.folded is not None and w.folded.key == h.key:
            return w.folded
        return None

    # ---------------------------------------------------------------- matrix products

    # Keep a tile-ordered copy of every matrix for the few-rows kernel: True, False, or "later", when they do
    # not all fit: then `finish_weights` makes those a number of bytes allows, once everything else is loaded.
    decode_copies = True

    def prepare_weight(self, w: torch.Tensor) -> PreparedWeight:
        """Called once per matrix when a part receives its tensors."""
        tiles = None
        fits = (self.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2
                and w.shape[0] % 16 == 0 and w.shape[1] % 128 == 0)
        if fits and self.decode_copies == "later":
            pw = PreparedWeight(w, None)
            self._later.append(pw)
            return pw
        if fits and self.decode_copies:
            tiles = tile_order(w)
        if self.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] % 8:
            inner = w.shape[1]
            return PreparedWeight(torch.nn.functional.pad(w, (0, 8 - inner % 8)).contiguous(), None, inner)
        return PreparedWeight(w, tiles)

    def finish_weights(self, budget_bytes: int) -> int:
        """The tile-ordered copies that `budget_bytes` allow, of the matrices that waited for them: those
        with the fewest rows first (measured at OPT-66B sizes, 8 rows: the copy saves 5 us of 37 for
        9,216 x 9,216, 20 of 134 for 9,216 x 36,864, 14 of 105 for 27,648 x 9,216 and 6 of 121 for
        36,864 x 9,216, that is 29, 29, 28 and 8 us a GB). Returns the bytes taken."""
        taken = 0
        waiting, self._later = self._later, []
        for pw in sorted(waiting, key=lambda pw: pw.tensor.shape[0]):      # (stable: layer order within a size)
            size = pw.tensor.numel() * pw.tensor.element_size()
            if pw.tiles is None and taken + size <= budget_bytes:
                pw.tiles = tile_order(pw.tensor)
                taken += size
        return taken

    def linear(self, x, w, bias=None, act=None, residual=None, out_f32=False, force_tiled=False):
        if isinstance(x, DeferredNorm):
            folded = self._folded_for(x, w) if (residual is None and not out_f32 and force_tiled != 1) else None
            if folded is not None and self._library_product(x.shape[0], w.tensor.shape[0], w.tensor.shape[1],
                                                              w.tensor, force_tiled):
                folded = None
            if folded is None:
                x = x.materialize()
            elif not self._norm_in_the_product(x.shape[0], w.tensor.shape[0], w.tensor.shape[1]):
                # the norm's kernel without weight and bias, then the plain product of the folded copy
                m, k = x.shape
                n = w.tensor.shape[0]
                out = torch.empty(m, n, dtype=self.dtype, device=x.x.device)
                rows, shift = x.normalised(), folded.d_with(bias)     # held until the launch is made
                self._call("gemm", "tnx_gemm_bf16", _ptr(rows), _ptr(w.tensor), _ptr(folded.tiles), _ptr(shift), None,
                           _ptr(out), _code(self.dtype), _ACT[act], m, n, k, int(force_tiled), _stream(),
                           work=self._product_work(m, n, k))
                return out
            else:
                if act not in _ACT:
                    raise ValueError(f"unknown activation {act!r}")
                m, k = x.shape
                n = w.tensor.shape[0]
                if bias is not None:
                    _want(bias, "bias", torch.float32, (n,))
                out = torch.empty(m, n, dtype=self.dtype, device=x.x.device)
                self._call("gemm", "tnx_gemm_bf16_normed", _ptr(x.x), _ptr(folded.tiles), _ptr(folded.c),
                           _ptr(folded.d), float(x.eps), _ptr(bias), _ptr(out), _code(self.dtype), _ACT[act], m, n, k,
                           int(force_tiled), int(bool(x.center)), _stream(), work=self._product_work(m, n, k, x_item=4))
                return out
        tiles = None
        if isinstance(w, PreparedWeight):
            if w.inner != w.tensor.shape[1] and x.shape[1] == w.inner:
                x = torch.nn.functional.pad(x, (0, w.tensor.shape[1] - w.inner))
            w, tiles = w.tensor, w.tiles
        _want(x, "x")
        _want(w, "w")
        if act not in _ACT:
            raise ValueError(f"unknown activation {act!r}")
        m, k = x.shape
        n, kw = w.shape
        if kw != k:
            raise ValueError(f"x is {k} wide, w takes {kw}")
        if bias is not None:
            _want(bias, "bias", torch.float32, (n,))
        if residual is not None:
            _want(residual, "residual", torch.float32, (m, n))
        out_dtype = torch.float32 if out_f32 else self.dtype
        if self._some_rows_product(m, n, k, w, tiles, residual, out_f32, force_tiled):
            # decode batches of 33 to 128 requests, a float32 result: our kernel for some rows
            out = torch.empty(m, n, dtype=out_dtype, device=x.device)
            space = self._library_workspace(x.device)
            self._call("gemm", "tnx_gemm_bf16_mid", _ptr(self.cast(x, torch.bfloat16)), _ptr(tiles), _ptr(bias),
                       _ptr(residual), _ptr(out), _code(out_dtype), _ACT[act], m, n, k, _ptr(space), space.numel() // 4,
                       0, 0, _stream(), work=self._product_work(m, n, k, out_item=4, residual=residual is not None))
            return out
        if (self._library_product(m, n, k, w, force_tiled) and (residual is not None or not out_f32)):
            # Many rows: the product goes to the vendor library (hipBLASLt), with what follows it where the
            # library can do that itself: bias and ReLU before it rounds a bfloat16 result, or bias and the
            # residual added to its float32 sums for a float32 result. The float32 head keeps our kernel.
            xa = self.cast(x, torch.bfloat16)
            # (its ReLU comes after everything it adds, so a product with both ReLU and a residual is not its)
            plain_act = act in (None, "none")
            if self.library_direct and (plain_act or (act == "relu" and residual is None)) \
                    and (residual is None or out_f32):
                out = torch.empty(m, n, dtype=out_dtype, device=x.device)
                if self._library_call(xa, w, bias, residual, out, act, m, n, k):
                    return out
            # Not to be had that way (another activation, no library to be found, no algorithm that fits):
            # the product through torch, and one kernel of ours for what follows it.
            if bias is not None and residual is None and not out_f32:
                b16 = self._bias_bf16(bias)
                if act == "relu":
                    return torch._addmm_activation(b16, xa, w.t(), use_gelu=False)
                y = torch.addmm(b16, xa, w.t())
                bias = None
            else:
                y = torch.mm(xa, w.t())
            out = torch.empty(m, n, dtype=out_dtype, device=x.device) if out_f32 else y
            if bias is not None or residual is not None or (act not in (None, "none")) or out_f32:
                self._call("elementwise", "tnx_epilogue", _ptr(y), _ptr(bias), _ACT[act], _ptr(residual), _ptr(out),
                           _code(out_dtype), m, n, _stream())
            return out
        out = torch.empty(m, n, dtype=out_dtype, device=x.device)
        if w.dtype == torch.float32:
            xa = self.cast(x, torch.float32)
            self._call("gemm", "tnx_gemm_f32", _ptr(xa), _ptr(w), _ptr(bias), _ptr(residual), _ptr(out),
                       _code(out_dtype), _ACT[act], m, n, k, _stream(),
                       work=self._product_work(m, n, k, 4, 4, out.element_size(), residual is not None))
        else:
            xa = self.cast(x, torch.bfloat16)
            self._call("gemm", "tnx_gemm_bf16", _ptr(xa), _ptr(w), _ptr(tiles), _ptr(bias), _ptr(residual),
                       _ptr(out), _code(out_dtype), _ACT[act], m, n, k, int(force_tiled), _stream(),
                       work=self._product_work(m, n, k, out_item=out.element_size(), residual=residual is not None))
        return out

    library_direct = True   # many-rows products as calls of the vendor library itself, with what follows them
    library_tune = 1        # and its algorithms timed once: 1, for products of few rows; 2, for every product
    _workspaces: Dict[str, torch.Tensor] = {}

    def _library_call(self, xa, w, bias, residual, out, act, m, n, k) -> bool:
        """`out = act(xa w^T + bias) + residual` by the vendor library; False where that is not to be had."""
        lib = library("gemm")
        space = self._library_workspace(xa.device)

        def call(flush, tune):
            return lib.tnx_gemm_library(_ptr(xa), _ptr(w), _ptr(bias), _ptr(residual), _ptr(out), _code(out.dtype),
                                        _ACT[act], m, n, k, _ptr(space), space.numel(), _ptr(flush),
                                        flush.numel() if flush is not None else 0, int(tune), _stream())
        timer = debug.timer()
        end = None
        if timer is not None:
            what, nbytes, flops = self._product_work(m, n, k, out_item=out.element_size(), residual=residual is not None)
            end = timer.start(f"tnx_gemm_library {what}", nbytes, flops)
        rc = call(None, self.library_tune)
        if end is not None:
            end.record()
        if rc == 3:
            # the algorithms for this size are timed now, once: with memory to push the operands out of the
            # caches, as large as the last-level cache; without it, if the device has no room, nothing is timed
            try:
                flush = torch.empty(256 << 20, dtype=torch.uint8, device=xa.device)
            except torch.OutOfMemoryError:
                flush = None
            rc = call(flush, int(self.library_tune) if flush is not None else 0)
        if rc == 1:
            raise RuntimeError(f"tnx_gemm_library: {lib.tnx_last_error().decode()}")
        return rc == 0

    @classmethod
    def _library_workspace(cls, device) -> torch.Tensor:
        """Memory the library's algorithms may ask for (those that split the inner dimension over blocks keep
        partial sums there, as does our kernel for some rows), one block per device, made at the first product
        and kept. Products on different streams of one device would share it: the engine runs its steps on
        one stream."""
        key = str(device)
        if key not in cls._workspaces:
            cls._workspaces[key] = torch.empty(32 << 20, dtype=torch.uint8, device=device)
        return cls._workspaces[key]

    # From this many rows on, plain bfloat16 products go to the vendor library (0: never). Up to 16 rows our
    # own kernel streams the weight as fast as the library does and fuses what follows the product.
    library_rows = 17

    def _bias_bf16(self, bias):
        """The bfloat16 copy of a float32 bias that the library's epilogue takes, made once. The original
        is held with it, so that its address names no other tensor while the copy is kept."""
        kept = self._bias_copies.get(bias.data_ptr())
        if kept is None or kept[0] is not bias:
            kept = (bias, bias.to(torch.bfloat16))
            self._bias_copies[bias.data_ptr()] = kept
        return kept[1]

    # Products of 17 to 128 rows with a float32 result (those that end in the residual sum, and the head): the
    # vendor library's kernels for such sizes leave much of the memory's rate unused (4,096 columns, K of
    # 16,384, 64 rows: 41 us against 31 here; 5,120 columns, K of 20,480, 32 rows: 68 against 41). Our kernel
    # gives a block 64 columns and shares K out until every compute unit has a block at most, so it is taken
    # where that leaves three units in four with one (9,216 columns make 144 blocks on 256 units, and there
    # the library is as good or better: 147 us against 195 at K of 36,864 and 64 rows), for matrices small
    # enough that the launches count and not the bytes, and for the head up to 64 rows (50,272 columns, more
    # column blocks than units; at 128 rows every block's reading of all rows costs more than it saves). Up to
    # 32 rows a small matrix stays with the few-rows kernel, one launch.
    some_rows = True

    def _some_rows_product(self, m, n, k, w, tiles, residual, out_f32, force_tiled) -> bool:
        if not (self.some_rows and tiles is not None and 16 < m <= 128 and out_f32 and not force_tiled
                and self.dtype == torch.bfloat16 and w.dtype == torch.bfloat16):
            return False
        small = n * k <= self.small_matrix
        if m <= self.few_rows and small:
            return False
        column_blocks = -(-n // 64)
        if column_blocks > self.compute_units:
            return residual is None and m <= 64
        shares = max(1, min(self.compute_units // column_blocks, k // 512))     # as the kernel shares K out
        return small or 4 * column_blocks * shares >= 3 * self.compute_units

    def _library_product(self, m, n, k, w, force_tiled) -> bool:
        if not (self.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and self.library_rows > 0
                and m >= self.library_rows and not force_tiled and n % 8 == 0 and k % 8 == 0):
            return False
        # small matrices at up to 32 rows: one launch of ours (5 to 10 us with its epilogue) beats the
        # library's product and the epilogue after it (11 to 15 us)
        return not (m <= 32 and n * k <= self.small_matrix)

    small_matrix = 1 << 23

    # ---------------------------------------------------------------- attention

    def _check_pages(self, k_pages, v_pages, num_kv, head_size, page_size):
        """The number of pages. A page's own elements lie together; from page to page there may be more than a
        page's elements, the same for keys and values (`_page_pad`: how many more)."""
        n = k_pages.shape[0]
        for t, name, shape in ((k_pages, "key pages", (n, num_kv, page_size, head_size)),
                               (v_pages, "value pages", (n, num_kv, head_size, page_size))):
            if not t.is_cuda or t.dtype != self.dtype:
                raise TypeError(f"{name} must be {self.dtype} on the GPU, got {t.dtype} on {t.device}")
            if tuple(t.shape) != shape:
                raise ValueError(f"{name} have shape {tuple(t.shape)}, expected {shape}")
            inner = (shape[2] * shape[3], shape[3], 1)
            if tuple(t.stride()[1:]) != inner or t.stride(0) < num_kv * inner[0] or (t.stride(0) - num_kv * inner[0]) % 8:
                raise ValueError(f"{name} must hold each page's elements together, pages a multiple of 8 elements "
                                 f"apart; strides {tuple(t.stride())}")
        if k_pages.stride(0) != v_pages.stride(0):
            raise ValueError("key and value pages must lie equally far apart")
        return n

    @staticmethod
    def _page_pad(pages, num_kv, head_size, page_size) -> int:
        return int(pages.stride(0) - num_kv * head_size * page_size) if pages is not None else 0

    @staticmethod
    def _turn_args(turn, head_size, ctx):
        """(a, b, positions, rows) of pair-turning tables as the entry points take them; all None / 0 without."""
        if turn is None:
            return None, None, None, 0
        a, b = turn
        _want(a, "turn a", torch.float32)
        _want(b, "turn b", torch.float32, tuple(a.shape))
        if a.dim() != 2 or a.shape[1] != head_size or head_size % 2:
            raise ValueError(f"pair-turning tables are [positions, head_size] with an even head size, got {tuple(a.shape)} "
                             f"for a head of {head_size}")
        return a, b, ctx.positions, a.shape[0]

    def qkv_project(self, h, w, bias, num_heads, num_kv_write, head_size, scale, ctx, view, k_pages, v_pages,
                    force_tiled=0, turn=None):
        """Queries, keys and values of the step's tokens: one matrix product whose epilogue scales the
        queries and stores keys and values in their pages (bfloat16), or product and `qkv_write` apart.
        `turn` = (a, b), float32 `[positions, head_size]`: element d of every query and key head of a token at
        position p becomes a[p, d] x[d] + b[p, d] x[d ^ 1] (bias added, before the scale), in the same launch."""
        turn_a, turn_b, turn_pos, turn_rows = self._turn_args(turn, head_size, ctx)
        if isinstance(h, DeferredNorm):
            folded = self._folded_for(h, w) if force_tiled != 1 else None
            if folded is not None and (ctx.num_tokens >= 128 or self._library_product(
                    ctx.num_tokens, w.tensor.shape[0], w.tensor.shape[1], w.tensor, force_tiled)):
                folded = None
            if folded is None:
                h = h.materialize()
            elif not self._norm_in_the_product(h.shape[0], w.tensor.shape[0], w.tensor.shape[1]):
                # the norm's kernel without weight and bias, then the fused projection of the folded copy
                h, w, bias = h.normalised(), PreparedWeight(w.tensor, folded.tiles), folded.d_with(bias)
            else:
                t = ctx.num_tokens
                total = (num_heads + 2 * num_kv_write) * head_size
                _want(h.x, "x", torch.float32, (t, w.tensor.shape[1]))
                if tuple(w.tensor.shape) != (total, h.x.shape[1]):
                    raise ValueError(f"w is {tuple(w.tensor.shape)}, the projections need {(total, h.x.shape[1])}")
                if bias is not None:
                    _want(bias, "qkv bias", torch.float32, (total,))
                num_pages = 0
                if num_kv_write:
                    num_pages = self._check_pages(k_pages, v_pages, num_kv_write, head_size, view.page_size)
                _want(view.token_page, "token pages", torch.int32, (t,))
                _want(view.token_offset, "token offsets", torch.int32, (t,))
                q = torch.empty(t, num_heads * head_size, dtype=self.dtype, device=h.x.device)
                self._call("gemm", "tnx_gemm_bf16_qkv_normed", _ptr(h.x), _ptr(folded.tiles), _ptr(folded.c),
                           _ptr(folded.d), float(h.eps), _ptr(bias), t, h.x.shape[1], _ptr(view.token_page),
                           _ptr(view.token_offset), _ptr(q), _ptr(k_pages) if num_kv_write else None,
                           _ptr(v_pages) if num_kv_write else None, float(scale), num_heads, num_kv_write, head_size,
                           view.page_size, num_pages, int(force_tiled), _ptr(turn_a), _ptr(turn_b), _ptr(turn_pos),
                           turn_rows, self._page_pad(k_pages if num_kv_write else None, num_kv_write, head_size,
                                                     view.page_size), int(bool(h.center)), _stream(),
                           work=self._product_work(t, total, h.x.shape[1], x_item=4))
                return q
        tiles = None
        if isinstance(w, PreparedWeight):
            w, tiles = w.tensor, w.tiles
        many = ctx.num_tokens >= 128 and w.shape[1] % 64 == 0 and w.shape[0] % 8 == 0 and not force_tiled
        if self.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and (many or self._library_product(
                ctx.num_tokens, w.shape[0], w.shape[1], w, force_tiled)):
            # many rows (the vendor library, or our wide-tile kernel where sizes allow): the bias joins the
            # product's float32 sums before they are rounded, once, as in the fused kernel below, so that keys
            # and values are cached with the same rounding whichever path a token took; the queries are
            # scaled after that
            return self.qkv_write(self.linear(h, w, bias), None, num_heads, num_kv_write, head_size, scale, ctx,
                                  view, k_pages, v_pages, turn)
        if self.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
            return self.qkv_write(self.linear(h, w, None), bias, num_heads, num_kv_write, head_size, scale, ctx,
                                  view, k_pages, v_pages, turn)
        t = ctx.num_tokens
        total = (num_heads + 2 * num_kv_write) * head_size
        _want(h, "h", torch.bfloat16, (t, w.shape[1]))
        _want(w, "w", torch.bfloat16, (total, h.shape[1]))
        if bias is not None:
            _want(bias, "qkv bias", torch.float32, (total,))
        num_pages = 0
        if num_kv_write:
            num_pages = self._check_pages(k_pages, v_pages, num_kv_write, head_size, view.page_size)
        _want(view.token_page, "token pages", torch.int32, (t,))
        _want(view.token_offset, "token offsets", torch.int32, (t,))
        q = torch.empty(t, num_heads * head_size, dtype=self.dtype, device=h.device)
        self._call("gemm", "tnx_gemm_bf16_qkv", _ptr(h), _ptr(w), _ptr(tiles), _ptr(bias), t, h.shape[1],
                   _ptr(view.token_page), _ptr(view.token_offset), _ptr(q),
                   _ptr(k_pages) if num_kv_write else None, _ptr(v_pages) if num_kv_write else None, float(scale),
                   num_heads, num_kv_write, head_size, view.page_size, num_pages, int(force_tiled), _ptr(turn_a),
                   _ptr(turn_b), _ptr(turn_pos), turn_rows,
                   self._page_pad(k_pages if num_kv_write else None, num_kv_write, head_size, view.page_size), _stream(),
                   work=self._product_work(t, total, h.shape[1]))
        return q

    def qkv_write(self, qkv, bias, num_heads, num_kv_write, head_size, scale, ctx, view, k_pages, v_pages, turn=None):
        turn_a, turn_b, _, turn_rows = self._turn_args(turn, head_size, ctx)
        t = ctx.num_tokens
        total = (num_heads + 2 * num_kv_write) * head_size
        _want(qkv, "qkv", self.dtype, (t, total))
        if bias is not None:
            _want(bias, "qkv bias", torch.float32, (total,))
        num_pages = 0
        if num_kv_write:
            num_pages = self._check_pages(k_pages, v_pages, num_kv_write, head_size, view.page_size)
        _want(view.block_table, "block table", torch.int32, (ctx.num_requests, view.width))
        q = torch.empty(t, num_heads * head_size, dtype=self.dtype, device=qkv.device)
        # the values of runs of several tokens are written by tiles (8 positions by 8 elements a thread, 16 bytes a store)
        by_tiles = (self.dtype == torch.bfloat16 and self.value_tiles and num_kv_write
                    and ctx.plan.get("tile_run") is not None and ctx.plan["tile_run"].numel() > 0)
        self._call("attention", "tnx_qkv_write", _ptr(qkv), _code(self.dtype), _ptr(bias), float(scale),
                   _ptr(ctx.positions), _ptr(ctx.token_request), _ptr(view.block_table), view.width, view.page_size,
                   num_pages, _ptr(q), _ptr(k_pages) if num_kv_write else None,
                   _ptr(v_pages) if num_kv_write else None, t, num_heads, num_kv_write, head_size,
                   _ptr(ctx.run_start), _ptr(ctx.cached_lens), _ptr(ctx.plan["tile_run"]), _ptr(ctx.plan["tile_start"]),
                   ctx.plan["tile_run"].numel() if by_tiles else 0, QUERY_TILE, _ptr(turn_a), _ptr(turn_b), turn_rows,
                   self._page_pad(k_pages if num_kv_write else None, num_kv_write, head_size, view.page_size), _stream())
        return q

    def attention(self, q, num_heads, num_kv_heads, head_size, ctx, view, k_pages, v_pages, window=None):
        t = ctx.num_tokens
        _want(q, "q", self.dtype, (t, num_heads * head_size))
        num_pages = self._check_pages(k_pages, v_pages, num_kv_heads, head_size, view.page_size)
        _want(view.block_table, "block table", torch.int32, (ctx.num_requests, view.width))
        if ctx.max_total > view.width * view.page_size:
            raise ValueError("a request is longer than its block table")
        out = torch.empty_like(q)
        window = int(window or 0)
        pad = self._page_pad(k_pages, num_kv_heads, head_size, view.page_size)
        fast = (self.dtype == torch.bfloat16 and not self.force_plain_attention
                and (ctx.plan["decode_runs"].numel() == 0
                     or view.page_size & (view.page_size - 1) == 0))
        if self.dtype == torch.bfloat16 and not fast and not self.force_plain_attention and not HipOps._warned_page_size:
            HipOps._warned_page_size = True
            build._log(f"a page size of {view.page_size} is no power of two: steps with decoding requests run on the "
                       "general attention kernel (one wave a query), several times slower than the matrix-unit "
                       "kernels that pages of 16, 32, 64, ... tokens get")
        if not fast:
            self._call("attention", "tnx_attention_any", _ptr(q), _code(self.dtype), _ptr(k_pages), _ptr(v_pages),
                       _ptr(ctx.positions), _ptr(ctx.token_request), _ptr(view.block_table), view.width,
                       view.page_size, num_pages, _ptr(out), t, num_heads, num_kv_heads, head_size, window, pad,
                       _stream())
            return out
        if ctx.plan["tile_run"].numel():
            self._call("attention", "tnx_attention_prefill", _ptr(q), _ptr(k_pages), _ptr(v_pages),
                       _ptr(ctx.run_start), _ptr(ctx.cached_lens), _ptr(view.block_table), view.width,
                       view.page_size, num_pages, _ptr(ctx.plan["tile_run"]), _ptr(ctx.plan["tile_start"]), ctx.plan["tile_run"].numel(),
                       _ptr(out), num_heads, num_kv_heads, head_size, window,
                       int(self.prefill_direct) or self._prefill_sets(ctx, num_heads, window), QUERY_TILE, pad,
                       _stream(), work=self._attention_work(ctx, "prompt", num_heads, num_kv_heads, head_size, window, 2)
                       if debug.timer() is not None else None)
        n_dec = ctx.plan["decode_runs"].numel()
        if n_dec:
            splits, waves = self._decode_splits(ctx, n_dec * self._decode_blocks(num_heads, num_kv_heads, head_size),
                                                window, head_size)
            part_o = part_ml = None
            if splits > 1:
                part_o = torch.empty(n_dec * num_heads * splits * head_size, dtype=torch.float32, device=q.device)
                part_ml = torch.empty(n_dec * num_heads * splits * 2, dtype=torch.float32, device=q.device)
            self._call("attention", "tnx_attention_decode", _ptr(q), _ptr(k_pages), _ptr(v_pages),
                       _ptr(ctx.run_start), _ptr(ctx.cached_lens), _ptr(view.block_table), view.width,
                       view.page_size, num_pages, _ptr(ctx.plan["decode_runs"]), n_dec, _ptr(out), _ptr(part_o),
                       _ptr(part_ml), num_heads, num_kv_heads, head_size, window, splits, waves,
                       _ptr(ctx.plan["longest_decode"]), pad,
                       _stream(), work=self._attention_work(ctx, "decode", num_heads, num_kv_heads, head_size, window, 2)
                       if debug.timer() is not None else None)
        return out

    # What the choice between one and two sets of waves a block rests on: the time of one 64-key step of a
    # block, in microseconds, measured on an MI355X at head size 128 (a block alone on its compute unit, two
    # blocks that share one, a block of two sets, and what a second round of blocks adds). Only the ratios
    # matter; another chip or head size changes which of two close estimates wins, not the results.
    prefill_step_cost = dict(alone=2.6, shared=3.9, two_sets=4.1, second_round=7.0)

    def _prefill_sets(self, ctx, num_heads, window) -> int:
        """How the staged prompt kernel runs this step: 0, two sets of four waves a block that halve a tile's
        keys between them, or 2, one set. One set lets two blocks share a compute unit and overlap each other's
        waits; two sets halve the time of the tile that sees the most keys, which the launch waits for when the
        blocks are few or uneven. The choice compares two estimates made from `prefill_step_cost`."""
        plan = ctx.plans.get(("prefill_sets", window))
        if plan is None:
            cost = self.prefill_step_cost
            lens, cached = ctx.run_lens_host, ctx.cached_lens_host
            steps = []
            for i in np.nonzero(lens > 1)[0]:
                for q0 in range(0, int(lens[i]), QUERY_TILE):
                    last = int(cached[i]) + min(q0 + QUERY_TILE, int(lens[i]))      # keys the tile's last query sees
                    first = max(0, int(cached[i]) + q0 - window + 1) // 64 if window > 0 else 0
                    steps.append(-(-last // 64) - first)
            steps = np.array(steps)
            halves = (steps + 1) // 2
            units = self.compute_units
            one = max(steps.max() * cost["alone"], steps.sum() * num_heads / units * cost["shared"] / 2)
            two = max(halves.max() * cost["two_sets"], halves.sum() * num_heads / units * cost["two_sets"])
            if len(steps) * num_heads > units:
                two += cost["second_round"]
            plan = ctx.plans[("prefill_sets", window)] = 0 if two < one else 2
        return plan

    _warned_page_size = False         # said once a process
    value_tiles = True                # tests clear it to write every value token by token
    prefill_direct = False            # tests set it: True, the prompt kernel that reads pages without LDS staging;
                                      # 2, the staged one with one set of four waves a block; 3, with two
    force_plain_attention = False     # tests set it to run the one-wave-per-query kernel in bfloat16 too
    decode_waves = 4                  # waves of a decode attention block (8 is kept for head sizes up to 128)
    decode_blocks_wanted = None       # the keys of decoding requests are split until about this many blocks run;
                                      # None: one block a compute unit

    @staticmethod
    def _decode_blocks(num_heads: int, num_kv_heads: int, head_size: int) -> int:
        """Blocks of the decode attention a request and a share of its keys: one a head, or, where heads share
        keys and values, one for every 16 heads of a group (8 at head sizes beyond 128), which read them once."""
        group = num_heads // num_kv_heads
        if group == 1:
            return num_heads
        return num_kv_heads * -(-group // (16 if head_size <= 128 else 8))

    def _decode_splits(self, ctx, pairs: int, window: int, head_size: int = 128):
        """(splits, waves): how many blocks share the keys of one decoding (request, head), and how many
        waves a block has. Blocks of four waves: with the products on the matrix unit a wave keeps the
        next tile's keys and values in flight by itself, and more waves bought nothing (measured at head
        size 128 and a context of 2,048: one request 8 x 4 waves 15.6 us against 16.9 for 4 x 8; eight
        requests 49.7 against 50.9; 64 requests 369 against 376).
        No block gets less than 256 keys of the longest request (a 64-key tile a wave). Requests about as
        long as one another are cut into as many blocks as that allows, up to 8: small blocks spread evenly
        over the compute units whatever the number of pairs (32 heads at 2,048 tokens, tokens a second: 9
        requests 1,582 -> 1,801, 20: 2,388 -> 2,545, 33: 3,067 -> 3,150, 128: 4,398 -> 4,487), except
        where the pairs alone give 0.7 to 1 block a compute unit (7 and 8 requests: whole requests, 1,548
        against 1,520 and 1,675 against 1,654) or a whole number of blocks each, within a twentieth (16, 24,
        32, 48, 64 requests: the many small blocks and the kernel that merges them cost 2 to 3 % there and
        have nothing to even out). Requests of very different lengths are not cut beyond what
        gives every compute unit a block: most blocks of a short request would be empty (64 requests of 16
        to 1,280 tokens: 6,430 tokens a second whole, 4,760 in eight blocks each). A recorded step is sized
        by the same two facts, which are part of what it is recorded under."""
        longest = ctx.length_bound if ctx.length_bound is not None else ctx.plan_host["longest_decode"]
        fills, alike = ctx.plan_host.get("decode_shape", (0, False))
        return self._splits_for(longest, fills, alike, pairs, window, head_size)

    def _splits_for(self, longest: int, fills: int, alike: bool, pairs: int, window: int, head_size: int):
        if not alike:
            fills = min(8, -(-longest // 256))
        if window:
            longest = min(longest, window + 64)
            fills = min(fills, -(-longest // 256))
        waves = 8 if self.decode_waves == 8 and head_size <= 128 else 4
        units = self.decode_blocks_wanted or self.compute_units
        if self.decode_blocks_wanted:                  # told how many blocks to make (measurements and tests)
            return max(1, min(-(-units // pairs), -(-longest // 256))), waves
        if 0.7 * units <= pairs <= units:
            return 1, waves
        fill_the_chip = max(1, min(-(-units // pairs), fills))
        if pairs > units and -(-pairs // units) * units <= 1.05 * pairs:
            alike = False         # whole requests already come out even over the compute units
        return (max(fill_the_chip, fills) if alike else fill_the_chip), waves

    def attention_launch_shape(self, step, num_heads: int, window, head_size: int, num_kv_heads: Optional[int] = None):
        """What the decode attention's launch in a recorded step is sized by beyond the number of requests: the
        blocks that share a request's keys (and their waves), for a `PackedStep` about to be replayed. A
        recorded step is sized for the longest request the model allows; how requests about as long as one
        another are cut depends on how long they are now, so a batch that grows is recorded again only when
        that changes the launch (8 requests of 32 heads: never; 9: at every 256 keys up to eight blocks)."""
        n_dec = int((step.run_lens == 1).sum())
        if n_dec == 0 or self.dtype != torch.bfloat16:
            return None
        fills, alike = step.plan_host.get("decode_shape", (0, False))
        blocks = self._decode_blocks(num_heads, num_kv_heads or num_heads, head_size)
        return ("decode", blocks, head_size) + self._splits_for(step.length_bound, fills, alike, n_dec * blocks,
                                                                int(window or 0), head_size)

    # ---------------------------------------------------------------- output end

    def ban_tokens(self, logits, tokens):
        """In place: `logits[i, tokens[i]] = -inf` where `tokens[i] >= 0`."""
        _want(logits, "logits", torch.float32)
        _want(tokens, "tokens", torch.int32, (logits.shape[0],))
        self._call("sampling", "tnx_ban_tokens", _ptr(logits), _ptr(tokens), logits.shape[0], logits.shape[1],
                   _stream())
        return logits

    def ban_pairs(self, logits, rows, tokens):
        """In place: `logits[rows[i], tokens[i]] = -inf` for every pair."""
        _want(logits, "logits", torch.float32)
        _want(rows, "rows", torch.int32)
        _want(tokens, "tokens", torch.int32, (rows.numel(),))
        self._call("sampling", "tnx_ban_pairs", _ptr(logits), _ptr(rows), _ptr(tokens), rows.numel(), logits.shape[0],
                   logits.shape[1], _stream())
        return logits

    def argmax(self, logits):
        _want(logits, "logits", torch.float32)
        out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
        self._call("sampling", "tnx_argmax", _ptr(logits), _ptr(out), logits.shape[0], logits.shape[1], _stream())
        return out

    def sample(self, logits, temperature, top_k, top_p, seeds, counters, min_keep=None):
        """See `ReferenceOps.sample`."""
        _want(logits, "logits", torch.float32)
        m = logits.shape[0]
        _want(temperature, "temperature", torch.float32, (m,))
        _want(top_k, "top_k", torch.int32, (m,))
        _want(top_p, "top_p", torch.float32, (m,))
        _want(seeds, "seeds", torch.int64, (m,))
        _want(counters, "counters", torch.int64, (m,))
        if min_keep is not None:
            _want(min_keep, "min_keep", torch.int32, (m,))
        out = torch.empty(m, dtype=torch.int32, device=logits.device)
        self._call("sampling", "tnx_sample", _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(seeds),
                   _ptr(counters), _ptr(min_keep), _ptr(out), m, logits.shape[1], _stream())
        return out

    def synchronize(self):
        torch.cuda.synchronize(self.device)
