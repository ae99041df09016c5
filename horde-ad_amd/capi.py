"""ctypes binding of the C ABI declared in include/hordead_gpu.h.

This is plumbing for the test-suite and the benchmark driver: it loads a
shared library that exports the ABI (the gfx950 library `libhordead_gpu.so`,
prefix `hgpu_`; the test-suite also loads its CPU checker, which exports the
same functions under another prefix) and wraps handles in small Python
objects.  Nothing here computes: every method is one call through the ABI.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
# HORDEAD_LIB_DIR points at another build of the libraries (the sanitizer build of the host layer)
LIB_DIR = os.environ.get("HORDEAD_LIB_DIR") or os.path.join(HERE, "lib")
GPU_LIB = os.path.join(LIB_DIR, "libhordead_gpu.so")
HOST_LIB = os.path.join(LIB_DIR, "libhordead_host.so")

F64, F32, I64, I32, I16, I8, BOOL = range(7)
_NP2DT = {np.dtype(np.float64): F64, np.dtype(np.float32): F32, np.dtype(np.int64): I64,
          np.dtype(np.int32): I32, np.dtype(np.int16): I16, np.dtype(np.int8): I8,
          np.dtype(np.bool_): BOOL}
_DT2NP = {v: k for k, v in _NP2DT.items()}

OP1 = {n: i for i, n in enumerate(
    ["neg", "abs", "signum", "recip", "exp", "log", "sqrt", "sin", "cos", "tan", "asin", "acos",
     "atan", "sinh", "cosh", "tanh", "asinh", "acosh", "atanh", "not"])}
OP2 = {n: i for i, n in enumerate(
    ["add", "mul", "sub", "div", "pow", "logbase", "atan2", "quot", "rem", "rem_scalar", "min",
     "max", "and"])}
CMP = {"leq": 0, "eq": 1, "lt": 2}

# name -> (restype, argtypes); P = opaque pointer, PP = pointer to pointer
P, PP, I, L = C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.c_int64
LP, IP = C.POINTER(C.c_int64), C.POINTER(C.c_int)
SIGNATURES = {
    "init": (I, [I, PP]), "shutdown": (I, [P]), "sync": (I, [P]), "last_error": (C.c_char_p, [P]),
    "upload": (I, [P, I, I, LP, P, PP]), "download": (I, [P, P, P]), "read_scalar": (I, [P, P, P]),
    "retain": (I, [P]), "release": (I, [P]), "rank": (I, [P]), "dtype_of": (I, [P]), "size": (L, [P]),
    "shape": (I, [P, LP]), "strides": (I, [P, LP]), "is_dense": (I, [P]),
    "transpose": (I, [P, P, I, IP, PP]), "reshape": (I, [P, P, I, LP, PP]),
    "slice": (I, [P, P, I, L, L, PP]), "reverse": (I, [P, P, I, PP]),
    "replicate": (I, [P, P, I, LP, PP]), "index_prefix": (I, [P, P, I, LP, PP]),
    "as_strided": (I, [P, P, I, LP, LP, L, PP]), "materialize": (I, [P, P, PP]),
    "pad": (I, [P, P, LP, LP, PP]), "ewise1": (I, [P, I, P, PP]), "ewise2": (I, [P, I, P, P, PP]),
    "compare": (I, [P, I, P, P, PP]), "compare_all": (I, [P, I, P, P, IP]),
    "select": (I, [P, P, P, P, PP]), "convert": (I, [P, P, I, I, PP]),
    "contract": (I, [P, P, P, I, PP]), "argminmax_last": (I, [P, P, I, PP]),
    "iota": (I, [P, L, I, PP]), "concat": (I, [P, I, PP, PP]),
    "gather": (I, [P, P, I, PP, I, LP, PP]), "scatter_add": (I, [P, P, I, PP, I, LP, I, PP]),
    "onehot": (I, [P, P, I, LP, LP, PP]), "get_api": (P, []),
    "scatter_affine": (I, [P, P, I, I, LP, LP, LP, PP]),
    "contract_sum": (I, [P, I, PP, PP, I, PP]),
    "assign": (I, [P, P, P]),
    "fused_map": (I, [P, I, PP, I, P, I, IP, PP]),
    "contract_sum_map": (I, [P, I, PP, PP, I, I, PP, I, P, I, IP, PP]),
    "fused_map_dimsum": (I, [P, I, PP, I, P, I, IP, PP, I, I, PP]),
}
# exported by the GPU library only
GPU_ONLY = {
    "extremum_last": (I, [P, P, I, PP, PP]),
    "fused_extremum": (I, [P, I, PP, I, P, I, I, I, PP, PP]),
    "fused_sum": (I, [P, I, PP, I, P, I, PP]),
    "mem_stats": (I, [P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "stream": (P, [P]), "inject_alloc_failure": (I, [P, L]),
    "profile_enable": (I, [P, I]), "profile_report": (I, [P, C.c_char_p, C.c_size_t]),
    "contract_noalloc": (I, [P, P, P, I, P]),
    "contract_map": (I, [P, P, P, I, I, PP, I, P, I, IP, PP, I, I, LP, LP, I, I, PP, PP]),
    "contract_operands": (I, [P, P, P, I, I, PP]),
    "mfma_probe": (I, [P, I, I, C.POINTER(C.c_double)]),
}


class Operand(C.Structure):
    """hgpu_operand: a plain array, or an elementwise program's result seen through a view."""
    _fields_ = [("array", C.c_void_p), ("n_in", C.c_int), ("inputs", C.POINTER(C.c_void_p)), ("n_instr", C.c_int),
                ("prog", C.c_void_p), ("slot", C.c_int), ("rank_m", C.c_int), ("mshape", C.POINTER(C.c_int64)),
                ("lo", C.POINTER(C.c_int64)), ("hi", C.POINTER(C.c_int64)), ("rank", C.c_int),
                ("shape", C.POINTER(C.c_int64)), ("strides", C.POINTER(C.c_int64)), ("offset", C.c_int64)]


class HgpuError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"status {code}: {msg}")
        self.code = code


def _larr(xs):
    xs = [int(x) for x in xs]
    return (C.c_int64 * max(len(xs), 1))(*xs)


class Lib:
    """One provider of the ABI: a shared library plus the symbol prefix."""

    def __init__(self, path=GPU_LIB, prefix="hgpu_", api_table="get_api"):
        if not os.path.exists(path):
            raise FileNotFoundError(
                f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
        self.path, self.prefix = path, prefix
        self.dll = C.CDLL(path)
        sigs = dict(SIGNATURES)
        if prefix == "hgpu_":
            sigs.update(GPU_ONLY)
        for name, (res, args) in sigs.items():
            fn = getattr(self.dll, prefix + name)
            fn.restype, fn.argtypes = res, args
            setattr(self, name, fn)
        if api_table != "get_api":   # another table of the same provider (the checker's one with the fused entry points)
            fn = getattr(self.dll, prefix + api_table)
            fn.restype, fn.argtypes = P, []
            self.get_api = fn

    def context(self, device=0):
        return Ctx(self, device)


class Ctx:
    def __init__(self, lib, device=0):
        self.lib = lib
        h = C.c_void_p()
        rc = lib.init(device, C.byref(h))
        if rc:
            raise HgpuError(rc, "init failed (no usable device?)")
        self.h = h

    def check(self, rc):
        if rc:
            raise HgpuError(rc, self.lib.last_error(self.h).decode())

    def sync(self):
        self.check(self.lib.sync(self.h))

    def shutdown(self):
        self.check(self.lib.shutdown(self.h))

    def mem_stats(self):
        a, b, c = C.c_uint64(), C.c_uint64(), C.c_uint64()
        self.check(self.lib.mem_stats(self.h, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def profile(self, on):
        self.check(self.lib.profile_enable(self.h, int(on)))

    def profile_report(self):
        """{kernel family: (launches, total_ms, algorithmic_bytes, algorithmic_flops)}"""
        buf = C.create_string_buffer(1 << 16)
        self.check(self.lib.profile_report(self.h, buf, len(buf)))
        out = {}
        for line in buf.value.decode().splitlines():
            name, cnt, ms, by, fl = line.rsplit(None, 4)   # (a label may hold blanks)
            out[name] = (int(cnt), float(ms), float(by), float(fl))
        return out

    def fused_map(self, inputs, prog, out_slots):
        """prog: list of (kind, op, dtype, a, b, c) over slots; returns the output arrays."""
        ins = (C.c_void_p * len(inputs))(*[p.h for p in inputs])
        flat = (C.c_int32 * (6 * len(prog)))(*[int(x) for q in prog for x in q])
        slots = (C.c_int * len(out_slots))(*out_slots)
        outs = (C.c_void_p * len(out_slots))()
        self.check(self.lib.fused_map(self.h, len(inputs), ins, len(prog), flat, len(out_slots), slots, outs))
        return [Array(self, C.c_void_p(o)) for o in outs]

    def fused_map_dimsum(self, inputs, prog, out_slots, sum_slot, keep_dim):
        """hgpu_fused_map_dimsum: (outs, sum of slot sum_slot over every dim but keep_dim)."""
        ins = (C.c_void_p * len(inputs))(*[p.h for p in inputs])
        flat = (C.c_int32 * (6 * len(prog)))(*[int(x) for q in prog for x in q])
        slots = (C.c_int * len(out_slots))(*out_slots)
        outs = (C.c_void_p * len(out_slots))()
        sm = C.c_void_p()
        self.check(self.lib.fused_map_dimsum(self.h, len(inputs), ins, len(prog), flat, len(out_slots), slots, outs, sum_slot, keep_dim, C.byref(sm)))
        return [Array(self, C.c_void_p(o)) for o in outs], Array(self, sm)

    def contract_map(self, a, b, n_keep, inputs, prog, out_slots, ext=None):
        """hgpu_contract_map: `inputs` holds None where the contraction of a and b stands;
        ext = (slot, view_shape, view_strides, n_reduce, want_max) asks for the extremum over
        windows.  Returns (outs, values, indices); the last two None without ext."""
        ins = (C.c_void_p * len(inputs))(*[None if p is None else p.h for p in inputs])
        flat = (C.c_int32 * max(6 * len(prog), 1))(*[int(x) for q in prog for x in q])
        slots = (C.c_int * max(len(out_slots), 1))(*out_slots)
        outs = (C.c_void_p * max(len(out_slots), 1))()
        v, i = C.c_void_p(), C.c_void_p()
        if ext is None:
            self.check(self.lib.contract_map(self.h, a.h, b.h, n_keep, len(inputs), ins, len(prog), flat, len(out_slots), slots, outs,
                                             0, 0, None, None, 0, 0, None, None))
            return [Array(self, C.c_void_p(o)) for o in outs[:len(out_slots)]], None, None
        slot, vshape, vstrides, n_reduce, want_max = ext
        self.check(self.lib.contract_map(self.h, a.h, b.h, n_keep, len(inputs), ins, len(prog), flat, len(out_slots), slots, outs,
                                         slot, len(vshape), _larr(vshape), _larr(vstrides), n_reduce, int(want_max), C.byref(v), C.byref(i)))
        return [Array(self, C.c_void_p(o)) for o in outs[:len(out_slots)]], Array(self, v), Array(self, i)

    def contract_sum_map(self, terms, n_keep, inputs, prog, out_slots):
        """hgpu_contract_sum_map: terms = [(a, b), ...]; `inputs` holds None where the sum of the
        contractions stands.  Returns the arrays of out_slots."""
        as_ = (C.c_void_p * len(terms))(*[a.h for a, _ in terms])
        bs_ = (C.c_void_p * len(terms))(*[b.h for _, b in terms])
        ins = (C.c_void_p * len(inputs))(*[None if p is None else p.h for p in inputs])
        flat = (C.c_int32 * max(6 * len(prog), 1))(*[int(x) for q in prog for x in q])
        slots = (C.c_int * max(len(out_slots), 1))(*out_slots)
        outs = (C.c_void_p * max(len(out_slots), 1))()
        self.check(self.lib.contract_sum_map(self.h, len(terms), as_, bs_, n_keep, len(inputs), ins, len(prog), flat, len(out_slots), slots, outs))
        return [Array(self, C.c_void_p(o)) for o in outs[:len(out_slots)]]

    def operand(self, inputs, prog, slot, mshape, view, pad=None):
        """An expression operand for contract_operands: view = (shape, strides, offset) over the
        dense layout of the program's result with dims merged to mshape and zero-extended by pad = (lo, hi)."""
        keep = []
        o = Operand()
        ins = (C.c_void_p * len(inputs))(*[p.h for p in inputs])
        flat = (C.c_int32 * max(6 * len(prog), 1))(*[int(x) for q in prog for x in q])
        ms, sh, st = _larr(mshape), _larr(view[0]), _larr(view[1])
        keep += [ins, flat, ms, sh, st, list(inputs)]
        o.array, o.n_in, o.inputs, o.n_instr, o.prog, o.slot = None, len(inputs), ins, len(prog), C.cast(flat, C.c_void_p), slot
        o.rank_m, o.mshape, o.rank, o.shape, o.strides, o.offset = len(mshape), ms, len(view[0]), sh, st, view[2]
        if pad is not None:
            lo, hi = _larr(pad[0]), _larr(pad[1])
            keep += [lo, hi]
            o.lo, o.hi = lo, hi
        o._keep = keep
        return o

    def contract_operands(self, a, b, n_keep, fused_only=False):
        """hgpu_contract_operands; a, b: Array or the result of operand()."""
        def conv(x):
            if x is None or isinstance(x, Operand):
                return x
            o = Operand()
            o.array = x.h
            o._keep = [x]
            return o
        oa, ob = conv(a), conv(b)
        return self._out(self.lib.contract_operands, C.byref(oa), C.byref(ob) if ob is not None else None, n_keep, int(fused_only))

    def fused_sum(self, inputs, prog, slot):
        """The sum of slot's values over all elements, a rank-0 array."""
        ins = (C.c_void_p * len(inputs))(*[p.h for p in inputs])
        flat = (C.c_int32 * max(6 * len(prog), 1))(*[int(x) for q in prog for x in q])
        return self._out(self.lib.fused_sum, len(inputs), ins, len(prog), flat, slot)

    def fused_extremum(self, inputs, prog, slot, n_reduce, want_max):
        """(values, indices) of the first extremum of slot's values over the trailing n_reduce dims."""
        ins = (C.c_void_p * len(inputs))(*[p.h for p in inputs])
        flat = (C.c_int32 * max(6 * len(prog), 1))(*[int(x) for q in prog for x in q])
        v, i = C.c_void_p(), C.c_void_p()
        self.check(self.lib.fused_extremum(self.h, len(inputs), ins, len(prog), flat, slot, n_reduce, int(want_max), C.byref(v), C.byref(i)))
        return Array(self, v), Array(self, i)

    def _wrap(self, h):
        return Array(self, h)

    def _out(self, fn, *args):
        o = C.c_void_p()
        self.check(fn(self.h, *args, C.byref(o)))
        return Array(self, o)

    # -- memory
    def upload(self, x):
        x = np.asarray(x)
        if not x.flags.c_contiguous:
            x = x.copy(order="C")
        dt = _NP2DT[x.dtype]
        return self._out(self.lib.upload, dt, x.ndim, _larr(x.shape), x.ctypes.data_as(C.c_void_p))

    def iota(self, n, dtype=I64):
        return self._out(self.lib.iota, n, dtype)

    def concat(self, parts):
        arr = (C.c_void_p * len(parts))(*[p.h for p in parts])
        return self._out(self.lib.concat, len(parts), arr)

    def gather(self, src, ix, shm):
        arr = (C.c_void_p * max(len(ix), 1))(*[p.h for p in ix])
        return self._out(self.lib.gather, src.h, len(ix), arr, len(shm), _larr(shm))

    def contract_sum(self, pairs, n_keep):
        a = (C.c_void_p * len(pairs))(*[x.h for x, _ in pairs])
        b = (C.c_void_p * len(pairs))(*[y.h for _, y in pairs])
        return self._out(self.lib.contract_sum, len(pairs), a, b, n_keep)

    def scatter_affine(self, src, rank_m, c0, coef, shp):
        """coef[d][j]: coefficient of position variable d in index component j."""
        flat = [int(v) for row in coef for v in row]
        return self._out(self.lib.scatter_affine, src.h, rank_m, len(shp), _larr(c0), _larr(flat), _larr(shp))

    def scatter_add(self, src, ix, rank_m, shp, flags=0):
        arr = (C.c_void_p * max(len(ix), 1))(*[p.h for p in ix])
        return self._out(self.lib.scatter_add, src.h, len(ix), arr, rank_m, _larr(shp), flags)


class Array:
    def __init__(self, ctx, h):
        self.ctx, self.h = ctx, h

    def __del__(self):
        try:
            if self.h:
                self.ctx.lib.release(self.h)
                self.h = None
        except Exception:
            pass

    # -- metadata
    @property
    def rank(self):
        return self.ctx.lib.rank(self.h)

    @property
    def dtype(self):
        return self.ctx.lib.dtype_of(self.h)

    @property
    def shape(self):
        r = self.rank
        buf = (C.c_int64 * max(r, 1))()
        self.ctx.lib.shape(self.h, buf)
        return tuple(buf[i] for i in range(r))

    @property
    def strides(self):
        r = self.rank
        buf = (C.c_int64 * max(r, 1))()
        self.ctx.lib.strides(self.h, buf)
        return tuple(buf[i] for i in range(r))

    @property
    def is_dense(self):
        return bool(self.ctx.lib.is_dense(self.h))

    def numpy(self):
        out = np.empty(self.shape, dtype=_DT2NP[self.dtype])
        self.ctx.check(self.ctx.lib.download(self.ctx.h, self.h, out.ctypes.data_as(C.c_void_p)))
        return out

    def item(self):
        out = np.empty((), dtype=_DT2NP[self.dtype])
        self.ctx.check(self.ctx.lib.read_scalar(self.ctx.h, self.h, out.ctypes.data_as(C.c_void_p)))
        return out[()]

    # -- views
    def _o(self, fn, *args):
        return self.ctx._out(fn, self.h, *args)

    def transpose(self, perm):
        return self._o(self.ctx.lib.transpose, len(perm), (C.c_int * max(len(perm), 1))(*perm))

    def reshape(self, shape):
        return self._o(self.ctx.lib.reshape, len(shape), _larr(shape))

    def slice(self, dim, start, length):
        return self._o(self.ctx.lib.slice, dim, start, length)

    def reverse(self, dim=0):
        return self._o(self.ctx.lib.reverse, dim)

    def replicate(self, prefix):
        return self._o(self.ctx.lib.replicate, len(prefix), _larr(prefix))

    def index_prefix(self, ix):
        return self._o(self.ctx.lib.index_prefix, len(ix), _larr(ix))

    def as_strided(self, shape, strides, offset=0):
        return self._o(self.ctx.lib.as_strided, len(shape), _larr(shape), _larr(strides), offset)

    def materialize(self):
        return self._o(self.ctx.lib.materialize)

    def pad(self, lo, hi):
        return self._o(self.ctx.lib.pad, _larr(lo), _larr(hi))

    # -- compute
    def ewise1(self, op):
        return self.ctx._out(self.ctx.lib.ewise1, OP1[op], self.h)

    def ewise2(self, op, other):
        return self.ctx._out(self.ctx.lib.ewise2, OP2[op], self.h, other.h)

    def compare(self, cmp, other):
        return self.ctx._out(self.ctx.lib.compare, CMP[cmp], self.h, other.h)

    def compare_all(self, cmp, other):
        r = C.c_int()
        self.ctx.check(self.ctx.lib.compare_all(self.ctx.h, CMP[cmp], self.h, other.h, C.byref(r)))
        return bool(r.value)

    def select(self, a, b):
        return self.ctx._out(self.ctx.lib.select, self.h, a.h, b.h)

    def convert(self, dtype, mode=0):
        return self._o(self.ctx.lib.convert, dtype, mode)

    def contract(self, other, n_keep):
        return self.ctx._out(self.ctx.lib.contract, self.h, other.h if other is not None else None, n_keep)

    def assign(self, src):
        """hgpu_assign: this array's memory takes src's elements."""
        self.ctx.check(self.ctx.lib.assign(self.ctx.h, self.h, src.h))
        return self

    def contract_noalloc(self, other, n_keep, out):
        """hgpu_contract into the caller's array `out`, without device allocation (gfx950 library only)."""
        self.ctx.check(self.ctx.lib.contract_noalloc(self.ctx.h, self.h, other.h if other is not None else None, n_keep, out.h))
        return out

    def argminmax_last(self, want_max):
        return self._o(self.ctx.lib.argminmax_last, int(want_max))

    def extremum_last(self, want_max):
        """(values, indices) of the first extremum along the last dim (gfx950 library only)."""
        v, i = C.c_void_p(), C.c_void_p()
        self.ctx.check(self.ctx.lib.extremum_last(self.ctx.h, self.h, int(want_max), C.byref(v), C.byref(i)))
        return Array(self.ctx, v), Array(self.ctx, i)

    def onehot(self, ix, shp):
        return self._o(self.ctx.lib.onehot, len(ix), _larr(ix), _larr(shp))
