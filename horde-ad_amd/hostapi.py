"""ctypes binding of include/hordead_host.h (libhordead_host.so).

`Host` is a context of the host layer on some provider of the array ABI, `V` a
tensor value whose methods carry the names of horde-ad's tensor operations
(`ssum`, `sgather`, `smatmul2`, ...; reference export list:
src/HordeAd/OpsTensor.hs:16-78), and `IxV` a lane-batched scalar with Python
operators, so that an index function is written as a lambda exactly like the
reference's `\\[i, k] -> [i + k]` and is called once, symbolically.
"""
import ctypes as C

import numpy as np

from . import capi
from .capi import _DT2NP, _NP2DT, CMP, OP1, OP2, HgpuError, _larr

P, PP, I, L = C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.c_int64
LP, IP = C.POINTER(C.c_int64), C.POINTER(C.c_int)
D = C.c_double
SIG = {
    "create_gpu": (I, [I, PP]), "create": (I, [P, I, PP]), "destroy": (I, [P]),
    "last_error": (C.c_char_p, [P]), "sync": (I, [P]), "array_ctx": (P, [P]), "tape_reset": (I, [P]), "set_fusion": (I, [P, I]),
    "upload": (I, [P, I, I, LP, P, I, PP]), "from_array": (I, [P, P, I, PP]),
    "constant": (I, [P, I, D, I, LP, PP]), "array": (I, [P, PP]), "download": (I, [P, P, P]),
    "val_rank": (I, [P]), "val_dtype": (I, [P]), "val_shape": (I, [P, LP]), "free": (I, [P]),
    "backward": (I, [P, P, P, I, PP, PP]),
    "ewise1": (I, [P, I, P, PP]), "ewise2": (I, [P, I, P, P, PP]), "compare": (I, [P, I, P, P, PP]),
    "compare_all": (I, [P, I, P, P, IP]), "select": (I, [P, P, P, P, PP]), "convert": (I, [P, P, I, I, PP]),
    "tssumN": (I, [P, P, I, PP]), "tssum0": (I, [P, P, PP]), "tsdot0": (I, [P, P, P, PP]),
    "tsdot1In": (I, [P, P, P, PP]), "tsdotNIn": (I, [P, P, P, I, PP]), "tD": (I, [P, P, P, PP]), "tprimalPart": (I, [P, P, PP]), "as_input": (I, [P, P, PP]), "tsmatvecmul": (I, [P, P, P, PP]), "tsmatmul2": (I, [P, P, P, PP]),
    "tsreplicateN": (I, [P, P, I, LP, PP]), "tsappend": (I, [P, P, P, PP]), "tsslice": (I, [P, P, L, L, PP]),
    "tsreverse": (I, [P, P, PP]), "tstranspose": (I, [P, P, I, IP, PP]), "tsreshape": (I, [P, P, I, LP, PP]),
    "tsindex": (I, [P, P, I, LP, PP]), "tsargminmax": (I, [P, P, I, PP]), "tsiota": (I, [P, L, I, PP]),
    "ix_var": (I, [P, I, LP, I, PP]), "ix_const": (I, [P, I, LP, I, D, PP]), "ix_lift": (I, [P, I, LP, P, PP]),
    "ix_op1": (I, [P, I, P, PP]), "ix_op2": (I, [P, I, P, P, PP]), "ix_compare": (I, [P, I, P, P, PP]),
    "ix_select": (I, [P, P, P, P, PP]), "ix_convert": (I, [P, P, I, I, PP]),
    "ix_index0": (I, [P, P, I, PP, PP]), "ix_argminmax": (I, [P, P, I, PP, I, PP]), "ix_free": (I, [P]),
    "ix_is_affine": (I, [P]), "counter": (L, [P, C.c_char_p]),
    "ix_from_val": (I, [P, P, PP]), "ix_to_val": (I, [P, P, PP]), "ix_dtype": (I, [P]),
    "tconvert": (I, [P, I, P, I, LP, PP]), "dense": (I, [P, P, PP]),
    "tsgather": (I, [P, P, I, LP, I, PP, PP]), "tsscatter": (I, [P, P, I, I, LP, PP, PP]),
    "capture_begin": (I, [P]), "capture_end": (I, [P, PP]), "graph_launch": (I, [P, P]), "graph_free": (I, [P, P]),
    "force": (I, [P, P]), "overwrite": (I, [P, P, P]), "assign": (I, [P, P, P]),
    "update_with_gradient": (I, [P, D, P, P, PP]),
    "update_with_gradient_adam": (I, [P, D, D, D, D, I, P, P, P, P, PP, PP, PP]),
    "adam_step_size": (I, [P, I, D, D, D, I, PP]),
    "adam_apply": (I, [P, P, D, D, D, P, P, P, P, PP, PP, PP]),
}

_dll = None


def _lib():
    global _dll
    if _dll is None:
        import os
        if not os.path.exists(capi.HOST_LIB):
            raise FileNotFoundError(f"{capi.HOST_LIB} is not built; run __graft_entry__.build()")
        dll = C.CDLL(capi.HOST_LIB)
        for name, (res, args) in SIG.items():
            fn = getattr(dll, "hh_" + name)
            fn.restype, fn.argtypes = res, args
        _dll = dll
    return _dll


def _values(x):
    if isinstance(x, V):
        yield x
    elif isinstance(x, (list, tuple)):
        for y in x:
            yield from _values(y)


class Graph:
    def __init__(self, host, h):
        self.host, self.h = host, h

    def launch(self):
        self.host.check(self.host.dll.hh_graph_launch(self.host.h, self.h))

    def free(self):
        if self.h:
            self.host.check(self.host.dll.hh_graph_free(self.host.h, self.h))
            self.h = None
            self.keeps = None


class Host:
    """A host-layer context: on the gfx950 library by default, or on the provider
    whose ABI table `api_lib.get_api()` returns."""

    def __init__(self, api_lib=None, device=0):
        self.dll = _lib()
        h = C.c_void_p()
        if api_lib is None:
            rc = self.dll.hh_create_gpu(device, C.byref(h))
        else:
            self._api_lib = api_lib  # keep the provider loaded
            rc = self.dll.hh_create(api_lib.get_api(), device, C.byref(h))
        if rc:
            raise HgpuError(rc, "cannot create a host-layer context (no usable device?)")
        self.h = h

    def check(self, rc):
        if rc:
            raise HgpuError(rc, self.dll.hh_last_error(self.h).decode())

    def _out(self, fn, *args):
        o = C.c_void_p()
        self.check(fn(self.h, *args, C.byref(o)))
        return V(self, o)

    def sync(self):
        self.check(self.dll.hh_sync(self.h))

    def set_fusion(self, on):
        self.check(self.dll.hh_set_fusion(self.h, int(on)))

    def counter(self, name):
        """How often the named rewrite onto a fused entry point was taken (diagnostic)."""
        return int(self.dll.hh_counter(self.h, name.encode()))

    def tape_reset(self):
        self.check(self.dll.hh_tape_reset(self.h))

    def destroy(self):
        self.dll.hh_destroy(self.h)

    # -- one recorded program, launched many times
    def capture(self, program):
        """Records the device work of `program()` (run it once without capture
        first) and returns (graph, what program returned); every value made
        inside is refreshed by graph.launch()."""
        self.check(self.dll.hh_capture_begin(self.h))
        try:
            result = program()
            for v in _values(result):
                self.check(self.dll.hh_force(self.h, v.h))
        except BaseException:
            g = C.c_void_p()
            self.dll.hh_capture_end(self.h, C.byref(g))
            if g:
                self.dll.hh_graph_free(self.h, g)
            raise
        g = C.c_void_p()
        self.check(self.dll.hh_capture_end(self.h, C.byref(g)))
        graph = Graph(self, g)
        # The recording reads, at every launch, the arrays that existed before it:
        # they must outlive it.  The recorded function holds them (its closure), so the graph holds the function.
        graph.keeps = program
        return graph, result

    # -- values
    def concrete(self, x, requires_grad=False):
        x = np.asarray(x)
        if not x.flags.c_contiguous:
            x = x.copy(order="C")
        return self._out(self.dll.hh_upload, _NP2DT[x.dtype], x.ndim, _larr(x.shape),
                         x.ctypes.data_as(C.c_void_p), int(requires_grad))

    def param(self, x):
        return self.concrete(x, requires_grad=True)

    def sconcrete(self, x):
        """A small constant of the program (`sconcrete (sfromListLinear ..)`: an index table,
        the [0.0, 1.0] of a mask): uploaded the first time its value is asked for and kept, so
        a program that names constants can be recorded after one eager run."""
        x = np.ascontiguousarray(x)
        key = (x.dtype.str, x.shape, x.tobytes())
        cache = self.__dict__.setdefault("_constants", {})
        if key not in cache:
            if x.nbytes > 1 << 16:
                return self.concrete(x)
            cache[key] = self.concrete(x)
        return cache[key]

    def srepl(self, shape, value, dtype=capi.F64):
        """sconcrete (sreplicate shape value)"""
        return self._out(self.dll.hh_constant, dtype, float(value), len(shape), _larr(shape))

    def siota(self, n, dtype=capi.I64):
        return self._out(self.dll.hh_tsiota, n, dtype)

    def grad(self, out, inputs, dt=None):
        """Cotangents of `inputs` for d(out) = dt (default: ones, as `grad` uses)."""
        if dt is None:
            dt = self.srepl(out.shape, 1.0, out.dtype)
        arr = (C.c_void_p * len(inputs))(*[v.h for v in inputs])
        outs = (C.c_void_p * len(inputs))()
        self.check(self.dll.hh_backward(self.h, out.h, dt.h, len(inputs), arr, outs))
        return [V(self, C.c_void_p(o)) for o in outs]

    # -- host loops of the tensor class (the reference's `Concrete` instance runs
    #    these closures once per index on the host as well)
    def sfromVector(self, vs):
        """tsfromVector (OpsConcrete.hs:144-151): stacks values of one shape along a new outermost dim."""
        out = None
        for v in vs:
            row = v.sreshape([1] + list(v.shape))
            out = row if out is None else out.sappend(row)
        return out

    def sbuild1(self, k, f):
        """tsbuild1 (OpsConcrete.hs:1761-1774): [f 0, ..., f (k-1)] stacked; f gets a concrete index."""
        return self.sfromVector([f(i) for i in range(k)])

    def kbuild(self, shm, f, dtype=None):
        """tkbuild @shm f (Ops.hs:863-880; Concrete: one vector generate, OpsConcrete.hs:1081-1087):
        f gets the position variables as lane values and runs once; its result (a lane
        value, or a Python number with `dtype`) is written out as an array of shape shm."""
        shm = tuple(int(s) for s in shm)
        r = f(*self.ix_space(shm))
        if not isinstance(r, IxV):
            r = IxV.const(self, shm, r, capi.I64 if dtype is None else dtype)
        elif dtype is not None and r.dtype != dtype:
            raise HgpuError(1, "kbuild: the closure's result is not of the element type asked for")
        return r.to_val()

    def kbuild1(self, k, f, dtype=None):
        """tkbuild1 @k f (Ops.hs:860-862)."""
        return self.kbuild((k,), f, dtype)

    def sbuild(self, shm, f):
        """tsbuild @shm f for a closure that yields arrays (Ops.hs:913-928, OpsConcrete.hs:1776-1789):
        the reference's nest of tsbuild1 host loops, f gets concrete indices.  With scalar
        elements (shn = []) the reference takes tbuildK instead: that is `kbuild`."""
        shm = tuple(int(s) for s in shm)

        def level(prefix, rest):
            if not rest:
                return f(*prefix)
            return self.sbuild1(rest[0], lambda i: level(prefix + [i], rest[1:]))
        return level([], list(shm))

    def smapAccumL(self, f, acc0, xs):
        """tmapAccumL (OpsConcrete.hs:990-1019): threads `acc` through the outermost
        dim of xs; f(acc, x) -> (acc', y).  Returns (final acc, stacked ys)."""
        acc, ys = acc0, []
        for t in range(xs.shape[0]):
            acc, y = f(acc, xs.sindex([t]))
            ys.append(y)
        return acc, self.sfromVector(ys)

    # -- index functions
    def ix_space(self, shm):
        return [IxV(self, self._ixo(self.dll.hh_ix_var, len(shm), _larr(shm), d), tuple(shm)) for d in range(len(shm))]

    def _ixo(self, fn, *args):
        o = C.c_void_p()
        self.check(fn(self.h, *args, C.byref(o)))
        return o

    def _apply_index_fn(self, shm, f):
        shm = tuple(int(s) for s in shm)
        vars_ = self.ix_space(shm)
        res = f(*vars_)
        res = [r if isinstance(r, IxV) else IxV.const(self, shm, int(r)) for r in res]
        return shm, res


def _ixarr(ixs):
    return (C.c_void_p * max(len(ixs), 1))(*[x.h for x in ixs])


class IxV:
    """A scalar inside an index function, for all positions at once."""

    def __init__(self, host, h, shm):
        self.host, self.h, self.shm = host, h, shm

    def __del__(self):
        try:
            self.host.dll.hh_ix_free(self.h)
        except Exception:
            pass

    @staticmethod
    def const(host, shm, value, dtype=capi.I64):
        return IxV(host, host._ixo(host.dll.hh_ix_const, len(shm), _larr(shm), dtype, float(value)), shm)

    @staticmethod
    def from_val(v):
        """The elements of an array as a lane value over the array's own index space
        (what the scalar closure of tsmap0N / tszipWith0N is applied to)."""
        return IxV(v.host, v.host._ixo(v.host.dll.hh_ix_from_val, v.h), tuple(v.shape))

    def to_val(self):
        """This lane value as an array of shape shm."""
        return self.host._out(self.host.dll.hh_ix_to_val, self.h)

    @property
    def dtype(self):
        return int(self.host.dll.hh_ix_dtype(self.h))

    def _coerce(self, o, dtype=None):
        """A Python number beside a lane value is a literal of the lane value's element type."""
        return o if isinstance(o, IxV) else IxV.const(self.host, self.shm, o, self.dtype if dtype is None else dtype)

    def _op2(self, op, o, dtype=None):
        o = self._coerce(o, dtype)
        return IxV(self.host, self.host._ixo(self.host.dll.hh_ix_op2, OP2[op], self.h, o.h), self.shm)

    def _rop2(self, op, o, dtype=None):
        return self._coerce(o, dtype)._op2(op, self)

    @property
    def is_affine(self):
        return bool(self.host.dll.hh_ix_is_affine(self.h))

    def __add__(self, o): return self._op2("add", o)
    def __radd__(self, o): return self._rop2("add", o)
    def __sub__(self, o): return self._op2("sub", o)
    def __rsub__(self, o): return self._rop2("sub", o)
    def __mul__(self, o): return self._op2("mul", o)
    def __rmul__(self, o): return self._rop2("mul", o)
    def __truediv__(self, o): return self._op2("div", o)
    def __rtruediv__(self, o): return self._rop2("div", o)
    def __pow__(self, o): return self._op2("pow", o)
    def atan2H(self, o): return self._op2("atan2", o)
    def __neg__(self): return IxV(self.host, self.host._ixo(self.host.dll.hh_ix_op1, OP1["neg"], self.h), self.shm)
    def quotH(self, o): return self._op2("quot", o)
    def remH(self, o): return self._op2("rem_scalar", o)      # scalar rule: remH a 0 = a (Types.hs:402-419)
    def minH(self, o): return self._op2("min", o)
    def maxH(self, o): return self._op2("max", o)
    def op1(self, name): return IxV(self.host, self.host._ixo(self.host.dll.hh_ix_op1, OP1[name], self.h), self.shm)

    def _cmp(self, c, o, dtype):
        o = self._coerce(o, dtype)
        return IxV(self.host, self.host._ixo(self.host.dll.hh_ix_compare, CMP[c], self.h, o.h), self.shm)

    def leq(self, o, dtype=None): return self._cmp("leq", o, dtype)     # <=.
    def lt(self, o, dtype=None): return self._cmp("lt", o, dtype)       # <.
    def eq(self, o, dtype=None): return self._cmp("eq", o, dtype)       # ==.
    def notB(self): return self.op1("not")
    def andB(self, o): return self._op2("and", o)                        # &&*

    def convert(self, dtype, mode=0):
        return IxV(self.host, self.host._ixo(self.host.dll.hh_ix_convert, self.h, dtype, mode), self.shm)


def ifH(cond, a, b, dtype=None):
    """ifH / kcond on lane-batched scalars.  Python numbers take the other branch's element
    type, or `dtype`, or Int."""
    if dtype is None:
        dtype = a.dtype if isinstance(a, IxV) else b.dtype if isinstance(b, IxV) else capi.I64
    a = a if isinstance(a, IxV) else IxV.const(cond.host, cond.shm, a, dtype)
    b = b if isinstance(b, IxV) else IxV.const(cond.host, cond.shm, b, dtype)
    return IxV(cond.host, cond.host._ixo(cond.host.dll.hh_ix_select, cond.h, a.h, b.h), cond.shm)


class V:
    """A tensor value of the `Gpu` carrier (possibly carrying a tape node)."""

    def __init__(self, host, h):
        self.host, self.h = host, h

    def __del__(self):
        try:
            if self.h:
                self.host.dll.hh_free(self.h)
                self.h = None
        except Exception:
            pass

    @property
    def shape(self):
        r = self.host.dll.hh_val_rank(self.h)
        buf = (C.c_int64 * max(r, 1))()
        self.host.dll.hh_val_shape(self.h, buf)
        return tuple(buf[i] for i in range(r))

    @property
    def dtype(self):
        return self.host.dll.hh_val_dtype(self.h)

    def numpy(self):
        out = np.empty(self.shape, dtype=_DT2NP[self.dtype])
        self.host.check(self.host.dll.hh_download(self.host.h, self.h, out.ctypes.data_as(C.c_void_p)))
        return out

    def overwrite(self, x):
        """New contents for an input of a recorded program (same shape and dtype)."""
        x = np.asarray(x, dtype=_DT2NP[self.dtype])
        if not x.flags.c_contiguous:
            x = x.copy(order="C")
        assert tuple(x.shape) == tuple(self.shape)
        self.host.check(self.host.dll.hh_overwrite(self.host.h, self.h, x.ctypes.data_as(C.c_void_p)))

    def assign(self, src):
        """This array's memory takes src's elements (how a recorded training step
        hands updated parameters to its next launch)."""
        self.host.check(self.host.dll.hh_assign(self.host.h, self.h, src.h))

    def _o(self, fn, *args):
        return self.host._out(fn, *args)

    def _lift(self, o):
        if isinstance(o, V):
            return o
        return self.host.srepl(self.shape, o, self.dtype)

    # -- Num / Fractional / Floating
    def op1(self, name): return self._o(self.host.dll.hh_ewise1, OP1[name], self.h)
    def op2(self, name, o):
        o = self._lift(o)   # keeps the lifted constant alive across the call
        return self._o(self.host.dll.hh_ewise2, OP2[name], self.h, o.h)

    def _cmp(self, c, o):
        o = self._lift(o)
        return self._o(self.host.dll.hh_compare, CMP[c], self.h, o.h)
    def __add__(self, o): return self.op2("add", o)
    def __radd__(self, o): return self._lift(o).op2("add", self)
    def __sub__(self, o): return self.op2("sub", o)
    def __rsub__(self, o): return self._lift(o).op2("sub", self)
    def __mul__(self, o): return self.op2("mul", o)
    def __rmul__(self, o): return self._lift(o).op2("mul", self)
    def __truediv__(self, o): return self.op2("div", o)
    def __rtruediv__(self, o): return self._lift(o).op2("div", self)
    def __pow__(self, o): return self.op2("pow", o)
    def __neg__(self): return self.op1("neg")
    def atan2H(self, o): return self.op2("atan2", o)
    def quotH(self, o): return self.op2("quot", o)
    def remH(self, o): return self.op2("rem", o)

    # -- comparisons, conditionals, conversions
    def leq(self, o): return self._cmp("leq", o)
    def lt(self, o): return self._cmp("lt", o)
    def eq(self, o): return self._cmp("eq", o)

    def compare_all(self, cmp, o):
        r = C.c_int()
        self.host.check(self.host.dll.hh_compare_all(self.host.h, CMP[cmp], self.h, o.h, C.byref(r)))
        return bool(r.value)

    def select(self, a, b):
        """Elementwise ifH on a Bool tensor."""
        return self._o(self.host.dll.hh_select, self.h, a.h, b.h)

    def scast(self, dtype): return self._o(self.host.dll.hh_convert, self.h, dtype, 0)
    def sfromIntegral(self, dtype): return self._o(self.host.dll.hh_convert, self.h, dtype, 0)
    def sfloor(self, dtype=capi.I64): return self._o(self.host.dll.hh_convert, self.h, dtype, 1)

    # -- maps of scalar closures (Ops.hs:929-941): the closure runs once, on lane values
    def smap0N(self, f):
        """tsmap0N f self"""
        return f(IxV.from_val(self)).to_val()

    def szipWith0N(self, f, o):
        """tszipWith0N f self o"""
        if tuple(self.shape) != tuple(o.shape):
            raise HgpuError(1, "szipWith0N: the two arrays differ in shape")
        return f(IxV.from_val(self), IxV.from_val(o)).to_val()

    # -- reductions and contractions
    def ssum(self): return self._o(self.host.dll.hh_tssumN, self.h, 1)
    def ssumN(self, k): return self._o(self.host.dll.hh_tssumN, self.h, k)
    def ssum0(self): return self._o(self.host.dll.hh_tssum0, self.h)
    def sdot0(self, o): return self._o(self.host.dll.hh_tsdot0, self.h, o.h)
    def sdot1In(self, o): return self._o(self.host.dll.hh_tsdot1In, self.h, o.h)
    def sdotNIn(self, o, n): return self._o(self.host.dll.hh_tsdotNIn, self.h, o.h, n)
    def as_input(self): return self._o(self.host.dll.hh_as_input, self.h)
    def sprimalPart(self): return self._o(self.host.dll.hh_tprimalPart, self.h)
    def tD(self, dual): return self._o(self.host.dll.hh_tD, self.h, dual.h)
    def tconvert(self, conv, shape=None):
        """ConvertTensor: "kfromS", "sfromK", "sfromR", "rfromS", "sfromX", "xfromS", "nest", "unnest";
        shape = the shape the shaped type names (sfromR / sfromX) or the outer dims (nest / unnest)."""
        kinds = ["kfromS", "sfromK", "sfromR", "rfromS", "sfromX", "xfromS", "nest", "unnest"]
        sh = list(shape) if shape is not None else []
        return self._o(self.host.dll.hh_tconvert, kinds.index(conv), self.h, len(sh), _larr(sh))

    def smatvecmul(self, v): return self._o(self.host.dll.hh_tsmatvecmul, self.h, v.h)
    def smatmul2(self, o): return self._o(self.host.dll.hh_tsmatmul2, self.h, o.h)
    def sargMax(self): return self._o(self.host.dll.hh_tsargminmax, self.h, 1)
    def sargMin(self): return self._o(self.host.dll.hh_tsargminmax, self.h, 0)

    # -- structure
    def sreplicate(self, k): return self._o(self.host.dll.hh_tsreplicateN, self.h, 1, _larr([k]))
    def sreplicateN(self, shm): return self._o(self.host.dll.hh_tsreplicateN, self.h, len(shm), _larr(shm))
    sreplicate0N = sreplicateN
    def sappend(self, o): return self._o(self.host.dll.hh_tsappend, self.h, o.h)
    def sslice(self, i, n): return self._o(self.host.dll.hh_tsslice, self.h, i, n)
    def sreverse(self): return self._o(self.host.dll.hh_tsreverse, self.h)
    def stranspose(self, perm): return self._o(self.host.dll.hh_tstranspose, self.h, len(perm), (C.c_int * max(len(perm), 1))(*perm))
    def str_(self): return self.stranspose([1, 0])
    def sreshape(self, shape): return self._o(self.host.dll.hh_tsreshape, self.h, len(shape), _larr(shape))
    def sindex(self, ix): return self._o(self.host.dll.hh_tsindex, self.h, len(ix), _larr(ix))   # `!$` with concrete indices

    # -- indexing with index functions
    def dense(self):
        """The primal part as a dense row-major array (a copy when the value is a strided view)."""
        return self._o(self.host.dll.hh_dense, self.h)

    def sgather(self, shm, f):
        """sgather @shm self (\\[i...] -> [ix...])"""
        shm, ix = self.host._apply_index_fn(shm, f)
        return self._o(self.host.dll.hh_tsgather, self.h, len(shm), _larr(shm), len(ix), _ixarr(ix))

    def sscatter(self, rank_m, shp, f):
        """sscatter @shm self (\\[i...] -> [ix...]) with shm = the first rank_m dims; result shp ++ rest"""
        shm, ix = self.host._apply_index_fn(self.shape[:rank_m], f)
        if len(ix) != len(shp):
            raise HgpuError(1, "sscatter: the index function must return one index per dim of shp")
        return self._o(self.host.dll.hh_tsscatter, self.h, rank_m, len(ix), _larr(shp), _ixarr(ix))

    # inside index functions
    def sindex0(self, ix):
        """self `sindex0` [ix...] with lane-batched indices"""
        first = next(x for x in ix if isinstance(x, IxV))
        ix = [x if isinstance(x, IxV) else IxV.const(self.host, first.shm, x) for x in ix]
        return IxV(self.host, self.host._ixo(self.host.dll.hh_ix_index0, self.h, len(ix), _ixarr(ix)), first.shm)

    def kargMax(self, ix, want_max=True):
        """kargMax (self !$ [ix...])"""
        first = next(x for x in ix if isinstance(x, IxV))
        ix = [x if isinstance(x, IxV) else IxV.const(self.host, first.shm, x) for x in ix]
        return IxV(self.host, self.host._ixo(self.host.dll.hh_ix_argminmax, self.h, len(ix), _ixarr(ix), int(want_max)), first.shm)

    def kargMin(self, ix):
        return self.kargMax(ix, want_max=False)

    def lift(self, shm):
        """A rank-0 tensor as a scalar of the position space shm."""
        return IxV(self.host, self.host._ixo(self.host.dll.hh_ix_lift, len(shm), _larr(shm), self.h), tuple(shm))


# Ranked (`tr*`, user-facing `r*`) and mixed (`tx*` / `x*`) methods of the tensor
# class (Ops.hs:297-1255): the ABI takes shapes at run time, so a ranked or
# mixed method is its shaped twin under another name -- the same entry point,
# the same kernel.  `rtr` = `str_`, `rmaxIndex` / `rminIndex` = `sargMax` /
# `sargMin` as in the reference's naming.
_TWINS = ["map0N", "zipWith0N", "cast", "fromIntegral", "floor", "sum", "sumN", "sum0", "dot0", "dot1In", "dotNIn", "matvecmul", "matmul2",
          "replicate", "replicateN", "append", "slice", "reverse", "transpose", "reshape", "index", "gather", "scatter", "index0"]
for _n in _TWINS:
    for _p in ("r", "x"):
        setattr(V, _p + _n, getattr(V, "s" + _n))
for _p in ("r", "x"):
    setattr(V, _p + "tr", V.str_)
    setattr(V, _p + "maxIndex", V.sargMax)
    setattr(V, _p + "minIndex", V.sargMin)
    setattr(Host, _p + "concrete", Host.sconcrete)
    setattr(Host, _p + "repl", Host.srepl)
    setattr(Host, _p + "iota", Host.siota)
    setattr(Host, _p + "fromVector", Host.sfromVector)
    setattr(Host, _p + "build1", Host.sbuild1)
    setattr(Host, _p + "build", Host.sbuild)
    setattr(Host, _p + "mapAccumL", Host.smapAccumL)
