"""Rows of the entity table that are looked up only when something needs their values.

Unchanged SMORE model code computes a step's negative logits as (smore/models/kg_reasoning.py:301-307,349-355)
    rows  = self.entity_embedding(negative_sample.view(-1), "negative_entity")      # sparse lookup
    rows  = self.entity_regularizer(rows.view(batch_size, negative_size, -1))        # identity, or clamp(rows + 1, .05, 1e9)
    logit = self.cal_logit(rows, None, query_embedding)                              # custom_cal_logit of the model
and custom_cal_logit (models/box.py:157-164, vec.py:85-90, rotate.py:137-142, beta.py:303-308) is
    gamma - dist(rows, query)            [box: gamma - box_dist_out(..) - cen * box_dist_in(..)]   then max over dim 1.
With an EmbeddingOptimizer attached, the lookup returns a `LazyRows` handle instead of a [B*K, row] tensor.
The handle understands exactly what that call sequence does to it -- `.view`, `.unsqueeze`, `+ base_add`,
`torch.clamp`, and ComplEx's `torch.chunk(rows, 2, dim=-1)` / `F.normalize` of each half / `torch.cat` of the two
(models/complex.py:142-146 in its 'norm' mode) -- and the distance operators of smore_amd.torchext.ext_ops, given a handle, return a `LazyLogit`:
a running affine expression  const + sum coef * dist  that scalar arithmetic extends.  The first operation that
needs values (torch.max in custom_cal_logit) evaluates the expression; when it has the shape of one of the
models' logits it becomes ONE launch of the gather-fused scorer (smx_score_forward) on the ids, and its autograd
node hands the entity gradient to the optimizer's fused entity pass.  Anything else -- an expression the fused
scorer has no model for, or any other use of the rows (cal_reg, indexing, printing) -- falls back to the plain
lookup (EmbedLookupFunc) and the dense operators, with the reference's results.

The native_cal_logit bodies (--logit_impl native, the default: config.py:119) write the same logits with torch
operators on the rows: box.py:147-155, vec.py:78-83, rotate.py:125-135, distmult.py:126-133, both branches
of complex.py:169-186 (`_LazyMat` for the shared negatives' torch.mm), and beta.py:293-301 (torch's own Beta-Beta
KL routine on the halves: `_Sym`).  Their intermediates on a handle are
`_LazyExpr` nodes (rows.unsqueeze(1) - center, its abs, relu(abs - offset), min(abs, offset), the stacked halves'
modulus, the products with the queries); torch.norm(.., p=1, dim=-1) or .sum(dim=-1) of the right node is the same
`LazyLogit` term the ext_ops call would have returned.  The fused scorer then computes them with ITS conventions where the two forms differ on a
set of measure zero: the subgradients at |e - c| = 0 and = offset are those of the CUDA functors
(dist_kernel.h:141), not autograd's of abs / relu / min, and RotatE's modulus carries the functor's 1e-20.
"""
import numbers
import weakref

import torch


_FUSED_MODEL = {"l1": "l1", "l2": "l2", "rotate": "rotate", "beta_kl": "beta_kl"}   # logit = const - dist
_FUSED_SIMILARITY = ("complex", "distmult")                                          # logit = const + similarity
UNIT_HALVES = "unit_halves"     # LazyRows.reg of ComplEx rows whose halves were scaled to unit length
UNIT_ROW = "unit_row"           # ... of rows scaled to unit length as a whole (DistMult's 'norm' mode)


def _is_lazy(x):
    return isinstance(x, _Delegating)


def _resolve(x):
    """Replaces every lazy object in a (possibly nested) argument by its tensor."""
    if _is_lazy(x):
        return x.materialize()
    if isinstance(x, (list, tuple)):
        return type(x)(_resolve(v) for v in x)
    if isinstance(x, dict):
        return {k: _resolve(v) for k, v in x.items()}
    return x


def _func_name(func):
    return getattr(func, "__name__", "")


_scalar_cache = {}     # id(tensor) -> (weak reference to that tensor, its version when read, value)


def _scalar(x):
    """Python float of a scalar operand: a number, or a one-element tensor that needs no gradient (the margin
    gamma is nn.Parameter(torch.Tensor([gamma]), requires_grad=False), models/kg_reasoning.py:97-100).  The value
    of such a tensor is read from the device once per version of the tensor, not once per step; the entry holds a
    weak reference, so it can never answer for another tensor that later gets the same id.  None: not a scalar."""
    if isinstance(x, bool):
        return None
    if isinstance(x, numbers.Real):
        return float(x)
    if isinstance(x, torch.Tensor) and x.numel() == 1 and not x.requires_grad and not _is_lazy(x):
        hit = _scalar_cache.get(id(x))
        if hit is None or hit[0]() is not x or hit[1] != x._version:
            key = id(x)
            ref = weakref.ref(x, lambda _, key=key: _scalar_cache.pop(key, None))
            hit = (ref, x._version, float(x.detach().reshape(()).item()))
            _scalar_cache[key] = hit
        return hit[2]
    return None


def _binary(name, reflected=False):
    def op(self, other):
        a, b = self.materialize(), _resolve(other)
        return getattr(torch, name)(b, a) if reflected else getattr(torch, name)(a, b)
    return op


class _Delegating:
    """Everything a handle does not know about is done by the tensor it stands for."""

    # Python's operators do not go through __getattr__: the defaults compute on the tensor (subclasses keep the
    # ones they can do lazily)
    __add__ = _binary("add")
    __radd__ = _binary("add", True)
    __sub__ = _binary("sub")
    __rsub__ = _binary("sub", True)
    __mul__ = _binary("mul")
    __rmul__ = _binary("mul", True)
    __truediv__ = _binary("div")
    __rtruediv__ = _binary("div", True)
    __floordiv__ = _binary("floor_divide")
    __rfloordiv__ = _binary("floor_divide", True)
    __mod__ = _binary("remainder")
    __rmod__ = _binary("remainder", True)
    __matmul__ = _binary("matmul")
    __rmatmul__ = _binary("matmul", True)
    __pow__ = _binary("pow")
    __rpow__ = _binary("pow", True)
    __and__ = _binary("bitwise_and")
    __rand__ = _binary("bitwise_and", True)
    __or__ = _binary("bitwise_or")
    __ror__ = _binary("bitwise_or", True)
    __xor__ = _binary("bitwise_xor")
    __rxor__ = _binary("bitwise_xor", True)
    __lt__ = _binary("lt")
    __le__ = _binary("le")
    __gt__ = _binary("gt")
    __ge__ = _binary("ge")
    # comparisons give a tensor, as they do for the tensor the handle stands for (object identity otherwise);
    # a class that defines __eq__ loses the inherited __hash__: handles stay hashable by identity
    __eq__ = _binary("eq")
    __ne__ = _binary("ne")
    __hash__ = object.__hash__

    def __setitem__(self, key, value):
        self.materialize()[key] = _resolve(value)

    def __invert__(self):
        return ~self.materialize()

    def __pos__(self):
        return +self.materialize()

    def __neg__(self):
        return -self.materialize()

    def __abs__(self):
        return abs(self.materialize())

    def __float__(self):
        return float(self.materialize())

    def __bool__(self):
        return bool(self.materialize())

    def materialize(self):
        raise NotImplementedError

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        handled = cls._try_lazy(func, args, kwargs)
        if handled is not NotImplemented:
            return handled
        return func(*_resolve(args), **_resolve(kwargs))

    @classmethod
    def _try_lazy(cls, func, args, kwargs):
        return NotImplemented

    def __getattr__(self, name):
        if name.startswith("__") and name.endswith("__"):
            raise AttributeError(name)
        return getattr(self.materialize(), name)

    def __getitem__(self, key):
        return self.materialize()[key]

    def __len__(self):
        return self.shape[0]

    def __iter__(self):
        return iter(self.materialize())

    def __repr__(self):
        return f"{type(self).__name__}(shape={tuple(self.shape)})"


class LazyRows(_Delegating):
    """rows-of(table, ids): logical shape ids.shape + (row,), optionally viewed / unsqueezed, optionally carrying the
    entity prologue clamp(rows + add, lo, hi) of smore/common/modules.py:29-36 (reg = (add, lo, hi)) or ComplEx's
    unit-length halves (reg = UNIT_HALVES)."""

    def __init__(self, opt, ids, name, shape=None, reg=None, pending_add=None, root=None):
        self.opt, self.ids, self.name = opt, ids, name
        row = opt.sparse_embed.embedding.shape[1]
        self.shape = torch.Size(tuple(ids.shape) + (row,)) if shape is None else torch.Size(shape)
        self.reg = reg                    # (add, lo, hi) once the clamp has been seen
        self.pending_add = pending_add    # `rows + c` that has not met its clamp yet
        self._root = root                 # None: this handle is the family's first (no reference to itself: the
        self.job_handle = opt.sparse_embed.dummy_job
        if root is None:                  # rows it may hold must go when the last user lets go, not at a later GC pass)
            self._looked_up = None        # the plain lookup, made at most once per handle family

    root = property(lambda self: self if self._root is None else self._root)

    # -- what the model code asks of a tensor before any value is needed
    device = property(lambda self: self.opt.sparse_embed.embedding.device)
    dtype = property(lambda self: self.opt.sparse_embed.embedding.dtype)
    requires_grad = True
    is_cuda = True

    def dim(self):
        return len(self.shape)

    ndim = property(dim)

    def size(self, d=None):
        return self.shape if d is None else self.shape[d]

    def numel(self):
        return self.shape.numel()

    def is_contiguous(self):
        return True

    def contiguous(self):
        return self

    def _like(self, shape):
        return LazyRows(self.opt, self.ids, self.name, shape, self.reg, self.pending_add, self.root)

    def view(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list, torch.Size)):
            shape = tuple(shape[0])
        shape = list(shape)
        if shape.count(-1) > 1 or any(not isinstance(s, int) for s in shape):
            return self.materialize().view(*shape)
        total = self.shape.numel()
        known = 1
        for s in shape:
            known *= s if s != -1 else 1
        if -1 in shape:
            if known == 0 or total % known:
                raise RuntimeError(f"shape {shape} is invalid for input of size {total}")
            shape[shape.index(-1)] = total // known
        elif known != total:
            raise RuntimeError(f"shape {shape} is invalid for input of size {total}")
        if shape[-1] != self.shape[-1]:          # rows are split or joined: values are needed
            return self.materialize().view(*shape)
        return self._like(shape)

    reshape = view

    def unsqueeze(self, d):
        n = len(self.shape)
        d = d + n + 1 if d < 0 else d
        if d > n - 1:                            # a new last dimension is no longer a stack of rows
            return self.materialize().unsqueeze(d)
        return self._like(tuple(self.shape[:d]) + (1,) + tuple(self.shape[d:]))

    def __add__(self, other):
        c = _scalar(other)
        if c is None or self.reg is not None or self.pending_add is not None:
            return torch.add(self.materialize(), _resolve(other))
        out = self._like(self.shape)
        out.pending_add = c
        return out

    __radd__ = __add__

    def __sub__(self, other):          # rows.unsqueeze(1) - center of the native_cal_logit bodies
        node = _LazyExpr.delta(self, other)
        return torch.sub(self.materialize(), _resolve(other)) if node is None else node

    def __mul__(self, other):          # query * rows.unsqueeze(1), distmult.py:131
        node = _LazyExpr.prod(self, other)
        return torch.mul(self.materialize(), _resolve(other)) if node is None else node

    __rmul__ = __mul__

    @classmethod
    def _try_lazy(cls, func, args, kwargs):
        name = _func_name(func)
        if name in ("mul", "multiply", "__mul__", "__rmul__") and len(args) == 2 and not kwargs:
            rows, other = (args[0], args[1]) if isinstance(args[0], LazyRows) else (args[1], args[0])
            if isinstance(rows, LazyRows):
                node = _LazyExpr.prod(rows, other)
                if node is not None:
                    return node
        if name == "clamp" and args and isinstance(args[0], LazyRows):
            x = args[0]
            lo = kwargs.get("min", args[1] if len(args) > 1 else None)
            hi = kwargs.get("max", args[2] if len(args) > 2 else None)
            lo, hi = _scalar(lo), _scalar(hi)
            if x.reg is None and lo is not None and hi is not None:
                out = x._like(x.shape)
                out.reg = (x.pending_add or 0.0, lo, hi)
                out.pending_add = None
                return out
        if name == "normalize" and len(args) == 1 and isinstance(args[0], LazyRows):      # distmult.py:129-130
            x = args[0]
            if (x.reg is None and x.pending_add is None and kwargs.get("p", 2.0) == 2 and
                    kwargs.get("dim", 1) in (-1, x.dim() - 1) and kwargs.get("eps", 1e-12) == 1e-12 and
                    kwargs.get("out") is None):
                out = x._like(x.shape)
                out.reg = UNIT_ROW
                return out
        if name == "chunk" and args and isinstance(args[0], LazyRows):
            x = args[0]
            chunks = kwargs.get("chunks", args[1] if len(args) > 1 else None)
            dim = kwargs.get("dim", args[2] if len(args) > 2 else 0)
            if (chunks == 2 and dim in (-1, x.dim() - 1) and x.pending_add is None and x.shape[-1] % 2 == 0 and
                    ((x.dim() == 3 and x.reg is None) or
                     (x.dim() == 4 and x.shape[1] == 1 and (x.reg is None or isinstance(x.reg, tuple))))):
                return _LazyHalf(x, 0), _LazyHalf(x, 1)    # (4-D with the clamp prologue: beta.py:295)
        if name in ("add", "__add__", "__radd__") and len(args) == 2 and not kwargs:
            rows, other = (args[0], args[1]) if isinstance(args[0], LazyRows) else (args[1], args[0])
            if isinstance(rows, LazyRows) and _scalar(other) is not None:
                return rows.__add__(other)
        return NotImplemented

    def materialize(self):
        """The plain lookup (one per handle family, through the optimizer's autograd node), then whatever views
        and prologue this handle carries, as torch operations."""
        root = self.root
        if root._looked_up is None:
            root._looked_up = self.opt.lookup_rows(self.ids, self.name, for_handle=True)
        rows = root._looked_up.view(self.shape)
        if self.pending_add is not None:
            rows = rows + self.pending_add
        if self.reg == UNIT_HALVES:
            re, im = torch.chunk(rows, 2, dim=-1)
            norm = torch.nn.functional.normalize
            rows = torch.cat((norm(re, p=2, dim=-1), norm(im, p=2, dim=-1)), dim=-1)
        elif self.reg == UNIT_ROW:
            rows = torch.nn.functional.normalize(rows, p=2, dim=-1)
        elif self.reg is not None:
            rows = torch.clamp(rows + self.reg[0], self.reg[1], self.reg[2])
        return rows


class _LazyHalf(_Delegating):
    """One of the two halves torch.chunk(rows, 2, dim=-1) returns for a LazyRows handle [Be, K, row], optionally
    scaled to unit length by F.normalize(half, p=2, dim=-1).  torch.cat of both halves of one handle, in order and
    both scaled, is that handle again with reg = UNIT_HALVES; of both unscaled, the handle itself."""

    def __init__(self, rows, which, unit=False):
        self.rows, self.which, self.unit = rows, which, unit
        self.shape = torch.Size(tuple(rows.shape[:-1]) + (rows.shape[-1] // 2,))

    device = property(lambda self: self.rows.device)
    dtype = property(lambda self: self.rows.dtype)
    requires_grad = True
    is_cuda = True

    def dim(self):
        return len(self.shape)

    ndim = property(dim)

    def size(self, d=None):
        return self.shape if d is None else self.shape[d]

    @classmethod
    def _try_lazy(cls, func, args, kwargs):
        name = _func_name(func)
        if name == "normalize" and args and isinstance(args[0], _LazyHalf) and len(args) == 1:
            x = args[0]
            if (not x.unit and x.rows.reg is None and kwargs.get("p", 2.0) == 2 and
                    kwargs.get("dim", 1) in (-1, x.dim() - 1) and kwargs.get("eps", 1e-12) == 1e-12 and
                    kwargs.get("out") is None):
                return _LazyHalf(x.rows, x.which, True)
        if name in ("mul", "multiply", "__mul__", "__rmul__") and len(args) == 2 and not kwargs:
            half, other = (args[0], args[1]) if isinstance(args[0], _LazyHalf) else (args[1], args[0])
            if isinstance(half, _LazyHalf):
                node = _LazyExpr.prod(half, other)
                if node is not None:
                    return node
        if name in ("digamma", "lgamma") and len(args) == 1 and not kwargs and isinstance(args[0], _LazyHalf):
            node = _Sym.make(name, args[0])
            if node is not None:
                return node
        if name == "cat" and args and isinstance(args[0], (tuple, list)) and len(args[0]) == 2:
            a, b = args[0]
            dim = kwargs.get("dim", args[1] if len(args) > 1 else 0)
            if (isinstance(a, _LazyHalf) and isinstance(b, _LazyHalf) and a.rows is b.rows and a.which == 0 and
                    b.which == 1 and a.unit == b.unit and dim in (-1, a.dim() - 1) and kwargs.get("out") is None):
                if not a.unit:
                    return a.rows
                out = a.rows._like(a.rows.shape)
                out.reg = UNIT_HALVES
                return out
        return NotImplemented

    def __sub__(self, other):          # entity_re_embedding - query_re_embedding of rotate.py:129-130
        node = _LazyExpr.delta(self, other)
        if node is None:
            node = _Sym.make("sub", self, other)
        return torch.sub(self.materialize(), _resolve(other)) if node is None else node

    def __mul__(self, other):          # entity_re_embedding * query_re_embedding of complex.py:176
        node = _LazyExpr.prod(self, other)
        return torch.mul(self.materialize(), _resolve(other)) if node is None else node

    __rmul__ = __mul__

    def __add__(self, other):          # p.concentration1 + p.concentration0 of torch's Beta KL (beta.py:298)
        node = _Sym.make("add", self, other)
        return torch.add(self.materialize(), _resolve(other)) if node is None else node

    def view(self, *shape):            # entity_re_embedding.view(nent, embed_dim) of complex.py:181-182
        if len(shape) == 1 and isinstance(shape[0], (tuple, list, torch.Size)):
            shape = tuple(shape[0])
        if (self.dim() == 4 and tuple(self.shape[:2]) == (1, 1) and tuple(shape) == tuple(self.shape[2:]) and
                self.rows.pending_add is None and (self.rows.reg is None or self.unit)):
            return _LazyMat(self, False)
        return self.materialize().view(*shape)

    def lgamma(self):
        node = _Sym.make("lgamma", self)
        return self.materialize().lgamma() if node is None else node

    def digamma(self):
        node = _Sym.make("digamma", self)
        return self.materialize().digamma() if node is None else node

    def materialize(self):
        half = torch.chunk(self.rows.materialize(), 2, dim=-1)[self.which]
        return torch.nn.functional.normalize(half, p=2, dim=-1) if self.unit else half


class _LazyMat(_Delegating):
    """The shared-negative branch of ComplEx's native_cal_logit (complex.py:178-186): one half of a [1, 1, K, 2h]
    handle viewed as the matrix [K, h] (`product` None, `transposed` False), its transpose [h, K], and
    torch.mm(query [B, h], that transpose) -> [B, K] (`product` = the query matrix).  The sum of the two halves'
    products is the ComplEx logit of the K shared rows against every query: the LazyLogit term of ext_ops.complex_sim,
    its single branch taken."""

    def __init__(self, half, transposed, product=None):
        self.half, self.transposed, self.product = half, transposed, product
        k, h = half.shape[2], half.shape[3]
        self.shape = torch.Size((product.shape[0], k) if product is not None else ((h, k) if transposed else (k, h)))

    device = property(lambda self: self.half.device)
    dtype = property(lambda self: self.half.dtype)
    requires_grad = True
    is_cuda = True

    def dim(self):
        return 2

    ndim = property(dim)

    def size(self, d=None):
        return self.shape if d is None else self.shape[d]

    def t(self):
        if self.product is None:
            return _LazyMat(self.half, not self.transposed)
        return self.materialize().t()

    def materialize(self):
        k, h = self.half.shape[2], self.half.shape[3]
        m = self.half.materialize().view(k, h)
        if self.product is not None:
            return torch.mm(self.product, m.t())
        return m.t() if self.transposed else m

    def __add__(self, other):
        a, b = self, other
        if (isinstance(b, _LazyMat) and a.product is not None and b.product is not None and a.half.which == 0 and
                b.half.which == 1 and a.half.rows is b.half.rows and a.half.unit == b.half.unit and
                a.product.shape == b.product.shape):
            handle = a.half.rows                                   # [1, 1, K, 2h]
            rows = handle._like((1, handle.shape[2], handle.shape[3]))
            if a.half.unit:
                rows.reg = UNIT_HALVES
            bq, h = a.product.shape
            term = lazy_dist("complex", rows, a.product.view(bq, 1, 1, h), b.product.view(bq, 1, 1, h))
            if term is not None:
                return torch.max(term, dim=1)[0]                   # one branch: [B, 1, K] -> [B, K]
        return torch.add(self.materialize(), _resolve(other))

    @classmethod
    def _try_lazy(cls, func, args, kwargs):
        name = _func_name(func)
        if name == "mm" and len(args) == 2 and not kwargs:
            q, m = args
            if (isinstance(m, _LazyMat) and m.product is None and m.transposed and isinstance(q, torch.Tensor) and
                    not _is_lazy(q) and q.dim() == 2 and q.shape[1] == m.shape[0] and q.dtype == m.dtype and
                    q.device == m.device):
                return _LazyMat(m.half, True, q)
        if name in ("add", "__add__") and len(args) == 2 and not kwargs and isinstance(args[0], _LazyMat):
            return args[0].__add__(args[1])
        if name == "t" and len(args) == 1 and isinstance(args[0], _LazyMat):
            return args[0].t()
        return NotImplemented


class _Sym(_Delegating):
    """A node of the expression torch's Beta-Beta KL routine builds from the two halves of a 4-D handle
    (native_cal_logit of beta.py:293-301 hands it BetaDist(alpha half, beta half) and BetaDist(*query)):
    add / sub / mul of nodes, halves and plain tensors, lgamma and digamma of nodes and halves.  Nothing is
    computed while the expression grows; torch.norm(.., p=1, dim=-1) of the finished one asks `beta_kl_operands`
    whether it IS that routine's expression of these halves and two query tensors, and if so becomes the same
    LazyLogit term ext_ops.beta_kl returns.  Any other use evaluates the expression with torch, node by node."""

    _BINARY = {"add": torch.add, "sub": torch.sub, "mul": torch.mul}
    _UNARY = {"lgamma": torch.lgamma, "digamma": torch.digamma}

    def __init__(self, op, args, handle, shape):
        self.op, self.args, self.handle = op, tuple(args), handle
        self.shape = torch.Size(shape)
        self._value = None

    device = property(lambda self: self.handle.device)
    dtype = property(lambda self: self.handle.dtype)
    requires_grad = True
    is_cuda = True

    def dim(self):
        return len(self.shape)

    ndim = property(dim)

    def size(self, d=None):
        return self.shape if d is None else self.shape[d]

    @staticmethod
    def _handle_of(x):
        if isinstance(x, _Sym):
            return x.handle
        if isinstance(x, _LazyHalf) and not x.unit and x.dim() == 4:
            return x.rows
        return None

    @staticmethod
    def make(op, *args):
        """The node op(args), or None when an operand is neither a node, a half of the same 4-D handle nor a plain
        tensor of the handle's dtype and device."""
        handle = None
        for a in args:
            h = _Sym._handle_of(a)
            if h is not None:
                if handle is not None and h is not handle:
                    return None
                handle = h
            elif not (isinstance(a, torch.Tensor) and not _is_lazy(a) and a.dim() == 4):
                return None
        if handle is None or any(isinstance(a, torch.Tensor) and (a.dtype != handle.dtype or a.device != handle.device)
                                 for a in args):
            return None
        try:
            shape = torch.broadcast_shapes(*[tuple(a.shape) for a in args])
        except RuntimeError:
            return None
        return _Sym(op, args, handle, shape)

    def materialize(self):
        if self._value is None:
            vals = [_resolve(a) for a in self.args]
            self._value = (self._BINARY.get(self.op) or self._UNARY[self.op])(*vals)
        return self._value

    def _binary(self, op, other, reflected=False):
        node = _Sym.make(op, other, self) if reflected else _Sym.make(op, self, other)
        if node is not None:
            return node
        a, b = (_resolve(other), self.materialize()) if reflected else (self.materialize(), _resolve(other))
        return self._BINARY[op](a, b)

    def __add__(self, other):
        return self._binary("add", other)

    def __radd__(self, other):
        return self._binary("add", other, True)

    def __sub__(self, other):
        return self._binary("sub", other)

    def __rsub__(self, other):
        return self._binary("sub", other, True)

    def __mul__(self, other):
        return self._binary("mul", other)

    def __rmul__(self, other):
        return self._binary("mul", other, True)

    def lgamma(self):
        return _Sym.make("lgamma", self)

    def digamma(self):
        return _Sym.make("digamma", self)

    def norm(self, p="fro", dim=None, keepdim=False, dtype=None):
        out = self._l1(p, dim, keepdim, dtype)
        return self.materialize().norm(p=p, dim=dim, keepdim=keepdim, dtype=dtype) if out is None else out

    def _l1(self, p, dim, keepdim, dtype):
        if p in (1, 1.0) and dim in (-1, self.dim() - 1) and not keepdim and dtype is None:
            try:
                found = beta_kl_operands(self)
            except (AttributeError, TypeError, ValueError, RuntimeError):   # an autograd graph of a shape this code
                found = None                                                # does not know: torch evaluates the expression
            if found is not None:
                return lazy_dist("beta_kl", *found)
        return None

    @classmethod
    def _try_lazy(cls, func, args, kwargs):
        name = _func_name(func)
        if len(args) == 2 and not kwargs:
            a, b = args
            op = {"add": "add", "__add__": "add", "__radd__": "add", "sub": "sub", "subtract": "sub", "__sub__": "sub",
                  "mul": "mul", "multiply": "mul", "__mul__": "mul", "__rmul__": "mul"}.get(name)
            if name in ("rsub", "__rsub__"):
                a, b, op = b, a, "sub"
            if op is not None:
                node = _Sym.make(op, a, b)
                if node is not None:
                    return node
        if name in cls._UNARY and len(args) == 1 and not kwargs:
            node = _Sym.make(name, args[0])
            if node is not None:
                return node
        if name == "norm" and len(args) == 1 and isinstance(args[0], _Sym) and kwargs.get("out") is None:
            out = args[0]._l1(kwargs.get("p", "fro"), kwargs.get("dim"), kwargs.get("keepdim", False), kwargs.get("dtype"))
            if out is not None:
                return out
        return NotImplemented


def _same_source(a, b):
    """Whether two tensors are the same value of the same autograd graph: one object, or one output of one node."""
    if a is b:
        return True
    return (isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor) and a.grad_fn is not None and
            a.grad_fn is b.grad_fn and a.output_nr == b.output_nr)


def _made_by(t, node_name, *inputs):
    """Whether autograd recorded tensor t as node_name(inputs) -- each input a tensor, or a nested (node_name,
    inputs...) tuple for an intermediate that nothing else holds."""
    fn = t if not isinstance(t, torch.Tensor) else t.grad_fn
    if fn is None or fn.name() != node_name or len(fn.next_functions) < len(inputs):
        return False
    for (nxt, nr), want in zip(fn.next_functions, inputs):
        if isinstance(want, tuple):
            if nxt is None or not _made_by(nxt, *want):
                return False
        elif want.grad_fn is not None:
            if nxt is not want.grad_fn or nr != want.output_nr:
                return False
        elif nxt is None or getattr(nxt, "variable", None) is not want:     # a leaf that requires grad
            return False
    return True


def beta_kl_operands(expr):
    """(rows, qa, qb) when `expr` is, node for node, what torch.distributions.kl._kl_beta_beta(p, q) builds for
    p = BetaDist(alpha half, beta half) of one 4-D handle and q = BetaDist(qa, qb):
        sp = a + b;  sq = qa + qb
        t1 = qa.lgamma() + qb.lgamma() + sp.lgamma();  t2 = a.lgamma() + b.lgamma() + sq.lgamma()
        t3 = (a - qa) * digamma(a);  t4 = (b - qb) * digamma(b);  t5 = (sq - sp) * digamma(sp)
        t1 - t2 + t3 + t4 + t5
    The query-side operands are plain tensors when they reach the expression; that they are lgamma(qa) + lgamma(qb),
    lgamma(qa + qb) and qa + qb of the very qa and qb the halves meet in t3 and t4 is read off the autograd graph
    torch recorded for them; where nothing carries a graph (evaluation under no_grad) they are compared by value.
    None otherwise."""
    def node(x, op, n):
        return x.args if isinstance(x, _Sym) and x.op == op and len(x.args) == n else None

    def half(x, which):
        return isinstance(x, _LazyHalf) and x.which == which and not x.unit and x.rows is expr.handle

    def is_sp(x):
        args = node(x, "add", 2)
        return args is not None and half(args[0], 0) and half(args[1], 1)

    def unary(x, op, inner):
        args = node(x, op, 1)
        return args is not None and inner(args[0])

    plain = lambda t: isinstance(t, torch.Tensor) and not _is_lazy(t)
    try:
        s4, t5 = node(expr, "add", 2)
        s3, t4 = node(s4, "add", 2)
        s2, t3 = node(s3, "add", 2)
        t1, t2 = node(s2, "sub", 2)
        x, lg_sp = node(t1, "add", 2)                     # (lgamma(qa) + lgamma(qb)) + lgamma(sp)
        lg_ab, y = node(t2, "add", 2)                     # (lgamma(a) + lgamma(b)) + lgamma(sq)
        lg_a, lg_b = node(lg_ab, "add", 2)
        d_a, psi_a = node(t3, "mul", 2)
        d_b, psi_b = node(t4, "mul", 2)
        d_s, psi_s = node(t5, "mul", 2)
        a0, qa = node(d_a, "sub", 2)
        b0, qb = node(d_b, "sub", 2)
        sq, sp2 = node(d_s, "sub", 2)
    except TypeError:                                      # some node was not of the expected kind
        return None
    a_is = lambda v: half(v, 0)
    b_is = lambda v: half(v, 1)
    if not (unary(lg_sp, "lgamma", is_sp) and unary(lg_a, "lgamma", a_is) and unary(lg_b, "lgamma", b_is) and
            unary(psi_a, "digamma", a_is) and unary(psi_b, "digamma", b_is) and unary(psi_s, "digamma", is_sp) and
            a_is(a0) and b_is(b0) and is_sp(sp2) and all(plain(t) for t in (x, y, qa, qb, sq))):
        return None
    if qa.shape != qb.shape or not _LazyExpr._query(qa, a0) or not _LazyExpr._query(qb, b0):
        return None
    if all(t.grad_fn is None and not t.requires_grad for t in (x, y, qa, qb, sq)):
        # no graph at all (evaluation under torch.no_grad()): the operands are compared by value instead -- three
        # small elementwise kernels and one wait for the device, nothing next to scoring every entity
        if not (torch.equal(sq, qa + qb) and torch.equal(y, sq.lgamma()) and torch.equal(x, qa.lgamma() + qb.lgamma())):
            return None
    elif not (_made_by(sq, "AddBackward0", qa, qb) and _made_by(y, "LgammaBackward0", ("AddBackward0", qa, qb)) and
              _made_by(x, "AddBackward0", ("LgammaBackward0", qa), ("LgammaBackward0", qb))):
        return None
    handle = expr.handle
    return handle._like((handle.shape[0], handle.shape[2], handle.shape[3])), qa, qb


class _LazyExpr(_Delegating):
    """An intermediate of a native_cal_logit body on a handle: `op` applied to rows [Be, 1, K, w] (a 4-D handle, or
    one half of it) and the query tensors [B, U, 1, w] in `queries`; logical shape [B, U, K, w].
      delta     rows - c                      box.py:150, vec.py:80, rotate.py:129-130 (half = 0 / 1)
      absdelta  |rows - c|                    box.py:150
      excess    |rows - c| - o                box.py:151
      box_out   relu(|rows - c| - o)          box.py:151
      box_in    min(|rows - c|, o)            box.py:152
      stack     stack([re - q_re, im - q_im], dim=0)     rotate.py:131
      modulus   its norm over dim 0                      rotate.py:132
      prod      rows * q                      distmult.py:131; one half (possibly at unit length): complex.py:176
      cprod     re * q_re + im * q_im         complex.py:176
    The value, if something else asks for it, is the torch expression itself."""

    def __init__(self, op, rows, queries, shape, compute, half=None, unit=False):
        self.op, self.rows, self.queries, self.half, self.unit = op, rows, tuple(queries), half, unit
        self.shape = torch.Size(shape)
        self._compute, self._value = compute, None

    device = property(lambda self: self.rows.device)
    dtype = property(lambda self: self.rows.dtype)
    requires_grad = True
    is_cuda = True

    def dim(self):
        return len(self.shape)

    ndim = property(dim)

    def size(self, d=None):
        return self.shape if d is None else self.shape[d]

    def materialize(self):
        if self._value is None:
            self._value = self._compute()
        return self._value

    @staticmethod
    def _query(t, like):
        """Whether t is a plain query tensor [B, U, 1, w] for rows / another query tensor `like`."""
        return (isinstance(t, torch.Tensor) and not _is_lazy(t) and t.dim() == 4 and t.shape[2] == 1 and
                t.shape[3] == like.shape[3] and t.dtype == like.dtype and t.device == like.device)

    @staticmethod
    def _binary_with_query(op, source, q, compute, unit_ok):
        """op(source, q) for a 4-D handle [Be, 1, K, w] or one of its halves; None when it is not that shape."""
        if isinstance(source, LazyRows):
            handle, half, unit = source, None, source.reg == UNIT_ROW
        elif isinstance(source, _LazyHalf) and (unit_ok or not source.unit):
            handle, half, unit = source.rows, source.which, source.unit
        else:
            return None
        plain = handle.reg is None or (half is None and unit and unit_ok)
        if (handle.dim() != 4 or handle.shape[1] != 1 or not plain or handle.pending_add is not None or
                not _LazyExpr._query(q, source) or q.shape[0] not in (1, handle.shape[0]) and handle.shape[0] != 1):
            return None
        rows = handle._like((handle.shape[0], handle.shape[2], handle.shape[3]))   # (keeps the handle's reg)
        shape = (max(q.shape[0], handle.shape[0]), q.shape[1], handle.shape[2], q.shape[3])
        return _LazyExpr(op, rows, (q,), shape, compute, half, unit)

    @staticmethod
    def delta(source, q):
        return _LazyExpr._binary_with_query("delta", source, q, lambda: source.materialize() - q, False)

    @staticmethod
    def prod(source, q):
        return _LazyExpr._binary_with_query("prod", source, q, lambda: source.materialize() * q, True)

    def __add__(self, other):
        if (self.op == "prod" and isinstance(other, _LazyExpr) and other.op == "prod" and self.half == 0 and
                other.half == 1 and self._same_rows(other) and self.unit == other.unit and self.shape == other.shape):
            return _LazyExpr("cprod", self.rows, self.queries + other.queries, self.shape,
                             lambda: self.materialize() + other.materialize(), None, self.unit)
        return torch.add(self.materialize(), _resolve(other))

    def _same_rows(self, other):
        return self.rows.root is other.rows.root and self.rows.shape == other.rows.shape

    def _follow(self, op, queries, compute):
        return _LazyExpr(op, self.rows, queries, self.shape, compute, self.half)

    # -- the steps of the bodies
    def abs(self):
        if self.op == "delta" and self.half is None:
            return self._follow("absdelta", self.queries, lambda: self.materialize().abs())
        return self.materialize().abs()

    __abs__ = abs

    def __sub__(self, other):
        if self.op == "absdelta" and self._query(other, self.queries[0]) and other.shape == self.queries[0].shape:
            return self._follow("excess", self.queries + (other,), lambda: self.materialize() - other)
        return torch.sub(self.materialize(), _resolve(other))

    def norm(self, p="fro", dim=None, keepdim=False, dtype=None):
        out = self._norm(p, dim, keepdim, dtype)
        return self.materialize().norm(p=p, dim=dim, keepdim=keepdim, dtype=dtype) if out is None else out

    def _norm(self, p, dim, keepdim, dtype):
        if keepdim or dtype is not None:
            return None
        if self.op == "stack" and p in ("fro", 2, 2.0) and dim == 0:
            shape = tuple(self.shape[1:])
            return _LazyExpr("modulus", self.rows, self.queries, shape, lambda: self.materialize().norm(dim=0))
        if p in (1, 1.0) and dim in (-1, self.dim() - 1):
            if self.op in ("box_out", "box_in"):
                return lazy_dist(self.op, self.rows, *self.queries)
            if self.op == "delta" and self.half is None:
                return lazy_dist("l1", self.rows, *self.queries)
        return None

    def sum(self, dim=None, keepdim=False, dtype=None):
        if dim in (-1, self.dim() - 1) and not keepdim and dtype is None:
            out = None
            if self.op == "modulus":
                out = lazy_dist("rotate", self.rows, *self.queries)
            elif self.op == "prod" and self.half is None:
                out = lazy_dist("distmult", self.rows, *self.queries)
            elif self.op == "cprod":
                rows = self.rows
                if self.unit:
                    rows = rows._like(rows.shape)
                    rows.reg = UNIT_HALVES
                out = lazy_dist("complex", rows, *self.queries)
            if out is not None:
                return out
        return self.materialize().sum(dim=dim, keepdim=keepdim, dtype=dtype)

    @classmethod
    def _try_lazy(cls, func, args, kwargs):
        name = _func_name(func)
        x = args[0] if args else None
        if name == "abs" and isinstance(x, _LazyExpr) and len(args) == 1 and not kwargs:
            return x.abs()
        if name == "relu" and isinstance(x, _LazyExpr) and len(args) == 1 and not kwargs.get("inplace", False):
            if x.op == "excess":
                return x._follow("box_out", x.queries, lambda: torch.relu(x.materialize()))
        if name in ("min", "minimum") and len(args) == 2 and not kwargs and isinstance(x, _LazyExpr):
            o = args[1]
            if x.op == "absdelta" and cls._query(o, x.queries[0]) and o.shape == x.queries[0].shape:
                return x._follow("box_in", x.queries + (o,), lambda: torch.min(x.materialize(), o))
        if name == "norm" and isinstance(x, _LazyExpr) and len(args) == 1:
            out = x._norm(kwargs.get("p", "fro"), kwargs.get("dim"), kwargs.get("keepdim", False), kwargs.get("dtype"))
            if out is not None and kwargs.get("out") is None:
                return out
        if name == "sum" and isinstance(x, _LazyExpr) and len(args) <= 2 and set(kwargs) <= {"dim"}:
            return x.sum(dim=kwargs.get("dim", args[1] if len(args) > 1 else None))
        if name in ("add", "__add__") and len(args) == 2 and not kwargs and isinstance(x, _LazyExpr):
            return x.__add__(args[1])
        if name == "stack" and isinstance(x, (list, tuple)) and len(x) == 2 and kwargs.get("out") is None:
            a, b = x
            dim = kwargs.get("dim", args[1] if len(args) > 1 else 0)
            if (isinstance(a, _LazyExpr) and isinstance(b, _LazyExpr) and a.op == b.op == "delta" and a.half == 0 and
                    b.half == 1 and a._same_rows(b) and a.shape == b.shape and dim == 0):
                return _LazyExpr("stack", a.rows, a.queries + b.queries, (2,) + tuple(a.shape),
                                 lambda: torch.stack([a.materialize(), b.materialize()], dim=0))
        return NotImplemented


class _Dist:
    """dist(kind, rows handle, query tensors), not yet evaluated."""

    def __init__(self, kind, rows, queries):
        self.kind, self.rows, self.queries = kind, rows, tuple(queries)

    def same_operands(self, other):
        return (self.rows.root is other.rows.root and self.rows.shape == other.rows.shape and
                self.rows.reg == other.rows.reg and self.rows.pending_add == other.rows.pending_add and
                len(self.queries) == len(other.queries) and all(a is b for a, b in zip(self.queries, other.queries)))

    def out_shape(self):
        q, e = self.queries[0], self.rows
        if q.dim() == 4:
            return torch.Size((max(e.shape[0], q.shape[0]), q.shape[1], max(e.shape[1], q.shape[2])))
        return torch.Size((max(e.shape[0], q.shape[0]), max(e.shape[1], q.shape[1])))

    def dense(self):
        from ..torchext.dist_func import _base
        rows = self.rows.materialize().contiguous()
        if self.kind == "l2":
            return torch.sqrt(_base.apply_dist("l2", rows, *self.queries))
        return _base.apply_dist(self.kind, rows, *self.queries)


class LazyLogit(_Delegating):
    """const + sum coef_i * dist_i over unevaluated distances; scalar arithmetic keeps it lazy."""

    def __init__(self, const, terms):
        self.const, self.terms = float(const), list(terms)
        self._value = None

    @staticmethod
    def of(kind, rows, queries):
        return LazyLogit(0.0, [(1.0, _Dist(kind, rows, queries))])

    shape = property(lambda self: self.terms[0][1].out_shape())
    device = property(lambda self: self.terms[0][1].rows.device)
    dtype = torch.float32

    def dim(self):
        return len(self.shape)

    def size(self, d=None):
        return self.shape if d is None else self.shape[d]

    # -- arithmetic that keeps the expression lazy
    def _scaled(self, c):
        return LazyLogit(self.const * c, [(k * c, d) for k, d in self.terms])

    def _plus(self, other, sign):
        if isinstance(other, LazyLogit):
            return LazyLogit(self.const + sign * other.const, self.terms + [(sign * k, d) for k, d in other.terms])
        c = _scalar(other)
        if c is None:
            return NotImplemented
        return LazyLogit(self.const + sign * c, self.terms)

    def __neg__(self):
        return self._scaled(-1.0)

    def __add__(self, other):
        out = self._plus(other, 1.0)
        return torch.add(self.materialize(), _resolve(other)) if out is NotImplemented else out

    __radd__ = __add__

    def __sub__(self, other):
        out = self._plus(other, -1.0)
        return torch.sub(self.materialize(), _resolve(other)) if out is NotImplemented else out

    def __rsub__(self, other):
        out = self._scaled(-1.0)._plus(other, 1.0)
        return torch.sub(_resolve(other), self.materialize()) if out is NotImplemented else out

    def __mul__(self, other):
        c = _scalar(other)
        return torch.mul(self.materialize(), _resolve(other)) if c is None else self._scaled(c)

    __rmul__ = __mul__

    def __truediv__(self, other):
        c = _scalar(other)
        return torch.div(self.materialize(), _resolve(other)) if c is None or c == 0.0 else self._scaled(1.0 / c)

    @classmethod
    def _try_lazy(cls, func, args, kwargs):
        name = _func_name(func)
        if len(args) == 2 and not kwargs:
            a, b = args
            if name in ("rsub", "__rsub__"):            # other - input
                a, b, name = b, a, "sub"
            lazy_first = isinstance(a, LazyLogit)
            if name in ("add", "__add__", "__radd__"):
                return a.__add__(b) if lazy_first else b.__add__(a)
            if name in ("sub", "subtract", "__sub__"):
                return a.__sub__(b) if lazy_first else b.__rsub__(a)
            if name in ("mul", "multiply", "__mul__", "__rmul__"):
                return a.__mul__(b) if lazy_first else b.__mul__(a)
        if name in ("neg", "negative", "__neg__") and len(args) == 1 and not kwargs:
            return -args[0]
        if name == "max" and args and isinstance(args[0], LazyLogit):
            # torch.max(logit, dim=1) of custom_cal_logit, the maximum over the union branches: the logits can wait
            # until something needs their values -- by then the step's other lookups against the same queries
            # (positives, negatives) have asked too, and all of them go into one launch
            dim = kwargs.get("dim", args[1] if len(args) > 1 else None)
            self = args[0]
            if (dim == 1 and len(args) <= 2 and set(kwargs) <= {"dim"} and self._value is None and
                    len(self.shape) == 3 and self._fusable() is not None):
                scores = LazyScores(self)
                if scores.request is not None:
                    return _MaxResult(scores, _LazyIndices(scores))
        return NotImplemented

    # -- evaluation
    def _fusable(self):
        """(model, cen) when the expression is one of the logits the fused scorer computes, else None."""
        if len(self.terms) == 1:
            k, d = self.terms[0]
            if k == -1.0 and d.kind in _FUSED_MODEL:
                return _FUSED_MODEL[d.kind], 0.0
            if k == -1.0 and d.kind == "box_out":
                return "box", 0.0
            if k == 1.0 and d.kind in _FUSED_SIMILARITY:        # models/complex.py:140-148: the similarity is the logit
                return d.kind, 0.0
        if len(self.terms) == 2:
            (k0, d0), (k1, d1) = self.terms
            if d0.kind == "box_in":
                (k0, d0), (k1, d1) = (k1, d1), (k0, d0)
            if d0.kind == "box_out" and d1.kind == "box_in" and k0 == -1.0 and d0.same_operands(d1):
                return "box", -k1
        return None

    def materialize(self):
        if self._value is not None:
            return self._value
        fused = self._fusable()
        value = None
        if fused is not None:
            model, cen = fused
            d = self.terms[0][1]
            value = d.rows.opt.score_lazy(model, d.rows, d.queries, self.const, cen)
        if value is None:      # not a shape the fused scorer takes: plain lookup + dense operators
            note = getattr(self.terms[0][1].rows.opt, "note_dense_fallback", None)
            if note is not None:
                note("a logit of " + " / ".join(sorted({d.kind for _, d in self.terms})) +
                     f" on rows {tuple(self.terms[0][1].rows.shape)}")
            value = self.const
            for k, d in self.terms:
                value = value + k * d.dense()
        self._value = value
        return value


class _MaxResult(tuple):
    """(values, indices) as torch.max(x, dim) returns them."""

    def __new__(cls, values, indices):
        return super().__new__(cls, (values, indices))

    values = property(lambda self: self[0])
    indices = property(lambda self: self[1])


class _LazyIndices(_Delegating):
    """Which branch held the maximum: known once the scores are, made only if somebody looks."""

    def __init__(self, scores):
        self.scores = scores
        self.dtype = torch.int64

    shape = property(lambda self: self.scores.shape)
    device = property(lambda self: self.scores.device)

    def materialize(self):
        self.scores.materialize()
        if self.scores._index is None:      # one branch
            self.scores._index = torch.zeros(self.shape, dtype=torch.int64, device=self.device)
        return self.scores._index


class LazyScores(_Delegating):
    """Logits [B, K] of one lookup against the queries (the maximum over their union branches), not yet computed.
    The optimizer keeps the step's pending ones; the first that is needed evaluates all that share its model,
    margin, parameters and query tensors in one launch of the fused scorer (ids side by side,
    [B, K_1 + K_2 + ..]), so that the step leaves one record with the optimizer, as if the caller had concatenated
    positives and negatives itself."""

    def __init__(self, logit):
        self.logit = logit
        self._value = None
        self._index = None      # branch of the maximum, [B, K]; None while there is one branch only
        d = logit.terms[0][1]
        self.opt = d.rows.opt
        model, cen = logit._fusable()
        self.request = self.opt.lazy_request(model, d.rows, d.queries, logit.const, cen)   # None: not a fused layout
        if self.request is not None:
            self.opt.pending_scores.append(weakref.ref(self))   # a placeholder nobody holds any more is never scored

    shape = property(lambda self: torch.Size((self.logit.shape[0], self.logit.shape[2])))
    device = property(lambda self: self.logit.device)
    dtype = torch.float32

    def dim(self):
        return 2

    def size(self, d=None):
        return self.shape if d is None else self.shape[d]

    def materialize(self):
        if self._value is None:
            self.opt.evaluate_pending(self)
        return self._value


def lazy_dist(kind, entity_embed, *queries):
    """What an operator of ext_ops returns for a LazyRows entity argument."""
    if kind not in ("l1", "l2", "rotate", "beta_kl", "box_out", "box_in", "complex", "distmult"):
        return None
    if any(_is_lazy(q) or not isinstance(q, torch.Tensor) for q in queries):
        return None
    if entity_embed.dim() != 3 or entity_embed.pending_add is not None:
        return None
    q = queries[0]
    if q.dim() not in (3, 4) or any(x.shape != q.shape for x in queries[1:]):
        return None
    return LazyLogit.of(kind, entity_embed, queries)
