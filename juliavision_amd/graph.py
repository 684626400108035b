"""A minimal loader/executor for exported op graphs, dispatching to the MI355X kernels.

The reference runs ``torch.export`` graphs serialised as JSON -- ``buffers``
(``weight`` / ``external`` / ``transient`` / ``view`` / ``host``) and ``ops``
(``aten`` name, ``in``, ``out``, ``attrs`` with positional constants as ``arg<j>``),
written by ``tools/export_graphs.py:111-230`` and read by ``graph.jl:125-149`` --
through one handler per ATen op (``runop!``, ``execute.jl:493-539``, ``ops.jl``).
This module reads the same schema, keeps the handler-per-op shape, and covers
the ops of the dense-contraction path:

    linear / addmm / mm / bmm, scaled_dot_product_attention (also written out
    as bmm + softmax + bmm), layer_norm / native_layer_norm, gelu, relu,
    add.Tensor, convolution, cat along the token axis, softmax over the last
    axis, mul / div by a constant, clamp, a per-feature or constant mul.Tensor
    after a linear (LayerScale, query scaling), contiguous clone, and the view
    ops between them.

Two of the reference's rewrites matter for that path and have counterparts here:

* ``foldrelu.jl:60-125`` folds an activation into the producing ``addmm``'s
  epilogue: ``fold_activations``.
* ``hoistcasts.jl:47-112`` (``hoistpermutes``) pre-transposes ``addmm`` weights
  at load time.  Nothing to hoist here: the GEMM reads ``[F][K]`` weights through
  a transposed view (``MI_W_FK``), so the permute stays a view.

and two more fall out of what the kernels accept: the residual ``add.Tensor``
after a linear rides in its GEMM store (``fold_residuals``; the reference's own
next item, plans/perf-plan.md:4074-4095), and attention writes its output
token-major when the graph transposes it straight back (``fold_sdpa_transpose``);
attention exported as ``bmm`` + ``_softmax`` + ``bmm`` (DINOv2) is put back together
(``fold_attention``).  A layer norm that only linear ops read, over enough rows for
the tiled GEMMs, gets no pass of its own (``fold_norms_away``): its readers run on
the raw rows with prepared weights, the row statistics come out of the GEMM that
wrote those rows.

The decoder step (tools/export_whisper_decoder.py:90-240) is functional: it takes
the self-attention cache, writes the new token's rows with ``index_copy`` /
``index_put``, masks the unwritten slots with ``arange <= cache_position`` and
returns the whole cache through ``stack`` / ``cat``; the reference copies the tensor
once per write and once more on the host (ops.jl:1018-1023, decode.jl:186-203).
``fold_cache_step`` turns that into an in-place write on the input cache fused with
the attention launch, the mask into a device-side count of valid keys, and the
returned cache into an alias of the input -- the "output aliases input" the
reference's schema cannot say.  ``embedding`` and the first-axis ``index.Tensor``
gather run as one kernel (``fold_embedding_sum`` joins the token and position rows).

An op outside the list raises :class:`UnsupportedOp`; there is no eager fallback.
``convert`` produces the schema from an ``ExportedProgram`` -- extents that
``torch.export`` left symbolic are written as expressions in the base symbols, as
the reference's exporter writes them (export_graphs.py:75-90) -- and ``Graph.load``
binds them to integers (``evalshape``, graph.jl:150-205), so a graph can be built
and run without the reference's tooling.
"""
from __future__ import annotations

import ast
import json
import math
from fractions import Fraction
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch

from . import kernels as K

VIEW_OPS = {"view.default", "_unsafe_view.default", "reshape.default", "transpose.int", "permute.default", "t.default",
            "unsqueeze.default", "squeeze.dim", "expand.default", "alias.default", "detach.default", "slice.Tensor",
            "select.int", "flatten.using_ints", "unflatten.int", "contiguous.default"}
DROP_OPS = {"_assert_tensor_metadata.default", "_assert_scalar.default", "sym_constrain_range_for_size.default"}
LINEAR_OPS = {"linear.default", "addmm.default", "mm.default"}
ACTIVATIONS = {"gelu.default": "gelu", "relu.default": "relu"}
# The fused-attention ops an exported graph can hold: the composite one, and the backend-specific ones it becomes
# when the program is decomposed on an accelerator (ops.jl:1365-1391).  Value: positions of (dropout_p, is_causal)
# among the positional arguments; the backend forms return a tuple whose first element is the attention output.
SDPA_OPS = {"scaled_dot_product_attention.default": (4, 5),
            "_scaled_dot_product_flash_attention.default": (3, 4),
            "_scaled_dot_product_flash_attention_for_cpu.default": (3, 4),
            "_scaled_dot_product_efficient_attention.default": (5, 6)}


def _mentions(text: str, names: set) -> bool:
    """Does ``text`` parse as an expression that uses one of ``names``?  (An attribute such as ``"float16"`` does not.)"""
    try:
        tree = ast.parse(text, mode="eval")
    except SyntaxError:
        return False
    return any(isinstance(n, ast.Name) and n.id in names for n in ast.walk(tree))


class UnsupportedOp(NotImplementedError):
    """An ATen op with no kernel on this path (the reference would route it to one of its other kernels)."""


# ----------------------------------------------------------------------------- schema

def _json_dtype(dt) -> str:
    return str(dt).replace("torch.", "")


# How a literal argument of an exported node is written into the JSON: first matching row wins.  Non-finite floats
# have no JSON form and travel as text; a device carries nothing the executor needs.
_LITERAL_FORMS = (
    (lambda x: isinstance(x, float) and math.isnan(x), lambda x: "nan"),
    (lambda x: isinstance(x, float) and math.isinf(x), lambda x: "inf" if x > 0 else "-inf"),
    (lambda x: x is None or isinstance(x, (bool, int, float, str)), lambda x: x),
    (lambda x: isinstance(x, (list, tuple)), lambda x: [_literal(v) for v in x]),
    (lambda x: isinstance(x, torch.dtype), _json_dtype),
    (lambda x: isinstance(x, torch.device), lambda x: None),
)


def _literal(x):
    for matches, encode in _LITERAL_FORMS:
        if matches(x):
            return encode(x)
    return str(x)


def _dim(d, symbols: set):
    """One extent: an int, or -- where the export left it symbolic -- its expression in the base symbols as text."""
    if isinstance(d, (int, bool)):
        return int(d)
    expr = d.node.expr if hasattr(d, "node") else d
    if getattr(expr, "is_Integer", False):
        return int(expr)
    symbols.update(str(x) for x in getattr(expr, "free_symbols", ()))
    return str(expr)


def _note_symbols(x, symbols: set):
    if isinstance(x, (list, tuple)):
        for v in x:
            _note_symbols(v, symbols)
    elif isinstance(x, (torch.SymInt, torch.SymFloat, torch.SymBool)):
        _dim(x, symbols)


_BINOPS = {ast.Add: lambda a, b: a + b, ast.Sub: lambda a, b: a - b, ast.Mult: lambda a, b: a * b,
           ast.FloorDiv: lambda a, b: a // b, ast.Div: lambda a, b: Fraction(a) / Fraction(b), ast.Mod: lambda a, b: a % b,
           ast.Pow: lambda a, b: a ** b}
_CALLS = {"Mod": lambda a, b: a % b, "Max": max, "Min": min, "Pow": lambda a, b: a ** b,
          "floor": lambda a, *b: math.floor(Fraction(a) / Fraction(b[0])) if b else math.floor(a),
          "floordiv": lambda a, b: a // b, "FloorDiv": lambda a, b: a // b,
          "ceiling": lambda a, *b: math.ceil(Fraction(a) / Fraction(b[0])) if b else math.ceil(a),
          "CeilDiv": lambda a, b: math.ceil(Fraction(a) / Fraction(b))}


def evalexpr(expr, dims: Dict[str, int]) -> int:
    """An extent expression -- sums, products, quotients, remainders and the function forms sympy prints (``Mod``,
    ``Max``, ``Min``, ``floor``, ``ceiling``, ``Pow``) over the base symbols -- as an integer under ``dims``; the
    operator set of ``evalexpr``, graph.jl:185-207.  ``/`` is the exact quotient while the expression is walked
    (``ceiling(h/3)`` is the ceiling of the fraction) and a value that is still fractional at the end is floored,
    which for a lone ``h/2`` is the floor division the reference applies.  Parsed with ``ast`` and walked by hand;
    nothing is ever handed to ``eval``."""
    if isinstance(expr, (int, bool)):
        return int(expr)

    def walk(n):
        if isinstance(n, ast.Constant) and isinstance(n.value, int):
            return int(n.value)
        if isinstance(n, ast.Name):
            if n.id not in dims:
                raise KeyError(f"extent expression {expr!r}: no value bound for symbol {n.id!r}")
            return int(dims[n.id])
        if isinstance(n, ast.UnaryOp) and isinstance(n.op, (ast.USub, ast.UAdd)):
            return -walk(n.operand) if isinstance(n.op, ast.USub) else walk(n.operand)
        if isinstance(n, ast.BinOp) and type(n.op) in _BINOPS:
            return _BINOPS[type(n.op)](walk(n.left), walk(n.right))
        if isinstance(n, ast.Call) and isinstance(n.func, ast.Name) and n.func.id in _CALLS and not n.keywords:
            return _CALLS[n.func.id](*[walk(a) for a in n.args])
        raise UnsupportedOp(f"unsupported shape expression: {expr!r}")

    return int(math.floor(walk(ast.parse(str(expr), mode="eval").body)))


class _SchemaWriter:
    """Collects the records of one exported program in the reference's JSON schema (export_graphs.py:111-230:
    ``buffers`` of kind weight / external / transient / view / host, ``ops`` with ``aten`` / ``in`` / ``out`` /
    ``attrs``).  One method per kind of fx node; liveness is worked out afterwards from the finished records."""

    SCALAR_RESULTS = (int, bool, float, torch.SymInt, torch.SymBool, torch.SymFloat)

    def __init__(self, state_keys: Dict[str, str]):
        self.state_keys = state_keys        # placeholder name -> state-dict key, for parameters, buffers and lifted constants
        self.buffers: Dict[str, Dict[str, Any]] = {}
        self.ops: List[Dict[str, Any]] = []
        self.inputs: List[str] = []
        self.outputs: List[str] = []
        self.symbols: set = set()

    # -- records
    def _tensor_fields(self, val) -> Dict[str, Any]:
        if isinstance(val, (tuple, list)):       # a tuple-returning op: one entry per element, None for non-tensors
            return {"shapes": [list(v.shape) if hasattr(v, "shape") else None for v in val],
                    "dtypes": [_json_dtype(v.dtype) if hasattr(v, "dtype") else None for v in val]}
        if val is not None and hasattr(val, "shape"):
            return {"shape": [_dim(d, self.symbols) for d in val.shape], "dtype": _json_dtype(val.dtype)}
        return {}

    def _buffer(self, nid: str, kind: str, val=None, **fields):
        self.buffers[nid] = {"id": nid, "kind": kind, **self._tensor_fields(val), **fields}

    # -- arguments of a call: tensor operands by name, everything else as attributes
    def _operands_and_attrs(self, node):
        import torch.fx as fx
        operands: List[str] = []
        attrs: Dict[str, Any] = {}

        def tensor(a):
            return isinstance(a, fx.Node)

        for pos, a in enumerate(node.args):
            key = f"arg{pos}"
            if tensor(a):
                operands.append(a.name)
            elif isinstance(a, (list, tuple)) and any(tensor(v) for v in a):
                # a list that mixes tensors and literals (cat's operands, index's indices): the tensors join the
                # operands, the attribute keeps the list's shape with "$name" where a tensor stood
                operands.extend(v.name for v in a if tensor(v))
                attrs[key] = ["$" + v.name if tensor(v) else _literal(v) for v in a]
            else:
                attrs[key] = _literal(a)
                _note_symbols(a, self.symbols)
        for key, a in node.kwargs.items():
            if tensor(a):
                operands.append(a.name)
            else:
                attrs[key] = _literal(a)
        return operands, attrs

    # -- one method per fx node kind
    def placeholder(self, node):
        val = node.meta.get("val")
        key = self.state_keys.get(node.name)
        if key is None:
            self._buffer(node.name, "external", val)
            self.inputs.append(node.name)
        else:
            self._buffer(node.name, "weight", val, key=key)

    def call_function(self, node):
        target = str(node.target).replace("aten.", "")
        if target in DROP_OPS:
            return
        operands, attrs = self._operands_and_attrs(node)
        val = node.meta.get("val")
        if isinstance(val, self.SCALAR_RESULTS):
            # a size computed on the host (sym_size, h * w): a named scalar that views refer to as "$name"
            self.buffers[node.name] = {"id": node.name, "kind": "host", "expr": _dim(val, self.symbols)}
        elif target in VIEW_OPS or "getitem" in target:
            self._buffer(node.name, "view", val, of=operands[0] if operands else None, op=target, attrs=attrs)
        else:
            self._buffer(node.name, "transient", val)
            self.ops.append({"id": node.name, "aten": target, "in": operands, "out": node.name,
                             "attrs": {k: v for k, v in attrs.items() if v is not None}})

    def output(self, node):
        import torch.fx as fx
        results = node.args[0]
        if not isinstance(results, (list, tuple)):
            results = [results]
        self.outputs.extend(r.name for r in results if isinstance(r, fx.Node))

    def get_attr(self, node):
        raise UnsupportedOp(f"get_attr node {node.name}: export the program with its constants lifted to inputs")

    # -- after the walk
    def _mark_liveness(self):
        """A transient's ``live`` interval, in op indices: from the op that writes it to the last op that reads it,
        directly or through any chain of views; a transient nobody reads lives to the end.  Results of the program
        are the caller's memory (``external``) and carry no interval."""
        def storage(bid):
            seen = set()
            while bid in self.buffers and self.buffers[bid]["kind"] == "view" and self.buffers[bid].get("of") and bid not in seen:
                seen.add(bid)
                bid = self.buffers[bid]["of"]
            return bid

        written = {op["out"]: i for i, op in enumerate(self.ops)}
        last_read: Dict[str, int] = {}
        for i, op in enumerate(self.ops):
            for operand in op["in"]:
                last_read[storage(operand)] = i
        for bid, b in self.buffers.items():
            if b["kind"] != "transient":
                continue
            if bid in self.outputs:
                b["kind"] = "external"
            else:
                b["live"] = [written.get(bid, 0), last_read.get(bid, len(self.ops))]

    def finish(self, name: str) -> Dict[str, Any]:
        self._mark_liveness()
        return {"name": name, "symbols": sorted(self.symbols), "inputs": self.inputs, "outputs": self.outputs,
                "buffers": list(self.buffers.values()), "ops": self.ops, "fusion_groups": [], "barriers": []}


def convert(ep, name: str = "graph") -> Dict[str, Any]:
    """``ExportedProgram`` -> the buffers/ops dictionary (the schema of export_graphs.py:111-230).  Parameters
    and buffers become ``weight`` buffers keyed by their state-dict name, user inputs and outputs ``external``,
    view ops ``view`` buffers that alias their parent, sizes computed on the host ``host`` scalars, everything
    else an op with a ``transient`` result and a ``live`` interval in op indices.  Symbolic extents stay
    expressions in torch's own symbol names (``s0`` ...), listed under ``symbols``."""
    sig = ep.graph_signature
    state_keys: Dict[str, str] = {}
    for table in ("inputs_to_parameters", "inputs_to_buffers", "inputs_to_lifted_tensor_constants"):
        state_keys.update(getattr(sig, table, {}))
    writer = _SchemaWriter(state_keys)
    for node in ep.graph.nodes:
        getattr(writer, node.op)(node)
    return writer.finish(name)


@dataclass
class Graph:
    """The parsed form (GraphSpec, graph.jl:125-149): buffers by id, ops in order."""
    name: str
    inputs: List[str]
    outputs: List[str]
    buffers: Dict[str, Dict[str, Any]]
    ops: List[Dict[str, Any]]
    notes: List[str] = field(default_factory=list)      # what the rewrites did, for inspection

    @classmethod
    def load(cls, src, dims: Optional[Dict[str, int]] = None) -> "Graph":
        """Parse the schema.  A graph with symbolic extents is bound here: ``dims`` gives every name in its
        ``symbols`` an integer, and each shape, ``host`` scalar and view / op argument written as an expression
        (or as ``"$name"`` of a host scalar) becomes the integer it evaluates to -- what the reference does per
        call (``call(model, name, ...; dims)``, ``evalshape``, graph.jl:150-167) happens once per binding, since
        the executor sizes its buffers when it is built.  One graph file serves any number of bindings."""
        d = json.load(open(src)) if isinstance(src, str) else src
        syms = list(d.get("symbols") or [])
        dims = dict(dims or {})
        missing = [x for x in syms if x not in dims]
        if missing:
            raise ValueError(f"graph {d.get('name')}: symbolic extents {missing} need values (dims={{...}})")
        buffers = {b["id"]: dict(b) for b in d["buffers"]}
        ops = [dict(o, attrs=dict(o.get("attrs", {}))) for o in d["ops"]]
        if syms:
            host = {b["id"]: evalexpr(b["expr"], dims) for b in buffers.values() if b["kind"] == "host" and b.get("expr") is not None}
            names = set(syms)

            def bind(v):
                if isinstance(v, list):
                    return [bind(x) for x in v]
                if isinstance(v, str):
                    if v.startswith("$") and v[1:] in host:
                        return host[v[1:]]
                    if _mentions(v, names):
                        return evalexpr(v, dims)
                return v

            for b in buffers.values():
                if "shape" in b:
                    b["shape"] = [evalexpr(x, dims) for x in b["shape"]]
                if "shapes" in b:
                    b["shapes"] = [None if sh is None else [evalexpr(x, dims) for x in sh] for sh in b["shapes"]]
                if b["kind"] == "view" and b.get("attrs"):
                    b["attrs"] = {k: bind(v) for k, v in b["attrs"].items()}
                if b["kind"] == "host":
                    b["value"] = host.get(b["id"])
            for o in ops:
                o["attrs"] = {k: bind(v) for k, v in o["attrs"].items()}
                o["in"] = [i for i in o["in"] if i not in host]
            for b in buffers.values():
                if b["kind"] == "view" and b.get("of") in host:
                    raise UnsupportedOp(f"{b['id']}: a view of the host scalar {b['of']}")
        return cls(d["name"], list(d["inputs"]), list(d["outputs"]), buffers, ops)

    # -- queries the rewrites share
    def root(self, bid: str) -> str:
        """The buffer a chain of views bottoms out in."""
        while self.buffers[bid]["kind"] == "view":
            bid = self.buffers[bid]["of"]
        return bid

    def readers(self, bid: str) -> List[str]:
        """Ops and views that take ``bid`` as an input."""
        r = [o["id"] for o in self.ops if bid in o["in"]]
        r += [b["id"] for b in self.buffers.values() if b["kind"] == "view" and b.get("of") == bid]
        return r

    def op(self, oid: str) -> Optional[Dict[str, Any]]:
        return next((o for o in self.ops if o["id"] == oid), None)


# ----------------------------------------------------------------------------- rewrites

RESHAPES = ("view.default", "_unsafe_view.default", "reshape.default", "alias.default", "detach.default")

def fold_activations(g: Graph) -> Graph:
    """gelu / relu whose only producer is a linear op -- directly or through a chain of views, as the
    decomposed ``addmm`` + ``view`` form of ``linear`` has it -- or an ordinary convolution, read by nothing
    else, becomes that op's epilogue (foldrelu.jl:60-125; the convolution kernels take it as ``act``); the
    activation's buffer then aliases what it used to read.  An elementwise function commutes with any view,
    so the chain may reshape or permute freely."""
    for act in [o for o in g.ops if o["aten"] in ACTIVATIONS]:
        if act["aten"] == "gelu.default" and act["attrs"].get("approximate", "none") != "none":
            continue                                    # only the erf form is the folded epilogue's arithmetic
        src = act["in"][0]
        chain = [src]
        while g.buffers[chain[-1]]["kind"] == "view":
            chain.append(g.buffers[chain[-1]]["of"])
        prod = g.op(chain[-1])
        single = g.readers(src) == [act["id"]] and all(len(g.readers(c)) == 1 for c in chain[1:]) and not any(c in g.outputs for c in chain)
        # an ordinary (not transposed) convolution takes relu, the reference's ``act`` (conv.jl:100-145); gelu after one stays an op
        conv = prod is not None and prod["aten"] == "convolution.default" and not prod["attrs"].get("arg6") and act["aten"] == "relu.default"
        if prod is None or not (prod["aten"] in LINEAR_OPS or conv) or not single or "epilogue" in prod["attrs"] or "residual" in prod["attrs"]:
            continue
        prod["attrs"]["epilogue"] = ACTIVATIONS[act["aten"]]
        g.ops.remove(act)
        g.buffers[act["id"]].update(kind="view", of=src, op="alias.default", attrs={})
        g.notes.append(f"fold {act['aten']} into {prod['id']}")
    return g


def fold_layerscale(g: Graph) -> Graph:
    """``mul.Tensor(y, gamma)`` with ``gamma`` a per-feature weight vector -- DINOv2's LayerScale after the attention
    projection and after the MLP -- or a constant -- Whisper's ``q_proj(x) * head_dim ** -0.5`` -- and ``y`` (a view chain
    of) a linear op's output that nothing else reads is applied to the linear's weight columns and bias once, when
    the executor binds the weights: ``(xW + b) * gamma = x (W gamma) + b gamma``.  The multiplication then costs
    nothing per run; the rounding moves from the activations to the weights (one fp16 rounding of ``W gamma``
    instead of one of the product)."""
    for mul in [o for o in g.ops if o["aten"] in ("mul.Tensor", "div.Tensor") and len(o["in"]) in (1, 2)]:
        const = _scalar_scale(mul)                      # x * c or x / c with a constant: the same fold, gamma = c
        if len(mul["in"]) == 1 and const is None:
            continue
        if const is None and mul["aten"] != "mul.Tensor":
            continue                                    # y / gamma and gamma / y are not a multiplication by gamma: left as written
        for mine, other in ((mul["in"][0], None),) if const is not None else (mul["in"], mul["in"][::-1]):
            gb = g.buffers[g.root(other)] if other is not None else None
            chain = [mine]
            while g.buffers[chain[-1]]["kind"] == "view":
                chain.append(g.buffers[chain[-1]]["of"])
            prod = g.op(chain[-1])
            if prod is None or prod["aten"] not in LINEAR_OPS or any(k in prod["attrs"] for k in ("epilogue", "residual", "colscale", "ln_out")):
                continue
            feat = (g.buffers[chain[-1]].get("shape") or [None])[-1]
            if other is not None:
                gshape = g.buffers[other].get("shape") or []
                if gb["kind"] != "weight" or not gshape or gshape[-1] != feat or any(d != 1 for d in gshape[:-1]):
                    continue
                if not all(g.buffers[c].get("op") in RESHAPES and (g.buffers[c].get("shape") or [None])[-1] == feat for c in chain[:-1]):
                    continue
            if not (_consumers(g, chain[-1]) <= {mul["id"]}):
                continue
            # the linear's own weight and bias must be constants too
            wpos = {"linear.default": (1, 2), "addmm.default": (2, 0), "mm.default": (1, None)}[prod["aten"]]
            ids = [prod["in"][wpos[0]]] + ([prod["in"][wpos[1]]] if wpos[1] is not None and len(prod["in"]) > wpos[1] else [])
            if any(g.buffers[g.root(i)]["kind"] != "weight" for i in ids):
                continue
            prod["attrs"]["colscale"] = other if other is not None else const
            g.ops.remove(mul)
            g.buffers[mul["id"]].update(kind="view", of=mine, op="alias.default", attrs={})
            g.notes.append(f"fold {mul['id']} (per-feature scale) into the weights of {prod['id']}")
            break
    return g


def group_linears(g: Graph) -> Graph:
    """Linear ops that read the same activations with the same extents -- the q, k and v projections of an attention
    written with three ``Linear`` modules -- become one op, ``linear_group``, run as a single batched GEMM launch over
    weights the executor stacks plane after plane when it binds them (three 1500 x 1280 x 1280 projections: 23 us
    as one launch of 180 tiles, 3 x 16 us apart).  The members keep their result buffers: planes of one allocation.
    Decode-sized members that all carry the same layer norm as their prologue (``fold_layernorm_prologues``) become one
    GEMV instead: the weights laid end to end along the output axis, the norm computed once, the results column bands
    of one buffer -- the fused q/k/v projection of the hand-composed decoder layer.  Members whose norm was folded
    away (``fold_norms_away``) run as the planes of one launch on the raw rows, their results column bands likewise."""
    def key(o):
        pos = {"linear.default": (0, 1, 2), "addmm.default": (1, 2, 0), "mm.default": (0, 1, None)}[o["aten"]]
        x, w = o["in"][pos[0]], o["in"][pos[1]]
        b = o["in"][pos[2]] if pos[2] is not None and len(o["in"]) > pos[2] else None
        return x, w, b
    plain = lambda o: o["aten"] in LINEAR_OPS and not any(k in o["attrs"] for k in ("epilogue", "residual", "ln_out", "clamp", "stats_out"))
    norm_keys = ("ln_in", "ln_in_gamma", "ln_in_beta", "ln_in_eps", "lnf", "lnf_gamma", "lnf_beta", "lnf_eps")
    norm_of = lambda o: tuple(o["attrs"].get(k) for k in norm_keys)
    done = set()
    for first in [o for o in g.ops if plain(o)]:
        if first["id"] in done or first not in g.ops:
            continue
        x0, w0, _ = key(first)
        xs = g.buffers[x0]

        def reshaped_root(bid):                          # the root, if only reshapes lie between: then equal shapes mean equal data
            while g.buffers[bid]["kind"] == "view":
                if g.buffers[bid].get("op") not in RESHAPES and "getitem" not in g.buffers[bid].get("op", ""):
                    return None
                bid = g.buffers[bid]["of"]
            return bid
        members = []
        for o in g.ops[g.ops.index(first):]:
            if not plain(o) or o["id"] in done:
                continue
            x, w, b = key(o)
            same_x = x == x0 or (reshaped_root(x) is not None and reshaped_root(x) == reshaped_root(x0) and
                                 g.buffers[x].get("shape") == xs.get("shape"))
            same_w = g.buffers[w].get("shape") == g.buffers[w0].get("shape") and g.buffers[g.root(w)]["kind"] == "weight"
            if same_x and same_w and (b is None or g.buffers[g.root(b)]["kind"] == "weight") and norm_of(o) == norm_of(first) and \
                    g.buffers[o["out"]].get("shape") == g.buffers[first["out"]].get("shape") and o["out"] not in g.outputs:
                members.append(o)
        # (buffers are written once, so a later member can run where the first one stands: its operands exist there)
        if len(members) < 2 or members[0] is not first:
            continue
        at = g.ops.index(first)
        spec = []
        for o in members:
            x, w, b = key(o)
            spec.append({"out": o["out"], "w": w, "b": b, "aten": o["aten"], "colscale": o["attrs"].get("colscale")})
            done.add(o["id"])
        g.ops = [o for o in g.ops if o not in members[1:]]
        attrs = {"members": spec}
        extra = []
        if first["attrs"].get("ln_in"):
            # decode-sized members that each carry the same norm as their prologue: one GEMV over the members' weights
            # laid end to end along the output axis, the norm computed once, the results column bands of one buffer
            attrs.update({k: first["attrs"].get(k) for k in ("ln_in", "ln_in_gamma", "ln_in_beta", "ln_in_eps")})
            extra = [first["attrs"][k] for k in ("ln_in_gamma", "ln_in_beta") if first["attrs"].get(k)]
        if first["attrs"].get("lnf"):
            # members whose norm was folded away (fold_norms_away): planes of one launch over the raw rows, the prepared
            # weights end to end along the output axis, the results column bands of one buffer
            attrs.update({k: first["attrs"].get(k) for k in ("lnf", "lnf_gamma", "lnf_beta", "lnf_eps")})
            extra = [first["attrs"][k] for k in ("lnf_gamma", "lnf_beta") if first["attrs"].get(k)]
        g.ops[at] = {"id": first["id"] + "_group", "aten": "linear_group", "in": [x0] + [m["w"] for m in spec] + [m["b"] for m in spec if m["b"]] + extra,
                     "out": first["out"], "attrs": attrs}
        g.notes.append("one launch for " + ", ".join(m["out"] for m in spec) + (" (norm prologue shared)" if attrs.get("ln_in") else " (on the raw rows)" if attrs.get("lnf") else ""))
    return g


def fold_residuals(g: Graph) -> Graph:
    """``add.Tensor(x, y)`` where one side is (a view chain of) a linear op's output that nothing else reads:
    the add moves into that GEMM's store, after the activation, with its own rounding -- bit-identical to
    the separate op."""
    for add in [o for o in g.ops if o["aten"] == "add.Tensor"]:
        if add["attrs"].get("alpha", 1) != 1 or len(add["in"]) != 2:
            continue
        for mine, other in (add["in"], add["in"][::-1]):
            chain = [mine]
            while g.buffers[chain[-1]]["kind"] == "view":
                chain.append(g.buffers[chain[-1]]["of"])
            prod = g.op(chain[-1])
            single = all(len(g.readers(c)) == 1 for c in chain) and not any(c in g.outputs for c in chain)
            if prod is None or prod["aten"] not in LINEAR_OPS or not single or "residual" in prod["attrs"]:
                continue
            if g.buffers[other].get("shape") != g.buffers[mine].get("shape") or other == mine:
                continue
            # the other operand must exist before the GEMM runs
            if g.op(g.root(other)) is not None and g.ops.index(g.op(g.root(other))) > g.ops.index(prod):
                continue
            prod["attrs"]["residual"] = "$" + other
            prod["in"].append(other)
            g.ops.remove(add)
            g.buffers[add["id"]].update(kind="view", of=mine, op="alias.default", attrs={})
            if add["id"] in g.outputs:                 # the GEMM's result is now what the caller gets
                g.buffers[chain[-1]]["kind"] = "external"
            g.notes.append(f"fold add {add['id']} into {prod['id']}")
            break
    return g


def fold_clamps(g: Graph) -> Graph:
    """``clamp(y, -c, c)`` with constant symmetric bounds whose input is (a view chain of) a linear op's result that
    nothing else reads -- the fp16 overflow guard exported encoder layers carry after their last residual add -- moves
    into that GEMM's store, after the residual (``matmul_ln_(clamp=)``): the same bits, one pass over the residual
    stream less, and the norm that reads the clamped stream can then ride in the same GEMM (``fold_layernorms``)."""
    for cl in [o for o in g.ops if o["aten"] == "clamp.default" and len(o["in"]) == 1]:
        a = cl["attrs"]
        lo, hi = a.get("arg1", a.get("min")), a.get("arg2", a.get("max"))
        if not isinstance(lo, (int, float)) or not isinstance(hi, (int, float)) or hi <= 0 or lo != -hi:
            continue
        chain = [cl["in"][0]]
        while g.buffers[chain[-1]]["kind"] == "view":
            chain.append(g.buffers[chain[-1]]["of"])
        prod = g.op(chain[-1])
        if prod is None or prod["aten"] not in LINEAR_OPS or any(k in prod["attrs"] for k in ("clamp", "ln_out", "ln_in")):
            continue
        if g.buffers[chain[-1]].get("dtype") != "float16" or not (_consumers(g, chain[-1]) <= {cl["id"]}):
            continue
        prod["attrs"]["clamp"] = float(hi)
        g.ops.remove(cl)
        g.buffers[cl["id"]].update(kind="view", of=cl["in"][0], op="alias.default", attrs={})
        if cl["id"] in g.outputs:
            g.buffers[chain[-1]]["kind"] = "external"
        g.notes.append(f"fold {cl['id']} into the store of {prod['id']}")
    return g


def fold_layernorm_prologues(g: Graph) -> Graph:
    """A layer norm over the last axis that only linear ops read (through reshapes at most) becomes their GEMMs'
    prologue (``ln_matmul_``) where the kernels can take it and it is the faster choice (``kernels.ln_matmul_folds``,
    ``ln_matmul_pays``): the rows are normalised on their way into LDS, so the normalised activations never exist in
    memory and the norm costs no launch.  Today that is the decode-sized case (at most 8 rows: a decoder step's norms);
    the tiled kernel's prologue exists (rows of at most 512) but is slower than the norm's own launch, so wider
    batches stay with ``fold_layernorms``.  The reference's plans/kernels-to-port.md, item 3."""
    for ln in [o for o in g.ops if o["aten"] in ("layer_norm.default", "native_layer_norm.default")]:
        a = ln["attrs"]
        xb = g.buffers[ln["in"][0]]
        feat = (xb.get("shape") or [None])[-1]
        if feat is None or list(a.get("arg1", [])) != [feat] or xb.get("dtype") != "float16":
            continue
        readers = _consumers(g, ln["out"])
        if not readers or "<output>" in readers:
            continue
        if any(g.op(g.root(i)) is not None for i in ln["in"][1:]):
            continue                                    # gamma / beta must be constants
        T = 1
        for d in (xb.get("shape") or [])[:-1]:
            T *= d
        # several readers are fine when each of them can take the norm (the q, k and v projections of a decoder layer:
        # group_linears then runs them as one GEMV with one norm); one that cannot keeps the norm as an op for all
        lins = []
        for rid in sorted(readers, key=lambda r: g.ops.index(g.op(r))):
            lin = g.op(rid)
            if lin is None or lin["aten"] not in LINEAR_OPS or any(k in lin["attrs"] for k in ("ln_in", "ln_out", "clamp")):
                break
            xpos = {"linear.default": 0, "addmm.default": 1, "mm.default": 0}[lin["aten"]]
            wpos = {"linear.default": 1, "addmm.default": 2, "mm.default": 1}[lin["aten"]]
            chain = [lin["in"][xpos]]
            ok = True
            while chain[-1] != ln["out"]:
                b = g.buffers[chain[-1]]
                if b["kind"] != "view" or not (b.get("op") in RESHAPES or "getitem" in b.get("op", "")) or \
                        ("getitem" not in b.get("op", "") and (b.get("shape") or [None])[-1] != feat):
                    ok = False
                    break
                chain.append(b["of"])
            if not ok or sum(1 for i in lin["in"] if i == lin["in"][xpos]) != 1:
                break
            wshape = g.buffers[lin["in"][wpos]].get("shape") or []
            if len(wshape) != 2 or g.buffers[g.root(lin["in"][wpos])]["kind"] != "weight":
                break
            F = wshape[0] if lin["aten"] == "linear.default" else wshape[1]
            if not (K.ln_matmul_folds(T, feat, F) and K.ln_matmul_pays(T, feat, F)):
                break
            lins.append(lin)
        if len(lins) != len(readers):
            continue
        for lin in lins:
            lin["attrs"].update(ln_in=True, ln_in_gamma=ln["in"][1] if len(ln["in"]) > 1 else None,
                                ln_in_beta=ln["in"][2] if len(ln["in"]) > 2 else None, ln_in_eps=a.get("arg4", a.get("eps", 1e-5)))
        lin = lins[0]
        g.ops.remove(ln)
        ob = g.buffers[ln["out"]]
        ob.update(kind="view", of=ln["in"][0], op="alias.default", attrs={})
        g.notes.append(f"fold {ln['id']} into the prologue of " + ", ".join(l["id"] for l in lins))
    return g


def fold_norms_away(g: Graph) -> Graph:
    """A layer norm over the last axis that only linear ops read (through reshapes at most), over enough rows that the
    tiled GEMMs run them (``kernels.lnfold_applies``), gets no pass of its own at all: ``LN(x) . W + b`` is
    ``r (x . gamma W) - r mu colsum(gamma W) + (b + beta . W)``, so the linears run on the RAW rows with constants the
    executor prepares once (``lnfold_prepare``) and need only each row's mean and reciprocal deviation, which come from
    partial sums the GEMM that wrote those rows leaves behind (``stats_out`` on a linear op: ``matmul_rowstats_``) or,
    for rows no linear op wrote (the graph's input, an embedding sum), from a small ``rowstats`` op where the norm
    stood.  The normalised activations never exist in memory.  Held to the parity gate against the separate norm, not
    to its bits.  Decode-sized norms are ``fold_layernorm_prologues``' (which runs first); what neither takes is left
    for ``fold_layernorms``."""
    for ln in [o for o in g.ops if o["aten"] in ("layer_norm.default", "native_layer_norm.default")]:
        a = ln["attrs"]
        x = ln["in"][0]
        xb = g.buffers[x]
        feat = (xb.get("shape") or [None])[-1]
        if feat is None or list(a.get("arg1", [])) != [feat] or xb.get("dtype") != "float16":
            continue
        readers = _consumers(g, ln["out"])
        if not readers or "<output>" in readers:
            continue
        if any(g.buffers[g.root(i)]["kind"] != "weight" for i in ln["in"][1:]):
            continue                                    # gamma / beta must be constants: they go into the weights
        T = math.prod(xb["shape"][:-1])
        lins = []
        for rid in sorted(readers, key=lambda r: g.ops.index(g.op(r))):
            lin = g.op(rid)
            if lin is None or lin["aten"] not in LINEAR_OPS or any(k in lin["attrs"] for k in ("ln_in", "ln_out", "lnf")):
                break
            xpos = {"linear.default": 0, "addmm.default": 1, "mm.default": 0}[lin["aten"]]
            wpos = {"linear.default": 1, "addmm.default": 2, "mm.default": 1}[lin["aten"]]
            at = lin["in"][xpos]
            ok = True
            while at != ln["out"]:
                b = g.buffers[at]
                if b["kind"] != "view" or not (b.get("op") in RESHAPES or "getitem" in b.get("op", "")) or \
                        ("getitem" not in b.get("op", "") and (b.get("shape") or [None])[-1] != feat):
                    ok = False
                    break
                at = b["of"]
            if not ok or sum(1 for i in lin["in"] if i == lin["in"][xpos]) != 1:
                break
            wshape = g.buffers[lin["in"][wpos]].get("shape") or []
            if len(wshape) != 2 or g.buffers[g.root(lin["in"][wpos])]["kind"] != "weight" or g.buffers[lin["out"]].get("dtype") != "float16":
                break
            if not K.lnfold_applies(T, feat, wshape[0] if lin["aten"] == "linear.default" else wshape[1]):
                break
            lins.append(lin)
        if len(lins) != len(readers):
            continue
        # where the rows' statistics come from: the linear op that wrote them, if its GEMM can leave them ...
        chain = [x]
        while g.buffers[chain[-1]]["kind"] == "view":
            chain.append(g.buffers[chain[-1]]["of"])
        prod = g.op(chain[-1])
        dense_rows = all(g.buffers[c].get("op") in RESHAPES and (g.buffers[c].get("shape") or [None])[-1] == feat for c in chain[:-1]) and \
            (g.buffers[chain[-1]].get("shape") or [None])[-1] == feat
        if not dense_rows:
            continue                                    # a permuted or sliced view: its rows are not what the GEMMs and rowstats read
        rides = prod is not None and prod["aten"] in LINEAR_OPS and not any(k in prod["attrs"] for k in ("ln_in", "ln_out")) and \
            g.buffers[chain[-1]].get("dtype") == "float16"
        if rides:
            wpos = {"linear.default": 1, "addmm.default": 2, "mm.default": 1}[prod["aten"]]
            wshape = g.buffers[prod["in"][wpos]].get("shape") or []
            rides = len(wshape) == 2 and K.rowstats_rides(T, wshape[1] if prod["aten"] == "linear.default" else wshape[0], feat)
        if rides and prod["attrs"].get("stats_out"):
            sid = prod["attrs"]["stats_out"]             # a second norm over the same rows
        else:
            sid = ln["id"] + "_rowstats"
            g.buffers[sid] = {"id": sid, "kind": "transient", "shape": [K.rowstats_segments(feat), T, 2], "dtype": "float32"}
            if rides:
                prod["attrs"]["stats_out"] = sid
            else:                                        # ... or one small pass over them where the norm stood
                g.ops.insert(g.ops.index(ln), {"id": sid, "aten": "rowstats", "in": [x], "out": sid, "attrs": {}})
        for lin in lins:
            lin["attrs"].update(lnf=sid, lnf_gamma=ln["in"][1] if len(ln["in"]) > 1 else None,
                                lnf_beta=ln["in"][2] if len(ln["in"]) > 2 else None, lnf_eps=a.get("arg4", a.get("eps", 1e-5)))
        g.ops.remove(ln)
        g.buffers[ln["out"]].update(kind="view", of=x, op="alias.default", attrs={})
        g.notes.append(f"fold {ln['id']} away: " + ", ".join(l["id"] for l in lins) + " run on the raw rows, statistics from " +
                       (prod["id"] if rides else "a rowstats op"))
    return g


def fold_layernorms(g: Graph) -> Graph:
    """A layer norm over the last axis whose input is (a reshaping view of) a linear op's output -- the residual
    stream after ``addmm`` + ``add``, normalised for the next block -- is written by that GEMM as a second result
    (``matmul_ln_``): one launch less where the GEMM splits K, the same bits everywhere.  The linear's own output
    stays what it was, so other readers (the next residual add) are untouched."""
    for ln in [o for o in g.ops if o["aten"] in ("layer_norm.default", "native_layer_norm.default")]:
        src, a = ln["in"][0], ln["attrs"]
        chain = [src]
        while g.buffers[chain[-1]]["kind"] == "view":
            chain.append(g.buffers[chain[-1]]["of"])
        prod = g.op(chain[-1])
        if prod is None or prod["aten"] not in LINEAR_OPS or any(k in prod["attrs"] for k in ("ln_out", "ln_in", "lnf", "stats_out")):
            continue
        feat = (g.buffers[chain[-1]].get("shape") or [None])[-1]
        shapes_ok = all(g.buffers[c].get("op") in RESHAPES and (g.buffers[c].get("shape") or [None])[-1] == feat for c in chain[:-1])
        if not shapes_ok or list(a.get("arg1", [])) != [feat]:
            continue
        if any(g.op(g.root(i)) is not None and g.ops.index(g.op(g.root(i))) > g.ops.index(prod) for i in ln["in"][1:]):
            continue                                    # gamma / beta must exist before the GEMM runs (weights always do)
        prod["attrs"].update(ln_out=ln["out"], ln_gamma=ln["in"][1] if len(ln["in"]) > 1 else None,
                             ln_beta=ln["in"][2] if len(ln["in"]) > 2 else None, ln_eps=a.get("arg4", a.get("eps", 1e-5)))
        g.ops.remove(ln)
        g.notes.append(f"fold {ln['id']} into {prod['id']}")
    return g


LAYOUT_VIEWS = RESHAPES + ("expand.default", "contiguous.default")
SOFTMAX_OPS = ("_softmax.default", "softmax.int")


def _layout_source(g: Graph, bid: str, used: List[str]) -> str:
    """Walk up from ``bid`` through steps that move no values -- reshaping views, expands to the same shape and
    contiguous ``clone`` ops -- to the buffer they all show; ``used`` collects the clone ops passed."""
    while True:
        b = g.buffers[bid]
        if b["kind"] == "view" and b.get("op") in LAYOUT_VIEWS:
            if b["op"] == "expand.default" and list(b.get("shape", [])) != list(g.buffers[b["of"]].get("shape", [])):
                return bid                              # a broadcasting expand does move values
            bid = b["of"]
            continue
        prod = g.op(bid)
        if prod is not None and prod["aten"] == "clone.default":
            used.append(prod["id"])
            bid = prod["in"][0]
            continue
        return bid


def _consumers(g: Graph, bid: str) -> set:
    """Ids of the ops that read ``bid`` directly or through any chain of views; ``"<output>"`` if the graph returns it."""
    seen, todo, ops = set(), [bid], set()
    while todo:
        x = todo.pop()
        if x in seen:
            continue
        seen.add(x)
        if x in g.outputs:
            ops.add("<output>")
        for r in g.readers(x):
            if g.op(r) is not None:
                ops.add(r)
            else:
                todo.append(r)
    return ops


def _scalar_scale(o) -> Optional[float]:
    """The factor of ``mul.Tensor(x, c)`` / ``div.Tensor(x, c)`` with a constant ``c``; None for anything else."""
    if o is None or o["aten"] not in ("mul.Tensor", "div.Tensor") or len(o["in"]) != 1:
        return None
    c = o["attrs"].get("arg1")
    if not isinstance(c, (int, float)) or isinstance(c, bool) or c == 0:
        return None
    return float(c) if o["aten"] == "mul.Tensor" else 1.0 / float(c)


def fold_attention(g: Graph) -> Graph:
    """Attention written out as ``bmm -> (scale) -> softmax -> bmm`` becomes the fused op.

    Models whose attention does not reach ``scaled_dot_product_attention`` export this way -- DINOv2 inside
    Depth Anything carries 24 ``bmm`` and 12 ``_softmax`` (DepthAnythingRunner.jl:38-42), which the reference runs
    through ``batchedmatmul!`` (ops.jl:1393-1399) and its softmax kernel (ops.jl:557-573).  Matched: a softmax over
    the last axis whose input is ``q3 @ k3^T``, optionally scaled by a constant before (on q) or after (on the
    scores), and whose only use is ``p3 @ v3``; the 3-D operands are reshapes (with or without the contiguous
    copies a batch > 1 puts in) of 4-D ``(B, H, L, E)`` tensors.  Everything between disappears: the scores never
    exist in memory."""
    for sm in [o for o in g.ops if o["aten"] in SOFTMAX_OPS]:
        sb = g.buffers[sm["out"]]
        nd = len(sb.get("shape", []))
        if nd < 3 or sm["attrs"].get("arg1") not in (-1, nd - 1) or sm["attrs"].get("arg2") not in (None, False):
            continue
        dead: List[str] = [sm["id"]]
        # -- up: the scores
        scale = 1.0
        src = _layout_source(g, sm["in"][0], dead)
        post = g.op(src)
        if _scalar_scale(post) is not None:
            scale *= _scalar_scale(post)
            dead.append(post["id"])
            src = _layout_source(g, post["in"][0], dead)
        bmm1 = g.op(src)
        if bmm1 is None or bmm1["aten"] != "bmm.default":
            continue
        dead.append(bmm1["id"])
        q4 = _layout_source(g, bmm1["in"][0], dead)
        pre = g.op(q4)
        if _scalar_scale(pre) is not None:
            scale *= _scalar_scale(pre)
            dead.append(pre["id"])
            q4 = _layout_source(g, pre["in"][0], dead)
        kt = g.buffers[_layout_source(g, bmm1["in"][1], dead)]
        swapped = kt["kind"] == "view" and (
            (kt.get("op") == "permute.default" and [x % 4 for x in kt["attrs"].get("arg1", [])] == [0, 1, 3, 2]) or
            (kt.get("op") == "transpose.int" and sorted(x % 4 for x in (kt["attrs"].get("arg1"), kt["attrs"].get("arg2"))) == [2, 3]))
        if not swapped:
            continue
        k4 = kt["of"]
        # -- down: the only use of the probabilities is the second product
        rd, cur = [], sm["out"]
        while True:
            rd = g.readers(cur)
            if len(rd) != 1:
                break
            nxt = g.buffers.get(rd[0])
            if nxt is not None and nxt["kind"] == "view" and nxt.get("op") in LAYOUT_VIEWS:
                cur = rd[0]
                continue
            o = g.op(rd[0])
            if o is not None and o["aten"] == "clone.default":
                dead.append(o["id"])
                cur = o["out"]
                continue
            break
        bmm2 = g.op(rd[0]) if len(rd) == 1 else None
        if bmm2 is None or bmm2["aten"] != "bmm.default" or g.root(bmm2["in"][0]) not in (sm["out"], *dead):
            continue
        v4 = _layout_source(g, bmm2["in"][1], dead)
        shapes = [g.buffers[x].get("shape") for x in (q4, k4, v4)]
        if any(sh is None or len(sh) != 4 for sh in shapes):
            continue
        (B, H, Lq, E), (_, _, Lk, _) = shapes[0], shapes[1]
        if shapes[1] != [B, H, Lk, E] or shapes[2] != [B, H, Lk, E] or g.buffers[bmm2["out"]].get("shape") != [B * H, Lq, E]:
            continue
        # every intermediate is read by this chain only, directly or through views, and is no output of the graph
        mine = set(dead) | {bmm2["id"]}
        if any(not _consumers(g, g.op(d)["out"]) <= mine for d in dead):
            continue
        new_id = bmm2["id"] + "_sdpa"
        g.buffers[new_id] = {"id": new_id, "kind": "transient", "shape": [B, H, Lq, E], "dtype": g.buffers[bmm2["out"]]["dtype"]}
        at = g.ops.index(bmm2)
        g.ops[at] = {"id": new_id, "aten": "scaled_dot_product_attention.default", "in": [q4, k4, v4], "out": new_id,
                     "attrs": {"scale": scale * 1.0}}
        g.ops = [o for o in g.ops if o["id"] not in dead]
        out3 = bmm2["out"]
        g.buffers[out3].update(kind="view", of=new_id, op="view.default", attrs={"arg1": [B * H, Lq, E]})
        # a view of the product back to (B, H, Lq, E) reads the fused op's result as it is
        back = [r for r in g.readers(out3) if g.buffers.get(r, {}).get("kind") == "view" and g.buffers[r].get("shape") == [B, H, Lq, E]]
        if back and len(g.readers(out3)) == 1 and out3 not in g.outputs:
            g.buffers[back[0]].update(of=new_id, op="alias.default", attrs={})
            del g.buffers[out3]
        g.notes.append(f"fold {bmm1['id']} / {sm['id']} / {bmm2['id']} into {new_id} (scale {scale:g})")
    return g


def fold_sdpa_transpose(g: Graph) -> Graph:
    """Attention whose only reader swaps the head and token axes back (``transpose(1, 2)`` /
    ``permute(0, 2, 1, 3)``): the kernel writes token-major, the swap becomes the view it already is, and
    the ``reshape`` that follows is a free view instead of a copy."""
    for o in g.ops:
        if o["aten"] not in SDPA_OPS and o["aten"] != "sdpa_append":
            continue
        rd = g.readers(o["id"])
        if len(rd) == 1 and "getitem" in g.buffers[rd[0]].get("op", "") and g.buffers[rd[0]]["attrs"].get("arg1", 0) == 0:
            rd = g.readers(rd[0])                       # the tuple-returning forms: look past the selection of element 0
        while len(rd) == 1 and g.buffers.get(rd[0], {}).get("kind") == "view" and g.buffers[rd[0]].get("op") == "alias.default":
            rd = g.readers(rd[0])
        if len(rd) != 1 or g.buffers.get(rd[0], {}).get("kind") != "view":
            continue
        v = g.buffers[rd[0]]
        swap = (v["op"] == "transpose.int" and sorted(x % 4 for x in (v["attrs"].get("arg1"), v["attrs"].get("arg2"))) == [1, 2]) or \
               (v["op"] == "permute.default" and [x % 4 for x in v["attrs"].get("arg1", [])] == [0, 2, 1, 3])
        if swap:
            o["attrs"]["token_major"] = True
            g.notes.append(f"{o['id']} writes token-major")
            # the contiguous copy a decomposed reshape puts after the swap has nothing left to do
            vr = g.readers(v["id"])
            cl = g.op(vr[0]) if len(vr) == 1 else None
            if cl is not None and cl["aten"] == "clone.default" and cl["attrs"].get("memory_format", "torch.contiguous_format") in (
                    "torch.contiguous_format", "contiguous_format"):
                g.ops.remove(cl)
                g.buffers[cl["out"]].update(kind="view", of=v["id"], op="alias.default", attrs={})
                g.notes.append(f"{cl['id']} is a view of the token-major result")
    return g


GATHER_OPS = ("embedding.default", "index.Tensor")


def _row_gather(g: Graph, o) -> Optional[tuple]:
    """``(table, ids)`` if ``o`` gathers whole rows of a constant 2-D table by an int64 tensor: ``embedding(table, ids)``
    or ``index.Tensor(table, [ids])`` (advanced indexing along the first axis only)."""
    if o is None or o["aten"] not in GATHER_OPS or len(o["in"]) != 2:
        return None
    table, ids = o["in"]
    if o["aten"] == "index.Tensor" and o["attrs"].get("arg1") != [f"${ids}"]:
        return None
    tb, ib = g.buffers[g.root(table)], g.buffers[ids]
    if tb["kind"] != "weight" or len(g.buffers[table].get("shape", [])) != 2 or ib.get("dtype") != "int64":
        return None
    if tb.get("dtype") != "float16" or g.buffers[o["out"]].get("dtype") != "float16":      # mi_embedding_f16 gathers fp16 rows
        return None
    return table, ids


def fold_embedding_sum(g: Graph) -> Graph:
    """``embedding(tokens, ids) + positions[cache_position]`` -- the first two lines of the decoder step
    (export_whisper_decoder.py:150-152) -- is one gather that adds the two rows on the way: one launch for three,
    and no broadcast add of a ``(1, D)`` row over ``B`` rows left in the graph."""
    for add in [o for o in g.ops if o["aten"] == "add.Tensor" and len(o["in"]) == 2 and o["attrs"].get("alpha", 1) == 1]:
        a, b = (g.op(i) for i in add["in"])
        ga, gb = _row_gather(g, a), _row_gather(g, b)
        if ga is None or gb is None:
            continue
        na, nb = (math.prod(g.buffers[x[1]]["shape"]) for x in (ga, gb))
        if nb != 1 and nb != na:
            if na != 1:
                continue
            (a, ga, na), (b, gb, nb) = (b, gb, nb), (a, ga, na)
        if g.buffers[ga[0]]["shape"][1] != g.buffers[gb[0]]["shape"][1]:
            continue
        if _consumers(g, a["out"]) != {add["id"]} or _consumers(g, b["out"]) != {add["id"]}:
            continue
        at = g.ops.index(add)
        g.ops[at] = {"id": add["id"], "aten": "embedding.default", "in": [ga[0], ga[1], gb[0], gb[1]], "out": add["out"], "attrs": {}}
        g.ops = [o for o in g.ops if o["id"] not in (a["id"], b["id"])]
        g.notes.append(f"fold {a['id']} + {b['id']} into one gather ({add['id']})")
    return g


def fold_patch_tokens(g: Graph) -> Graph:
    """``cat(cls.expand(B, -1, -1), conv(img).flatten(2).transpose(1, 2), dim=1) + pos`` -- a ViT's patch embedding -- is
    one op: the convolution's GEMM writes token rows 1.. itself with the position embedding as its residual
    (``mi_conv2d_tokens_f16``), row 0 is ``cls + pos[0]``.  No channel-major result, no transposing copy, no add."""
    for cat in [o for o in g.ops if o["aten"] == "cat.default" and len(o["in"]) == 2]:
        sh = g.buffers[cat["out"]].get("shape") or []
        if len(sh) != 3 or cat["attrs"].get("arg1", 0) % 3 != 1 or sh[1] < 2:
            continue
        B, T, C = sh
        first, second = cat["in"]
        # the class token: a weight of C values shown as (B, 1, C) through reshapes and an expand
        cls, x, plain = g.root(first), first, True
        while g.buffers[x]["kind"] == "view":
            plain = plain and g.buffers[x]["op"] in RESHAPES + ("expand.default",)
            x = g.buffers[x]["of"]
        cb = g.buffers[cls]
        if not plain or cb["kind"] != "weight" or math.prod(cb["shape"]) != C or list(g.buffers[first].get("shape", [])) != [B, 1, C]:
            continue
        # the patches: the last two axes of a (B, C, P) reshape of an ordinary convolution's (B, C, gh, gw) result, swapped
        v = g.buffers[second]
        if v["kind"] != "view" or list(v.get("shape", [])) != [B, T - 1, C]:
            continue
        va = v.get("attrs", {})
        if v["op"] == "permute.default":
            swapped = list(va.get("arg1", [])) == [0, 2, 1]
        else:
            swapped = v["op"] == "transpose.int" and {va.get("arg1", 0) % 3, va.get("arg2", 0) % 3} == {1, 2}
        x = v["of"]
        while swapped and g.buffers[x]["kind"] == "view":
            w = g.buffers[x]
            if w["op"] not in RESHAPES + ("flatten.using_ints",) or list(w.get("shape", [])) != [B, C, T - 1]:
                swapped = False
            x = w["of"]
        conv = g.op(x) if swapped else None
        if conv is None or conv["aten"] != "convolution.default" or conv["attrs"].get("arg6") or conv["attrs"].get("arg8", 1) != 1 \
                or len(conv["attrs"].get("arg3", [])) != 2 or len(conv["in"]) not in (2, 3):
            continue
        csh = g.buffers[conv["out"]].get("shape") or []
        if len(csh) != 4 or csh[0] != B or csh[1] != C or csh[2] * csh[3] != T - 1:
            continue
        users = _consumers(g, cat["out"])
        if _consumers(g, conv["out"]) != {cat["id"]} or len(users) != 1:
            continue
        add = g.op(next(iter(users)))
        if add is None or add["aten"] != "add.Tensor" or len(add["in"]) != 2 or add["attrs"].get("alpha", 1) != 1 or cat["out"] not in add["in"]:
            continue
        other = add["in"][1] if add["in"][0] == cat["out"] else add["in"][0]
        pos = g.root(other)
        pb = g.buffers[pos]
        if pb["kind"] != "weight" or math.prod(pb["shape"]) != T * C or list(pb["shape"][-2:]) != [T, C] or \
                list(g.buffers[other].get("shape", [])[-2:]) != [T, C]:
            continue
        # what the fused launch needs (mi_conv2d_tokens_f16): fp16 throughout, and token rows that start on 16 bytes --
        # row 1 of every image, so C and T * C in whole 16-byte chunks.  Otherwise the ops stay as written.
        f16 = lambda bid: g.buffers[bid].get("dtype") == "float16"
        if C % 8 or (T * C) % 8 or not all(f16(b) for b in list(conv["in"]) + [cls, pos, conv["out"], add["out"]]):
            continue
        at = g.ops.index(add)
        g.ops[at] = {"id": add["id"], "aten": "patch_tokens", "in": list(conv["in"]) + [cls, pos], "out": add["out"],
                     "attrs": dict(conv["attrs"], has_bias=len(conv["in"]) == 3)}
        g.ops = [o for o in g.ops if o["id"] not in (conv["id"], cat["id"])]
        g.notes.append(f"fold {conv['id']} -> tokens, {cat['id']} and {add['id']} into one patch embedding")
    return g


CACHE_WRITES = ("index_copy.default", "index_put.default")
MASK_VIEWS = RESHAPES + ("expand.default", "unsqueeze.default")


def _cache_write(g: Graph, o) -> Optional[Dict[str, Any]]:
    """``dst.index_copy(2, position, rows)`` / ``index_put(dst, [None, None, position], rows)`` with ``dst`` an input of the
    graph (or a ``select`` of one: the layer's plane of a stacked cache) of shape (B, H, T, E), ``position`` a one-element
    int64 input and ``rows`` (B, H, 1, E): the decoder step's cache update (export_whisper_decoder.py:170-177)."""
    if o is None or o["aten"] not in CACHE_WRITES or len(o["in"]) != 3:
        return None
    dst, pos, rows = o["in"]
    a = o["attrs"]
    if o["aten"] == "index_copy.default":
        if a.get("arg1") not in (2, -2):
            return None
    elif a.get("arg1") != [None, None, f"${pos}"] or a.get("arg3") or a.get("accumulate"):
        return None
    db, pb, rb = g.buffers[dst], g.buffers[pos], g.buffers[rows]
    sh = db.get("shape") or []
    if len(sh) != 4 or pb["kind"] != "external" or pos not in g.inputs or pb.get("dtype") != "int64" or list(pb.get("shape", [])) != [1]:
        return None
    if list(rb.get("shape", [])) != [sh[0], sh[1], 1, sh[3]] or db.get("dtype") != "float16" or rb.get("dtype") != "float16":
        return None
    plane, x = None, dst
    while g.buffers[x]["kind"] == "view":                # the input itself, or select(input, 0, layer) through aliases
        v = g.buffers[x]
        if v["op"] == "select.int" and plane is None and v["attrs"].get("arg1") == 0 and len(g.buffers[v["of"]].get("shape", [])) == 5:
            plane = v["attrs"].get("arg2")
        elif v["op"] not in ("alias.default", "detach.default"):
            return None
        x = v["of"]
    if x not in g.inputs:
        return None
    if plane is not None and plane < 0:
        plane += g.buffers[x]["shape"][0]
    return {"cache": x, "plane": plane, "dst": dst, "pos": pos, "rows": rows}


def _position_mask(g: Graph, bid: str, pos: str, T: int) -> Optional[List[str]]:
    """The ops behind ``bid`` if it is ``where(arange(T) <= position, 0, lowest)`` shown through reshapes and broadcasts
    along every axis but the keys': slots up to and including ``position`` take part, the rest are masked out
    (export_whisper_decoder.py:158-166).  ``lowest`` is -inf or the dtype's most negative value: next to any real
    score its exponential is exactly 0 in fp32, so the masked softmax equals the softmax over the first
    ``position + 1`` keys."""
    x = bid
    while g.buffers[x]["kind"] == "view":
        v = g.buffers[x]
        sh = v.get("shape") or []
        if v["op"] not in MASK_VIEWS or not sh or sh[-1] != T:
            return None
        x = v["of"]
    wh = g.op(x)
    if wh is None or wh["aten"] != "where.self" or len(wh["in"]) != 3 or list(g.buffers[x].get("shape", [])) != [T]:
        return None
    cond, keep, drop = (g.op(i) for i in wh["in"])

    def filled(o):
        if o is None or o["in"]:
            return None
        if o["aten"] == "zeros.default":
            return 0.0
        if o["aten"] == "full.default":
            v = o["attrs"].get("arg1")
            return float(v) if isinstance(v, (int, float, str)) and not isinstance(v, bool) else None
        return None

    lo = filled(drop)
    if cond is None or cond["aten"] != "le.Tensor" or cond["in"] != [cond["in"][0], pos] or filled(keep) != 0.0 or lo is None or lo > -6.0e4:
        return None
    ar = g.op(cond["in"][0])
    a = ar["attrs"] if ar is not None else {}
    steps = ar is not None and not ar["in"] and (
        (ar["aten"] == "arange.default" and a.get("arg0") == T) or
        (ar["aten"] == "arange.start_step" and a.get("arg0") == 0 and a.get("arg1") == T and a.get("arg2", 1) == 1) or
        (ar["aten"] == "arange.start" and a.get("arg0") == 0 and a.get("arg1") == T))
    return [wh["id"], cond["id"], keep["id"], drop["id"], ar["id"]] if steps else None


def fold_cache_step(g: Graph) -> Graph:
    """The functional cache update of an exported decoder step becomes an in-place one.

    Matched, per attention: ``K = cache_k[layer].index_copy(2, position, k_new)``, the same for ``V``, and
    ``scaled_dot_product_attention(q, K, V, mask)`` with one query row, where the only other reader of ``K`` / ``V`` is
    the ``stack`` (``cat`` + ``view`` once decomposed) that returns every layer's plane as the new cache, in layer order
    and in the input's shape.  The three ops become ``sdpa_append``: the new rows go into slot ``position`` of the
    *input* cache, and attention runs over it -- in one launch where the single-workgroup kernel covers the shape.
    If the mask is the position mask (``_position_mask``) it goes away: the kernel takes ``position + 1`` as the number
    of valid keys, which a ``kv_len_from_position`` op computes on the device once per step; any other mask stays
    an operand.  The returned cache becomes an alias of the input (the caller's tensor is updated, and is what the
    call returns), which removes the 2 x 18 MB of copies per token the reference pays for a functional graph
    (ops.jl:1018-1023, decode.jl:186-203).  Requires that nothing else reads the cache plane, so no op can observe the
    difference between "a new tensor" and "the same tensor, updated"."""
    writes = {o["id"]: w for o in g.ops if (w := _cache_write(g, o)) is not None}
    if not writes:
        return g
    # which attention reads which pair of writes
    plans = []
    for att in [o for o in g.ops if o["aten"] in SDPA_OPS]:
        if len(att["in"]) < 3 or att["in"][1] not in writes or att["in"][2] not in writes:
            continue
        wk, wv = writes[att["in"][1]], writes[att["in"][2]]
        qsh = g.buffers[att["in"][0]].get("shape") or []
        a = att["attrs"]
        pd, pc = SDPA_OPS[att["aten"]]
        if wk["pos"] != wv["pos"] or wk["plane"] != wv["plane"] or wk["cache"] == wv["cache"] or len(qsh) != 4 or qsh[2] != 1:
            continue
        if a.get("is_causal", a.get(f"arg{pc}", False)) or a.get("dropout_p", a.get(f"arg{pd}", 0.0)) not in (0, 0.0):
            continue
        plans.append((att, att["in"][1], att["in"][2]))
    # per cache input: every plane written once, each write read by its attention and by the op that returns the planes
    by_cache: Dict[str, Dict[Any, str]] = {}
    for att, ik, iv in plans:
        for wid in (ik, iv):
            by_cache.setdefault(writes[wid]["cache"], {})[writes[wid]["plane"]] = wid
    returned: Dict[str, tuple] = {}
    for cache, planes in by_cache.items():
        shape = g.buffers[cache]["shape"]
        order = [planes.get(i) for i in range(shape[0])] if len(shape) == 5 else [planes.get(None)]
        if any(w is None for w in order):
            continue
        joins = [o for o in g.ops if o["aten"] in ("stack.default", "cat.default") and o["in"] == order and o["attrs"].get("arg1", 0) == 0]
        if len(shape) == 4:                              # a single-layer cache returned as it is
            if order[0] in g.outputs:
                returned[cache] = (None, order[0])
            continue
        for j in joins:
            outs = [x for x in ([j["out"]] + [v for v in g.readers(j["out"]) if g.buffers.get(v, {}).get("kind") == "view"])
                    if x in g.outputs and g.buffers[x].get("shape") == shape]
            if outs and _consumers(g, j["out"]) == {"<output>"}:
                returned[cache] = (j, outs[0])
                break
    done = []
    for att, ik, iv in plans:
        wk, wv = writes[ik], writes[iv]
        if wk["cache"] not in returned or wv["cache"] not in returned:
            continue
        jk, jv = returned[wk["cache"]][0], returned[wv["cache"]][0]
        allowed_k = {att["id"]} | ({jk["id"]} if jk else {"<output>"})
        allowed_v = {att["id"]} | ({jv["id"]} if jv else {"<output>"})
        if _consumers(g, ik) != allowed_k or _consumers(g, iv) != allowed_v:
            continue
        if any(_consumers(g, c) != set(by_cache[c].values()) for c in (wk["cache"], wv["cache"])):
            continue                                    # someone else reads the cache, through whatever view: it would see the new rows
        done.append((att, ik, iv))
    if not done:
        return g
    # all or nothing per cache: a returned tensor that aliases the input must have had every plane written in place
    covered: Dict[str, set] = {}
    for att, ik, iv in done:
        for wid in (ik, iv):
            covered.setdefault(writes[wid]["cache"], set()).add(wid)
    ok_cache = {c for c, ws in covered.items() if ws == set(by_cache[c].values())}
    done = [d for d in done if writes[d[1]]["cache"] in ok_cache and writes[d[2]]["cache"] in ok_cache]
    lens: Dict[tuple, str] = {}
    for att, ik, iv in done:
        wk, wv = writes[ik], writes[iv]
        B, H, T, E = g.buffers[wk["dst"]]["shape"]
        key = (wk["pos"], B, T)
        if key not in lens:                             # position + 1 as the per-row key count, once per step
            lid = f"kv_len_{wk['pos']}_{T}"
            g.buffers[lid] = {"id": lid, "kind": "transient", "shape": [B], "dtype": "int32"}
            g.ops.insert(0, {"id": lid, "aten": "kv_len_from_position", "in": [wk["pos"]], "out": lid, "attrs": {"cap": T + 1}})
            lens[key] = lid
        ins = [att["in"][0], wk["dst"], wv["dst"], wk["rows"], wv["rows"], lens[key]]
        attrs = {k: v for k, v in att["attrs"].items() if k in ("scale", "token_major")}
        mask = att["in"][3] if len(att["in"]) > 3 else None
        if mask is not None:
            if _position_mask(g, mask, wk["pos"], T) is None:
                ins.append(mask)
                attrs["masked"] = True
        else:
            attrs["all_slots"] = True                   # no mask in the export: every slot takes part, written or not
        at = g.ops.index(att)
        g.ops[at] = {"id": att["id"], "aten": "sdpa_append", "in": ins, "out": att["out"], "attrs": attrs}
        g.ops = [o for o in g.ops if o["id"] not in (ik, iv)]
        for wid in (ik, iv):                            # the "new" plane is the input's plane
            g.buffers[wid].update(kind="view", of=writes[wid]["dst"], op="alias.default", attrs={})
        g.notes.append(f"fold {ik} / {iv} / {att['id']} into an in-place sdpa_append on {wk['cache']} / {wv['cache']}")
    for cache in ok_cache:
        j, out = returned[cache]
        if j is not None:
            g.ops.remove(j)
            for x in [j["out"]] + [v for v in g.readers(j["out"]) if g.buffers.get(v, {}).get("kind") == "view"]:
                g.buffers[x].update(kind="view", of=cache, op="alias.default", attrs={})
        g.notes.append(f"output {out} is the input {cache}, updated in place")
    return prune(g)


def prune(g: Graph) -> Graph:
    """Drop ops whose result nothing reads any more (the mask arithmetic once the mask became a length)."""
    while True:
        dead = [o for o in g.ops if not _consumers(g, o["out"]) and o["aten"] != "sdpa_append" and
                not any(_consumers(g, m["out"]) for m in o["attrs"].get("members", []))]
        if not dead:
            return g
        for o in dead:
            g.ops.remove(o)
            g.notes.append(f"drop {o['id']} (unused)")


def optimize(g: Graph) -> Graph:
    g = fold_patch_tokens(fold_cache_step(fold_embedding_sum(g)))
    return group_linears(fold_sdpa_transpose(fold_attention(fold_layernorms(fold_norms_away(fold_layernorm_prologues(
        fold_clamps(fold_residuals(fold_layerscale(fold_activations(g))))))))))


# ----------------------------------------------------------------------------- execution

_DTYPES = {"float16": torch.float16, "float32": torch.float32, "int64": torch.int64, "int32": torch.int32, "bool": torch.bool}


class Executor:
    """Binds a graph to weights and a context and runs it op by op (Model / call, execute.jl:493-539).
    Transient buffers are allocated once at construction; nothing is allocated per run."""

    def __init__(self, graph: Graph, weights: Dict[str, torch.Tensor], ctx: Optional[K.Ctx] = None, device="cuda"):
        self.g = graph
        self.ctx = ctx if ctx is not None else K.Ctx(device)
        self.device = torch.device(device)
        self.t: Dict[str, torch.Tensor] = {}
        self.scaled: Dict[str, Any] = {}                  # op id -> (weight, bias) with a folded per-feature scale
        for b in graph.buffers.values():
            if b["kind"] == "weight":
                w = weights[b["key"]]
                if list(w.shape) != list(b["shape"]):
                    raise ValueError(f"weight {b['key']}: shape {tuple(w.shape)} but the graph declares {b['shape']}")
                self.t[b["id"]] = w.to(self.device, _DTYPES[b["dtype"]]).contiguous()
        for o in graph.ops:                               # check every op has a handler before anything runs
            if o["aten"] not in self.HANDLERS:
                raise UnsupportedOp(f"{graph.name}: no kernel on this path for aten.{o['aten']} (op {o['id']})")
        for o in graph.ops:                               # row statistics a GEMM leaves for a folded norm
            sid = o["attrs"].get("stats_out")
            if sid is not None and sid not in self.t:
                self.t[sid] = torch.empty(list(graph.buffers[sid]["shape"]), dtype=torch.float32, device=self.device)
        for o in graph.ops:                               # a norm folded into its producer: its result still needs a home
            nid = o["attrs"].get("ln_out")
            if nid is not None:
                nb = graph.buffers[nid]
                shape, dtype = (nb["shape"], nb["dtype"]) if "shape" in nb else (nb["shapes"][0], nb["dtypes"][0])
                self.t[nid] = torch.empty(list(shape), dtype=_DTYPES[dtype], device=self.device)
        for o in graph.ops:
            if o["aten"] == "linear_group":               # the members' results are planes of one allocation
                mem = o["attrs"]["members"]
                b0 = graph.buffers[mem[0]["out"]]
                if o["attrs"].get("ln_in") or o["attrs"].get("lnf"):      # ... or column bands of one (rows, n F) matrix
                    F, rows = b0["shape"][-1], math.prod(b0["shape"][:-1])
                    bands = torch.empty((rows, len(mem) * F), dtype=_DTYPES[b0["dtype"]], device=self.device)
                    for i, m in enumerate(mem):
                        self.t[m["out"]] = bands[:, i * F:(i + 1) * F].view(list(b0["shape"]))
                    self.t[o["id"]] = bands
                    continue
                planes = torch.empty([len(mem)] + list(b0["shape"]), dtype=_DTYPES[b0["dtype"]], device=self.device)
                for i, m in enumerate(mem):
                    self.t[m["out"]] = planes[i]
                self.t[o["id"]] = planes
                continue
            b = graph.buffers[o["out"]]
            if "shape" in b:
                shape, dtype = list(b["shape"]), b["dtype"]
            elif o["aten"] in SDPA_OPS or o["aten"] == "sdpa_append":   # a tuple result: only the attention output is materialised
                shape, dtype = list(b["shapes"][0]), b["dtypes"][0]
            else:
                continue
            if o["attrs"].get("token_major"):             # (B, H, L, E) stored as (B, L, H, E)
                self.t[o["out"]] = torch.empty([shape[0], shape[2], shape[1], shape[3]], dtype=_DTYPES[dtype],
                                               device=self.device).transpose(1, 2)
            else:
                self.t[o["out"]] = torch.empty(shape, dtype=_DTYPES[dtype], device=self.device)

    # -- operands
    def get(self, bid: str) -> torch.Tensor:
        if bid in self.t:
            return self.t[bid]
        b = self.g.buffers[bid]
        if b["kind"] != "view":
            raise KeyError(f"buffer {bid} ({b['kind']}) has no value yet")
        return self._view(b)

    def _view(self, b) -> torch.Tensor:
        src, a, op = self.get(b["of"]), b.get("attrs", {}), b["op"]
        if "getitem" in op:
            if a.get("arg1", 0) != 0:
                raise UnsupportedOp(f"{b['id']}: only the first result of a multi-result op is kept")
            return src
        if op in ("view.default", "_unsafe_view.default", "reshape.default"):
            want = list(a["arg1"])
            try:
                return src.view(want)
            except RuntimeError:
                raise UnsupportedOp(f"{b['id']}: reshape of {tuple(src.shape)} strides {src.stride()} to {want} needs a copy")
        if op == "transpose.int":
            return src.transpose(a["arg1"], a["arg2"])
        if op == "permute.default":
            return src.permute(a["arg1"])
        if op == "t.default":
            return src.t()
        if op == "unsqueeze.default":
            return src.unsqueeze(a["arg1"])
        if op == "squeeze.dim":
            return src.squeeze(a["arg1"])
        if op == "expand.default":
            return src.expand(a["arg1"])
        if op in ("alias.default", "detach.default"):
            return src
        if op == "contiguous.default":
            if not src.is_contiguous():
                raise UnsupportedOp(f"{b['id']}: contiguous() of a strided tensor needs a copy")
            return src
        if op == "slice.Tensor":
            dim, lo, hi, step = a.get("arg1", 0), a.get("arg2"), a.get("arg3"), a.get("arg4", 1)
            idx = [slice(None)] * src.dim()
            idx[dim] = slice(lo, None if hi is None or hi >= 2 ** 62 else hi, step)
            return src[tuple(idx)]
        if op == "select.int":
            return src.select(a["arg1"], a["arg2"])
        if op == "flatten.using_ints":
            return src.flatten(a.get("arg1", 0), a.get("arg2", -1))
        if op == "unflatten.int":
            return src.unflatten(a["arg1"], a["arg2"])
        raise UnsupportedOp(f"view op {op}")

    @staticmethod
    def _rows(t: torch.Tensor) -> torch.Tensor:
        """(..., K) -> (T, K) without a copy."""
        if t.dim() == 2:
            return t
        try:
            return t.view(-1, t.shape[-1])
        except RuntimeError:
            raise UnsupportedOp(f"linear over a tensor of shape {tuple(t.shape)} strides {t.stride()} needs a copy")

    # -- handlers (runop!, ops.jl)
    def _linear(self, o):
        at, ins, attrs = o["aten"], o["in"], o["attrs"]
        res_id = attrs["residual"][1:] if "residual" in attrs else None
        ins = ins[:-1] if res_id else ins                # fold_residuals appended it last
        if at == "linear.default":                       # (x, weight[F,K], bias?)
            x, w = self.get(ins[0]), self.get(ins[1]).t()
            bias = self.get(ins[2]) if len(ins) > 2 else None
        elif at == "addmm.default":                      # (bias, x, w[K,F]); ops.jl:1347-1363
            if attrs.get("beta", 1) != 1 or attrs.get("alpha", 1) != 1:
                raise UnsupportedOp(f"{o['id']}: addmm with beta/alpha other than 1")
            bias, x, w = self.get(ins[0]), self.get(ins[1]), self.get(ins[2])
        else:                                            # mm (x, w[K,F])
            x, w, bias = self.get(ins[0]), self.get(ins[1]), None
        if "colscale" in attrs:                          # LayerScale folded into the constants, once
            if o["id"] not in self.scaled:
                cs = attrs["colscale"]
                gamma = self.get(cs).reshape(-1).float() if isinstance(cs, str) else float(cs)
                self.scaled[o["id"]] = ((w.float() * gamma).to(w.dtype), None if bias is None else (bias.float() * gamma).to(bias.dtype))
            w, bias = self.scaled[o["id"]]
        out = self.t[o["out"]]
        res = self._rows(self.get(res_id)) if res_id else None
        self.ctx.ws.reset()
        stats_out = self.t[attrs["stats_out"]] if attrs.get("stats_out") else None
        if attrs.get("lnf"):                             # the norm in front folded away: prepared constants, raw rows
            if ("lnf", o["id"]) not in self.scaled:
                self.scaled[("lnf", o["id"])] = K.lnfold_prepare(self.ctx, w, self.get(attrs["lnf_gamma"]) if attrs.get("lnf_gamma") else None,
                                                                 self.get(attrs["lnf_beta"]) if attrs.get("lnf_beta") else None, bias)
            K.lnfold_matmul_(self.ctx, self._rows(out), self.scaled[("lnf", o["id"])], self._rows(x), self.t[attrs["lnf"]], attrs.get("lnf_eps", 1e-5),
                             epi=attrs.get("epilogue", "none"), residual=res, stats_out=stats_out, clamp=attrs.get("clamp"))
            return
        if stats_out is not None:
            K.matmul_rowstats_(self.ctx, self._rows(out), stats_out, w, self._rows(x), bias, epi=attrs.get("epilogue", "none"),
                               residual=res, clamp=attrs.get("clamp"))
            return
        if attrs.get("ln_out") is not None or attrs.get("clamp") is not None:
            has_ln = attrs.get("ln_out") is not None
            gamma = self.get(attrs["ln_gamma"]) if has_ln and attrs.get("ln_gamma") else None
            beta = self.get(attrs["ln_beta"]) if has_ln and attrs.get("ln_beta") else None
            K.matmul_ln_(self.ctx, self._rows(out), self._rows(self.t[attrs["ln_out"]]) if has_ln else None, w, self._rows(x), gamma, beta,
                         attrs.get("ln_eps", 0.0), bias, epi=attrs.get("epilogue", "none"), residual=res, clamp=attrs.get("clamp"))
            return
        if attrs.get("ln_in"):
            gamma = self.get(attrs["ln_in_gamma"]) if attrs.get("ln_in_gamma") else None
            beta = self.get(attrs["ln_in_beta"]) if attrs.get("ln_in_beta") else None
            K.ln_matmul_(self.ctx, self._rows(out), w, self._rows(x), gamma, beta, attrs.get("ln_in_eps", 1e-5), bias,
                         epi=attrs.get("epilogue", "none"), residual=res)
            return
        K.matmul_(self.ctx, self._rows(out), w, self._rows(x), bias, epi=attrs.get("epilogue", "none"), residual=res)

    def _linear_group(self, o):
        mem = o["attrs"]["members"]
        if o["id"] not in self.scaled:                    # stack the members' constants once: (n, K, F) or (n, F, K), (n, F)
            ws, bs = [], []
            for m in mem:
                w = self.get(m["w"]).t() if m["aten"] == "linear.default" else self.get(m["w"])       # (K, F) view
                b = self.get(m["b"]) if m["b"] else None
                if m["colscale"] is not None:
                    cs = m["colscale"]
                    gamma = self.get(cs).reshape(-1).float() if isinstance(cs, str) else float(cs)
                    w = (w.float() * gamma).to(w.dtype)
                    b = None if b is None else (b.float() * gamma).to(b.dtype)
                ws.append(w)
                bs.append(b)
            fk = all(w.stride(0) == 1 and w.stride(1) == w.shape[0] for w in ws)       # every member a transposed [F][K] matrix
            filled = [torch.zeros_like(next(x for x in bs if x is not None)) if b is None else b for b in bs] if any(b is not None for b in bs) else None
            if o["attrs"].get("ln_in") or o["attrs"].get("lnf"):      # end to end along the output axis, in the members' own memory layout
                W = torch.cat([w.t() for w in ws]).t() if fk else torch.cat([w.contiguous() for w in ws], dim=1)
                B = None if filled is None else torch.cat(filled)
                if o["attrs"].get("lnf"):
                    a = o["attrs"]
                    W = K.lnfold_prepare(self.ctx, W, self.get(a["lnf_gamma"]) if a.get("lnf_gamma") else None,
                                         self.get(a["lnf_beta"]) if a.get("lnf_beta") else None, B, planes=len(mem))
            else:
                W = torch.stack([w.t() for w in ws]).transpose(1, 2) if fk else torch.stack([w.contiguous() for w in ws])
                B = None if filled is None else torch.stack(filled)
            self.scaled[o["id"]] = (W, B)
        W, B = self.scaled[o["id"]]
        x = self._rows(self.get(o["in"][0]))
        planes = self.t[o["id"]]
        if o["attrs"].get("lnf"):
            self.ctx.ws.reset()
            K.lnfold_matmul_(self.ctx, planes, W, x, self.t[o["attrs"]["lnf"]], o["attrs"].get("lnf_eps", 1e-5))
            return
        if o["attrs"].get("ln_in"):
            a = o["attrs"]
            self.ctx.ws.reset()
            K.ln_matmul_(self.ctx, planes, W, x, self.get(a["ln_in_gamma"]) if a.get("ln_in_gamma") else None,
                         self.get(a["ln_in_beta"]) if a.get("ln_in_beta") else None, a.get("ln_in_eps", 1e-5), B)
            return
        K.batchedmatmul_(self.ctx, planes.view(len(mem), -1, planes.shape[-1]), W, x.unsqueeze(0), B)

    def _sdpa(self, o):
        a = o["attrs"]
        pd, pc = SDPA_OPS[o["aten"]]
        dropout = a.get("dropout_p", a.get(f"arg{pd}", 0.0))
        causal = a.get("is_causal", a.get(f"arg{pc}", False))
        if causal or dropout not in (0, 0.0) or a.get("enable_gqa"):
            raise UnsupportedOp(f"{o['id']}: causal flag / dropout / gqa are not exported on this path (masks arrive as attn_mask)")
        q, k, v = (self.get(i) for i in o["in"][:3])
        bias = self.get(o["in"][3]) if len(o["in"]) > 3 else None       # attn_mask / attn_bias, positional or keyword
        self.ctx.ws.reset()
        K.sdpa(self.ctx, q, k, v, bias, a.get("scale"), out=self.t[o["out"]])

    def _cat(self, o):
        """cat of (B, N_i, C) tensors along the token axis (class token + patch tokens): each operand is copied into its
        rows of the result with the layout kernel, whatever its strides -- the patch tokens arrive as the transposed
        view of the convolution's (B, C, N) output, and the copy is that transpose."""
        ins = [self.get(i) for i in o["in"]]
        out = self.t[o["out"]]
        dim = o["attrs"].get("arg1", 0) % out.dim()
        if out.dim() != 3 or dim != 1 or any(t.dim() != 3 for t in ins):
            raise UnsupportedOp(f"{o['id']}: cat of {[tuple(t.shape) for t in ins]} along {dim} (only (B, N, C) along N)")
        at = 0
        for t in ins:
            n = t.shape[1]
            K.transposeLE_(self.ctx, out[:, at:at + n].unsqueeze(1), t.permute(0, 2, 1).unsqueeze(1))
            at += n

    def _softmax(self, o):
        """aten::_softmax / softmax over the last axis (softmax_kernel!, ops.jl:557-573); inside bmm + softmax + bmm
        optimize() replaces it, on its own -- or where the probabilities are a result -- it runs as written."""
        x, out = self.get(o["in"][0]), self.t[o["out"]]
        if o["attrs"].get("arg1") not in (-1, x.dim() - 1) or o["attrs"].get("arg2") not in (None, False) or not x.is_contiguous():
            raise UnsupportedOp(f"{o['id']}: softmax over an axis other than the last, or of a strided tensor")
        K.softmax_(self.ctx, out, x)

    def _scale(self, o):
        c = _scalar_scale(o)
        if c is None:
            raise UnsupportedOp(f"{o['id']}: {o['aten']} other than a tensor times a constant")
        x, out = self.get(o["in"][0]), self.t[o["out"]]
        if not x.is_contiguous():                         # a strided operand (a head slice of a packed projection): copy, then scale in place
            self._copy(o, out, x)
            x = out
        K.scale_(self.ctx, out, x, c)

    def _copy(self, o, out, x):
        """out (contiguous) = x (any strides), up to four axes, with the layout kernel."""
        if x.dim() > 4 or x.dim() < 2:
            raise UnsupportedOp(f"{o['id']}: a contiguous copy of a {x.dim()}-axis strided tensor")
        while x.dim() < 4:
            x, out = x.unsqueeze(0), out.unsqueeze(0)
        K.transposeLE_(self.ctx, out, x.transpose(2, 3))

    def _clone(self, o):
        if o["attrs"].get("memory_format", "torch.contiguous_format") not in ("torch.contiguous_format", "contiguous_format"):
            raise UnsupportedOp(f"{o['id']}: clone to another memory format")
        self._copy(o, self.t[o["out"]], self.get(o["in"][0]))

    def _bmm(self, o):
        """bmm(a (B,m,k), b (B,k,n)) -- batchedmatmul!, ops.jl:1393-1399."""
        a, b = self.get(o["in"][0]), self.get(o["in"][1])
        K.batchedmatmul_(self.ctx, self.t[o["out"]], b, a)

    def _rowstats(self, o):
        """The partial sums a folded norm's linears read, for rows no GEMM here wrote (``fold_norms_away``)."""
        K.rowstats_(self.ctx, self.t[o["out"]], self._rows(self.get(o["in"][0])))

    def _layer_norm(self, o):
        ins, a = o["in"], o["attrs"]
        x = self.get(ins[0])
        shape = a["arg1"]
        if len(shape) != 1 or shape[0] != x.shape[-1]:
            raise UnsupportedOp(f"{o['id']}: layer_norm over {shape} (only the last axis)")
        gamma = self.get(ins[1]) if len(ins) > 1 else None
        beta = self.get(ins[2]) if len(ins) > 2 else None
        eps = a.get("arg4", a.get("eps", 1e-5))
        K.layernorm_(self.ctx, self.t[o["out"]], None, None, x, gamma, beta, x.shape[-1], eps)

    def _native_layer_norm(self, o):
        ins, a = o["in"], o["attrs"]
        x = self.get(ins[0])
        shape = a["arg1"]
        if len(shape) != 1 or shape[0] != x.shape[-1]:
            raise UnsupportedOp(f"{o['id']}: layer_norm over {shape} (only the last axis)")
        b = self.g.buffers[o["out"]]
        if o["out"] not in self.t:                        # multi-result: only the normalised tensor is materialised
            self.t[o["out"]] = torch.empty(b["shapes"][0], dtype=_DTYPES[b["dtypes"][0]], device=self.device)
        K.layernorm_(self.ctx, self.t[o["out"]], None, None, x, self.get(ins[1]) if len(ins) > 1 else None,
                     self.get(ins[2]) if len(ins) > 2 else None, x.shape[-1], a.get("arg4", 1e-5))

    def _add(self, o):
        if o["attrs"].get("alpha", 1) != 1 or len(o["in"]) != 2:
            raise UnsupportedOp(f"{o['id']}: add with a scalar operand or alpha")
        a, b = self.get(o["in"][0]), self.get(o["in"][1])
        out = self.t[o["out"]]
        drop1 = lambda t: [d for d in t.shape if d != 1]
        if a.shape != b.shape and drop1(a) != drop1(b):   # (1, T, D) + (T, D) is the same elements; anything else would broadcast
            raise UnsupportedOp(f"{o['id']}: broadcasting add {tuple(a.shape)} + {tuple(b.shape)}")
        if not a.is_contiguous():                         # e.g. the permuted output of a convolution stem + its position embedding
            self._copy(o, out.view(a.shape), a)
            a = out
        if not b.is_contiguous():
            raise UnsupportedOp(f"{o['id']}: add of two strided tensors")
        K.add_(self.ctx, out, a, b)

    def _activation(self, o):
        """gelu / relu that no linear op could take as its epilogue (after a convolution stem): on its own."""
        a = o["attrs"]
        if o["aten"] == "gelu.default" and a.get("approximate", "none") not in ("none", "tanh"):
            raise UnsupportedOp(f"{o['id']}: gelu approximate={a.get('approximate')}")
        x, out = self.get(o["in"][0]), self.t[o["out"]]
        if not x.is_contiguous():
            self._copy(o, out, x)
            x = out
        kind = "relu" if o["aten"] == "relu.default" else ("gelu_tanh" if a.get("approximate") == "tanh" else "gelu")
        K.act_(self.ctx, out, x, kind)

    def _clamp(self, o):
        a = o["attrs"]
        lo, hi = a.get("arg1", a.get("min")), a.get("arg2", a.get("max"))
        x, out = self.get(o["in"][0]), self.t[o["out"]]
        if len(o["in"]) != 1 or not x.is_contiguous():
            raise UnsupportedOp(f"{o['id']}: clamp with tensor bounds or of a strided tensor")
        K.clamp_(self.ctx, out, x, float("-inf") if lo is None else float(lo), float("inf") if hi is None else float(hi))

    def _convolution(self, o):
        """aten::convolution, ordinary and transposed (arg6), 2-D and -- lifted to a singleton second spatial
        axis -- 1-D (runop! for convolution.default, ops.jl:1114-1200)."""
        a, ins = o["attrs"], o["in"]
        x, w = self.get(ins[0]), self.get(ins[1])
        bias = self.get(ins[2]) if len(ins) > 2 else None
        stride, padding, dilation = list(a["arg3"]), list(a["arg4"]), list(a["arg5"])
        outpad = list(a.get("arg7") or [0] * len(stride))
        out = self.t[o["out"]]
        if len(stride) == 1:                               # (N,C,L) -> (N,C,1,L); the added axis has stride 1, no padding
            x, w, out = x.unsqueeze(2), w.unsqueeze(2), out.unsqueeze(2)
            stride, padding, dilation, outpad = [1] + stride, [0] + padding, [1] + dilation, [0] + outpad
        elif len(stride) != 2:
            raise UnsupportedOp(f"{o['id']}: {len(stride)}-D convolution")
        xy = lambda p: tuple(p[::-1])                      # ATen's (h, w) pairs to the kernels' (x, y)
        self.ctx.ws.reset()
        if a.get("arg6"):
            K.convolutiontranspose_(self.ctx, out, x, w, bias, xy(stride), xy(padding), xy(dilation), xy(outpad), a.get("arg8", 1))
        else:
            K.convolution_(self.ctx, out, x, w, bias, xy(stride), xy(padding), xy(dilation), a.get("arg8", 1), act=a.get("epilogue", "none"))

    def _patch_tokens(self, o):
        """The folded patch embedding: convolution -> token rows 1.. with the position embedding joined in the GEMM's
        store, and the class row ``cls + pos[0]`` of every image."""
        a, ins = o["attrs"], o["in"]
        nb = 3 if a["has_bias"] else 2
        x, w = self.get(ins[0]), self.get(ins[1])
        bias = self.get(ins[2]) if a["has_bias"] else None
        out = self.t[o["out"]]
        B, T, C = out.shape
        cls, pos = self.get(ins[nb]).view(1, C), self.get(ins[nb + 1]).view(T, C)
        xy = lambda p: tuple(list(p)[::-1])
        self.ctx.ws.reset()
        K.convolution_tokens_(self.ctx, out[:, 1:], x, w, bias, xy(a["arg3"]), xy(a["arg4"]), xy(a["arg5"]), residual=pos[1:],
                              act=a.get("epilogue", "none"))
        if ("cls", o["id"]) not in self.scaled:          # cls + pos[0]: constants, added once
            row = torch.empty((1, C), dtype=out.dtype, device=out.device)
            K.add_(self.ctx, row, cls, pos[:1])
            self.scaled[("cls", o["id"])] = row
        row = self.scaled[("cls", o["id"])]
        if B == 1:
            K.add_(self.ctx, out[0, :1], cls, pos[:1])
        else:                                           # one launch for every image: the row read with stride 0 along the batch
            K.transposeLE_(self.ctx, out[:, :1].view(B, 1, C).unsqueeze(0), row.view(1, 1, C, 1).expand(1, B, C, 1))

    def _embedding(self, o):
        """embedding(table, ids) / index.Tensor(table, [ids]) along the first axis (ops.jl:1754-1783, 1524-1640); with
        four operands the sum of two gathers ``fold_embedding_sum`` made."""
        ins = o["in"]
        if o["aten"] == "index.Tensor" and o["attrs"].get("arg1") != [f"${ins[1]}"]:
            raise UnsupportedOp(f"{o['id']}: index.Tensor other than a gather of rows along the first axis")
        t2, i2 = (self.get(ins[2]), self.get(ins[3])) if len(ins) == 4 else (None, None)
        K.embedding_(self.ctx, self.t[o["out"]], self.get(ins[0]), self.get(ins[1]), t2, i2)

    def _kv_len(self, o):
        K.kv_len_from_position_(self.ctx, self.t[o["out"]], self.get(o["in"][0]), o["attrs"]["cap"])

    def _sdpa_append(self, o):
        """The folded cache step: write the new rows into the input cache and attend over it.  One launch where the
        single-workgroup kernel covers the shape and the mask became a length; two (append, attention) otherwise."""
        a = o["attrs"]
        q, ck, cv, kn, vn, kv_len = (self.get(i) for i in o["in"][:6])
        out = self.t[o["out"]]
        self.ctx.ws.reset()
        if not a.get("masked") and not a.get("all_slots"):
            try:
                K.sdpa_append(self.ctx, q, ck, cv, kn, vn, kv_len, a.get("scale"), out=out)
                return
            except K.DeclineError as e:
                if e.status != K.L.DECLINE_UNSUPPORTED:
                    raise
        K.kv_append_(self.ctx, ck, cv, kn, vn, kv_len)
        if a.get("masked"):
            K.sdpa(self.ctx, q, ck, cv, self.get(o["in"][6]), a.get("scale"), out=out)
        else:
            K.sdpa(self.ctx, q, ck, cv, None, a.get("scale"), out=out, kv_len=None if a.get("all_slots") else kv_len)

    HANDLERS = {"linear.default": _linear, "addmm.default": _linear, "mm.default": _linear,
                **dict.fromkeys(SDPA_OPS, _sdpa), "layer_norm.default": _layer_norm,
                "native_layer_norm.default": _native_layer_norm, "add.Tensor": _add,
                "gelu.default": _activation, "relu.default": _activation, "convolution.default": _convolution,
                "bmm.default": _bmm, "cat.default": _cat, **dict.fromkeys(SOFTMAX_OPS, _softmax),
                "mul.Tensor": _scale, "div.Tensor": _scale, "clone.default": _clone, "clamp.default": _clamp,
                "linear_group": _linear_group, "embedding.default": _embedding, "index.Tensor": _embedding,
                "kv_len_from_position": _kv_len, "sdpa_append": _sdpa_append, "patch_tokens": _patch_tokens,
                "rowstats": _rowstats}

    def replayable(self, *inputs: torch.Tensor):
        """Run once eagerly (binds inputs, sizes the workspace, stacks folded constants), then capture the whole graph as
        one device graph (the reference's ``Lava.capture/replay``).  Returns ``(replay, outputs)``: ``replay()`` re-runs
        the captured launches on the same input tensors -- refill them in place -- and ``outputs`` are the tensors it writes."""
        from .decode import StepGraph
        outs = self(*inputs)
        sg = StepGraph(lambda: self(*inputs))
        return sg.replay, outs

    def __call__(self, *inputs: torch.Tensor):
        if len(inputs) != len(self.g.inputs):
            raise ValueError(f"{self.g.name} takes {len(self.g.inputs)} inputs")
        for bid, x in zip(self.g.inputs, inputs):
            b = self.g.buffers[bid]
            if list(x.shape) != list(b["shape"]) or x.dtype != _DTYPES[b["dtype"]] or not x.is_cuda:
                raise ValueError(f"input {bid}: expected cuda {b['dtype']} {b['shape']}")
            self.t[bid] = x
        for o in self.g.ops:
            self.HANDLERS[o["aten"]](self, o)
        outs = [self.get(bid) for bid in self.g.outputs]
        return outs[0] if len(outs) == 1 else outs
