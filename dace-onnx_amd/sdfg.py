"""The slice of the DaCe graph API that ONNX expansions are written against.

DaCeML expansions receive ``(node, state, sdfg)``, read data descriptors off
the edges of the node and return either a replacement node or a nested SDFG
whose non-transient arrays are named like the node's connectors
(``daceml/onnx/op_implementations/utils.py:94-128``,
``daceml/onnx/nodes/onnx_op.py:652-683``). This module provides exactly those
objects -- ``SDFG``, ``SDFGState``, ``AccessNode``, ``Memlet``, data descriptors
with ``shape``/``strides``/``dtype``/``storage``, ``LibraryNode`` -- plus the one
node kind the ``"mi355x"`` expansions produce: :class:`KernelCall`, the
counterpart of the C++ tasklet a vendor-library expansion emits
(``daceml/onnx/op_implementations/cudnn_implementations.py:303-334``).

A :class:`KernelCall` is declarative (C function name + argument list), so the
same object can be executed from Python through ctypes -- what
:class:`CompiledSDFG` does, on torch's current HIP stream, optionally replayed
as a HIP graph -- or printed as the body of a DaCe C++ tasklet
(:meth:`KernelCall.as_cpp`).

Execution never leaves the GPU: arrays live in HBM as torch tensors, numpy
arguments are staged in and out, and there is no host implementation of any
node; a library node that was not expanded to kernels cannot run.
"""
import collections
import itertools
import typing

import numpy as np

from . import _lib

# --------------------------------------------------------------------------- dtypes


class typeclass:
    """Element type, the subset of ``dace.typeclass`` the ONNX path touches."""

    def __init__(self, name: str, np_dtype, ctype: str):
        self.name = name
        self.type = np.dtype(np_dtype).type
        self.np_dtype = np.dtype(np_dtype)
        self.bytes = self.np_dtype.itemsize
        self.ctype = ctype

    @property
    def base_type(self):
        return self

    def to_string(self) -> str:
        return self.name

    def as_torch(self):
        import torch
        return getattr(torch, self.name if self.name != "bool_" else "bool")

    def __call__(self, value):
        return self.type(value)

    def __repr__(self):
        return self.name

    def __eq__(self, other):
        return isinstance(other, typeclass) and other.name == self.name

    def __hash__(self):
        return hash(self.name)


float16 = typeclass("float16", np.float16, "half")
float32 = typeclass("float32", np.float32, "float")
float64 = typeclass("float64", np.float64, "double")
int8 = typeclass("int8", np.int8, "int8_t")
uint8 = typeclass("uint8", np.uint8, "uint8_t")
int16 = typeclass("int16", np.int16, "int16_t")
int32 = typeclass("int32", np.int32, "int32_t")
int64 = typeclass("int64", np.int64, "int64_t")
bool_ = typeclass("bool_", np.bool_, "bool")

_ALL_TYPES = [float16, float32, float64, int8, uint8, int16, int32, int64, bool_]
_BY_NP = {t.np_dtype: t for t in _ALL_TYPES}


def typeclass_of(dtype) -> typeclass:
    """typeclass for a numpy / torch dtype or a typeclass."""
    if isinstance(dtype, typeclass):
        return dtype
    try:
        import torch
        if isinstance(dtype, torch.dtype):
            dtype = str(dtype).split(".")[-1]
            dtype = "bool_" if dtype == "bool" else dtype
            return {t.name: t for t in _ALL_TYPES}[dtype]
    except ImportError:  # pragma: no cover
        pass
    return _BY_NP[np.dtype(dtype)]


class StorageType:
    Default = "Default"
    GPU_Global = "GPU_Global"
    CPU_Heap = "CPU_Heap"


class ScheduleType:
    Default = "Default"
    GPU_Default = "GPU_Default"
    GPU_Device = "GPU_Device"


# --------------------------------------------------------------------------- data


def _contiguous_strides(shape):
    strides, acc = [], 1
    for s in reversed(shape):
        strides.append(acc)
        acc *= int(s)
    return tuple(reversed(strides))


class Array:
    """Data descriptor (``dace.data.Array``): shape, element strides, dtype, storage."""

    def __init__(self, dtype, shape, strides=None, transient=False, storage=StorageType.GPU_Global):
        self.dtype = typeclass_of(dtype)
        self.shape = tuple(int(s) for s in shape)
        self.strides = tuple(int(s) for s in strides) if strides is not None else _contiguous_strides(self.shape)
        if len(self.strides) != len(self.shape):
            raise ValueError(f"strides {self.strides} do not match shape {self.shape}")
        self.transient = transient
        self.storage = storage

    @property
    def total_size(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    def is_contiguous(self) -> bool:
        return self.strides == _contiguous_strides(self.shape)

    def __repr__(self):
        return f"Array({self.dtype}, shape={self.shape}, strides={self.strides}, transient={self.transient})"


class Scalar(Array):
    def __init__(self, dtype, transient=False, storage=StorageType.GPU_Global):
        super().__init__(dtype, (), None, transient, storage)


class Memlet:
    """Data movement annotation. Only whole-array memlets occur on the ONNX path."""

    def __init__(self, data: str):
        self.data = data

    def __repr__(self):
        return f"Memlet({self.data})"


# --------------------------------------------------------------------------- nodes


class Node:
    def __init__(self, label: str, inputs=(), outputs=()):
        self.label = label
        self.in_connectors = {c: None for c in inputs}
        self.out_connectors = {c: None for c in outputs}

    @property
    def name(self):
        return self.label

    def add_in_connector(self, name):
        self.in_connectors[name] = None

    def add_out_connector(self, name):
        self.out_connectors[name] = None

    def remove_in_connector(self, name):
        self.in_connectors.pop(name, None)

    def remove_out_connector(self, name):
        self.out_connectors.pop(name, None)

    def __repr__(self):
        return f"{type(self).__name__}({self.label})"


class AccessNode(Node):
    def __init__(self, data: str):
        super().__init__(data)
        self.data = data


class LibraryNode(Node):
    """A node with several named implementations, expanded before execution."""
    implementations: typing.Dict[str, typing.Any] = {}
    default_implementation: typing.Optional[str] = None

    def __init__(self, name, location=None, inputs=(), outputs=()):
        super().__init__(name, inputs, outputs)
        self.implementation = None
        self.location = location or {}
        self.schedule = ScheduleType.GPU_Default

    @classmethod
    def register_implementation(cls, name, transformation_type):
        # per-class dict (the class attribute of the base must not be shared)
        if "implementations" not in cls.__dict__:
            cls.implementations = dict(cls.implementations)
        cls.implementations[name] = transformation_type
        transformation_type._match_node = cls

    def expand(self, sdfg, state, implementation=None):
        """Replace this node by its expansion; returns the implementation name used.

        Selection order follows DaCe: the node's ``implementation``, then the
        class's ``default_implementation``, then the library default.
        """
        impl = implementation or self.implementation or type(self).default_implementation
        if impl is None:
            impl = library_default_implementation(self)
        if impl not in self.implementations:
            raise KeyError(f"{type(self).__name__} has no implementation '{impl}' "
                           f"(available: {sorted(self.implementations)})")
        result = self.implementations[impl].expansion(self, state, sdfg)
        state.replace_node(self, result, sdfg)
        return impl


def library_default_implementation(node) -> str:
    from . import onnx as donnx  # late: avoids an import cycle
    return donnx.default_implementation


class Ptr:
    """Kernel argument: device pointer of the array attached to a connector."""

    def __init__(self, connector: typing.Optional[str], offset: int = 0):
        self.connector = connector  # None -> NULL
        self.offset = offset        # in elements

    def __repr__(self):
        return f"Ptr({self.connector}{'+%d' % self.offset if self.offset else ''})"


class Stream:
    """Kernel argument: the HIP stream the state is executing on."""


class I64Array:
    """Kernel argument: a small constant ``const int64_t[]`` (shapes, strides, pads)."""

    def __init__(self, values):
        self.values = [int(v) for v in values]

    def __repr__(self):
        return f"I64Array({self.values})"


class U32Array:
    """Kernel argument: a small constant ``const uint32_t[]`` (an elementwise program)."""

    def __init__(self, values):
        self.values = [int(v) & 0xFFFFFFFF for v in values]

    def __repr__(self):
        return f"U32Array({[hex(v) for v in self.values]})"


class F32Array:
    """Kernel argument: a small constant ``const float[]`` (immediates of an elementwise program)."""

    def __init__(self, values):
        self.values = [float(v) for v in values]

    def __repr__(self):
        return f"F32Array({self.values})"


class PtrArray:
    """Kernel argument: ``const float* const[]`` built from the arrays attached to several connectors."""

    def __init__(self, connectors):
        self.connectors = list(connectors)

    def __repr__(self):
        return f"PtrArray({self.connectors})"


class KernelCall(Node):
    """One call into ``libmi355x_onnx.so``; what a ``"mi355x"`` expansion returns.

    ``args`` are given in the order of the C prototype; plain Python ints/floats
    are passed by value.
    """

    def __init__(self, label, function: str, args, inputs, outputs):
        super().__init__(label, inputs, outputs)
        self.function = function
        self.args = list(args)
        if function not in _lib.SIGNATURES:
            raise KeyError(f"{function} is not part of the C ABI")

    def as_cpp(self) -> str:
        """Body of the equivalent DaCe C++ tasklet (connectors ``_<name>`` are
        ``dace.pointer`` typed, as in cudnn_implementations.py:324-327)."""
        lines, call_args = [], []
        for i, a in enumerate(self.args):
            if isinstance(a, Ptr):
                if a.connector is None:
                    call_args.append("nullptr")
                else:
                    call_args.append(f"_{a.connector}" + (f" + {a.offset}" if a.offset else ""))
            elif isinstance(a, Stream):
                call_args.append("__dace_current_stream")
            elif isinstance(a, I64Array):
                lines.append(f"const int64_t __arg{i}[] = {{{', '.join(str(v) for v in a.values)}}};")
                call_args.append(f"__arg{i}")
            elif isinstance(a, U32Array):
                lines.append(f"const uint32_t __arg{i}[] = {{{', '.join(hex(v) + 'u' for v in a.values) or '0u'}}};")
                call_args.append(f"__arg{i}")
            elif isinstance(a, F32Array):
                lines.append(f"const float __arg{i}[] = {{{', '.join(repr(v) + 'f' for v in a.values) or '0.0f'}}};")
                call_args.append(f"__arg{i}")
            elif isinstance(a, PtrArray):
                lines.append(f"const float* const __arg{i}[] = {{{', '.join('_' + c for c in a.connectors) or 'nullptr'}}};")
                call_args.append(f"__arg{i}")
            elif a is None:
                call_args.append("nullptr")
            elif isinstance(a, float):
                call_args.append(repr(a) + "f")
            else:
                call_args.append(str(int(a)))
        lines.append(f"int __status = {self.function}({', '.join(call_args)});")
        lines.append(f'if (__status != 0) {{ printf("{self.function}: %s\\n", mi355x_last_error()); exit(1); }}')
        return "\n".join(lines)


class AliasNode(Node):
    """Output is the input's storage seen under another shape (ONNX Reshape /
    Flatten / Identity on contiguous data): no kernel, no bytes moved."""

    def __init__(self, label, in_conn, out_conn):
        super().__init__(label, [in_conn], [out_conn])
        self.in_conn, self.out_conn = in_conn, out_conn


class NestedSDFG(Node):
    def __init__(self, label, sdfg, inputs, outputs):
        super().__init__(label, inputs, outputs)
        self.sdfg = sdfg


class MultiConnectorEdge:
    def __init__(self, src, src_conn, dst, dst_conn, data: Memlet):
        self.src, self.src_conn, self.dst, self.dst_conn, self.data = src, src_conn, dst, dst_conn, data

    def __repr__(self):
        return f"{self.src}:{self.src_conn} -> {self.dst}:{self.dst_conn} [{self.data}]"


# --------------------------------------------------------------------------- state / sdfg


class SDFGState:
    def __init__(self, label, sdfg):
        self.label = label
        self.parent = sdfg
        self._nodes: typing.List[Node] = []
        self._edges: typing.List[MultiConnectorEdge] = []
        self.nosync = False

    def nodes(self):
        return list(self._nodes)

    def edges(self):
        return list(self._edges)

    def node_id(self, node):
        return self._nodes.index(node)

    def add_node(self, node):
        if node not in self._nodes:
            self._nodes.append(node)
        return node

    def add_access(self, data):
        return self.add_node(AccessNode(data))

    add_read = add_access
    add_write = add_access

    def add_edge(self, src, src_conn, dst, dst_conn, memlet):
        self.add_node(src)
        self.add_node(dst)
        e = MultiConnectorEdge(src, src_conn, dst, dst_conn, memlet)
        self._edges.append(e)
        return e

    def remove_edge(self, edge):
        self._edges.remove(edge)

    def remove_node(self, node):
        self._nodes.remove(node)
        self._edges = [e for e in self._edges if e.src is not node and e.dst is not node]

    def in_edges(self, node):
        return [e for e in self._edges if e.dst is node]

    def out_edges(self, node):
        return [e for e in self._edges if e.src is node]

    def in_degree(self, node):
        return len(self.in_edges(node))

    def out_degree(self, node):
        return len(self.out_edges(node))

    def replace_node(self, old, new, sdfg):
        """Put an expansion result in place of a library node, keeping its edges."""
        if isinstance(new, SDFG):
            inputs = [e.dst_conn for e in self.in_edges(old)]
            outputs = [e.src_conn for e in self.out_edges(old)]
            for conn in inputs + outputs:
                if conn not in new.arrays:
                    raise ValueError(f"expansion of {old} has no array for connector '{conn}'")
            new = NestedSDFG(old.label, new, inputs, outputs)
        idx = self._nodes.index(old)
        self._nodes[idx] = new
        for e in self._edges:
            if e.src is old:
                if e.src_conn not in new.out_connectors:
                    raise ValueError(f"expansion of {old} lost output connector '{e.src_conn}'")
                e.src = new
            if e.dst is old:
                if e.dst_conn in new.in_connectors:
                    e.dst = new
        # inputs the expansion does not consume (e.g. Reshape's constant `shape`)
        self._edges = [e for e in self._edges if e.dst is not old]
        self._prune_dangling_reads()

    def _prune_dangling_reads(self):
        for n in list(self._nodes):
            if isinstance(n, AccessNode) and not self.in_edges(n) and not self.out_edges(n):
                self._nodes.remove(n)

    def topological_nodes(self):
        """Nodes in dependency order. Two access nodes of the same array are
        ordered write-before-read, which is how DaCe sequences them across the
        access-node chain of a state."""
        indeg = {id(n): 0 for n in self._nodes}
        succ = collections.defaultdict(list)
        for e in self._edges:
            succ[id(e.src)].append(e.dst)
            indeg[id(e.dst)] += 1
        writers, readers = collections.defaultdict(list), collections.defaultdict(list)
        for n in self._nodes:
            if isinstance(n, AccessNode):
                (writers if self.in_edges(n) else readers)[n.data].append(n)
        for data, ws in writers.items():
            for w in ws:
                for r in readers.get(data, []):
                    succ[id(w)].append(r)
                    indeg[id(r)] += 1
        ready = [n for n in self._nodes if indeg[id(n)] == 0]
        order = []
        while ready:
            n = ready.pop(0)
            order.append(n)
            for m in succ[id(n)]:
                indeg[id(m)] -= 1
                if indeg[id(m)] == 0:
                    ready.append(m)
        if len(order) != len(self._nodes):
            raise ValueError(f"state {self.label} has a dependency cycle")
        return order


class SDFG:
    _ids = itertools.count()

    def __init__(self, name: str):
        self.name = name
        self.sdfg_id = next(SDFG._ids)
        self.arrays: typing.Dict[str, Array] = collections.OrderedDict()
        self._states: typing.List[SDFGState] = []
        self._compiled = None

    # -- construction ------------------------------------------------------------
    def add_array(self, name, shape, dtype, strides=None, transient=False, storage=StorageType.GPU_Global):
        if name in self.arrays:
            raise NameError(f"array '{name}' already exists in {self.name}")
        self.arrays[name] = Array(dtype, shape, strides, transient, storage)
        self._compiled = None
        return name, self.arrays[name]

    def add_transient(self, name, shape, dtype, strides=None, storage=StorageType.GPU_Global):
        return self.add_array(name, shape, dtype, strides, True, storage)

    def add_scalar(self, name, dtype, transient=False):
        return self.add_array(name, (), dtype, None, transient)

    def add_datadesc(self, name, desc: Array):
        if name in self.arrays:
            raise NameError(f"array '{name}' already exists in {self.name}")
        self.arrays[name] = desc
        self._compiled = None
        return name

    def add_state(self, label=None):
        st = SDFGState(label or f"state_{len(self._states)}", self)
        self._states.append(st)
        self._compiled = None
        return st

    def add_state_before(self, state, label=None):
        st = SDFGState(label or f"state_{len(self._states)}", self)
        self._states.insert(self._states.index(state), st)
        self._compiled = None
        return st

    def nodes(self):
        return list(self._states)

    states = nodes

    def node(self, i):
        return self._states[i]

    def node_id(self, state):
        return self._states.index(state)

    def make_array_memlet(self, name):
        if name not in self.arrays:
            raise KeyError(f"no array '{name}' in {self.name}")
        return Memlet(name)

    def all_nodes_recursive(self):
        for st in self._states:
            yield st, self
            for n in st.nodes():
                yield n, st
                if isinstance(n, NestedSDFG):
                    yield from n.sdfg.all_nodes_recursive()

    # -- expansion ------------------------------------------------------------------
    def expand_library_nodes(self, recursive=True):
        """Expand every library node (``dace.SDFG.expand_library_nodes``)."""
        self._compiled = None
        changed = True
        while changed:
            changed = False
            for st in self._states:
                for n in st.nodes():
                    if isinstance(n, LibraryNode):
                        n.expand(self, st)
                        changed = True
                    elif isinstance(n, NestedSDFG) and recursive:
                        before = sum(1 for x, _ in n.sdfg.all_nodes_recursive() if isinstance(x, LibraryNode))
                        if before:
                            n.sdfg.expand_library_nodes(recursive)
                            changed = True

    # -- execution --------------------------------------------------------------------
    def compile(self) -> "CompiledSDFG":
        if self._compiled is None:
            self._compiled = CompiledSDFG(self)
        return self._compiled

    def __call__(self, **kwargs):
        self.expand_library_nodes()
        return self.compile()(**kwargs)


# --------------------------------------------------------------------------- executor


class CompiledSDFG:
    """Executable form of an expanded SDFG: a flat list of kernel launches.

    Transients are allocated once, when the launch list is first bound, and kept. ``__call__`` binds the
    non-transient arrays, enqueues every launch on torch's current HIP stream and returns
    without synchronising. ``capture_graph`` records the launches into a HIP
    graph; afterwards ``replay`` re-runs them against the same buffers with a
    single launch.
    """

    def __init__(self, sdfg: SDFG, device="cuda:0"):
        import torch
        self.sdfg = sdfg
        self.device = torch.device(device)
        for n, _ in sdfg.all_nodes_recursive():
            if isinstance(n, LibraryNode):
                raise RuntimeError(f"{n} was not expanded; call expand_library_nodes() first")
        self._lib = _lib.library()  # raises if the HIP library is not built
        self._external = [k for k, d in sdfg.arrays.items() if not d.transient]
        self._written = self._find_written(sdfg)
        self._transients = {}   # flattened key -> descriptor
        self._transient_tensors = {}   # flattened key -> its allocation (made on first use, kept)
        self._plan = []         # ("call", node, connector -> key) | ("alias", src key, dst key, dst descriptor)
        self._bound_key = None
        self._graph = None
        self._build(sdfg, prefix="", outer_map={})

    @staticmethod
    def _find_written(sdfg):
        written = set()
        for st in sdfg.nodes():
            for e in st.edges():
                if isinstance(e.dst, AccessNode) and not isinstance(e.src, AccessNode):
                    written.add(e.dst.data)
        return written

    def _build(self, sdfg, prefix, outer_map):
        """Flatten (possibly nested) states into launches. ``outer_map`` maps a
        non-transient array name of ``sdfg`` to the key of the enclosing scope."""
        import torch

        def key_of(name):
            return outer_map.get(name, prefix + name)

        for name, desc in sdfg.arrays.items():
            if name in outer_map:
                continue
            if desc.transient:
                self._transients[key_of(name)] = desc
        for st in sdfg.nodes():
            for n in st.topological_nodes():
                if isinstance(n, (AccessNode,)):
                    continue
                conn_to_key = {}
                for e in st.in_edges(n):
                    conn_to_key[e.dst_conn] = key_of(e.data.data)
                for e in st.out_edges(n):
                    conn_to_key[e.src_conn] = key_of(e.data.data)
                if isinstance(n, KernelCall):
                    self._plan.append(("call", n, conn_to_key))
                elif isinstance(n, AliasNode):
                    src_e = [e for e in st.in_edges(n) if e.dst_conn == n.in_conn][0]
                    dst_e = [e for e in st.out_edges(n) if e.src_conn == n.out_conn][0]
                    self._plan.append(("alias", key_of(src_e.data.data), key_of(dst_e.data.data),
                                       sdfg.arrays[dst_e.data.data]))
                elif isinstance(n, NestedSDFG):
                    inner_map = {c: k for c, k in conn_to_key.items()}
                    self._build(n.sdfg, prefix=f"{prefix}{n.label}_{st.node_id(n)}.", outer_map=inner_map)
                else:
                    raise RuntimeError(f"cannot execute node {n!r}")

    # -- binding ---------------------------------------------------------------------
    def _bind(self, env):
        """Resolve every pointer argument against ``env`` (key -> tensor). Transient tensors are allocated on the
        first call and kept: binding again (the caller passed other buffers) only resolves pointers anew."""
        import torch
        env = dict(env)
        launches = []
        # A Reshape-like alias whose result is caller-owned memory: let the producer of its source write there
        # directly (the source, a transient, becomes a view of the caller's buffer). Walking the aliases backwards
        # carries this through chains of them. What cannot be redirected (the source is caller-owned too, or
        # already a view of something else) is copied on the device.
        # The redirect moves the write of the caller's buffer from the alias's place in the plan to the producer's,
        # which is earlier: it is only taken when nothing before the alias reads that buffer (an array that is both
        # an input of an earlier node and the reshaped output keeps its old contents until the copy).
        def read_before(position, key):
            for earlier in self._plan[:position]:
                if earlier[0] == "alias":
                    if earlier[1] == key:
                        return True
                elif any(earlier[2].get(c) == key for c in earlier[1].in_connectors):
                    return True
            return False

        redirected = set()
        for position in range(len(self._plan) - 1, -1, -1):
            item = self._plan[position]
            if item[0] != "alias":
                continue
            _, src_key, dst_key, _ = item
            if dst_key in env and src_key not in env and src_key in self._transients and not read_before(position, dst_key):
                env[src_key] = env[dst_key].reshape(self._transients[src_key].shape)
                redirected.add((src_key, dst_key))
        for item in self._plan:
            if item[0] == "alias":
                _, src_key, dst_key, dst_desc = item
                if (src_key, dst_key) in redirected:
                    continue
                src = self._tensor(env, src_key)
                if dst_key in env:
                    launches.append(("copy", env[dst_key], src))
                else:
                    env[dst_key] = src.reshape(dst_desc.shape)  # contiguous -> view
                continue
            _, node, conn_to_key = item
            fn = getattr(self._lib, node.function)
            args, keep, stream_slots = [], [], []
            for i, a in enumerate(node.args):
                if isinstance(a, Ptr):
                    if a.connector is None:
                        args.append(None)
                    else:
                        t = self._tensor(env, conn_to_key[a.connector])
                        args.append(t.data_ptr() + a.offset * t.element_size())
                elif isinstance(a, Stream):
                    stream_slots.append(i)
                    args.append(None)
                elif isinstance(a, I64Array):
                    arr = _lib.i64_array(a.values)
                    keep.append(arr)
                    args.append(arr)
                elif isinstance(a, (U32Array, F32Array, PtrArray)):
                    if isinstance(a, PtrArray):
                        arr = _lib.pointer_array([self._tensor(env, conn_to_key[c]).data_ptr() for c in a.connectors])
                    else:
                        arr = (_lib.u32_array if isinstance(a, U32Array) else _lib.f32_array)(a.values)
                    keep.append(arr)
                    args.append(arr)
                else:
                    args.append(a)
            launches.append(("call", fn, node.function, args, stream_slots, keep, node))
        return env, launches

    def _tensor(self, env, key):
        """The tensor bound to ``key``; a transient that has none yet gets its allocation, made once per
        compiled SDFG and reused by every later binding."""
        if key not in env:
            import torch
            if key not in self._transient_tensors:
                d = self._transients[key]
                self._transient_tensors[key] = torch.empty(d.shape, dtype=d.dtype.as_torch(), device=self.device)
            env[key] = self._transient_tensors[key]
        return env[key]

    def _run(self, launches):
        import torch
        stream = torch.cuda.current_stream(self.device).cuda_stream
        for item in launches:
            if item[0] == "copy":
                item[1].copy_(item[2].reshape(item[1].shape))
                continue
            _, fn, name, args, stream_slots, _, _ = item
            for s in stream_slots:
                args[s] = stream
            status = fn(*args)
            if status != 0:
                _lib.check(status, name)

    def __call__(self, **kwargs):
        import torch
        sdfg = self.sdfg
        unknown = set(kwargs) - set(sdfg.arrays)
        if unknown:
            raise TypeError(f"unknown arguments {sorted(unknown)} for SDFG {sdfg.name}")
        env, staged_back = {}, []
        any_torch = any(isinstance(v, torch.Tensor) for v in kwargs.values())
        for name in self._external:
            desc = sdfg.arrays[name]
            if name not in kwargs:
                if name == "__return" or name.startswith("__return"):
                    env[name] = torch.empty(desc.shape, dtype=desc.dtype.as_torch(), device=self.device)
                    continue
                raise TypeError(f"missing argument '{name}' for SDFG {sdfg.name}")
            v = kwargs[name]
            if isinstance(v, torch.Tensor):
                if tuple(v.shape) != desc.shape or typeclass_of(v.dtype) != desc.dtype:
                    raise TypeError(f"argument '{name}': expected {desc.dtype}{list(desc.shape)}, "
                                    f"got {v.dtype}{list(v.shape)}")
                if v.device.type != "cuda":
                    d = v.to(self.device)
                    if name in self._written:
                        staged_back.append((v, d))
                    v = d
                if not v.is_contiguous():
                    raise TypeError(f"argument '{name}' must be contiguous")
                env[name] = v
            else:
                a = np.asarray(v)
                if a.shape != desc.shape:
                    raise TypeError(f"argument '{name}': expected shape {desc.shape}, got {a.shape}")
                if typeclass_of(a.dtype) != desc.dtype:
                    a = a.astype(desc.dtype.np_dtype)  # python scalars / default float64
                d = torch.from_numpy(np.ascontiguousarray(a)).to(self.device)
                if name in self._written and isinstance(v, np.ndarray):
                    staged_back.append((v, d))
                env[name] = d
        key = tuple((n, env[n].data_ptr()) for n in self._external)
        if key != self._bound_key:
            self._env, self._launch_list = self._bind(env)
            self._bound_key = key
            self._graph = None
        self._run(self._launch_list)
        for host, dev in staged_back:
            if isinstance(host, np.ndarray):
                host[...] = dev.cpu().numpy()
            else:
                host.copy_(dev)
        rets = [n for n in self._external if n.startswith("__return")]
        if rets:
            outs = [self._env[n] if any_torch else self._env[n].cpu().numpy() for n in rets]
            return outs[0] if len(outs) == 1 else tuple(outs)
        return None

    # -- HIP graph -------------------------------------------------------------------
    def capture_graph(self):
        """Record the currently bound launch list into a HIP graph."""
        import torch
        if self._bound_key is None:
            raise RuntimeError("call the compiled SDFG once before capturing it")
        # (a device copy left over from a Reshape into caller-owned memory is issued on the capture stream like
        # the kernels and becomes a node of the graph)
        g = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.graph(g):
            self._run(self._launch_list)
        self._graph = g
        return g

    def replay(self):
        if self._graph is None:
            raise RuntimeError("capture_graph() has not been called for the current buffers")
        self._graph.replay()

    @property
    def num_launches(self):
        return sum(1 for item in self._plan if item[0] == "call")

    # -- the same launch sequence as C++ -----------------------------------------------
    def program_source(self, name: typing.Optional[str] = None) -> typing.Tuple[str, typing.List[str]]:
        """The launch sequence as a C++ translation unit, the code DaCe would emit around the tasklets of
        :meth:`KernelCall.as_cpp` (each tasklet a block with ``dace.pointer`` typed connectors ``_<name>``
        and the stream as ``__dace_current_stream``: ``cudnn_implementations.py:324-334``,
        ``environments/cudnn.py:44``).

        Returns ``(source, arrays)``. The source includes only ``mi355x_onnx.h`` and defines
        ``extern "C" int __program_<name>(void** __arrays, void* __dace_current_stream)``; ``arrays`` lists, in
        the order of ``__arrays``, the arrays whose device pointers the caller passes: the SDFG's non-transient
        arrays by name, then its transients by their flattened key (see :meth:`transient_descriptors`). A
        Reshape-like alias of a transient is a pointer assignment; one into caller-owned memory would need a
        copy and is not supported here.
        """
        name = name or self.sdfg.name
        arrays = list(self._external) + [k for k in self._transients if k not in self._external]
        index = {k: i for i, k in enumerate(arrays)}
        desc_of = {**{k: self.sdfg.arrays[k] for k in self._external}, **self._transients}
        lines = ['#include <stdint.h>', '#include <stdio.h>', '#include <stdlib.h>', '#include "mi355x_onnx.h"', '',
                 f'extern "C" int __program_{name}(void** __arrays, void* __dace_current_stream) {{']
        for item in self._plan:
            if item[0] == "alias":
                _, src_key, dst_key, dst_desc = item
                if dst_key in self._external:
                    raise NotImplementedError(f"alias into caller-owned array '{dst_key}' needs a device copy")
                if dst_key not in index:
                    index[dst_key] = len(arrays)
                    arrays.append(dst_key)
                desc_of[dst_key] = dst_desc   # the view's own element type (an int64 or int8 view is not a float*)
                lines.append(f"    __arrays[{index[dst_key]}] = __arrays[{index[src_key]}];  // {dst_key} is a view of {src_key}")
                continue
            _, node, conn_to_key = item
            lines.append(f"    {{  // {node.label}")
            for conn, key in conn_to_key.items():
                ctype = desc_of[key].dtype.ctype if key in desc_of else "float"
                lines.append(f"        {ctype}* _{conn} = ({ctype}*)__arrays[{index[key]}];")
                lines.append(f"        (void)_{conn};")
            lines.extend("        " + ln for ln in node.as_cpp().splitlines())
            lines.append("    }")
        lines += ["    return 0;", "}", ""]
        return "\n".join(lines), arrays

    def transient_descriptors(self):
        """Flattened key -> descriptor of every transient array (what :meth:`program_source` expects the caller
        to allocate besides the SDFG's own arguments)."""
        return dict(self._transients)

    def bound_launches(self):
        """[(KernelCall node, zero-argument callable)] for the currently bound buffers:
        each callable re-issues that one launch on torch's current stream (profiling)."""
        import torch
        if self._bound_key is None:
            raise RuntimeError("call the compiled SDFG once first")
        out = []
        for item in self._launch_list:
            if item[0] != "call":
                continue
            out.append((item[6], (lambda it: (lambda: self._run([it])))(item)))
        return out
