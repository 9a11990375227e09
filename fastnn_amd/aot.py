"""Host-side mirror of fastnn's Python entry to the quantised path:

    fastnn.AotExecutor(nodes, params, input_names, output_names, input_shapes=None, quantize=None)
    executor.forward({name: array}) -> {name: array}

(fastnn/__init__.py:102, fastnn/io/__init__.py:352; Rust side src/python/nn.rs:1222-1431.)  `nodes` are
ONNX-style dicts whose values are all strings ("name", "op_type", "inputs": "[a, b]", "outputs": "[y]",
attributes as strings); `params` maps initialiser names to arrays; `quantize` is 4, 8 or one of
"i4", "i8", "u4", "u8", "f8", "f8r", "f4", "i4cb" (src/python/nn.rs:1320-1358).

The graph is lowered the way the reference's compile step does for a quantised model
(src/compiler/passes/quantization.rs:36-273, src/backend/cpu/mod.rs:385-626,776-979): a constant that is
input[1] of a MatMul (2-D, stored [K,N], packed transposed as [N,K]) or of a Conv is quantised with the
reference's packer; MatMul + Add(bias) + Relu/Gelu/Silu collapse into one epilogue-tagged kernel
(src/compiler/passes/fusion/matmul_add_relu.rs:92-110); every value gets a 64-byte aligned slot of one arena
(src/compiler/passes/memory_planning.rs:652-654); the result is an ExecutablePlan for HipBackend.
Only the operators of that path are accepted; anything else raises FnnError(UnsupportedOp) naming the op.
No compute happens here: building an executor needs no GPU, forward() does."""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np

from . import lib as _l
from .backend import BITS_OF, KERNEL_OF, ExecutablePlan, HipBackend, meta_of
from .lib import FnnError

_QUANTIZE_STR = {"i4": _l.DT_I4, "i8": _l.DT_I8, "u4": _l.DT_U4, "u8": _l.DT_U8, "f8": _l.DT_F8,
                 "f8r": _l.DT_F8R, "f4": _l.DT_F4, "i4cb": _l.DT_I4CB}
_CONV_KERNEL = {_l.DT_I8: "conv2d_i8", _l.DT_I4: "conv2d_i4", _l.DT_U8: "conv2d_u8", _l.DT_U4: "conv2d_u4",
                _l.DT_F8: "conv2d_f8", _l.DT_F8R: "conv2d_f8r", _l.DT_F4: "conv2d_f4", _l.DT_I4CB: "conv2d_i4"}
_ACT_SUFFIX = {"Relu": "_relu", "Gelu": "_gelu", "Silu": "_silu"}
_ACT_KERNEL = {"Relu": "relu_f32", "Gelu": "gelu_f32", "Silu": "silu_f32"}


def weight_dtype_of(quantize) -> Optional[int]:
    """`quantize` argument -> weight type, with the reference's errors (src/python/nn.rs:1320-1358).
    None and "f32" mean unquantised weights (returns None)."""
    if quantize is None:
        return None
    if isinstance(quantize, (bool, np.bool_)):
        raise TypeError("quantize must be int (4, 8) or str (f32, f8, f8r, f4) or None")
    if isinstance(quantize, (int, np.integer)):
        if int(quantize) == 4:
            return _l.DT_I4
        if int(quantize) == 8:
            return _l.DT_I8
        raise ValueError(f"unsupported quantize value for integer: {int(quantize)} (expected 4 or 8)")
    if isinstance(quantize, str):
        if quantize == "f32":
            return None
        if quantize in _QUANTIZE_STR:
            return _QUANTIZE_STR[quantize]
        raise ValueError(f"unsupported quantize string: '{quantize}' (expected f32, i4, i8, u4, u8, f8, f8r, f4, i4cb, 4, or 8)")
    raise TypeError("quantize must be int (4, 8) or str (f32, f8, f8r, f4) or None")


def _names(field: Optional[str]) -> List[str]:
    """"[a, b]" -> ["a", "b"] (src/python/nn.rs:1242-1262)."""
    if not field:
        return []
    return [x.strip() for x in field.strip("[]").split(",") if x.strip()]


def _attr_int(node: dict, *keys: str, default: int) -> int:
    for k in keys:
        if k in node:
            try:
                return int(node[k])
            except ValueError:
                pass
    return default


class _Value:
    __slots__ = ("shape", "slot", "view_of")

    def __init__(self, shape: Sequence[int], slot, view_of=None):
        self.shape = tuple(int(d) for d in shape)
        self.slot = slot
        self.view_of = view_of     # (name of the value whose slot holds this one, byte offset inside it) or None

    @property
    def nbytes(self) -> int:
        return int(np.prod(self.shape, dtype=np.int64)) * 4


class AotExecutor:
    """Compiles the node list into an ExecutablePlan once; forward() writes the inputs into the arena,
    dispatches (graph replay from the second call on) and reads the outputs.

    concat_in_place (default on): the parts of a Concat with one outer block (a channel Concat of one image) get
    their slots inside the Concat's result, so their producers store there and the Concat copies only the parts
    that cannot move (a graph input, a value that lives in another Concat already, a part that comes twice)."""

    def __init__(self, nodes: Sequence[Dict[str, str]], params: Dict[str, np.ndarray], input_names: Sequence[str],
                 output_names: Sequence[str], input_shapes: Optional[Dict[str, Sequence[int]]] = None, quantize=None,
                 device: int = 0, concat_in_place: bool = True):
        self.weight_dtype = weight_dtype_of(quantize)
        if self.weight_dtype is None:
            raise FnnError(3, "AotExecutor: only quantised weights run on this backend (quantize=None / 'f32' is the f32 path)")
        self.input_names, self.output_names = list(input_names), list(output_names)
        self.device = device
        self._params = {k: np.ascontiguousarray(v, dtype=np.float32) for k, v in params.items()}
        shapes = dict(input_shapes or {})
        for n in self.input_names:
            if n not in shapes:
                raise FnnError(4, f"AotExecutor: input_shapes must give the shape of '{n}'")
            if any(int(d) < 0 for d in shapes[n]):
                raise FnnError(3, f"AotExecutor: symbolic dimension in the shape of '{n}' (static shapes only)")
        # Two passes when a Concat joins its parts in one outer block (a channel concat of one image): the first gives
        # every value its shape, then the values that are such parts get their slot INSIDE the Concat result's slot
        # (the producers store there, the Concat copies nothing), and the second pass lowers with those slots
        self._placement: Dict[str, tuple] = {}  # value name -> (name of the Concat result, byte offset inside it)
        self._sizes: Dict[str, int] = {}
        self._reserved: Dict[str, tuple] = {}
        for lowering in (0, 1):
            self._top = 0
            self._values: Dict[str, _Value] = {}
            self.instructions: List[tuple] = []     # (kernel_name, input names, output name, params): for inspection
            self._consts: List[tuple] = []          # (offset, array)
            self._calls: List[tuple] = []           # (kernel, [slots], slot, params, meta)
            self._reserved = {}
            self._split_of: Dict[str, tuple] = {}   # copied Split part -> (source, axis, first index, indices, source's size along axis)
            for n in self.input_names:
                self._new_value(n, shapes[n])
            self._lower([dict(n) for n in nodes])
            self._drop_unread()
            if lowering == 1 or not concat_in_place:
                break
            self._placement = self._place_concat_parts([dict(n) for n in nodes])
            if not self._placement:
                break
            self._sizes = {k: v.nbytes for k, v in self._values.items()}
        for n in self.output_names:
            if n not in self._values:
                raise FnnError(4, f"AotExecutor: output '{n}' is produced by no node")
        self._plan: Optional[ExecutablePlan] = None
        self._backend: Optional[HipBackend] = None

    # ---- memory planning: one slot per value, 64-byte aligned
    def _take(self, nbytes: int):
        off = self._top
        self._top += (int(nbytes) + 63) // 64 * 64
        return (off, int(nbytes))

    def _slot_for(self, name: str, nbytes: int):
        """A value's slot: inside the slot of the Concat result it is a part of (reserved on first use), the slot
        reserved for it by one of its parts, or a new one."""
        if name in self._reserved:
            return self._reserved[name]
        if name in self._placement:
            parent, off = self._placement[name]
            base = self._slot_for(parent, self._sizes[parent])
            slot = (base[0] + off, int(nbytes))
        else:
            slot = self._take(nbytes)
        self._reserved[name] = slot
        return slot

    def _new_value(self, name: str, shape) -> _Value:
        v = _Value(shape, self._slot_for(name, int(np.prod(shape, dtype=np.int64)) * 4))
        self._values[name] = v
        return v

    def _drop_unread(self):
        """Instructions whose result nothing reads (no later instruction, no view of it, not a graph output) are
        taken out: the copy of a Split part that only a Concat wanted, once that Concat reads the Split's source."""
        inside: Dict[str, list] = {}     # Concat result -> the values stored in place inside it
        for child, (parent, _) in self._placement.items():
            inside.setdefault(parent, []).append(child)
        needed = set()

        def need(name):
            name = self._root_of(name)[0]
            if name not in needed:
                needed.add(name)
                for child in inside.get(name, []):
                    if child in self._values:
                        need(child)

        for n in self.output_names:
            if n in self._values:
                need(n)
        keep = [False] * len(self.instructions)
        for idx in range(len(self.instructions) - 1, -1, -1):
            _, ins, out, _ = self.instructions[idx]
            if out in needed:
                keep[idx] = True
                for i in ins:
                    if i in self._values:
                        need(i)
        self._dropped = set(x[2] for x, k in zip(self.instructions, keep) if not k)
        self.instructions = [x for x, k in zip(self.instructions, keep) if k]
        self._calls = [x for x, k in zip(self._calls, keep) if k]

    def kept(self, name: str) -> bool:
        """False for a value that no instruction of the plan writes (nothing reads it and it is no output)."""
        return name in self._values and name not in self._dropped

    def _root_of(self, name: str):
        """(value that owns the slot `name` lives in, byte offset of `name` inside it)."""
        off = 0
        while self._values[name].view_of is not None:
            name, o = self._values[name].view_of
            off += o
        return name, off

    def _place_concat_parts(self, nodes: List[dict]) -> Dict[str, tuple]:
        """After a first lowering: which values can live inside the slot of a Concat result.  A Concat with one
        outer block lays its parts end to end; a part (or the value a part is a Split view of) takes that place
        when it is produced by an instruction of the plan, is not placed already, lands 64-byte aligned, and all
        of its bytes are parts of this Concat at the same relative position."""
        placed: Dict[str, tuple] = {}
        for nd in nodes:
            if nd.get("op_type") != "Concat":
                continue
            ins, outs = _names(nd.get("inputs")), _names(nd.get("outputs"))
            if not outs or outs[0] not in self._values or any(i not in self._values for i in ins):
                continue
            out = self._values[outs[0]]
            rank = len(out.shape)
            axis = _attr_int(nd, "axis", default=0)
            axis = axis + rank if axis < 0 else axis
            axis = min(max(axis, 0), rank - 1)
            if int(np.prod(out.shape[:axis], dtype=np.int64)) != 1:
                continue
            claims: Dict[str, tuple] = {}       # root -> (offset of the root inside the result, [(first byte, size) of its parts])
            off = 0
            for x in ins:
                size = self._values[x].nbytes
                root, delta = self._root_of(x)
                want = off - delta
                if root in claims and claims[root][0] == want:
                    claims[root][1].append((delta, size))
                elif root not in claims and root not in placed and root not in self.input_names and root != outs[0]:
                    claims[root] = (want, [(delta, size)])
                off += size
            spans = []
            for root, (want, parts) in claims.items():
                rsize = self._values[root].nbytes
                covered, end = True, 0
                for d, s in sorted(parts):
                    covered = covered and d <= end
                    end = max(end, d + s)
                if not (covered and end >= rsize and want >= 0 and want % 64 == 0 and want + rsize <= out.nbytes):
                    continue
                if any(want < o + s and o < want + rsize for o, s in spans):
                    continue
                spans.append((want, rsize))
                placed[root] = (outs[0], want)
        return placed

    def _const_slot(self, arr: np.ndarray):
        slot = self._take(arr.nbytes)
        self._consts.append((slot[0], arr))
        return slot

    def _emit(self, kernel: str, ins: List[str], out: str, in_slots, out_slot, params, meta=None):
        self.instructions.append((kernel, list(ins), out, [int(p) for p in params]))
        self._calls.append((kernel, list(in_slots), out_slot, [int(p) for p in params], meta))

    # ---- lowering
    def _lower(self, nodes: List[dict]):
        uses: Dict[str, int] = {}
        for nd in nodes:
            for i in _names(nd.get("inputs")):
                uses[i] = uses.get(i, 0) + 1
        for o in self.output_names:
            uses[o] = uses.get(o, 0) + 1
        producer_of_next = {}   # value name -> index of the single node that consumes it
        for idx, nd in enumerate(nodes):
            for i in _names(nd.get("inputs")):
                producer_of_next.setdefault(i, []).append(idx)
        done = set()
        for idx, nd in enumerate(nodes):
            if idx in done:
                continue
            op = nd.get("op_type", "")
            ins, outs = _names(nd.get("inputs")), _names(nd.get("outputs"))
            if op in ("MatMul", "Gemm"):
                self._lower_matmul(nodes, idx, nd, ins, outs, uses, producer_of_next, done)
            elif op in ("Conv", "Conv2d"):
                self._lower_conv(nodes, idx, nd, ins, outs, uses, producer_of_next, done)
            elif op == "Add":
                a, b = self._val_or_const(ins[0]), self._val_or_const(ins[1])
                if int(np.prod(b.shape)) > int(np.prod(a.shape)):
                    a, b = b, a
                na, nb = int(np.prod(a.shape)), int(np.prod(b.shape))
                # add_f32 repeats its second operand modulo its length (src/backend/cpu/mod.rs:2699-2751):
                # that is an elementwise add or a broadcast along the last dimension, nothing else
                if nb != na and not (len(a.shape) >= 1 and a.shape[-1] == nb):
                    raise FnnError(3, f"Add: broadcast of {b.shape} onto {a.shape} is not a last-dimension broadcast")
                out = self._new_value(outs[0], a.shape)
                self._emit("add_f32", ins, outs[0], [a.slot, b.slot], out.slot, [int(np.prod(a.shape))])
            elif op in _ACT_KERNEL:
                a = self._val(ins[0])
                out = self._new_value(outs[0], a.shape)
                self._emit(_ACT_KERNEL[op], ins, outs[0], [a.slot], out.slot, [int(np.prod(a.shape))])
            elif op in ("MaxPool", "AvgPool"):
                a = self._val(ins[0])
                k = _attr_int(nd, "kernel_size", "kernel_shape", default=2)
                s = _attr_int(nd, "stride", "strides", default=k)
                p = _attr_int(nd, "padding", "pads", default=0)
                n, c, h, w = a.shape
                ho, wo = max(h + 2 * p - k, 0) // s + 1, max(w + 2 * p - k, 0) // s + 1
                out = self._new_value(outs[0], (n, c, ho, wo))
                self._emit("pool_f32", ins, outs[0], [a.slot], out.slot, [k, s, p, 1 if op == "MaxPool" else 0, n, c, h, w])
            elif op == "Concat":
                rank = len(self._val(ins[0]).shape)
                axis = _attr_int(nd, "axis", default=0)
                axis = axis + rank if axis < 0 else axis
                axis = min(max(axis, 0), rank - 1)
                # consecutive parts that are, in order, ALL the copied parts of one Split along this axis: the Split's
                # source is read instead (the copies of parts that nothing else reads are then dropped)
                merged, i = [], 0
                while i < len(ins):
                    sp = self._split_of.get(ins[i])
                    if sp and sp[1] == axis and sp[2] == 0:
                        j, at = i, 0
                        while j < len(ins) and self._split_of.get(ins[j], (None,))[0] == sp[0] and self._split_of[ins[j]][1] == axis and \
                                self._split_of[ins[j]][2] == at:
                            at += self._split_of[ins[j]][3]
                            j += 1
                        if at == sp[4]:
                            merged.append(sp[0])
                            i = j
                            continue
                    merged.append(ins[i])
                    i += 1
                ins = merged
                vals = [self._val(i) for i in ins]
                shape = list(vals[0].shape)
                shape[axis] = sum(v.shape[axis] for v in vals)
                out = self._new_value(outs[0], shape)
                inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
                outer = int(np.prod(shape[:axis], dtype=np.int64))
                # parts that live at their place inside the result already (their producers stored them there) are
                # not copied; each run of the others is one concat into its stretch of the result
                run, run_at, off = [], 0, 0
                for name, v in list(zip(ins, vals)) + [(None, None)]:
                    at_home = v is not None and outer == 1 and v.slot == (out.slot[0] + off, v.nbytes)
                    if (v is None or at_home) and run:
                        size = sum(r.nbytes for _, r in run)
                        self._emit("concat", [n for n, _ in run], outs[0], [r.slot for _, r in run],
                                   out.slot if size == out.nbytes else (out.slot[0] + run_at, size), [axis, inner, outer])
                        run = []
                    if v is None:
                        break
                    if not at_home:
                        if not run:
                            run_at = off
                        run.append((name, v))
                    off += v.nbytes
            elif op == "Split":
                # one slice_f32 per output (src/onnx/converter.rs:549-612): explicit `split` sizes, else equal
                # parts with the remainder in the last one
                a = self._val(ins[0])
                rank = len(a.shape)
                axis = _attr_int(nd, "axis", default=0)
                axis = axis + rank if axis < 0 else axis
                axis = min(max(axis, 0), rank - 1)
                sizes = [int(v) for v in nd.get("split", "").split(",") if v.strip()]
                if not (len(sizes) == len(outs) and all(v > 0 for v in sizes)):
                    part = a.shape[axis] // max(len(outs), 1)
                    if part < 1:
                        raise FnnError(4, f"Split: {a.shape[axis]} values along axis {axis} into {len(outs)} outputs")
                    sizes = [part] * (len(outs) - 1) + [a.shape[axis] - part * (len(outs) - 1)]
                inner = int(np.prod(a.shape[axis + 1:], dtype=np.int64))
                outer = int(np.prod(a.shape[:axis], dtype=np.int64))
                start = 0
                for o, sz in zip(outs, sizes):
                    shape = list(a.shape)
                    shape[axis] = sz
                    byte0 = start * inner * 4
                    if outer == 1 and byte0 % 64 == 0:
                        # one outer block: the part is a contiguous, aligned range of the input's slot; values are
                        # never overwritten (one slot per value), so it needs no copy
                        self._values[o] = _Value(shape, (a.slot[0] + byte0, sz * inner * 4), view_of=(ins[0], byte0))
                    else:
                        out = self._new_value(o, shape)
                        self._emit("slice_f32", ins, o, [a.slot], out.slot, [axis, start, start + sz, inner])
                        self._split_of[o] = (ins[0], axis, start, sz, a.shape[axis])
                    start += sz
            elif op == "Resize":
                a = self._val(ins[0])
                if nd.get("mode", "nearest") != "nearest":
                    raise FnnError(3, "Resize: only mode=nearest runs on this backend")
                sh, sw = _attr_int(nd, "scale_h", default=2), _attr_int(nd, "scale_w", default=2)
                n, c, h, w = a.shape
                out = self._new_value(outs[0], (n, c, h * sh, w * sw))
                self._emit("upsample_nearest2d", ins, outs[0], [a.slot], out.slot, [sh, sw, h, w])
            else:
                raise FnnError(3, op)
            done.add(idx)

    def _val(self, name: str) -> _Value:
        if name not in self._values:
            raise FnnError(4, f"AotExecutor: '{name}' is used before it is produced")
        return self._values[name]

    def _val_or_const(self, name: str) -> _Value:
        if name in self._values:
            return self._values[name]
        if name in self._params:
            arr = self._params[name]
            v = _Value(arr.shape, self._const_slot(arr))
            self._values[name] = v
            return v
        raise FnnError(4, f"AotExecutor: '{name}' is neither a value nor a parameter")

    def _single_consumer(self, nodes, name, uses, consumers, op_types):
        """The node that is the only consumer of `name`, when its op type is one of `op_types`."""
        if uses.get(name, 0) != 1 or name in self.output_names:
            return None
        idxs = consumers.get(name, [])
        if len(idxs) != 1 or nodes[idxs[0]].get("op_type") not in op_types:
            return None
        return idxs[0]

    def _fold_bias_act(self, nodes, out_name, n_cols, uses, consumers, done, has_bias):
        """MatMul/Conv -> Add(constant bias of n_cols) -> Relu|Gelu|Silu, each link only when the value has
        no other consumer.  Returns (bias array or None, activation op or None, final output name)."""
        bias = None
        act = None
        if not has_bias:
            j = self._single_consumer(nodes, out_name, uses, consumers, ("Add",))
            if j is not None:
                ai = _names(nodes[j].get("inputs"))
                other = ai[1] if ai[0] == out_name else ai[0]
                if other in self._params and self._params[other].size == n_cols:
                    bias = self._params[other].reshape(-1)
                    done.add(j)
                    out_name = _names(nodes[j].get("outputs"))[0]
        j = self._single_consumer(nodes, out_name, uses, consumers, tuple(_ACT_SUFFIX))
        if j is not None:
            act = nodes[j]["op_type"]
            done.add(j)
            out_name = _names(nodes[j].get("outputs"))[0]
        return bias, act, out_name

    def _lower_matmul(self, nodes, idx, nd, ins, outs, uses, consumers, done):
        a = self._val(ins[0])
        if ins[1] not in self._params:
            raise FnnError(3, f"{nd.get('op_type')}: the second operand must be a constant weight on this backend")
        w = self._params[ins[1]]
        if w.ndim != 2:
            raise FnnError(3, f"{nd.get('op_type')}: rank-{w.ndim} weight (the quantisation pass takes 2-D MatMul weights)")
        if nd.get("op_type") == "Gemm":
            alpha = float(nd.get("alpha", "1.0"))
            if abs(alpha - 1.0) > np.finfo(np.float32).eps:
                raise FnnError(3, "Gemm: alpha != 1 keeps the weight unquantised in the reference; not run here")
            trans_b = str(nd.get("transB", nd.get("trans_b", "0"))).lower() in ("1", "true")
            w_kn = w.T if trans_b else w
        else:
            w_kn = w
        k, n = w_kn.shape
        m = int(np.prod(a.shape[:-1], dtype=np.int64))
        if a.shape[-1] != k:
            raise FnnError(4, f"{nd.get('op_type')}: activation [..., {a.shape[-1]}] x weight [{k}, {n}]")
        pw = _l.quantize_weights_kn(self.weight_dtype, w_kn)
        bias = None
        if nd.get("op_type") == "Gemm" and len(ins) > 2:
            if ins[2] not in self._params or self._params[ins[2]].size != n:
                raise FnnError(3, "Gemm: the third operand must be a constant bias of N values")
            bias = self._params[ins[2]].reshape(-1)
        fbias, act, out_name = self._fold_bias_act(nodes, outs[0], n, uses, consumers, done, bias is not None)
        bias = bias if bias is not None else fbias
        w_slot = self._const_slot(pw.words)
        in_slots = [a.slot, w_slot]
        in_names = [ins[0], ins[1]]
        if bias is not None:
            in_slots.append(self._const_slot(np.ascontiguousarray(bias, np.float32)))
            in_names.append("bias")
        out = self._new_value(out_name, tuple(a.shape[:-1]) + (n,))
        kernel = KERNEL_OF[self.weight_dtype] + (_ACT_SUFFIX[act] if act else "")
        self._emit(kernel, in_names, out_name, in_slots, out.slot, [m, k, n], meta_of(pw))

    def _lower_conv(self, nodes, idx, nd, ins, outs, uses, consumers, done):
        a = self._val(ins[0])
        if ins[1] not in self._params:
            raise FnnError(3, "Conv: the weight must be a constant on this backend")
        w = self._params[ins[1]]
        if w.ndim != 4 or len(a.shape) != 4:
            raise FnnError(3, "Conv: only 2-D convolutions (NCHW input, [OC, IC/g, KH, KW] weight)")
        stride = _attr_int(nd, "stride", "strides", default=1)
        pad = _attr_int(nd, "padding", "pads", default=0)
        dil = _attr_int(nd, "dilation", "dilations", default=1)
        groups = _attr_int(nd, "group", default=1)
        oc, icg, kh, kw = w.shape
        n, c, h, wd = a.shape
        if groups < 1 or c != icg * groups or oc % groups:
            raise FnnError(4, f"Conv: input channels {c}, weight {w.shape}, group {groups}")
        pw = _l.quantize_weights(self.weight_dtype, w.reshape(oc, icg * kh * kw))
        bias = None
        if len(ins) > 2:
            if ins[2] not in self._params or self._params[ins[2]].size != oc:
                raise FnnError(3, "Conv: the bias must be a constant of OC values")
            bias = self._params[ins[2]].reshape(-1)
        _, act, out_name = self._fold_bias_act(nodes, outs[0], oc, uses, consumers, done, True)
        ho = (h + 2 * pad - (dil * (kh - 1) + 1)) // stride + 1
        wo = (wd + 2 * pad - (dil * (kw - 1) + 1)) // stride + 1
        if ho < 1 or wo < 1:
            raise FnnError(4, "Conv: kernel larger than the padded input")
        in_slots = [a.slot, self._const_slot(pw.words)]
        in_names = [ins[0], ins[1]]
        if bias is not None:
            in_slots.append(self._const_slot(np.ascontiguousarray(bias, np.float32)))
            in_names.append(ins[2])
        out = self._new_value(out_name, (n, oc, ho, wo))
        kernel = _CONV_KERNEL[self.weight_dtype] + (_ACT_SUFFIX[act] if act else "")
        self._emit(kernel, in_names, out_name, in_slots, out.slot, [stride, pad, dil, groups, c, h, wd, kh, kw],
                   meta_of(pw, [oc, icg, kh, kw]))

    # ---- execution
    @property
    def arena_size(self) -> int:
        return self._top

    def _ensure_plan(self):
        if self._plan is not None:
            return
        plan = ExecutablePlan(self._top)
        for off, arr in self._consts:
            plan.write_const(off, arr)
        for kernel, in_slots, out_slot, params, meta in self._calls:
            plan.call_kernel(kernel, in_slots, out_slot, params, meta)
        self._backend = HipBackend(self.device)
        self._backend.allocate_arena(self._top)
        self._plan = plan

    def forward(self, inputs: Dict[str, np.ndarray]) -> Dict[str, np.ndarray]:
        self._ensure_plan()
        for name in self.input_names:
            if name not in inputs:
                raise FnnError(1, f"forward: missing input '{name}'")
            v = self._values[name]
            x = np.ascontiguousarray(inputs[name], dtype=np.float32)
            if x.shape != v.shape:
                raise FnnError(1, f"forward: input '{name}' has shape {x.shape}, compiled for {v.shape}")
            self._backend.write_arena(v.slot[0], x)
        self._backend.dispatch(self._plan)
        out = {}
        for name in self.output_names:
            v = self._values[name]
            out[name] = self._backend.read_arena(*v.slot, np.float32).reshape(v.shape).copy()
        return out

    def set_option(self, option: int, value: int):
        """Kernel-selection option of the backend's context (lib.OPT_* constants)."""
        self._ensure_plan()
        self._backend.set_option(option, value)

    def set_graph_replay(self, enabled: bool):
        """Resident plan as one HIP-graph replay (default) or instruction by instruction."""
        self._ensure_plan()
        self._backend.set_graph_replay(enabled)

    def write_inputs(self, inputs: Dict[str, np.ndarray]):
        """Copies the inputs into their arena slots (what forward() does first)."""
        self._ensure_plan()
        for name in self.input_names:
            v = self._values[name]
            x = np.ascontiguousarray(inputs[name], dtype=np.float32)
            if x.shape != v.shape:
                raise FnnError(1, f"input '{name}' has shape {x.shape}, compiled for {v.shape}")
            self._backend.write_arena(v.slot[0], x)

    def dispatch(self):
        """Runs the plan on whatever the input slots hold (inputs resident on the device) and synchronises."""
        self._ensure_plan()
        self._backend.dispatch(self._plan)

    def read_output(self, name: str) -> np.ndarray:
        """A graph output, or any other value the plan computes (every value keeps its slot)."""
        if name in self._dropped:
            raise FnnError(4, f"AotExecutor: '{name}' is not computed: nothing reads it; name it in output_names to keep it")
        v = self._values[name]
        return self._backend.read_arena(*v.slot, np.float32).reshape(v.shape).copy()

    @property
    def replayed(self) -> bool:
        return bool(self._plan is not None and self._plan.replayed)

    @property
    def ranges_used(self) -> int:
        """Conv instructions of the plan that took their activation ranges from the instruction before them."""
        return 0 if self._plan is None else self._plan.ranges_used

    @property
    def residuals_fused(self) -> int:
        """Add instructions of the plan whose sum the MatMul before them stored."""
        return 0 if self._plan is None else self._plan.residuals_fused

    def close(self):
        if self._plan is not None:
            self._plan.close()
            self._plan = None
        if self._backend is not None:
            self._backend.close()
            self._backend = None
