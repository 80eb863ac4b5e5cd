"""Fold chains of element-wise ops behind a GEMM into the fused GEMM ops.

Counterpart of python/aitemplate/compiler/transform/fuse_mm_elementwise.py:31-215 with the pattern table of
fuse_mm_elementwise_patterns.py:46-200 (the bmm alpha fold is left out: the kernels take no alpha).  Matching is by chain: starting at a gemm_rcr / gemm_rcr_bias output, follow
tensors that have exactly one consumer, an element-wise op, and are not graph outputs; the longest prefix of
the chain that is a row of the table is replaced.  Binary steps (ADD, MUL) take the other operand as the
fused op's residual, and the replacement's own `is_valid_inputs` decides whether it fits (the residual must
have the GEMM's shape; gemm_rcr + ADD needs a 1-D bias of size N).  Swish, x * sigmoid(x), is matched
separately because x has two consumers there."""
from typing import List, Optional, Tuple

from .. import ops
from ..base import Operator, Tensor
from ..ops.common.epilogue import FuncEnum
from .toposort import toposort

_F = FuncEnum
_UNARY = {_F.RELU, _F.SIGMOID, _F.TANH, _F.GELU, _F.FASTGELU}
_BINARY = {_F.ADD, _F.MUL}

# (first op, element-wise chain) -> fused op, as in the reference's table
PATTERNS = {
    ("bmm_ccr", (_F.ADD,)): "bmm_ccr_add",
    ("bmm_crr", (_F.ADD,)): "bmm_crr_add",
    ("bmm_rrr", (_F.ADD,)): "bmm_rrr_add",
    ("gemm_rcr", (_F.ADD,)): "gemm_rcr_bias",
    ("gemm_rcr_bias", (_F.RELU,)): "gemm_rcr_bias_relu",
    ("gemm_rcr_bias", (_F.SIGMOID, _F.MUL, _F.TANH)): "gemm_rcr_bias_sigmoid_mul_tanh",
    ("gemm_rcr_bias", (_F.SIGMOID, _F.MUL)): "gemm_rcr_bias_sigmoid_mul",
    ("gemm_rcr_bias", (_F.SIGMOID,)): "gemm_rcr_bias_sigmoid",
    ("gemm_rcr_bias", (_F.TANH,)): "gemm_rcr_bias_tanh",
    ("gemm_rcr_bias", (_F.GELU,)): "gemm_rcr_bias_gelu",
    ("gemm_rcr_bias", (_F.FASTGELU,)): "gemm_rcr_bias_fast_gelu",
    ("gemm_rcr_bias", (_F.ADD, _F.RELU)): "gemm_rcr_bias_add_relu",
    ("gemm_rcr_bias", (_F.ADD, _F.ADD, _F.RELU)): "gemm_rcr_bias_add_add_relu",
    ("gemm_rcr_bias", (_F.ADD, _F.ADD)): "gemm_rcr_bias_add_add",
    ("gemm_rcr_bias", (_F.ADD,)): "gemm_rcr_bias_add",
    ("gemm_rcr_bias", (_F.MUL, _F.ADD)): "gemm_rcr_bias_mul_add",
    ("gemm_rcr_bias", (_F.MUL, _F.TANH)): "gemm_rcr_bias_mul_tanh",
    ("gemm_rcr_bias", (_F.MUL,)): "gemm_rcr_bias_mul",
}
_MAX_CHAIN = max(len(k[1]) for k in PATTERNS)
_START_OPS = {k[0] for k in PATTERNS}


def _only_consumer(t: Tensor) -> Optional[Operator]:
    consumers = list(t.dst_ops())
    if t._attrs["is_output"] or len(consumers) != 1:
        return None
    return consumers[0]


def _chain_from(t: Tensor) -> List[Tuple[Operator, Optional[Tensor]]]:
    """[(element-wise op, its other operand or None)] following `t` while the chain stays linear."""
    chain = []
    while len(chain) < _MAX_CHAIN:
        op = _only_consumer(t)
        if op is None or op._attrs["op"] != "elementwise":
            break
        func, args = op._attrs["func"], op._attrs["args"]
        if func in _UNARY and len(args) == 1:
            other = None
        elif func in _BINARY and len(args) == 2 and sum(a is t for a in args) == 1:
            other = args[0] if args[1] is t else args[1]
            if other.is_a_const_num():
                break
        else:
            break
        chain.append((op, other))
        t = op._attrs["outputs"][0]
    return chain


def _detach(op: Operator) -> None:
    for inp in op._attrs["inputs"]:
        inp._attrs["dst_ops"].discard(op)


def _take_over(old: Tensor, new: Tensor, outputs: List[Tensor]) -> None:
    """`new` replaces `old` for every consumer and as a graph output."""
    for consumer in list(old.dst_ops()):
        consumer.replace_input_tensor(old, new)
        new._attrs["dst_ops"].add(consumer)
    for key in ("name", "is_output", "check_nan_and_inf", "check_outputs", "original_name"):
        new._attrs[key] = old._attrs[key]
    for i, t in enumerate(outputs):
        if t is old:
            outputs[i] = new


def _fuse_chain(gemm: Operator, outputs: List[Tensor]) -> bool:
    start = gemm._attrs["op"]
    chain = _chain_from(gemm._attrs["outputs"][0])
    for length in range(len(chain), 0, -1):
        fused_name = PATTERNS.get((start, tuple(op._attrs["func"] for op, _ in chain[:length])))
        if fused_name is None:
            continue
        extra = [other for _, other in chain[:length] if other is not None]
        inputs = list(gemm._attrs["inputs"]) + extra
        fused_cls = getattr(ops, fused_name)
        ok, _ = fused_cls.is_valid_inputs(*inputs)
        if not ok:
            continue
        last = chain[length - 1][0]._attrs["outputs"][0]
        if list(last._attrs["shape"]) != list(gemm._attrs["outputs"][0]._attrs["shape"]):
            continue  # a broadcast changed the shape: not an epilogue
        _detach(gemm)
        for op, _ in chain[:length]:
            _detach(op)
        new = fused_cls()(*inputs)
        _take_over(last, new, outputs)
        return True
    return False


def _fuse_swish(gemm: Operator, outputs: List[Tensor]) -> bool:
    """gemm_rcr_bias -> x; x * sigmoid(x)  ==>  gemm_rcr_bias_swish (reference: fuse_mm_elementwise.py:113-178)."""
    if gemm._attrs["op"] != "gemm_rcr_bias":
        return False
    x = gemm._attrs["outputs"][0]
    consumers = list(x.dst_ops())
    if x._attrs["is_output"] or len(consumers) != 2:
        return False
    for sig, mul in (consumers, consumers[::-1]):
        if not (sig._attrs["op"] == "elementwise" and sig._attrs["func"] == _F.SIGMOID
                and mul._attrs["op"] == "elementwise" and mul._attrs["func"] == _F.MUL):
            continue
        s = sig._attrs["outputs"][0]
        args = mul._attrs["args"]
        if len(args) != 2 or not ((args[0] is x and args[1] is s) or (args[0] is s and args[1] is x)):
            continue
        if _only_consumer(s) is not mul:
            continue
        _detach(gemm)
        _detach(sig)
        _detach(mul)
        new = ops.gemm_rcr_bias_swish()(*gemm._attrs["inputs"])
        _take_over(mul._attrs["outputs"][0], new, outputs)
        return True
    return False


def fuse_mm_elementwise(sorted_graph: List[Tensor], output_tensors: List[Tensor]) -> List[Tensor]:
    """Returns the re-sorted graph; `output_tensors` is updated in place where an output was replaced."""
    changed = True
    while changed:
        changed = False
        for t in sorted_graph:
            for op in list(t.src_ops()):
                if op._attrs["op"] in _START_OPS and op._attrs["outputs"][0] is t:
                    if _fuse_chain(op, output_tensors) or _fuse_swish(op, output_tensors):
                        changed = True
                        break
            if changed:
                break
        if changed:
            sorted_graph = toposort(output_tensors)
    return sorted_graph


def check_leftover_elementwise(sorted_graph: List[Tensor]) -> None:
    """Element-wise ops that no epilogue absorbed run as stand-alone launches; raise for those the stand-alone
    kernel cannot take, naming the tensor."""
    for t in sorted_graph:
        for op in t.src_ops():
            if op._attrs["op"] == "elementwise":
                try:
                    op.standalone_plan()
                except NotImplementedError as e:
                    raise NotImplementedError(
                        f"{e}; the op producing {t._attrs['name'] or 'an unnamed tensor'} could not be fused into a "
                        "GEMM epilogue either") from None
