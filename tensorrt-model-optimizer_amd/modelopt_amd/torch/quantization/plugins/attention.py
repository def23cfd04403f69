"""KV-cache / attention-operand quantizers.

Follows the call site of the reference's HF plugin (plugins/huggingface.py:52-139): an attention
module gains ``q_bmm_quantizer``, ``k_bmm_quantizer`` and ``v_bmm_quantizer`` (disabled until a
config such as ``FP8_KV_CFG`` enables ``*[kv]_bmm_quantizer``) that are applied to the query, key
and value states ``[B, H, S, D]`` right before the attention product.  Any module class that
calls ``self._quantize_qkv(q, k, v)`` can be registered with :func:`register_attention_class`.
"""

import ast
import inspect
import textwrap

from torch import nn

from ..nn.modules.quant_module import QuantModule, QuantModuleRegistry
from ..nn.modules.tensor_quantizer import TensorQuantizer

__all__ = ["QuantAttentionMixin", "register_attention_class", "register_attention_for_kv_quant"]


class QuantAttentionMixin(QuantModule):
    """Adds the three BMM quantizers; the host attention calls ``_quantize_qkv``."""

    def _setup(self):
        for name in ("q_bmm_quantizer", "k_bmm_quantizer", "v_bmm_quantizer"):
            q = TensorQuantizer()
            q.disable()
            self.add_module(name, q)

    def _quantize_qkv(self, query, key, value):
        query = self.q_bmm_quantizer(query)
        key, value = TensorQuantizer.forward_pair(self.k_bmm_quantizer, key, self.v_bmm_quantizer, value)
        return query, key, value


def register_attention_class(attn_cls: type):
    """Make ``mtq.quantize`` attach BMM quantizers to instances of ``attn_cls``.  Until then the
    class-level ``_quantize_qkv`` of the attention implementation is expected to be an identity."""
    QuantModuleRegistry.register({attn_cls: attn_cls.__name__})(QuantAttentionMixin)


_HOLE = "_kvq_operand_"
_BASE = "_kvq_original_class_"
_WRAP = {
    "plain": f"self.{{q}}({_HOLE})",
    # quantise the key as [.., S, D] even where the product takes it as [.., D, S]
    "method_t": f"self.{{q}}({_HOLE}.transpose(-1, -2)).transpose(-1, -2)",
    "torch_t": f"torch.transpose(self.{{q}}(torch.transpose({_HOLE}, -1, -2)), -1, -2)",
}


def _wrapped(operand: ast.expr, quantizer: str, form: str) -> ast.expr:
    """``operand`` inside the quantizer call that ``form`` spells."""
    expr = ast.parse(_WRAP[form].format(q=quantizer), mode="eval").body
    for parent in ast.walk(expr):
        for field, value in ast.iter_fields(parent):
            if isinstance(value, ast.Name) and value.id == _HOLE:
                setattr(parent, field, operand)
            elif isinstance(value, list):
                value[:] = [operand if isinstance(v, ast.Name) and v.id == _HOLE else v for v in value]
    return expr


def register_attention_for_kv_quant(attention_cls: type) -> bool:
    """Derive, from the source of ``attention_cls``, a subclass whose attention products read
    their operands through ``q_bmm_quantizer`` / ``k_bmm_quantizer`` / ``v_bmm_quantizer``, and
    register it as the quantised form of ``attention_cls``.  Returns False (and registers
    nothing) when the source does not have one of the three shapes below.

    Same recognition rules and operand choice as the reference
    (plugins/attention.py:45-216), found in breadth-first order over the class's syntax tree:

    * two method calls named ``matmul`` / ``bmm`` / ``baddbmm``: the second one found is
      ``q x k^T`` (both operands quantised in ``[.., S, D]`` layout, i.e. around a transpose of
      the last two dims), the first is ``p x v`` (second operand quantised);
    * two ``@`` products: likewise, with only ``k`` taken through the transposes;
    * one ``scaled_dot_product_attention`` call: its first three positional arguments.

    The derived class is built by executing the rewritten method definitions in the namespace of
    the module that defines ``attention_cls``; only the methods that hold a rewritten product are
    redefined, everything else is inherited.
    """
    tree = ast.parse(textwrap.dedent(inspect.getsource(attention_cls)))
    cls_def = tree.body[0]
    assert isinstance(cls_def, ast.ClassDef), f"{attention_cls} has no class definition to read"

    def named_call(node, names):
        return (isinstance(node, ast.Call) and isinstance(node.func, ast.Attribute)
                and node.func.attr in names)

    order = list(ast.walk(cls_def))
    bmm = [n for n in order if named_call(n, ("matmul", "bmm", "baddbmm"))]
    sdpa = [n for n in order if named_call(n, ("scaled_dot_product_attention",))]
    at = [n for n in order if isinstance(n, ast.BinOp) and isinstance(n.op, ast.MatMult)]
    if len(bmm) != 2 and len(sdpa) != 1 and len(at) != 2:
        print(f"{attention_cls.__name__}: expected 2 matmul/bmm calls (found {len(bmm)}), 1 "
              f"scaled_dot_product_attention call (found {len(sdpa)}) or 2 @ products (found "
              f"{len(at)}); the KV cache quantizers were not attached")
        return False

    touched = []
    if len(bmm) == 2:
        pv, qk = bmm
        pv.args[1] = _wrapped(pv.args[1], "v_bmm_quantizer", "plain")
        qk.args[0] = _wrapped(qk.args[0], "q_bmm_quantizer", "method_t")
        qk.args[1] = _wrapped(qk.args[1], "k_bmm_quantizer", "method_t")
        touched += [pv, qk]
    if len(at) == 2:
        pv, qk = at
        qk.left = _wrapped(qk.left, "q_bmm_quantizer", "plain")
        qk.right = _wrapped(qk.right, "k_bmm_quantizer", "torch_t")
        pv.right = _wrapped(pv.right, "v_bmm_quantizer", "plain")
        touched += [pv, qk]
    if len(sdpa) == 1:
        for i, name in enumerate(("q_bmm_quantizer", "k_bmm_quantizer", "v_bmm_quantizer")):
            sdpa[0].args[i] = _wrapped(sdpa[0].args[i], name, "plain")
        touched += sdpa

    def holds(fn, node):
        return any(n is node for n in ast.walk(fn))

    methods = [m for m in cls_def.body if isinstance(m, (ast.FunctionDef, ast.AsyncFunctionDef))
               and any(holds(m, t) for t in touched)]
    for m in methods:                      # the method now lives one class further down
        for call in ast.walk(m):
            if (isinstance(call, ast.Call) and isinstance(call.func, ast.Name)
                    and call.func.id == "super" and not call.args):
                me = m.args.args[0].arg
                call.args = [ast.Attribute(value=ast.Name(id=me, ctx=ast.Load()), attr=_BASE, ctx=ast.Load()),
                             ast.Name(id=me, ctx=ast.Load())]
    cls_def.name = "_Quant" + attention_cls.__name__
    cls_def.bases, cls_def.keywords, cls_def.decorator_list = [ast.Name(id=_BASE, ctx=ast.Load())], [], []
    cls_def.body = methods or [ast.Pass()]
    code = compile(ast.fix_missing_locations(tree), f"<kv quantizers for {attention_cls.__qualname__}>", "exec")

    # the class statement finds its base in the local namespace; the methods keep the defining
    # module's globals, which stay untouched
    made = {_BASE: attention_cls}
    exec(code, vars(inspect.getmodule(attention_cls)), made)   # noqa: S102 - the user's own class source
    quant_cls = made[cls_def.name]
    setattr(quant_cls, _BASE, attention_cls)

    def _setup(self):
        self.q_bmm_quantizer = TensorQuantizer()
        self.k_bmm_quantizer = TensorQuantizer()
        self.v_bmm_quantizer = TensorQuantizer()

    assert "_setup" not in vars(quant_cls), "the attention class already defines _setup"
    quant_cls._setup = _setup
    QuantModuleRegistry.register({attention_cls: attention_cls.__name__})(quant_cls)
    return True
