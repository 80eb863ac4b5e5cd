"""Turns a planned graph into the sources of a model library.

Counterpart of python/aitemplate/backend/codegen.py:69-135,330-1246 and
backend/main_templates.py:21-403.  Emitted files, all host C++:

  <func>.cpp            one per distinct op function ("rocm.<op>.gen_function")
  model-generated.cpp   class Model : ait::ModelBase  - tensor / dim members, parameter table
                        with dim ranges, one OpEntry per op (the func_call strings), constant
                        binding, alias handling - plus the graph's static description and the
                        factory the prebuilt runtime calls
  constants.bin         bytes of the bound constants (only when there are any)
"""
from __future__ import annotations

import os
from typing import Dict, List, Tuple

from ..compiler.base import IntImm, Tensor
from ..compiler.dtype import dtype_to_enumerator, get_dtype_size
from ..compiler.transform.mark_param_tensor import storage_offset_bytes, storage_root
from ..compiler.transform.transform_utils import get_sorted_ops, is_view_op
from . import registry
from .target import Target


def gen_function_src(sorted_graph: List[Tensor], workdir: str, model_name: str = "") -> List[Tuple[str, str]]:
    """Write one source per distinct op function; returns [(source, object)] pairs."""
    target = Target.current()
    prefix = os.path.join(workdir, model_name)
    os.makedirs(prefix, exist_ok=True)
    pairs, seen = [], set()
    for op in get_sorted_ops(sorted_graph):
        if is_view_op(op):
            continue
        name = op._attrs["name"]
        if name in seen:
            continue
        seen.add(name)
        src = os.path.join(prefix, name + target.src_extension())
        with open(src, "w") as f:
            f.write(op.gen_function())
        pairs.append((src, os.path.join(prefix, name + ".o")))
    return pairs


def _dims_of(t: Tensor):
    return t._attrs["shape"]


def _numel_expr(t: Tensor) -> str:
    return " * ".join(d._attrs["name"] for d in _dims_of(t)) or "1"


def _shape_literal(values) -> str:
    return "{" + ", ".join(str(v) for v in values) + "}"


class ModelSource:
    """Collects the pieces of model-generated.cpp while walking the graph."""

    def __init__(self, sorted_graph: List[Tensor], output_tensors: List[Tensor], blob_size: int, workspace_size: int):
        self.graph = sorted_graph
        self.blob_size = blob_size
        self.workspace_size = workspace_size
        self.inputs = [t for t in sorted_graph if t._attrs["is_input"]]
        self.outputs = list(output_tensors)
        self.constants = [t for t in sorted_graph
                          if not t.src_ops() and not t._attrs["is_input"] and not t.is_a_const_num()]
        self.bound = [t for t in self.constants if t._attrs["data"] is not None]
        self.unbound = [t for t in self.constants if t._attrs["data"] is None]
        # parameter table order: inputs, outputs, unbound constants
        self.param_index: Dict[int, int] = {}
        for i, t in enumerate(self.inputs + self.outputs + self.unbound):
            self.param_index.setdefault(id(t), i)
        self.constant_offsets: Dict[int, int] = {}
        off = 0
        for t in self.bound:
            self.constant_offsets[id(t)] = off
            size = len(t._attrs["data"])
            off += (size + 63) // 64 * 64
        self.constants_size = off

    # ---- pieces ---------------------------------------------------------------
    def members(self) -> str:
        lines, seen_dims = [], set()
        for t in self.graph:
            if t.is_a_const_num():
                continue
            lines.append(f"  void* {t._attrs['name']} {{nullptr}};")
            for d in _dims_of(t):
                n = d._attrs["name"]
                if n in seen_dims:
                    continue
                seen_dims.add(n)
                init = d.value() if isinstance(d, IntImm) else d.upper_bound()
                lines.append(f"  int64_t {n} {{{init}}};")
        # dims of views that a split / concatenate fusion left only in an op's accessor
        for op in get_sorted_ops(self.graph):
            for acc in (op._attrs.get("input_accessors") or []) + (op._attrs.get("output_accessors") or []):
                for d in acc.original_shapes:
                    n = d._attrs["name"]
                    if n in seen_dims:
                        continue
                    seen_dims.add(n)
                    init = d.value() if isinstance(d, IntImm) else d.upper_bound()
                    lines.append(f"  int64_t {n} {{{init}}};")
        return "\n".join(lines)

    def param_table(self) -> str:
        lines = []
        for t in self.inputs + self.outputs + self.unbound:
            idx = self.param_index[id(t)]
            dims = ", ".join(f"ParamDim({d.lower_bound()}, {d.upper_bound()}, &{d._attrs['name']})" for d in _dims_of(t))
            lines.append(f'    params_[{idx}].name = "{t._attrs["name"]}";')
            lines.append(f"    params_[{idx}].shape_ptrs = {{{dims}}};")
        return "\n".join(lines)

    def internal_bindings(self) -> str:
        lines = []
        for t in self.graph:
            if t._attrs["offset"] is not None:
                lines.append(f"    {t._attrs['name']} = blob_ + {t._attrs['offset']};")
        for t in self.unbound:
            lines.append(f'    constant_name_to_ptr_["{t._attrs["name"]}"] = '
                         f"const_cast<const void**>(reinterpret_cast<void**>(&{t._attrs['name']}));")
        return "\n".join(lines)

    def bound_constant_bindings(self) -> str:
        return "\n".join(f"    {t._attrs['name']} = base + {self.constant_offsets[id(t)]};" for t in self.bound)

    def op_entries(self) -> str:
        target = Target.current()
        lines = []
        for op in get_sorted_ops(self.graph):
            if is_view_op(op):
                continue
            call = registry.get(f"{target.name()}.{op._attrs['op']}.func_call")(op._attrs, indent="      ")
            shown = op._attrs.get("original_name") or op._attrs["name"]
            lines.append(f'    ops_.push_back(OpEntry{{"{shown}", [this](StreamType stream) {{\n{call}\n    }}}});')
        return "\n".join(lines)

    def func_decls(self) -> str:
        target = Target.current()
        seen, lines = set(), []
        for op in get_sorted_ops(self.graph):
            if is_view_op(op) or op._attrs["name"] in seen:
                continue
            seen.add(op._attrs["name"])
            lines.append(registry.get(f"{target.name()}.{op._attrs['op']}.func_decl")(op._attrs))
        return "\n".join(lines)

    def setup_inputs_outputs(self) -> Tuple[str, str]:
        """(SetUpInputsOutputs body, DeviceToDeviceCopies body).

        Tensors that own their memory are bound first (inputs and owning outputs from the
        parameter table; planned buffers and constants were bound in the constructor), then
        every other tensor takes its owner's pointer; outputs that do not own their memory
        are filled by a device-to-device copy after the ops ran."""
        not_set = "was not set! Set the value with set_constant."
        lines, copies = [], []
        for t in self.inputs:
            idx, n = self.param_index[id(t)], t._attrs["name"]
            lines.append(f"    {n} = params_[{idx}].ptr;")
            lines.append(f'    if ({n} == nullptr && ({_numel_expr(t)}) != 0) throw std::runtime_error("Constant {n} {not_set}");')
        for t in self.unbound:
            n = t._attrs["name"]
            lines.append(f'    if ({n} == nullptr) throw std::runtime_error("Constant {n} {not_set}");')
        for t in self.outputs:
            idx, n = self.param_index[id(t)], t._attrs["name"]
            owner = t._attrs["external_tensor"]
            if owner is None:
                lines.append(f"    {n} = params_[{idx}].ptr;")
                lines.append(f'    if ({n} == nullptr && ({_numel_expr(t)}) != 0) throw std::runtime_error("Constant {n} {not_set}");')
            else:
                nbytes = f"({_numel_expr(t)}) * {get_dtype_size(t.dtype())}"
                copies.append(
                    f"    if (params_[{idx}].ptr != nullptr && params_[{idx}].ptr != {n})\n"
                    f"      AIT_DEVICE_CHECK(hipMemcpyAsync(params_[{idx}].ptr, {n}, {nbytes}, "
                    f"hipMemcpyDeviceToDevice, stream));")
        for t in self.graph:
            owner = t._attrs["external_tensor"]
            if owner is not None and not t.is_a_const_num():
                rel = storage_offset_bytes(t) - storage_offset_bytes(owner)
                if rel == 0:
                    lines.append(f"    {t._attrs['name']} = {owner._attrs['name']};")
                else:  # a piece of a split: same buffer, shifted
                    lines.append(f"    {t._attrs['name']} = static_cast<uint8_t*>({owner._attrs['name']}) + ({rel});")
        return "\n".join(lines), "\n".join(copies)

    def meta(self) -> str:
        def tensor_meta(t):
            shape = _shape_literal(d.upper_bound() for d in _dims_of(t))
            return f'{{"{t._attrs["name"]}", {dtype_to_enumerator(t.dtype())}, {shape}}}'

        ins = ",\n      ".join(tensor_meta(t) for t in self.inputs)
        outs = ",\n      ".join(tensor_meta(t) for t in self.outputs)
        consts = []
        for t in self.unbound + self.bound:
            bound = t._attrs["data"] is not None
            shape = _shape_literal(d.upper_bound() for d in _dims_of(t))
            orig = t._attrs.get("original_name") or t._attrs["name"]
            off = self.constant_offsets.get(id(t), 0)
            consts.append(f'{{"{t._attrs["name"]}", "{orig}", {dtype_to_enumerator(t.dtype())}, {shape}, '
                          f'{"true" if bound else "false"}, {off}, {t.size_bytes(alignment=1)}}}')
        return ins, outs, ",\n      ".join(consts)

    def render(self) -> str:
        setup, copies = self.setup_inputs_outputs()
        ins, outs, consts = self.meta()
        has_blob = self.constants_size > 0
        blob_decl = ("extern \"C\" const uint8_t _binary_constants_bin_start[];\n"
                     "extern \"C\" const uint8_t _binary_constants_bin_end[];\n") if has_blob else ""
        blob_begin = "_binary_constants_bin_start" if has_blob else "nullptr"
        blob_end = "_binary_constants_bin_end" if has_blob else "nullptr"
        n_in, n_out, n_unbound = len(self.inputs), len(self.outputs), len(self.unbound)
        return f"""// generated by aitemplate_amd - do not edit
#include <stdexcept>

#include "model_base.h"

{blob_decl}
namespace ait {{

{self.func_decls()}

namespace {{

class Model : public ModelBase {{
 public:
  Model(uint8_t* constants, AITemplateAllocator& allocator)
      : ModelBase({self.blob_size}, {self.workspace_size}, {n_in}, {n_out}, {n_unbound}, constants, allocator) {{
{self.param_table()}
{self.internal_bindings()}
    BindBoundConstants(constants);
{self.op_entries()}
  }}

 protected:
  void SetUpInputsOutputs() override {{
{setup}
  }}

  void BindBoundConstants(uint8_t* base) override {{
    (void)base;
{self.bound_constant_bindings()}
  }}

  void DeviceToDeviceCopies(StreamType stream) override {{
    (void)stream;
{copies}
  }}

 private:
{self.members()}
}};

}}  // namespace
}}  // namespace ait

extern "C" const ait::ModelMeta* aitamd_model_meta() {{
  static const ait::ModelMeta meta = [] {{
    ait::ModelMeta m;
    m.inputs = {{
      {ins}
    }};
    m.outputs = {{
      {outs}
    }};
    m.constants = {{
      {consts}
    }};
    m.blob_size = {self.blob_size};
    m.workspace_size = {self.workspace_size};
    m.constants_size = {self.constants_size};
    m.constants_begin = {blob_begin};
    m.constants_end = {blob_end};
    return m;
  }}();
  return &meta;
}}

extern "C" ait::ModelBase* aitamd_model_create(uint8_t* constants, AITemplateAllocator* allocator) {{
  return new ait::Model(constants, *allocator);
}}
"""

    def constants_bytes(self) -> bytes:
        buf = bytearray(self.constants_size)
        for t in self.bound:
            off = self.constant_offsets[id(t)]
            raw = t._attrs["data"].to_bytes()
            buf[off:off + len(raw)] = raw
        return bytes(buf)


def gen_library_src(sorted_graph: List[Tensor], blob_size: int, workspace_size: int, workdir: str,
                    output_tensors: List[Tensor], model_name: str = "") -> List[Tuple[str, str]]:
    """Write model-generated.cpp (and constants.bin); returns [(source, object)] pairs."""
    prefix = os.path.join(workdir, model_name)
    os.makedirs(prefix, exist_ok=True)
    ms = ModelSource(sorted_graph, output_tensors, blob_size, workspace_size)
    src = os.path.join(prefix, "model-generated.cpp")
    with open(src, "w") as f:
        f.write(ms.render())
    pairs = [(src, os.path.join(prefix, "model-generated.o"))]
    if ms.constants_size > 0:
        bin_path = os.path.join(prefix, "constants.bin")
        with open(bin_path, "wb") as f:
            f.write(ms.constants_bytes())
        pairs.append((bin_path, os.path.join(prefix, "constants.o")))
    return pairs
