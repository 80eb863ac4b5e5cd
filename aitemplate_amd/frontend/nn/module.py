"""nn.Module: attribute-tree container with name_parameter_tensor()
(counterpart of python/aitemplate/frontend/nn/module.py, reduced to parameter naming and call)."""
from typing import Iterator, Tuple

from .parameter import Parameter


class Module:
    def __call__(self, *args, **kwargs):
        return self.forward(*args, **kwargs)

    def forward(self, *args, **kwargs):
        raise NotImplementedError

    def named_children(self) -> Iterator[Tuple[str, "Module"]]:
        for k, v in vars(self).items():
            if isinstance(v, Module):
                yield k, v

    def named_parameters(self, prefix: str = "") -> Iterator[Tuple[str, Parameter]]:
        for k, v in vars(self).items():
            full = f"{prefix}.{k}" if prefix else k
            if isinstance(v, Parameter):
                yield full, v
            elif isinstance(v, Module):
                yield from v.named_parameters(full)

    def name_parameter_tensor(self, prefix: str = "") -> None:
        """Name every parameter tensor after its attribute path, with '.' replaced by '_'."""
        for name, p in self.named_parameters(prefix):
            p.tensor()._attrs["name"] = name.replace(".", "_")
