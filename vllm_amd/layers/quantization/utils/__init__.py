import torch


def replace_parameter(mod: torch.nn.Module, name: str, new: torch.Tensor | torch.nn.Parameter) -> None:
    """Replace ``mod.<name>`` by a plain non-trainable Parameter holding ``new``
    (reference: vllm/model_executor/layers/quantization/utils/layer_utils.py)."""
    if not isinstance(new, torch.nn.Parameter):
        new = torch.nn.Parameter(new, requires_grad=False)
    if name in mod._parameters:
        del mod._parameters[name]
    elif hasattr(mod, name):
        delattr(mod, name)
    mod.register_parameter(name, torch.nn.Parameter(new.data, requires_grad=False))
