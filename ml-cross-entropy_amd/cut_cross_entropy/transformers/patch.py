"""``cce_patch``: make a Hugging Face causal LM compute its loss with ``linear_cross_entropy``.

Same entry point, arguments and error behaviour as ref: transformers/patch.py:53-95.  The reference
carries one rewritten ``forward`` per model family (ref: transformers/llama.py:26-131, gemma2.py,
mistral.py, phi3.py, qwen2.py) because the library's forwards differed; in the installed library every
supported family has the same three steps -- ``self.model(...)``, ``self.lm_head``, ``self.loss_function``
-- so one forward serves them all.  With labels (and not ``train_only`` in eval mode) the logits are
never formed: the hidden states and ``lm_head.weight`` go straight to the fused loss.
"""

import importlib
from types import MethodType
from typing import Optional, Union

import torch
import transformers
from transformers.modeling_outputs import CausalLMOutputWithPast

from cut_cross_entropy.cce_utils import LinearCrossEntropyImpl
from cut_cross_entropy.linear_cross_entropy import LCE_IMPL_DEFAULT
from cut_cross_entropy.transformers.utils import PatchOptions, apply_lce

# model_type -> (module, class) of the causal LM the patch applies to (ref: transformers/patch.py:15-21)
PATCH_TARGETS = {
    "llama": ("transformers.models.llama.modeling_llama", "LlamaForCausalLM"),
    "phi3": ("transformers.models.phi3.modeling_phi3", "Phi3ForCausalLM"),
    "gemma2": ("transformers.models.gemma2.modeling_gemma2", "Gemma2ForCausalLM"),
    "mistral": ("transformers.models.mistral.modeling_mistral", "MistralForCausalLM"),
    "qwen2": ("transformers.models.qwen2.modeling_qwen2", "Qwen2ForCausalLM"),
}

_OPTS_ATTR = "_cce_patch_options"


def cce_forward(
    self,
    input_ids: Optional[torch.LongTensor] = None,
    attention_mask: Optional[torch.Tensor] = None,
    position_ids: Optional[torch.LongTensor] = None,
    past_key_values=None,
    inputs_embeds: Optional[torch.FloatTensor] = None,
    labels: Optional[torch.LongTensor] = None,
    use_cache: Optional[bool] = None,
    logits_to_keep: Union[int, torch.Tensor] = 0,
    **kwargs,
) -> CausalLMOutputWithPast:
    """Causal-LM forward whose loss never materialises the logits (ref: transformers/llama.py:84-131)."""
    outputs = self.model(
        input_ids=input_ids,
        attention_mask=attention_mask,
        position_ids=position_ids,
        past_key_values=past_key_values,
        inputs_embeds=inputs_embeds,
        use_cache=use_cache,
        **kwargs,
    )
    hidden_states = outputs.last_hidden_state
    opts: Optional[PatchOptions] = getattr(self, _OPTS_ATTR, None)
    softcap = getattr(self.config, "final_logit_softcapping", None)

    loss = None
    logits = None
    if opts is not None and opts.use_lce(labels, self.training):
        loss = apply_lce(
            hidden_states,
            self.lm_head.weight,
            labels,
            opts,
            bias=getattr(self.lm_head, "bias", None),
            softcap=softcap,
            **kwargs,
        )
    else:
        slice_indices = slice(-logits_to_keep, None) if isinstance(logits_to_keep, int) else logits_to_keep
        logits = self.lm_head(hidden_states[:, slice_indices, :])
        if softcap is not None:
            logits = torch.tanh(logits / softcap) * softcap
        if labels is not None:
            loss = self.loss_function(logits=logits, labels=labels, vocab_size=self.config.vocab_size, **kwargs)

    return CausalLMOutputWithPast(
        loss=loss,
        logits=logits,
        past_key_values=outputs.past_key_values,
        hidden_states=outputs.hidden_states,
        attentions=outputs.attentions,
    )


def _target_class(model_type: str):
    module_name, class_name = PATCH_TARGETS[model_type]
    return getattr(importlib.import_module(module_name), class_name)


def _impl_name(impl) -> str:
    """Lower-case name of an implementation given as enum member or string; ValueError for an unknown one."""
    name = impl.name.lower() if isinstance(impl, LinearCrossEntropyImpl) else impl
    known = {member.name.lower() for member in LinearCrossEntropyImpl}
    if name not in known:
        raise ValueError(f"Unknown impl={name!r}")
    return name


def _model_type_of(target) -> str:
    """The ``model_type`` string of a model, a config, or the string itself; RuntimeError if no patch exists."""
    if isinstance(target, transformers.PreTrainedModel):
        target = target.config
    model_type = target.model_type if isinstance(target, transformers.PretrainedConfig) else target
    if model_type not in PATCH_TARGETS:
        raise RuntimeError(f"Unknown model type {model_type}")
    return model_type


def cce_patch(
    model_type_or_model,
    impl: Union[str, LinearCrossEntropyImpl] = LCE_IMPL_DEFAULT,
    reduction: str = "mean",
    filter_eps: Union[float, str, None] = "auto",
    accum_e_fp32: bool = False,
    accum_c_fp32: bool = False,
    filter_e_grad: bool = True,
    filter_c_grad: bool = True,
    train_only: bool = False,
):
    """Patch a model instance (returned), or a model family named by type string / config (returns None:
    every instance created afterwards is patched).  ref: transformers/patch.py:53-95.
    """
    target = model_type_or_model
    impl = _impl_name(impl)  # (an unknown impl is reported before an unknown model type, as in the reference)
    is_instance = isinstance(target, transformers.PreTrainedModel)
    cls = _target_class(_model_type_of(target))
    options = PatchOptions(impl=impl, reduction=reduction, filter_eps=filter_eps,
                           accum_e_fp32=accum_e_fp32, accum_c_fp32=accum_c_fp32,
                           filter_e_grad=filter_e_grad, filter_c_grad=filter_c_grad, train_only=train_only)
    if is_instance:
        # one model: its own bound forward and its own options; other instances of the class stay as they are
        assert isinstance(target, cls), f"Expected a {cls.__name__} model. Got {type(target)}."
        setattr(target, _OPTS_ATTR, options)
        target.forward = MethodType(cce_forward, target)
        return target
    setattr(cls, _OPTS_ATTR, options)
    cls.forward = cce_forward
    return None
