"""Binds the MoA attention path into a loaded model, like the reference's MoA/models/interface.py:3-28."""


def update_model_function(model, model_name):
    """Update the model function based on the model name: for Llama-family names
    (``llama``, ``Llama``, ``vicuna``, ``longchat``) binds ``set_mixture_of_attention`` (and the
    deprecated ``use_block_sparse_attention_lut``, which raises here) to ``model.model``; other names
    raise NotImplementedError, as in the reference.  Usage, as in the reference's scripts:

        model = update_model_function(model, model_name)
        model.model.set_mixture_of_attention(moa_config, permute_head=True)
    """
    if ("llama" in model_name) or ("Llama" in model_name) or ("vicuna" in model_name) or ("longchat" in model_name):
        print("Update functions from `modeling_llama` in `moa_amd`")
        from moa_amd.models.llama.modeling_llama import (LlamaModel_set_mixture_of_attention,
                                                         LlamaModel_use_block_sparse_attention_lut)

        model.model.use_block_sparse_attention_lut = LlamaModel_use_block_sparse_attention_lut.__get__(model.model)
        model.model.set_mixture_of_attention = LlamaModel_set_mixture_of_attention.__get__(model.model)
    else:
        raise NotImplementedError("Model {} not implemented".format(model_name))
    return model
