"""Puts the HIP-backed functions in place of the reference's Triton-backed ones.

The reference binds its kernels by module-level name: composites and tests do
``from model_triton import t_layernorm_fwd_t, ...`` and the trainer does
``from loss_and_optimizer_triton import t_acc_grad_loss3_t, init_adam_w, ...``
(train_gpt2_triton.py:56).  ``install`` therefore overwrites those attributes on the
reference's OWN, already imported modules -- every other name of those modules (the
torch.func side: loss_train, loss_eval, grad_loss, predict, log_probs, the Jacobian ladder)
stays the reference's -- and rebinds the names that ``loss_and_optimizer_triton`` copied out
of ``model_triton`` at import time.
"""
import importlib

# kernel wrappers and composites of model_triton.py that the HIP library replaces
MODEL_NAMES = (
    "t_log_softmax_fwd_t", "t_log_softmax_bkwd2_t", "t_gelu_fwd_t", "t_gelu_bkwd2_t", "t_matmul_t",
    "t_tlayer_ffn_fwd_t", "t_tlayer_ffn_bkwd2_t", "t_softmax_attn_fwd_t", "t_softmax_attn_bkwd2_t",
    "t_scaled_dot_prod_attn_fwd3_t", "t_scaled_dot_prod_attn_bkwd3_t",
    "t_dropout_fwd_t", "t_dropout_bkwd2_t", "t_layernorm_fwd_t", "t_layernorm_bkwd2_p_t", "t_layernorm_bkwd2_x_t",
    "t_gpt2_tlayer_fwd3_t", "t_gpt2_tlayer_bkwd3_t", "t_gpt2_tlayers_fwd3_t", "t_gpt2_forward_with_acts_t",
    "t_gpt2_bkwd3_p_t",
)
# loss / optimizer side of loss_and_optimizer_triton.py
LOSS_NAMES = (
    "t_avg_cross_entropy_loss_bkwd3_t", "t_loss_bkwd3_t", "t_acc_grad_loss3_t", "_acc_grad_loss", "sample_p_gen_aux",
    "init_adam_w", "adam_w_in_place", "grads_l2norm", "grads_grps_l2norms",
)


def install(ref_model_triton, ref_loss_and_optimizer_triton=None):
    """Overwrite the names above on the reference's modules.  Returns the list of
    (module name, attribute) pairs that were replaced."""
    mt = importlib.import_module(__package__ + ".model_triton")
    lo = importlib.import_module(__package__ + ".loss_and_optimizer_triton")
    done = []
    for name in MODEL_NAMES:
        setattr(ref_model_triton, name, getattr(mt, name))
        done.append((ref_model_triton.__name__, name))
    if ref_loss_and_optimizer_triton is not None:
        for name in LOSS_NAMES:
            setattr(ref_loss_and_optimizer_triton, name, getattr(lo, name))
            done.append((ref_loss_and_optimizer_triton.__name__, name))
        # names the loss module imported from model_triton by value
        for name in MODEL_NAMES:
            if hasattr(ref_loss_and_optimizer_triton, name):
                setattr(ref_loss_and_optimizer_triton, name, getattr(mt, name))
                done.append((ref_loss_and_optimizer_triton.__name__, name))
    return done
