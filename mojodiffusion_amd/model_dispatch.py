"""Per-model attention dispatchers with a `*_SDPA_SAGE` arm: the host mirror of the reference's
`comptime if <MODEL>_SDPA_FLASH:` switches, which is where a new attention backend plugs in.

  zimage_sdpa_product_fwd       serenitymojo/models/zimage/lora_block.mojo:99-123
  ideogram4_sdpa_product_fwd    serenitymojo/models/dit/ideogram4_dit.mojo:29-49
  ltx2_sdpa_product_fwd, _rect  serenitymojo/models/dit/ltx2_dit.mojo:80-130
  krea2_attention_sdpa          serenitymojo/models/dit/krea2_dit.mojo:707-732 (step 6 of krea2_attention)
  klein_sdpa_train_fwd          serenitymojo/models/klein/double_block.mojo:1445-1454 (`KLEIN_SDPA_FLASH`, F32 activations)

Same dtype flow as the reference arms: BF16 q/k/v go straight in; anything else is cast to BF16
at the op boundary and the result cast back to q's dtype; the returned tensor owns its memory.
There is no other backend behind these functions: with an arm switched off, or for a head dim the
library does not cover (64, 128 and, forward only, 256 are covered), they raise.
"""
import torch

from . import attention_sage as A
from .attention_sage import Error, PV_FP16

ZIMAGE_SDPA_SAGE = True
LTX2_SDPA_SAGE = True
KREA2_SDPA_SAGE = True
KLEIN_SDPA_SAGE = True
# Ideogram-4 attends with Dh = 256 (ideogram4_dit.mojo:39-40): forward only, as in the reference.
IDEOGRAM4_SDPA_SAGE = True


def _product_fwd(name, enabled, q, k, v, scale, variant, rect):
    if not enabled:
        raise Error("%s: the quantized-attention arm is switched off and this package has no other backend" % name)
    fwd_fn = A.sdpa_flash_train_fwd_rect if rect else A.sdpa_flash_train_fwd
    if q.dtype == torch.bfloat16 and k.dtype == torch.bfloat16 and v.dtype == torch.bfloat16:
        # (the reference clones because its O may be a view into a padded buffer; O here is
        # already an owning, unpadded tensor)
        return fwd_fn(q, k, v, scale, variant).o
    out = fwd_fn(q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16), scale, variant).o
    return out.to(q.dtype)


def zimage_sdpa_product_fwd(q, k, v, scale, variant=PV_FP16):
    """[B,S,H,Dh] q/k/v (BF16, or F32 from the norm / projection math) -> attention in q's dtype."""
    return _product_fwd("zimage_sdpa_product_fwd", ZIMAGE_SDPA_SAGE, q, k, v, scale, variant, False)


def ideogram4_sdpa_product_fwd(q, k, v, scale, variant=PV_FP16):
    return _product_fwd("ideogram4_sdpa_product_fwd", IDEOGRAM4_SDPA_SAGE, q, k, v, scale, variant, False)


def ltx2_sdpa_product_fwd(q, k, v, scale, variant=PV_FP16):
    return _product_fwd("ltx2_sdpa_product_fwd", LTX2_SDPA_SAGE, q, k, v, scale, variant, False)


def ltx2_sdpa_product_fwd_rect(q, k, v, scale, variant=PV_FP16):
    """q [B,SQ,H,DH], k/v [B,SKV,H,DH] (cross-attention of the video and audio streams)."""
    return _product_fwd("ltx2_sdpa_product_fwd_rect", LTX2_SDPA_SAGE, q, k, v, scale, variant, True)


def krea2_attention_sdpa(q_rot, k_full, v_full, real_len=None, mask=None, variant=PV_FP16):
    """Step 6 of krea2_attention: F32 [1,L,heads,Dh] q/k/v after RoPE and repeat_kv, scale
    1/sqrt(Dh), result F32.  Three paths as in the reference: real_len set -> flash with the
    trailing key positions [real_len, L) masked (needs L % 128 == 0, as there); an additive mask
    [1,heads,L,L] -> the masked call; neither -> plain."""
    if not KREA2_SDPA_SAGE:
        raise Error("krea2_attention_sdpa: the quantized-attention arm is switched off and this package has no other backend")
    scale = 1.0 / float(q_rot.shape[-1]) ** 0.5
    q_bf, k_bf, v_bf = (t.to(torch.bfloat16) for t in (q_rot, k_full, v_full))     # round-to-nearest-even
    if real_len is not None:
        out = A.sdpa_flash_fwd_padmask(q_bf, k_bf, v_bf, int(real_len), scale, variant).o
    elif mask is not None:
        out = A.sdpa_tiled(q_bf, k_bf, v_bf, mask.to(torch.bfloat16), scale, variant)
    else:
        out = A.sdpa_nomask_tiled(q_bf, k_bf, v_bf, scale, variant)
    return out.to(torch.float32)


def klein_sdpa_train_fwd(q, k, v, scale, variant=PV_FP16):
    """Klein blocks carry F32 activations: returns (attention in F32, the BF16 forward set —
    q, k, v, o and Stats — that the block keeps for sdpa_flash_backward_f32)."""
    if not KLEIN_SDPA_SAGE:
        raise Error("klein_sdpa_train_fwd: the quantized-attention arm is switched off and this package has no other backend")
    return A.sdpa_flash_train_fwd_f32(q, k, v, scale, variant)
