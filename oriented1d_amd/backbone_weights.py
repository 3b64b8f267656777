"""Classification checkpoint -> dense-prediction backbone checkpoint.

Working counterpart of the reference's ``scripts/convert_to_backbone_weights.py:42-55`` (whose
``reshape_kernel`` is not defined anywhere): the backbone holds every oriented convolution in a
wrapper (``.weight`` -> ``.conv.weight``, likewise ``.bias`` and ``.theta``;
``semantic_segmentation/backbone/convnext.py:74-80``) and uses shorter kernels in the coarse
stages (``:316-327``), so ``[C,1,1,K]`` weights are cropped around their centre tap to the target's
kernel size.  Centre cropping keeps every remaining tap at its offset from the centre, i.e. the
cropped operator is the original one restricted to the inner taps.
"""
import torch


def centre_crop_kernel(weight, kernel_size):
    """``[C,1,1,K] -> [C,1,1,kernel_size]`` around the centre tap (both sizes odd, K >= kernel_size)."""
    K = weight.shape[-1]
    if kernel_size > K or (K - kernel_size) % 2:
        raise ValueError("cannot centre-crop a kernel of size %d to %d" % (K, kernel_size))
    lo = (K - kernel_size) // 2
    return weight[..., lo:lo + kernel_size].clone()


def convert_to_backbone_state_dict(state_dict, target_state_dict):
    """Renames the oriented-convolution entries of a classification ``state_dict`` to the
    backbone's wrapped names and crops their weights to the shapes in ``target_state_dict`` (the
    backbone model's own ``state_dict()``).  Entries the backbone does not have (the classifier
    head and its norm) are dropped; the backbone's per-stage output norms are not in the source
    and keep their initial values when the result is loaded with ``strict=False``."""
    out = {}
    for key, value in state_dict.items():
        new_key = key
        if "dw" in key:
            for leaf in (".weight", ".bias", ".theta"):
                if new_key.endswith(leaf):
                    new_key = new_key[:-len(leaf)] + ".conv" + leaf
        if new_key not in target_state_dict:
            continue
        target = target_state_dict[new_key]
        if "dw" in key and key.endswith(".weight") and value.dim() == 4 and value.shape[2] == 1 \
                and value.shape[-1] != target.shape[-1]:
            value = centre_crop_kernel(value, target.shape[-1])
        if tuple(value.shape) != tuple(target.shape):
            raise ValueError("%s: %s does not fit %s" % (new_key, tuple(value.shape),
                                                         tuple(target.shape)))
        out[new_key] = value.clone() if isinstance(value, torch.Tensor) else value
    return out
