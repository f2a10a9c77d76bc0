"""``utils.rec_update_fwm_tanh``: the reference's module of this name (language_modeling/src/utils/rec_update_fwm_tanh/__init__.py), served by the
MI355X implementation: Recurrent Delta Net update with tanh feedback.  Imported as ``from utils.rec_update_fwm_tanh import rec_update_fwm_tanh``
(language_modeling/src/utils/cuda_fast_weight_layer.py:9-23)."""
from _fwp_dropin import package as _package

FastWeightRecUpdateTanh = _package().FastWeightRecUpdateTanh
rec_update_fwm_tanh = _package().rec_update_fwm_tanh

__all__ = ["FastWeightRecUpdateTanh", "rec_update_fwm_tanh"]
