"""``rec_update_fwm_tanh``: the reference's module of this name (algorithmic/rec_update_fwm_tanh/__init__.py), served by the
MI355X implementation: Recurrent Delta Net update with tanh feedback.  Imported as ``from rec_update_fwm_tanh import rec_update_fwm_tanh``
(algorithmic/layers.py:7-10)."""
from _fwp_dropin import package as _package

FastWeightRecUpdateTanh = _package().FastWeightRecUpdateTanh
rec_update_fwm_tanh = _package().rec_update_fwm_tanh

__all__ = ["FastWeightRecUpdateTanh", "rec_update_fwm_tanh"]
