from .muon_math import (
    DEFAULT_NS_COEFFICIENTS,
    OwnedMuon,
    _adjust_muon_learning_rate,
    _apply_muon_update,
    _compute_muon_direction,
    _estimate_muon_compute_cost,
    _prepare_muon_input,
    _zeropower_via_newtonschulz,
)

__all__ = [
    "DEFAULT_NS_COEFFICIENTS",
    "OwnedMuon",
    "_adjust_muon_learning_rate",
    "_apply_muon_update",
    "_compute_muon_direction",
    "_estimate_muon_compute_cost",
    "_prepare_muon_input",
    "_zeropower_via_newtonschulz",
]
