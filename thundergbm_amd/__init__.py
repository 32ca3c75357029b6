"""MI355X-native histogram GBDT trainer behind ThunderGBM's C ABI and Python estimator names."""
from ._lib import LIB_PATH, load  # noqa: F401
from .estimator import TGBMClassifier, TGBMModel, TGBMRegressor  # noqa: F401
from .session import Session  # noqa: F401
