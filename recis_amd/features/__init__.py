from .feature import Feature  # noqa: F401
from .feature_engine import FeatureEngine  # noqa: F401
from .op import (Bucketize, FeatureCross, Hash, IDMultiHash, Mod, SelectField, SelectFields,  # noqa: F401
                 SequenceTruncate)
