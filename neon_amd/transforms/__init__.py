"""Activation functions, cost functions and metrics: callers of the op-tree
path (each returns an op-tree, or assigns a few into small buffers)."""
from neon_amd.transforms.activation import (Explin, Identity, Logistic, Normalizer,  # noqa: F401
                                            PixelwiseSoftmax, Rectlin, Rectlinclip, Sign, Softmax, Tanh)
from neon_amd.transforms.cost import (Accuracy, Cost, CrossEntropyBinary, CrossEntropyMulti,  # noqa: F401
                                      GANCost, LogLoss, MeanSquared, Metric, Misclassification, MultiMetric,
                                      PrecisionRecall, SmoothL1Loss, SquareHingeLoss, SumSquared,
                                      TopKMisclassification)
from neon_amd.transforms.transform import Transform  # noqa: F401
