"""Layers that are thin callers of the backend's tensor API (dense, bias,
activation, batch norm, dropout, embedding lookup, plain, LSTM and GRU recurrence), the
cost wrapper and the sequential container that chains them."""
from neon_amd.layers.layer import (Activation, Affine, BatchNorm, Bias, Dropout, GeneralizedCost,  # noqa: F401
                                   Layer, Linear, LookupTable, ParameterLayer, interpret_in_shape)
from neon_amd.layers.container import DeltasTree, Sequential  # noqa: F401
from neon_amd.layers.recurrent import (GRU, LSTM, Recurrent, RecurrentLast, RecurrentMean, RecurrentOutput,  # noqa: F401
                                       RecurrentSum, get_steps)
