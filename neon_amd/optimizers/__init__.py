"""Parameter update rules: callers of the op-tree path (each update is a few
``tensor[:] = expr`` statements, fused by the hip backend into one kernel)."""
from neon_amd.optimizers.optimizer import (Adadelta, Adagrad, Adam, ExpSchedule,  # noqa: F401
                                           GradientDescentMomentum, MultiOptimizer, Optimizer,
                                           PolySchedule, PowerSchedule, RMSProp, Schedule,
                                           ShiftAdaMax, ShiftSchedule, StepSchedule, get_param_list)
