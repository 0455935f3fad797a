"""
Backend factory (reference neon/backends/__init__.py:49-127).

Importing this package registers the ``hip`` backend; ``gen_backend('hip')``
(the ``-b hip`` choice) instantiates it and installs it as the process-wide
backend.
"""
import atexit
import logging

import numpy as np

from neon_amd import NervanaObject
from neon_amd.backends.backend import Backend, Block, OpTreeNode, OpCollection, Tensor  # noqa: F401
from neon_amd.backends import nervanahip
from neon_amd.backends.hip.bf16 import bfloat16  # noqa: F401  (storage dtype for be.empty / be.array)

# registers 'hip' in this package's own registry; a host package (neon) binds the
# backend to ITS classes instead -- see nervanahip.bind
NervanaHIP, HIPTensor = nervanahip.bind(Backend, OpTreeNode, Tensor, Block)

# this package's own API copy builds its elementwise nodes in C when the extension is there
# (a host package's API classes are its own business)
from neon_amd.backends import backend as _api                   # noqa: E402
from neon_amd.backends.hip import fastpath as _fastpath         # noqa: E402
if _fastpath.enabled():
    try:
        _api.use_c_node_builder(_fastpath.load())
    except ImportError:
        pass

_atexit_registered = False


def gen_backend(backend='hip', rng_seed=None, datatype=np.float32,
                batch_size=0, stochastic_round=False, device_id=0,
                max_devices=1, compat_mode=None,
                deterministic_update=None, deterministic=None):
    """Construct the named backend and make it the global one."""
    global _atexit_registered
    logger = logging.getLogger(__name__)
    if NervanaObject.be is not None:
        cleanup_backend()
    elif not _atexit_registered:
        atexit.register(cleanup_backend)
        _atexit_registered = True
    if deterministic_update is not None or deterministic is not None:
        logger.warning('deterministic_update and deterministic args are deprecated '
                       'in favor of specifying random seed')
        deterministic = None
    be = Backend.allocate_backend(backend,
                                  rng_seed=rng_seed,
                                  default_dtype=datatype,
                                  stochastic_round=stochastic_round,
                                  device_id=device_id,
                                  num_devices=max_devices,
                                  compat_mode=compat_mode,
                                  deterministic=deterministic)
    logger.info("Backend: {}, RNG seed: {}".format(backend, rng_seed))
    NervanaObject.be = be
    be.bsz = batch_size
    return be


def cleanup_backend():
    if NervanaObject.be is None:
        return
    NervanaObject.be.cleanup_backend()
    NervanaObject.be = None
