"""Backend dispatcher with the reference's selection protocol (BCPNN/__init__.py:8-36 there): the
BCPNN_BACKEND environment variable picks the module whose DenseLayer, StructuralPlasticityLayer and
Network become the package's API, so a StreamBrain training script runs unchanged.

This repository ships one backend, `hip` (MI355X); it is also the default.  A StreamBrain checkout
selects it by adding the same `elif _BACKEND == 'hip'` branch to its own dispatcher.
"""
import os
import sys

_BACKEND = os.environ.get('BCPNN_BACKEND', 'hip')

if _BACKEND == 'hip':
    sys.stderr.write('Using HIP (MI355X) backend.\n')
    from streambrain_amd.backend.hip_backend import *  # noqa: F401,F403
    from streambrain_amd.backend.hip_backend import DenseLayer, Network, StructuralPlasticityLayer  # noqa: F401
else:
    raise ValueError('Unable to import backend : ' + str(_BACKEND))


def backend():
    return _BACKEND
