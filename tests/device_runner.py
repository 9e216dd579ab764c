"""The device-side problem runner lives in the package (ruy_amd/device_problem.py);
the tests import it under its old name."""
from ruy_amd.device_problem import *  # noqa: F401,F403
from ruy_amd.device_problem import DeviceProblem, device_mul, host_pointer_mul, to_dev, GUARD_ELEMENTS  # noqa: F401
