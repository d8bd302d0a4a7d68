"""The kernels that the tests' toy parts bring along, each registered with the framework's one
call for that.  Imported by the tests that use them and by ``__graft_entry__.build()``, which
compiles every library that is registered."""
import ctypes as C
import os

from zse_amd.parts import register_kernels

HERE = os.path.dirname(os.path.abspath(__file__))
_VP, _I, _F = C.c_void_p, C.c_int, C.c_float

# the toy state mixer's recurrence (toy_decay_device.py)
register_kernels("toy_decay", os.path.join(HERE, "toy_decay.hip"),
                 {"zk_toy_decay": [_VP, _VP, _VP, _I, _I, _VP, _VP, _I, _I, _F, _VP]})
# query and key heads scaled to unit length between product and rotation (test_gpu_parts.py)
register_kernels("toy_head_norm", os.path.join(HERE, "toy_head_norm.hip"),
                 {"zk_toy_head_norm": [_VP, _I, _I, _I, _I, _VP]})
