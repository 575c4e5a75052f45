from .Cacheton import Cacheton
from .TensorAxes import TensorAxes
from .TensorShape import TensorShape
from .hip import HipDevice, HipBuffer, HipDevicesBuffers, devices
from .module.ModuleBase import ModuleBase
