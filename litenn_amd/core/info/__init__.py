from .InfoBroadcast import InfoBroadcast
from .InfoConv2D import InfoConv2D
from .InfoReduction import InfoReduction
from .InfoReshape import InfoReshape
from .InfoTranspose import InfoTranspose
