from .inception_v3 import inception_v3
from .randwire import randwire_small, randwire_large
from .squeezenet import squeezenet, squeezenet_1_1
from .nasnet import nasnet_mobile, nasnet_large
from .sample import sample_network
