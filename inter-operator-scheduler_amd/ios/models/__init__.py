from .inception_v3 import inception_v3
from .randwire import randwire_small, randwire_large, randwire_xlarge
from .squeezenet import squeezenet, squeezenet_1_1
from .nasnet import nasnet_mobile, nasnet_large
from .sample import sample_network
from .vgg import vgg_11, vgg_13, vgg_16, vgg_19
from .alexnet import alexnet
from .resnet import resnet18, resnet34, resnet50
