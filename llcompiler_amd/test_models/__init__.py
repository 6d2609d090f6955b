"""Model and op definitions the parity tests and benchmarks run, in the spirit of the reference's
llcompiler/test_models: tiny modules per op plus the five benchmark configurations."""
from .models import (MLP, BertEncoder, EncoderBlock, ResNet18BN, ResNet18Folded, make_bert_inputs, make_encoder_inputs,
                     make_mlp_inputs, make_resnet_inputs)
from .ops import *  # noqa: F401,F403
