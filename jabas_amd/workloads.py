"""Gradient-set shapes of the five benchmark configurations.

Each builder returns a list of ``ParamSpec(name, numel, group)`` in module registration
order, i.e. the order ``model.named_parameters()`` yields in the reference's example
scripts. ``group`` is the optimizer parameter group the reference's
``build_param_groups_in_optimizer`` puts the tensor in. No model code is needed here:
the synchronisation path sees only flat sizes.

Shape sources (JABAS repository):
  ResNet-50    examples/resnet50/image_classification/resnet.py:166-187,245-300,366-372
               groups: examples/resnet50/main.py:340-349 ("bn" in name -> weight_decay 0)
  ViT-B/L      examples/vit/models/vit.py:426-431,465-470
               groups: examples/vit/main.py:405-423 (1-D tensors and biases -> no decay)
  GNMT         examples/gnmt/seq2seq/models/{gnmt,encoder,decoder,attention}.py,
               defaults examples/gnmt/train.py:143-150 (hidden 1024, 4 layers, shared embedding)
  Faster R-CNN synthetic list (torchvision is not installed here): the large R50-FPN
               tensors by their real shapes plus a seeded tail of small tensors.
"""
from collections import namedtuple
import random

ParamSpec = namedtuple("ParamSpec", "name numel group")

MiB = 1024 * 1024


def resnet50(num_classes=1000):
    """161 tensors, 25,557,032 elements. group 0 = BN (wd 0), group 1 = rest (wd 1e-4)."""
    specs = []

    def conv(name, cout, cin, k):
        specs.append(ParamSpec(name + ".weight", cout * cin * k * k, 1))

    def bn(name, c):
        specs.append(ParamSpec(name + ".weight", c, 0))
        specs.append(ParamSpec(name + ".bias", c, 0))

    conv("conv1", 64, 3, 7)
    bn("bn1", 64)
    inplanes = 64
    for li, (planes, blocks) in enumerate(zip((64, 128, 256, 512), (3, 4, 6, 3))):
        for b in range(blocks):
            pre = f"layers.{li}.{b}"
            conv(pre + ".conv1", planes, inplanes, 1)
            bn(pre + ".bn1", planes)
            conv(pre + ".conv2", planes, planes, 3)
            bn(pre + ".bn2", planes)
            conv(pre + ".conv3", planes * 4, planes, 1)
            bn(pre + ".bn3", planes * 4)
            if b == 0:
                # downsample = Sequential(conv1x1, batchnorm): names "downsample.0/1" carry no
                # "bn", so the reference's name filter leaves both in the decayed group
                conv(pre + ".downsample.0", planes * 4, inplanes, 1)
                specs.append(ParamSpec(pre + ".downsample.1.weight", planes * 4, 1))
                specs.append(ParamSpec(pre + ".downsample.1.bias", planes * 4, 1))
                inplanes = planes * 4
    specs.append(ParamSpec("fc.weight", num_classes * 2048, 1))
    specs.append(ParamSpec("fc.bias", num_classes, 1))
    return specs


def _vit(dim, depth, mlp, num_classes=1000, patch=16, img=224):
    n_tok = (img // patch) ** 2 + 1
    specs = [
        ParamSpec("cls_token", dim, 0),                      # in no_weight_decay()
        ParamSpec("pos_embed", n_tok * dim, 0),              # in no_weight_decay()
        ParamSpec("patch_embed.proj.weight", dim * 3 * patch * patch, 1),
        ParamSpec("patch_embed.proj.bias", dim, 0),
    ]
    for b in range(depth):
        pre = f"blocks.{b}"
        specs += [
            ParamSpec(pre + ".norm1.weight", dim, 0), ParamSpec(pre + ".norm1.bias", dim, 0),
            ParamSpec(pre + ".attn.qkv.weight", 3 * dim * dim, 1), ParamSpec(pre + ".attn.qkv.bias", 3 * dim, 0),
            ParamSpec(pre + ".attn.proj.weight", dim * dim, 1), ParamSpec(pre + ".attn.proj.bias", dim, 0),
            ParamSpec(pre + ".norm2.weight", dim, 0), ParamSpec(pre + ".norm2.bias", dim, 0),
            ParamSpec(pre + ".mlp.fc1.weight", mlp * dim, 1), ParamSpec(pre + ".mlp.fc1.bias", mlp, 0),
            ParamSpec(pre + ".mlp.fc2.weight", dim * mlp, 1), ParamSpec(pre + ".mlp.fc2.bias", dim, 0),
        ]
    specs += [
        ParamSpec("norm.weight", dim, 0), ParamSpec("norm.bias", dim, 0),
        ParamSpec("head.weight", num_classes * dim, 1), ParamSpec("head.bias", num_classes, 0),
    ]
    return specs


def vit_b16():
    """152 tensors, 86,567,656 elements. group 0 = no decay, group 1 = wd 0.05."""
    return _vit(768, 12, 3072)


def vit_l16():
    """296 tensors, 304,326,632 elements."""
    return _vit(1024, 24, 4096)


def gnmt(hidden=1024, layers=4, vocab=32317):
    """160,665,150 elements; one parameter group (Adam, wd 0)."""
    specs = []

    def lstm(name, inp, bidir=False):
        for suffix in ([""] + (["_reverse"] if bidir else [])):
            specs.append(ParamSpec(f"{name}.weight_ih_l0{suffix}", 4 * hidden * inp, 0))
            specs.append(ParamSpec(f"{name}.weight_hh_l0{suffix}", 4 * hidden * hidden, 0))
            specs.append(ParamSpec(f"{name}.bias_ih_l0{suffix}", 4 * hidden, 0))
            specs.append(ParamSpec(f"{name}.bias_hh_l0{suffix}", 4 * hidden, 0))

    lstm("encoder.rnn_layers.0", hidden, bidir=True)
    lstm("encoder.rnn_layers.1", 2 * hidden)
    for i in range(2, layers):
        lstm(f"encoder.rnn_layers.{i}", hidden)
    specs.append(ParamSpec("encoder.embedder.weight", vocab * hidden, 0))
    lstm("decoder.att_rnn.rnn", hidden)
    specs.append(ParamSpec("decoder.att_rnn.attn.linear_att", hidden, 0))
    specs.append(ParamSpec("decoder.att_rnn.attn.normalize_scalar", 1, 0))
    specs.append(ParamSpec("decoder.att_rnn.attn.normalize_bias", hidden, 0))
    specs.append(ParamSpec("decoder.att_rnn.attn.linear_q.weight", hidden * hidden, 0))
    specs.append(ParamSpec("decoder.att_rnn.attn.linear_k.weight", hidden * hidden, 0))
    for i in range(layers - 1):
        lstm(f"decoder.rnn_layers.{i}", 2 * hidden)
    specs.append(ParamSpec("decoder.classifier.classifier.weight", vocab * hidden, 0))
    specs.append(ParamSpec("decoder.classifier.classifier.bias", vocab, 0))
    return specs


GNMT_EMBEDDING = "encoder.embedder.weight"
GNMT_EMBEDDING_ROWS, GNMT_EMBEDDING_COLS = 32317, 1024


def faster_rcnn_r50_fpn(seed=0):
    """About 41 M elements over about 280 tensors: ResNet-50 trunk convolutions (frozen-BN
    backbones carry no BN parameters), FPN, RPN and box heads by their real shapes, then a
    seeded tail of 64..2048-element tensors standing in for the many small biases/scales.
    group 0 = biases / 1-D (the reference keeps one group, examples/faster_r_cnn/train.py:266-276;
    the tag only marks which tensors are small)."""
    specs = []
    inplanes = 64
    specs.append(ParamSpec("backbone.body.conv1.weight", 64 * 3 * 49, 0))
    for li, (planes, blocks) in enumerate(zip((64, 128, 256, 512), (3, 4, 6, 3))):
        for b in range(blocks):
            pre = f"backbone.body.layer{li + 1}.{b}"
            specs.append(ParamSpec(pre + ".conv1.weight", planes * inplanes, 0))
            specs.append(ParamSpec(pre + ".conv2.weight", planes * planes * 9, 0))
            specs.append(ParamSpec(pre + ".conv3.weight", planes * 4 * planes, 0))
            if b == 0:
                specs.append(ParamSpec(pre + ".downsample.0.weight", planes * 4 * inplanes, 0))
                inplanes = planes * 4
    for i, cin in enumerate((256, 512, 1024, 2048)):
        specs.append(ParamSpec(f"backbone.fpn.inner_blocks.{i}.weight", 256 * cin, 0))
        specs.append(ParamSpec(f"backbone.fpn.inner_blocks.{i}.bias", 256, 0))
        specs.append(ParamSpec(f"backbone.fpn.layer_blocks.{i}.weight", 256 * 256 * 9, 0))
        specs.append(ParamSpec(f"backbone.fpn.layer_blocks.{i}.bias", 256, 0))
    specs += [
        ParamSpec("rpn.head.conv.weight", 256 * 256 * 9, 0), ParamSpec("rpn.head.conv.bias", 256, 0),
        ParamSpec("rpn.head.cls_logits.weight", 3 * 256, 0), ParamSpec("rpn.head.cls_logits.bias", 3, 0),
        ParamSpec("rpn.head.bbox_pred.weight", 12 * 256, 0), ParamSpec("rpn.head.bbox_pred.bias", 12, 0),
        ParamSpec("roi_heads.box_head.fc6.weight", 1024 * 12544, 0), ParamSpec("roi_heads.box_head.fc6.bias", 1024, 0),
        ParamSpec("roi_heads.box_head.fc7.weight", 1024 * 1024, 0), ParamSpec("roi_heads.box_head.fc7.bias", 1024, 0),
        ParamSpec("roi_heads.box_predictor.cls_score.weight", 91 * 1024, 0),
        ParamSpec("roi_heads.box_predictor.cls_score.bias", 91, 0),
        ParamSpec("roi_heads.box_predictor.bbox_pred.weight", 364 * 1024, 0),
        ParamSpec("roi_heads.box_predictor.bbox_pred.bias", 364, 0),
    ]
    rng = random.Random(seed)
    i = 0
    while len(specs) < 280:
        specs.append(ParamSpec(f"tail.{i}", rng.choice((64, 128, 256, 512, 1024, 2048)), 0))
        i += 1
    return specs


Config = namedtuple("Config", "name specs K batches grad_dtype grad_std opt stats")

# optimizer dictionaries: kind + hyper-parameters + per-group (lr, weight_decay)
_SGD_RESNET = dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
                   groups=[dict(lr=0.1, weight_decay=0.0), dict(lr=0.1, weight_decay=1e-4)])
_ADAMW_VIT = dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8,
                  groups=[dict(lr=5e-4, weight_decay=0.0), dict(lr=5e-4, weight_decay=0.05)])
_SGD_FRCNN = dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
                  groups=[dict(lr=0.02, weight_decay=1e-4)])
_ADAM_GNMT = dict(kind="adam", betas=(0.9, 0.999), eps=1e-8,
                  groups=[dict(lr=2e-3, weight_decay=0.0)])


def configs():
    """The five configurations the benchmark is specified on, in order."""
    return [
        Config("resnet50", resnet50(), 2, (32, 32), "fp32", 1e-3, _SGD_RESNET, False),
        Config("vit_b16", vit_b16(), 4, (48, 32, 32, 16), "fp32", 5e-4, _ADAMW_VIT, True),
        Config("faster_rcnn_r50_fpn", faster_rcnn_r50_fpn(), 3, (4, 2, 2), "fp32", 1e-3, _SGD_FRCNN, False),
        Config("gnmt", gnmt(), 4, (128, 128, 64, 64), "fp32", 1e-3, _ADAM_GNMT, True),
        Config("vit_l16", vit_l16(), 8, tuple(range(64, 0, -8)), "bf16", 2e-4, _ADAMW_VIT, True),
    ]


def config(name):
    for c in configs():
        if c.name == name:
            return c
    raise KeyError(name)
