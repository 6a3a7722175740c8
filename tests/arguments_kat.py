"""Known answers for the shape -> MLP feature extraction of the four
MLP-predicted operations.

Each case gives the recorded call as literal ``Arguments(args, kwargs)`` content
(tensors already reduced to their sizes, as the reference's tracker stores them,
analyzer/habitat/analysis/arguments.py:13-38) and the feature list in the
network's own order, written out BY HAND from reading
analyzer/habitat/analysis/predictor.py:150-283 and the `features` lists of
analyzer/habitat/analysis/mlp/mlp.py:38,57,76-77,97.  Nothing here is computed
by the code under test.

Feature orders:
  conv2d  bias, batch, image_size, in_channels, out_channels, kernel_size, stride, padding
  linear  bias, batch, in_features, out_features
  bmm     batch, left, middle, right
  lstm    bias, bidirectional, batch, seq_len, input_size, hidden_size, num_layers
"""

FEATURE_ORDER = {
    "conv2d": ["bias", "batch", "image_size", "in_channels", "out_channels", "kernel_size",
               "stride", "padding"],
    "linear": ["bias", "batch", "in_features", "out_features"],
    "bmm": ["batch", "left", "middle", "right"],
    "lstm": ["bias", "bidirectional", "batch", "seq_len", "input_size", "hidden_size",
             "num_layers"],
}

_W = ["w_ih", "w_hh", "b_ih", "b_hh"]          # stands for the list of flat weight sizes

# (kind, label, args, kwargs, special, expected features)
CASES = [
    # F.conv2d(input, weight, bias, stride, padding, dilation, groups), all positional,
    # tuples as nn.Conv2d passes them: batch = input[0], image = input[2],
    # in = input[1], out = weight[0], kernel = weight[2], stride[0], padding[0].
    ("conv2d", "tuple stride and padding",
     ((32, 64, 56, 56), (128, 64, 3, 3), (128,), (2, 2), (1, 1), (1, 1), 1), {}, None,
     [1, 32, 56, 64, 128, 3, 2, 1]),
    # int stride / padding (predictor.py:164-171 keeps a non-tuple as is), no bias
    ("conv2d", "int stride and padding, bias None",
     ((8, 3, 224, 224), (64, 3, 7, 7), None, 2, 3, 1, 1), {}, None,
     [0, 8, 224, 3, 64, 7, 2, 3]),
    # everything after the weight by keyword (utils.py:54-63 merges by name)
    ("conv2d", "keyword arguments",
     ((16, 256, 14, 14), (512, 256, 1, 1)),
     {"bias": None, "stride": (1, 1), "padding": (0, 0), "dilation": (1, 1), "groups": 1}, None,
     [0, 16, 14, 256, 512, 1, 1, 0]),
    # not square: the image size is the height input[2], the kernel size weight[2],
    # stride and padding their first entries
    ("conv2d", "rectangular image, kernel, stride, padding",
     ((4, 16, 30, 40), (32, 16, 5, 3), (32,), (1, 2), (2, 1), (1, 1), 1), {}, None,
     [1, 4, 30, 16, 32, 5, 1, 2]),
    # F.linear(input, weight, bias): in = weight[1], out = weight[0]
    ("linear", "two-dimensional input",
     ((64, 512), (1000, 512), (1000,)), {}, None,
     [1, 64, 512, 1000]),
    # leading dimensions multiply into the batch (predictor.py:201-204): 32 * 50
    ("linear", "three-dimensional input, bias None",
     ((32, 50, 512), (2048, 512), None), {}, None,
     [0, 1600, 512, 2048]),
    # 2 * 3 * 5 = 30, weight and bias by keyword
    ("linear", "four-dimensional input, keyword weight and bias",
     ((2, 3, 5, 128),), {"weight": (10, 128), "bias": (10,)}, None,
     [1, 30, 128, 10]),
    # torch.bmm(input, mat2): batch, left, middle = input; right = mat2[2]
    ("bmm", "positional",
     ((16, 128, 64), (16, 64, 256)), {}, None,
     [16, 128, 64, 256]),
    ("bmm", "keyword mat2",
     ((3, 7, 11),), {"mat2": (3, 11, 13)}, None,
     [3, 7, 11, 13]),
    # _VF.lstm(input, hx, flat_weights, bias, num_layers, dropout, training,
    # bidirectional, batch_first): position 4 is an int -> unpacked overload;
    # batch = input[1], seq_len = input[0], input_size = input[2], hidden = hx[0][2]
    ("lstm", "unpacked, two layers, one direction",
     ((35, 20, 650), ((2, 20, 650), (2, 20, 650)), _W * 2, True, 2, 0.5, True, False, False), {},
     None,
     [1, 0, 20, 35, 650, 650, 2]),
    # bias False is still "not None" -> 1 (predictor.py:252); bidirectional True -> 1
    ("lstm", "unpacked, bias False, bidirectional",
     ((50, 8, 256), ((6, 8, 512), (6, 8, 512)), _W * 6, False, 3, 0.0, False, True, False), {},
     None,
     [1, 1, 8, 50, 256, 512, 3]),
    # _VF.lstm(input, batch_sizes, hx, flat_weights, bias, num_layers, dropout,
    # training, bidirectional): position 4 is the bool `bias` -> packed overload;
    # input is (sum of batch sizes, input_size); batch = max(batch_sizes) = 32,
    # seq_len = 1200 // 32 = 37, input_size = input[1], hidden = hx[0][2]
    ("lstm", "packed sequence",
     ((1200, 300), (40,), ((4, 32, 1024), (4, 32, 1024)), _W * 4, True, 2, 0.2, True, True), {},
     {"batch_sizes": [32] * 35 + [16] * 5},
     [1, 1, 32, 37, 300, 1024, 2]),
    # packed, one step: batch sizes [5], 5 // 5 = 1
    ("lstm", "packed sequence of one step",
     ((5, 64), (1,), ((1, 5, 128), (1, 5, 128)), _W, False, 1, 0.0, False, False), {},
     {"batch_sizes": [5]},
     [1, 0, 5, 1, 64, 128, 1]),
]


def arguments_of(case):
    """The case's call as a habitat_amd Arguments object."""
    from habitat_amd.analysis.arguments import Arguments
    _, _, args, kwargs, special, _ = case
    a = Arguments(args, dict(kwargs))
    if special:
        a.special.update(special)
    return a
