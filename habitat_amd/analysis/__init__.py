from habitat_amd.device import _Device

Device = _Device()

# Operations predicted by an MLP rather than by wave scaling
# (analyzer/habitat/analysis/__init__.py:5-18).  gru / rnn_tanh / rnn_relu are
# listed but have no predictor: their measured times pass through unscaled.
SPECIAL_OPERATIONS = {
    "conv2d",
    "linear",
    "bmm",
    "lstm",
    "gru",
    "rnn_tanh",
    "rnn_relu",
}
