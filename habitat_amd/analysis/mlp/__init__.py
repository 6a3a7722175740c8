"""Per-operation MLP predictors: model classes and RuntimePredictor (mlp), the
device-feature table (devices)."""
