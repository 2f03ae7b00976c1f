"""Plain-PyTorch definitions of the model families the reference's training
scripts use (bench_models/models/train_vit.py, train_llama.py, train_sdxl.py),
built from a config and a seed: the reference fetches them by name from the
network, which is not available here."""
