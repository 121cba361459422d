"""HIP sources of libs2cnn_hip.so and the script that builds it (build.py)."""
