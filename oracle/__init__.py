"""CPU restatement of the reference algorithms: test infrastructure only (tests/, smoke(), the cpu_baseline leg of bench.py); nothing in s2cnn_amd imports it."""
