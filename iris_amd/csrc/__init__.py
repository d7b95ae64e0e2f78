"""HIP sources of libiris_hip.so and the script that builds it."""
