"""HIP sources of libnklq.so and the script that compiles them."""
