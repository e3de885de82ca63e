"""MI355X-native W4A16 Marlin GEMM: HIP kernels behind the reference's
`marlin` module interface (see marlin.py in this package)."""
