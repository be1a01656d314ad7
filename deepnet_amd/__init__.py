"""MI355X-native matrix backend for deepnet: `cudamat` (CUDAMatrix API) and
`cudamat_conv` (cuda-convnet style conv / pool / norm entry points) over two
C-ABI HIP libraries built from csrc/."""
