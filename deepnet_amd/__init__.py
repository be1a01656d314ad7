"""MI355X-native matrix backend for deepnet: `cudamat` (CUDAMatrix API) and
`cudamat_conv` (cuda-convnet style conv / pool / norm entry points) over two
C-ABI HIP libraries built from csrc/, plus the callers either side of it that a
training step runs: `convolutions` (the conv stage of an edge), `parameter`, `layer`,
`neuralnet` (layers, edges, back-propagation step),
`pbtxt` / `trainer` (deepnet's text-format model files -> nets on the device), `datahandler`
(device-resident data cache) and `util` (checkpoint byte format, model / operation readers)."""
