"""Launch sequence for counter collection (run under rocprofv3 --pmc FETCH_SIZE, then
WRITE_SIZE; the summary of such a run is kept under profiles/): per repetition a cache-flushing fill, a plain copy
of known size, the quantizer and the FP8 GEMM at the headline shape."""
import sys, os
sys.path.insert(0, os.getcwd())
import torch
from cache_dit_amd import ops
FP8 = torch.float8_e4m3fn
dev = torch.device("cuda")
g = torch.Generator(device=dev).manual_seed(0)
M, K, N = 4608, 3072, 12288
x = [torch.randn(M, K, device=dev, generator=g).to(torch.bfloat16) for _ in range(4)]
q = [torch.empty(M, K, dtype=FP8, device=dev) for _ in range(4)]
s = torch.empty(M, dtype=torch.float32, device=dev)
w = [(torch.randint(0, 256, (N, K), dtype=torch.uint8, device=dev, generator=g) & 0xBF).view(FP8) for _ in range(4)]
ws = torch.rand(N, device=dev, generator=g) * 1e-3
b = torch.randn(N, device=dev, generator=g).to(torch.bfloat16)
out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
y = torch.empty(M, K, dtype=torch.bfloat16, device=dev)
# a big flush buffer to push earlier data out of the caches between measured launches
flush = torch.empty(1 << 29, dtype=torch.uint8, device=dev)
for i in range(4):
    flush.zero_()
    y.copy_(x[i])                     # plain copy: reads 2MK, writes 2MK bytes
    flush.zero_()
    ops.quant_rowwise_into(x[i], q[i], s, 0)
    flush.zero_()
    ops.gemm_rowwise_into(q[i], s, w[i], ws, b, out, 0)
torch.cuda.synchronize()
print("done")
