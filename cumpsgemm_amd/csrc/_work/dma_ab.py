import os, sys, hashlib, torch
sys.path.insert(0, os.getcwd())
import cumpsgemm_amd as cg
from cumpsgemm_amd import _lib
tag = "default"
if len(sys.argv) > 1 and sys.argv[1] != ".":
    _lib._LIB = os.path.join(os.getcwd(), sys.argv[1], "libcumpsgemm.so"); tag = sys.argv[1]
L = cg.lib()
dev = torch.device('cuda:0'); h = cg.Handle(); h.set_stream(torch.cuda.current_stream())
def bench(fn, steps=10, warm=3):
    best = 1e9
    for _ in range(3):
        for _ in range(warm): fn()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps): fn()
        e1.record(); torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / steps)
    return best
os.environ["CUMPSGEMM_PACKED"] = "1"; os.environ["CUMPSGEMM_PACKED_WALK"] = "0"; L.cuMpSGEMM_reload_tuning_env()
g = torch.Generator(device=dev).manual_seed(1)
for (m, n, k, mode) in [(8192, 8192, 8192, 1), (4096, 4096, 4096, 1), (8192, 8192, 1024, 1), (5000, 4100, 2050, 1), (8192, 8192, 8192, 2), (4096, 4096, 4096, 2)]:
    a = torch.rand(m * k, generator=g, device=dev) * 2 - 1; b = torch.rand(k * n, generator=g, device=dev) * 2 - 1; c = torch.zeros(m * n, device=dev)
    fn = lambda: h.gemm(111, 111, m, n, k, 1.0, a, m, b, k, 0.0, c, m, mode)
    t = bench(fn)
    _, mid = h.gemm(111, 111, m, n, k, 1.0, a, m, b, k, 0.0, c, m, mode, want_module_id=True); torch.cuda.synchronize()
    digest = hashlib.md5(c.cpu().numpy().tobytes()).hexdigest()[:12]
    print(f"[{tag}] {m}x{n}x{k} mode {mode}: {t*1e3:.0f}us {2*m*n*k/t/1e9:.1f}TF id={mid} md5={digest}", flush=True)
    del a, b, c
