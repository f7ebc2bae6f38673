"""tga_moe_route_static (the routing entry point that allocates nothing: its workspace is a device array inside the library) against
tga_moe_route, bit for bit, through the C-ABI: two calls in a row on the same GPU, the second with a smaller input (the shared workspace
still holds the first call's contents), then the size limits."""
import ctypes
import numpy as np, pytest

pytestmark = pytest.mark.gpu

def _route(gpu, logits, k, static):
  T, E = logits.shape
  L = gpu.lib()
  lg = gpu.Buffer.from_numpy(logits)
  w, topi, dest, off, cnt = (gpu.Buffer(s, d) for s, d in (((T, k), np.float32), ((T, k), np.int32), ((T * k,), np.int32), ((E + 1,), np.int32), ((E,), np.int32)))
  for b in (w, topi, dest, off, cnt): gpu.check(L.tga_memset(b.ptr, 0xEE, b.nbytes, None))
  if static: gpu.check(L.tga_moe_route_static(lg.ptr, T, E, k, w.ptr, topi.ptr, dest.ptr, off.ptr, cnt.ptr, None))
  else:
    ws = gpu.Buffer((T * k + ((T * k + 1023) // 1024) * E,), np.int32)
    gpu.check(L.tga_moe_route(lg.ptr, T, E, k, w.ptr, topi.ptr, dest.ptr, off.ptr, cnt.ptr, ws.ptr, None))
  gpu.synchronize()
  return [b.numpy() for b in (w, topi, dest, off, cnt)]

def test_route_static_equals_route_on_two_calls_in_a_row(gpu):
  rng = np.random.default_rng(1005)
  E, k = 128, 8
  pop = 1.0 / np.arange(1, E + 1) ** 1.1
  big = (np.log(pop[rng.permutation(E)])[None, :] + rng.gumbel(size=(4096, E))).astype(np.float32)      # benchmark configuration 5's routing: 32768 assignments
  small = rng.standard_normal((1000, 48)).astype(np.float32); small[::7, 3] = small[::7, 5]              # fewer tokens, fewer experts, some ties
  for logits, kk in ((big, k), (small, 6)):
    got, ref = _route(gpu, logits, kk, True), _route(gpu, logits, kk, False)
    for g, r, name in zip(got, ref, ("weights", "topi", "dest_row", "off", "counts")):
      assert g.tobytes() == r.tobytes(), name
    T = logits.shape[0]
    assert len(set(got[2].tolist())) == T * kk and got[3][-1] % 256 == 0

def test_route_static_rejects_what_does_not_fit(gpu):
  L = gpu.lib()
  d = gpu.Buffer((64,), np.int32)
  assert L.tga_moe_route_static(d.ptr, 65536 // 8 + 1, 64, 8, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, None) != 0
  assert b"exceeds the static workspace" in L.tga_last_error()
  assert L.tga_moe_route_static(d.ptr, 8192, 2048, 8, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, None) != 0       # 65536 + 64 * 2048 words
  assert b"workspace words" in L.tga_last_error()
