"""numpy restatement of the linear the reference runs over a dequantized GGUF weight.  Test infrastructure only.

Linear.__call__ = x.linear(W.T) (tinygrad/nn/__init__.py:177) -> Tensor.dot (tinygrad/mixin/op.py:367-392): operands are
promoted to least_upper_dtype, multiplied in that dtype, summed with sum_acc_dtype (float32 for every float type,
tinygrad/dtype.py:212-216, tinygrad/mixin/reduce.py:44-45) and, when the product dtype was fp16, cast back to fp16."""
import numpy as np
from oracle import ggml

def weight_f32(data, n, k, ggml_type) -> np.ndarray:
  """gguf.py:148: W = ggml_data_to_tensor(...).reshape(*reversed(dims)) -> (N, K) row-major, quant blocks along K."""
  return ggml.ggml_data_to_tensor(data, n * k, ggml_type).reshape(n, k)

def linear_f64(x: np.ndarray, w: np.ndarray) -> np.ndarray:
  """Tolerance anchor: textbook x @ W.T in float64 on the exact operand values."""
  return x.astype(np.float64) @ w.astype(np.float64).T

def linear_model(x_f32: np.ndarray, w_f32: np.ndarray) -> np.ndarray:
  """Model path (tinygrad/llm/model.py:359,376): x float32, W cast to fp16 at load (lossy for Q4_0), product and
  accumulation in float32.  Returned as float32 of the float64-accumulated sum: summation order is not part of the spec."""
  wh = w_f32.astype(np.float16).astype(np.float32)
  return (x_f32.astype(np.float64) @ wh.astype(np.float64).T).astype(np.float32)

def linear_standalone_f16(x_f16: np.ndarray, w_f32: np.ndarray) -> np.ndarray:
  """Config-1 semantics (fp16 x, fp16 W): each product rounded to fp16 (mixin/op.py:392), float32 accumulation,
  result cast to fp16.  O(M*N*K) memory-light loop over rows of x."""
  wh = w_f32.astype(np.float16)
  out = np.empty((x_f16.shape[0], wh.shape[0]), dtype=np.float16)
  for m in range(x_f16.shape[0]):
    prod = (x_f16[m].astype(np.float16)[None, :] * wh)            # fp16 * fp16 -> fp16 (RNE)
    out[m] = prod.astype(np.float32).sum(axis=1, dtype=np.float64).astype(np.float32).astype(np.float16)
  return out

def rel_err(y: np.ndarray, ref: np.ndarray) -> float:
  """max |y - ref| / max |ref|: the 'rel-err' every GEMV/GEMM parity test states its bound in."""
  ref = ref.astype(np.float64)
  return float(np.abs(y.astype(np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))
