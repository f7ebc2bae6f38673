"""numpy restatement of the GGUF container parse and of from_gguf's weight preparation.  Test infrastructure only.
_gguf_parse: tinygrad/llm/gguf.py:132-149.  from_gguf: tinygrad/llm/model.py:370-451 (fp16 cast :376, tied embeddings :379,
llama q/k permutation :409-419, config extraction :420-444)."""
import io, struct
import numpy as np
from oracle import ggml

def _rd(fmt, n, r): return struct.unpack("<" + fmt, r.read(n))[0]
def _str(r): return str(r.read(_rd("Q", 8, r)), "utf-8")
def _arr(r):
  t, n = _rd("i", 4, r), _rd("Q", 8, r)
  return [_val(t, r) for _ in range(n)]
def _val(t, r):
  if t == 8: return _str(r)
  if t == 9: return _arr(r)
  f, nb = {0: ("c", 1), 1: ("b", 1), 2: ("H", 2), 3: ("h", 2), 4: ("I", 4), 5: ("i", 4), 6: ("f", 4), 7: ("?", 1), 10: ("Q", 8), 11: ("q", 8), 12: ("d", 8)}[t]
  return _rd(f, nb, r)

def parse(raw: bytes):
  r = io.BytesIO(raw)
  magic, version, n_tensors, n_kv = r.read(4), _rd("i", 4, r), _rd("q", 8, r), _rd("q", 8, r)
  if magic != b"GGUF" or version not in (2, 3): raise ValueError("Invalid GGUF format!")
  kv = {}
  for _ in range(n_kv):
    k = _str(r); kv[k] = _val(_rd("i", 4, r), r)
  infos = [(_str(r), tuple(_rd("Q", 8, r) for _ in range(_rd("I", 4, r))), _rd("i", 4, r), _rd("Q", 8, r)) for _ in range(n_tensors)]
  align = kv.get("general.alignment", 32)
  start = (r.tell() + align - 1) // align * align
  arr = np.frombuffer(raw, dtype=np.uint8)
  sd = {}
  for name, dims, typ, off in infos:
    n = int(np.prod(dims))
    sd[name] = ggml.ggml_data_to_tensor(arr[start + off:], n, typ).astype(np.float32).reshape(*reversed(dims))
  return kv, sd

def from_gguf_weights(raw: bytes):
  """-> (cfg dict, {name: float32 weight after the reference's load-time preparation})."""
  kv, sd = parse(raw)
  sd = {k: v.astype(np.float16).astype(np.float32) for k, v in sd.items()}                      # model.py:376
  if "output.weight" not in sd: sd["output.weight"] = sd["token_embd.weight"]                    # model.py:379
  arch = kv["general.architecture"]
  if arch in ("qwen35", "qwen35moe", "glm4moe"): sd = {k.replace("post_attention_norm", "ffn_norm"): v for k, v in sd.items()}   # model.py:403-404
  H, KV = kv[f"{arch}.attention.head_count"], kv[f"{arch}.attention.head_count_kv"]
  for name in list(sd):
    if arch == "llama" and "attn_q.weight" in name:
      w = sd[name].reshape(H, sd[name].shape[0] // H, -1)
      sd[name] = w.reshape(H, -1, 2, w.shape[-1]).transpose(0, 2, 1, 3).reshape(-1, w.shape[-1])   # "n (h two) d -> n (two h) d"
    elif arch == "llama" and "attn_k.weight" in name:
      w = sd[name].reshape(KV, sd[name].shape[0] // KV, -1)
      sd[name] = w.reshape(KV, -1, 2, w.shape[-1]).transpose(0, 2, 1, 3).reshape(-1, w.shape[-1])
  dim = kv[f"{arch}.embedding_length"]
  cfg = dict(num_blocks=kv[f"{arch}.block_count"] - kv.get(f"{arch}.nextn_predict_layers", 0), dim=dim,
             leading_dense_blocks=kv.get(f"{arch}.leading_dense_block_count", 0),                  # model.py:438; the other MoE extras are read off the tensors hidden_dim=kv.get(f"{arch}.expert_feed_forward_length", kv.get(f"{arch}.feed_forward_length", 0)),
             n_heads=H, n_kv_heads=KV, norm_eps=kv[f"{arch}.attention.layer_norm_rms_epsilon"], vocab_size=len(kv["tokenizer.ggml.tokens"]),
             head_dim=kv.get(f"{arch}.attention.key_length", dim // H), rope_theta=kv[f"{arch}.rope.freq_base"],
             rope_dim=kv.get(f"{arch}.rope.dimension_count", kv.get(f"{arch}.attention.key_length", dim // H)),   # model.py:406
             qk_norm=int(sd["blk.0.attn_q_norm.weight"].shape[0]) if "blk.0.attn_q_norm.weight" in sd else 0,
             num_experts=kv.get(f"{arch}.expert_count", 0), num_experts_per_tok=kv.get(f"{arch}.expert_used_count", 0),
             norm_topk_prob=kv.get(f"{arch}.expert_weights_norm", arch in ("qwen3moe", "qwen35moe", "kimi-linear")),   # model.py:432
             expert_gating_func=kv.get(f"{arch}.expert_gating_func", 1), routed_scaling_factor=kv.get(f"{arch}.expert_weights_scale", 1.0))
  return cfg, sd, kv
