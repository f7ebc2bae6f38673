"""Shared by the GPU decode tests: step-by-step greedy decoding on the GPU against the oracle fed the same token history."""
import numpy as np

def greedy_vs_reference_numerics(model, oracle, prompt, n_new):
  """Decodes n_new tokens on the GPU and, step by step, on the oracle fed the SAME history; returns (gpu tokens, oracle tokens, worst logits
  rel-err, minimum oracle top-2 margin, logit rms).  The oracle follows the GPU's token after a step, so one flipped near-tie cannot hide
  behind a diverged history; a flip still fails the caller's token assertion."""
  from oracle import linear as ol
  model.prefill(prompt)
  pos = 0
  for t in prompt[:-1]: oracle.forward(t, pos); pos += 1
  cur, got, ref, worst, margin, rms = prompt[-1], [], [], 0.0, np.inf, 0.0
  for i in range(n_new):
    model.decode_step()
    lg_gpu = model.logits()
    tok = int(model.s.out_tokens.view(4 * i, (1,), np.int32).numpy()[0])
    lg = oracle.forward(cur, pos); pos += 1
    top2 = np.partition(lg, -2)[-2:]
    margin, rms = min(margin, float(top2[1] - top2[0])), float(np.sqrt(np.mean(lg ** 2)))
    worst = max(worst, ol.rel_err(lg_gpu, lg))
    got.append(tok); ref.append(int(np.argmax(lg)))
    cur = tok
  model.check_state()
  return got, ref, worst, margin, rms

