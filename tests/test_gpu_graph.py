"""The entry points under HIP graph capture: they only enqueue kernels on the caller's stream (no allocation, no
synchronisation, no memset nodes), so a captured step must replay to the eager result every time."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import to_dev_bf16
from maxdiffusion_amd import ops

pytestmark = pytest.mark.gpu


def _step(q, k, v, wq, wk, cos, sin, heads, o_run, l_run):
  """prologue -> attention with lse -> two fused ring hops into (o_run, l_run) -> fp8 quantisation + fp8 attention."""
  qn, kn = ops.norm_rope_fullrow(q, k, wq, wk, cos, sin, heads, q_mul=ops.folded_q_mul(128))
  b, s = q.shape[0], q.shape[1]
  v4 = v.view(b, s, heads, 128)
  out, lse = ops.flash_attention(qn, kn, v4, scale=ops.FOLDED_SCALE, return_lse=True)
  o_run.zero_()
  l_run.fill_(ops.LSE_INIT)
  half = s // 2 + 3
  ops.flash_attention_merge(qn, kn[:, :half], v4[:, :half], o_run, l_run, scale=ops.FOLDED_SCALE)
  ops.flash_attention_merge(qn, kn[:, half:], v4[:, half:], o_run, l_run, scale=ops.FOLDED_SCALE)
  q8, sq = ops.quant_e4m3(qn, pow2_scale=True)
  k8, sk = ops.quant_e4m3(kn, pow2_scale=True)
  v8, sv = ops.quant_e4m3(v4)
  out8 = ops.flash_attention_fp8(q8, k8, v8, sq, sk, sv, scale=ops.FOLDED_SCALE)
  return out, lse, out8


def test_captured_step_replays_to_the_eager_result(dev):
  H, grid = 4, (3, 10, 11)
  S = grid[0] * grid[1] * grid[2]
  q, k, v = (to_dev_bf16(O.normal_bf16((1, S, H * 128), s), dev) for s in (0, 1, 2))
  wq, wk = (to_dev_bf16(O.norm_weight(H * 128, s), dev) for s in (3, 4))
  cos, sin = (torch.from_numpy(t).to(dev) for t in O.wan_rope_table(grid, 128))
  o_run, l_run = ops.new_merge_state(1, S, H, 128, dev)
  o_ref, l_ref = ops.new_merge_state(1, S, H, 128, dev)

  eager = _step(q, k, v, wq, wk, cos, sin, H, o_ref, l_ref)
  torch.cuda.synchronize()
  want = [t.clone() for t in eager] + [o_ref.clone(), l_ref.clone()]

  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):  # warm-up on the capture stream, as torch asks for
    _step(q, k, v, wq, wk, cos, sin, H, o_run, l_run)
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()

  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    captured = _step(q, k, v, wq, wk, cos, sin, H, o_run, l_run)
  for rep in range(4):
    # eager work and a synchronisation between replays; the carry is dirtied so that a replay must rebuild it
    o_run.fill_(float(rep) + 0.5)
    l_run.fill_(7.0)
    for t in captured:
      t.zero_()
    ops.flash_attention(to_dev_bf16(O.normal_bf16((1, 64, 2, 128), 9 + rep), dev),
                        to_dev_bf16(O.normal_bf16((1, 80, 2, 128), 19), dev),
                        to_dev_bf16(O.normal_bf16((1, 80, 2, 128), 29), dev))
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    got = list(captured) + [o_run, l_run]
    for i, (g, w) in enumerate(zip(got, want)):
      assert torch.equal(g, w), f"replay {rep}: output {i} differs from the eager result"


def test_captured_forward_and_static_backward_replay_to_the_eager_result(dev):
  """A training step under capture: forward with lse, then the backward through the entry point that allocates nothing
  (its scratch is the library's static device array; the per-device address lookup happens on the warm-up call)."""
  B, H, Sq, Skv = 2, 3, 333, 500
  q, do = (to_dev_bf16(O.normal_bf16((B, Sq, H, 128), s), dev) for s in (0, 3))
  k, v = (to_dev_bf16(O.normal_bf16((B, Skv, H, 128), s), dev) for s in (1, 2))
  out, lse = ops.flash_attention(q, k, v, return_lse=True)
  want = [t.clone() for t in ops.flash_attention_backward(q, k, v, out, do, lse)]
  grads = [torch.empty_like(t) for t in (q, k, v)]

  def step():
    o, l = ops.flash_attention(q, k, v, return_lse=True)  # torch's capture-time allocator; the library allocates nothing
    ops.flash_attention_backward_static(q, k, v, o, do, l, *grads)
    return o, l

  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    step()
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    out_c, lse_c = step()
  for rep in range(3):
    for t in grads + [out_c, lse_c]:
      t.fill_(float(rep) + 0.25)
    # eager work between the replays, including a backward that uses the same static scratch with another shape
    qq, kk = (to_dev_bf16(O.normal_bf16((1, 70 + rep, 2, 128), 40 + s), dev) for s in (0, 1))
    oo, ll = ops.flash_attention(qq, kk, kk, return_lse=True)
    ops.flash_attention_backward_static(qq, kk, kk, oo, oo, ll, torch.empty_like(qq), torch.empty_like(kk), torch.empty_like(kk))
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out_c, out) and torch.equal(lse_c, lse), f"replay {rep}: forward differs"
    for i, (g, w) in enumerate(zip(grads, want)):
      assert torch.equal(g, w), f"replay {rep}: gradient {i} differs from the eager result"


def test_captured_training_step_with_the_prologue_backward(dev):
  """Prologue -> attention -> attention backward -> prologue backward in one captured graph: the backward entry points
  enqueue kernels only (their workspaces are the caller's; the weight gradients come from a two-stage sum, no atomics,
  so every replay reproduces the eager gradients bit for bit)."""
  H, grid = 3, (2, 6, 11)
  S, N = grid[0] * grid[1] * grid[2], 3 * 128
  q, k, v, do = (to_dev_bf16(O.normal_bf16((2, S, N), s), dev) for s in (0, 1, 2, 5))
  wq, wk = (to_dev_bf16(O.norm_weight(N, s), dev) for s in (3, 4))
  cos, sin = (torch.from_numpy(t).to(dev) for t in O.wan_rope_table(grid, 128))
  q_mul = ops.folded_q_mul(128)

  def step():
    qn, kn = ops.norm_rope_fullrow(q, k, wq, wk, cos, sin, H, q_mul=q_mul)
    v4, do4 = v.view(2, S, H, 128), do.view(2, S, H, 128)
    out, lse = ops.flash_attention(qn, kn, v4, scale=ops.FOLDED_SCALE, return_lse=True)
    dqn, dkn, dv = ops.flash_attention_backward(qn, kn, v4, out, do4, lse, scale=ops.FOLDED_SCALE)
    dq, dk, dwq, dwk = ops.norm_rope_fullrow_backward(q, k, wq, wk, cos, sin, H, dqn, dkn, q_mul=q_mul)
    return out, dv, dq, dk, dwq, dwk

  want = [t.clone() for t in step()]
  torch.cuda.synchronize()
  assert all(bool(torch.isfinite(t.float()).all()) and float(t.float().abs().max()) > 0 for t in want)
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):  # warm-up on the capture stream (also: the prologue backward sizes its grid on first use)
    step()
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    captured = step()
  for rep in range(3):
    for t in captured:
      t.fill_(float(rep) + 0.25)
    # eager work between the replays: another prologue backward of a different shape
    x = to_dev_bf16(O.normal_bf16((1, 37 + rep, N), 50 + rep), dev)
    ops.norm_rope_fullrow_backward(x, x, wq, wk, None, None, H, x.view(1, -1, H, 128), x.view(1, -1, H, 128))
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    for i, (g, w) in enumerate(zip(captured, want)):
      assert torch.equal(g, w), f"replay {rep}: output {i} differs from the eager result"
