"""CPU oracle for the trainer-side per-token hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``axon_amd/`` imports this package; it is
used by ``tests/``, by ``__graft_entry__.smoke()`` and by ``bench.py``'s
``cpu_baseline`` leg as the checker and the timed CPU baseline, never as the
product path.

Each module restates, in plain torch on the CPU, the arithmetic of the reference
(modelcorp/axon) functions it cites.  The reference is pure Python; none of its
code is imported or executed, here or in the tests.

What pins each function (see tests/test_oracle_*.py):

  lmhead.forward / backward   the reference's own tests hold no vector for the fused
      LM head, so parity rests on mathematics: ``log_softmax().gather()`` and
      ``-sum p log p`` (library routines), closed forms (zero weight -> -ln V / ln V),
      shift and temperature invariances, fp64 brute force, autograd of the textbook
      forward and fp64 finite differences for the backward.
  loss.agg_loss / masked_mean / ppo_loss / gspo_loss
      every known-answer row of the reference's tests/trainer/algos/loss/test_utils.py
      and test_loss.py, a scalar pure-Python evaluation over all clip regions, and
      autograd-vs-closed-form gradients including tie handling.
  sampler.correction          the known answers of tests/utils/test_rl_sampler.py
      plus a per-token scalar loop.
  advantage.group_mean_std / grpo / filter_zero_advantage
      the known answers of tests/utils/test_rl_advantage.py,
      tests/trainer/algos/advantages/test_advantages.py, tests/utils/test_rl_utils.py
      and ``torch.std`` per group.
  layout.*                    the ``get_unpad_data`` vectors of tests/utils/torch/test_ops.py.
"""
