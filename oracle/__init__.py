"""CPU oracle: TEST INFRASTRUCTURE ONLY.

Plain numpy / C restatements of the reference algorithms on the rollout hot
path.  Nothing under ``ksim_amd/`` may import this package; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do,
and only as the checker.

Pinning status (what independent evidence fixes each restatement):

* ``ppo.compute_ppo_inputs`` / ``compute_ppo_loss``: pinned by brute-force
  O(T^2) sums, closed forms and special cases (tests/test_oracle_ppo.py).
* ``terms.action_*_penalty``: pinned by the reference's own known-answer
  vectors (tests/golden/reward_kats.json, from reference tests/test_rewards.py).
* ``terms.*_termination``: pinned by the reference's known answers
  (reference tests/test_terminations.py) and an exhaustive truth table.
* ``dyn`` kinematics / mass matrix / bias forces / integrator / contact
  geometry / solver fixed point: pinned by brute-force Jacobians, Lagrangian
  identities, free-fall closed forms and KKT residuals
  (tests/test_oracle_dyn.py).
* ``dyn`` Newton *iterates* of the third-party MJX solver at a fixed iteration
  count, impedance details and pyramidal regulariser scaling: restated from
  the public MuJoCo documentation; **parity with MJX unpinned** (MJX is not
  vendored in the reference and not installed).
"""
