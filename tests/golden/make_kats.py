"""Writes the known-answer fixtures transcribed from the reference's own unit tests.

The numbers are the input/expected literals of reference tests/test_rewards.py:63-271
and tests/test_terminations.py:22-124 (data only; nothing of the reference is
imported or executed).  Run: python tests/golden/make_kats.py
"""
import json
import os

lin = [[float(i)] * 3 for i in range(5)]
quad = [[float(i * i)] * 3 for i in range(5)]
reward_kats = [
    # name, fn, norm, actions, done, expected, atol          (reference test line)
    dict(ref="test_rewards.py:63-73", fn="velocity", norm="l2", actions=[[2.0] * 3] * 5, done=None,
         expected=[0.0] * 5, atol=1e-6),
    dict(ref="test_rewards.py:75-98", fn="velocity", norm="l2", actions=lin, done=None,
         expected=[0.0, 1.0, 1.0, 1.0, 1.0], atol=1e-6),
    dict(ref="test_rewards.py:100-123", fn="velocity", norm="l1",
         actions=[[1.0, 0.0, 0.0]] * 3 + [[3.0, 2.0, -1.0]] * 2, done=None,
         expected=[0.0, 0.0, 0.0, 5.0 / 3.0, 0.0], atol=1e-6),
    dict(ref="test_rewards.py:125-147", fn="velocity", norm="l2",
         actions=[[0.0, 0.0, 0.0], [2.0, 0.0, 0.0], [4.0, 0.0, 0.0], [5.0, 0.0, 0.0]],
         done=[False, True, False, False], expected=[0.0, 4.0 / 3.0, 0.0, 1.0 / 3.0], atol=1e-6),
    dict(ref="test_rewards.py:153-174", fn="acceleration", norm="l2", actions=lin, done=None,
         expected=[0.0] * 5, atol=1e-6),
    dict(ref="test_rewards.py:176-199", fn="acceleration", norm="l2", actions=quad, done=None,
         expected=[0.0, 0.0, 4.0, 4.0, 4.0], atol=1e-6),
    dict(ref="test_rewards.py:201-224", fn="acceleration", norm="l1",
         actions=[[0.0, 0, 0], [1.0, 0, 0], [2.0, 0, 0], [2.0, 0, 0], [1.0, 0, 0]], done=None,
         expected=[0.0, 0.0, 0.0, 1.0 / 3.0, 1.0 / 3.0], atol=1e-6),
    dict(ref="test_rewards.py:230-252", fn="jerk", norm="l2", actions=[[float(i * i)] * 3 for i in range(6)],
         done=None, expected=[0.0] * 6, atol=1e-6),
    dict(ref="test_rewards.py:254-271", fn="jerk", norm="l2", actions=[[float(i ** 3)] * 3 for i in range(6)],
         done=None, expected=[0.0, 0.0, 0.0, 36.0, 36.0, 36.0], atol=1e-5),
]

qpos = [1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0, 9.0]
termination_kats = [
    dict(ref="test_terminations.py:66-79", fn="not_upright", qpos=qpos, max_radians=0.1, expected=-1),
    dict(ref="test_terminations.py:66-79", fn="not_upright", qpos=qpos, max_radians=10.0, expected=0),
    dict(ref="test_terminations.py:85-99", fn="minimum_height", qpos=qpos, min_height=4.0, expected=-1),
    dict(ref="test_terminations.py:85-99", fn="minimum_height", qpos=qpos, min_height=2.0, expected=0),
    dict(ref="test_terminations.py:105-113", fn="illegal_contact", ncon=2, geom1=[0, 2], geom2=[1, 3],
         dist=[-0.01, -0.02], illegal=[0, 3], expected=-1),
    dict(ref="test_terminations.py:115-118", fn="illegal_contact", ncon=2, geom1=[0, 2], geom2=[1, 3],
         dist=[-0.01, -0.02], illegal=[4, 5], expected=0),
    dict(ref="test_terminations.py:120-124", fn="illegal_contact", ncon=0, geom1=[0, 2], geom2=[1, 3],
         dist=[-0.01, -0.02], illegal=[0, 1], expected=0),
]

here = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(here, "reward_kats.json"), "w") as f:
    json.dump(reward_kats, f, indent=1)
with open(os.path.join(here, "termination_kats.json"), "w") as f:
    json.dump(termination_kats, f, indent=1)
print("wrote", len(reward_kats), "reward and", len(termination_kats), "termination KATs")
