"""Known-answer vectors for the decode loops, as plain data.

Inputs and expected outputs are the literal arrays held by the reference's own
tests (t5x/decoding_test.py; line ranges given per case).  They are shared by
the CPU oracle tests and by the GPU tests of the HIP-backed decode loops, so
both are checked against the same answers.
"""

import numpy as np

NEG = -1e7
F = np.float32

PICK_2_3 = np.array([[NEG, NEG, 0, NEG], [NEG, NEG, NEG, 0]], dtype=F)
PICK_3_3 = np.array([[NEG, NEG, NEG, 0], [NEG, NEG, NEG, 0]], dtype=F)

# Constant-logit sampling cases: dict(logits, inputs, kwargs, expected[, scores])
SAMPLE_CASES = {
    # decoding_test.py:36-56
    'uneven_prefix': dict(
        logits=PICK_2_3,
        inputs=[[0, 5, 7, 1, 0, 0], [0, 6, 1, 0, 0, 0]],
        kwargs=dict(topk=0, initial_index=np.array([3, 2], np.int32)),
        expected=[[5, 7, 1, 2, 2, 2], [6, 1, 3, 3, 3, 3]]),
    # :58-75
    'no_prefix': dict(
        logits=PICK_2_3, inputs=np.zeros((2, 3), np.int32).tolist(),
        kwargs=dict(topk=0), expected=[[2, 2, 2], [3, 3, 3]]),
    # :77-93
    'prefix': dict(
        logits=PICK_2_3, inputs=[[0, 5, 6, 7, 0], [0, 8, 9, 0, 0]],
        kwargs=dict(topk=0), expected=[[5, 6, 7, 2, 2], [8, 9, 3, 3, 3]]),
    # :95-119 (near-equal large logits, greedy)
    'zero_temperature': dict(
        logits=np.array([[1700.47, 1700.48, 1700.51, 1700.45],
                         [3.2, 4.8, -5.3, 5.6]], dtype=F),
        inputs=np.zeros((2, 3), np.int32).tolist(),
        kwargs=dict(topk=4, temperature=0.0),
        expected=[[2, 2, 2], [3, 3, 3]]),
    # :121-138
    'prefix_ending_with_eos': dict(
        logits=PICK_2_3, inputs=[[0, 5, 6, 1, 0], [0, 8, 1, 0, 0]],
        kwargs=dict(topk=1), expected=[[5, 6, 1, 2, 2], [8, 1, 3, 3, 3]]),
    # :256-281
    'greedy_topk_rescaled': dict(
        logits=np.array([[NEG, NEG, -0.510825624, -0.916290732]], dtype=F),
        inputs=[[0, 2, 2, 2, 0]],
        kwargs=dict(topk=1, rescale_log_probs=True),
        expected=[[2, 2, 2, 2, 2]], scores=[0.0]),
    # :283-299
    'greedy_topk_not_rescaled': dict(
        logits=np.array([[NEG, NEG, -0.510825624, -0.916290732]], dtype=F),
        inputs=[[0, 2, 2, 3, 0]],
        kwargs=dict(topk=1, rescale_log_probs=False),
        expected=[[2, 2, 3, 2, 2]], scores=[-1.02165125]),
}

# `temperature_sample` (outer function) cases with call counts.
# dict(logits, inputs, kwargs, expected [B, L], scores, calls)
OUTER_SAMPLE_CASES = {
    # :451-506
    'max_steps_no_initial_index': dict(
        logits=PICK_3_3,
        inputs=[[0, 2, 0, 0, 0, 0, 0, 0], [0, 2, 2, 0, 0, 0, 0, 0]],
        kwargs=dict(topk=4, max_decode_steps=4, initial_index=None),
        expected=[[2, 3, 3, 3, 3, 0, 0, 0], [2, 2, 3, 3, 3, 3, 0, 0]],
        scores=[[0.0], [0.0]], calls=6),
    'max_steps_initial_index': dict(
        logits=PICK_3_3,
        inputs=[[0, 2, 0, 0, 0, 0, 0, 0], [0, 2, 2, 0, 0, 0, 0, 0]],
        kwargs=dict(topk=4, max_decode_steps=4,
                    initial_index=np.array([1, 2], np.int32)),
        expected=[[2, 3, 3, 3, 3, 0, 0, 0], [2, 2, 3, 3, 3, 3, 0, 0]],
        scores=[[0.0], [0.0]], calls=4),
    'max_steps_lower_initial_index': dict(
        logits=PICK_3_3,
        inputs=[[0, 2, 0, 0, 0, 0, 0, 0], [0, 2, 2, 0, 0, 0, 0, 0]],
        kwargs=dict(topk=4, max_decode_steps=4,
                    initial_index=np.array([1, 1], np.int32)),
        expected=[[2, 3, 3, 3, 3, 0, 0, 0], [2, 2, 3, 3, 3, 3, 0, 0]],
        scores=[[0.0], [0.0]], calls=5),
    # :508-564
    'max_steps_endpad': dict(
        logits=np.array([[NEG, NEG, NEG, 0]] * 3, dtype=F),
        inputs=[[0, 2, 0, 0, 0, 0, 0, 0], [0, 2, 2, 2, 2, 2, 2, 0],
                [0, 2, 2, 2, 0, 0, 0, 0]],
        kwargs=dict(topk=4, max_decode_steps=4,
                    initial_index=np.array([1, 6, 0])),
        expected=[[2, 3, 3, 3, 3, 0, 0, 0], [2, 2, 2, 2, 2, 2, 3, 3],
                  [2, 2, 2, 3, 3, 3, 3, 0]],
        scores=[[0.0], [0.0], [0.0]], calls=7),
    # :566-600
    'docstring_ex4': dict(
        logits=PICK_2_3,
        inputs=[[0, 2, 0, 0, 0, 0, 0, 0], [0, 3, 4, 0, 0, 0, 0, 0]],
        kwargs=dict(topk=4, max_decode_steps=2,
                    initial_index=np.array([1, 2])),
        expected=[[2, 2, 2, 0, 0, 0, 0, 0], [3, 4, 3, 3, 0, 0, 0, 0]],
        scores=None, calls=2),
    # :602-637
    'hard_limit': dict(
        logits=PICK_3_3,
        inputs=[[0, 2, 0, 0, 0, 0, 0, 0], [0, 2, 2, 0, 0, 0, 0, 0]],
        kwargs=dict(topk=4, max_decode_steps=10,
                    max_decode_steps_hard_limit=4),
        expected=[[2, 3, 3, 3, 3, 0, 0, 0], [2, 2, 3, 3, 3, 3, 0, 0]],
        scores=[[0.0], [0.0]], calls=None),
    # :639-659  logits ~ probs (0.3, 0, 0.1, 0.6)
    'topp_055': dict(
        logits=np.array([[-1.2, NEG, -2.3, -0.51]], dtype=F),
        inputs=np.zeros((1, 20), np.int32).tolist(),
        kwargs=dict(topp=0.55, topk=0),
        expected=[[3] * 20], scores=[[0.0]], calls=None),
    # :661-678
    'topp_063_temp_08': dict(
        logits=np.array([[-1.2, NEG, -2.3, -0.51]], dtype=F),
        inputs=np.zeros((1, 20), np.int32).tolist(),
        kwargs=dict(temperature=0.8, topp=0.63, topk=0),
        expected=[[3] * 20], scores=[[0.0]], calls=None),
    # :736-769
    'topp_max_decode_steps': dict(
        logits=np.array([[-1.2, NEG, -2.3, -0.51]], dtype=F),
        inputs=np.zeros((1, 20), np.int32).tolist(),
        kwargs=dict(temperature=0.8, topp=0.63, topk=0, max_decode_steps=10),
        expected=[[3] * 10 + [0] * 10], scores=[[0.0]], calls=None),
}

# :680-734  per-item temperature, 4 items x 2 decodes.
PER_ITEM_TEMPERATURE = dict(
    logits=np.repeat(np.array([[-1.2, NEG, -2.3, -0.51],
                               [-0.51, -1.2, NEG, -2.3],
                               [-1.2, NEG, -0.51, -2.3],
                               [-1.2, -0.51, NEG, -2.3]], dtype=F), 2, axis=0),
    inputs=np.zeros((4, 20), np.int32),
    kwargs=dict(temperature=np.array([0.5, 0, 0.3, 0.2]), topp=0.63, topk=0,
                num_decodes=2),
    expected=np.repeat(np.array([[3] * 20, [0] * 20, [2] * 20,
                                 [1] + [0] * 19])[:, None, :], 2, axis=1),
    scores=[[0.0, 0.0]] * 4)

# :214-254 / :301-344  forced draws per loop step (categorical seam).
FORCED_DRAWS = dict(
    draws=[[2, 3], [2, 3], [2, 3], [2, 1], [1, 3], [2, 3], [2, 3]],
    inputs=[[0, 5, 1, 0, 0, 0, 0], [0, 8, 0, 0, 0, 0, 0]],
    expected=[[5, 1, 2, 2, 1, 0, 0], [8, 3, 3, 1, 0, 0, 0]],
    # log-prob terms per row: (row, token) pairs whose log-probs are summed.
    logprob_terms=[[(0, 2), (0, 2), (0, 1)], [(1, 3), (1, 3), (1, 1)]])

# :346-449
NUM_DECODES = dict(
    inputs=[[0, 5, 1, 0], [0, 8, 7, 0]],
    trial_decodes=[[5, 1, 4, 4], [5, 1, 5, 5], [5, 1, 3, 3],
                   [8, 7, 5, 5], [8, 7, 3, 3], [8, 7, 4, 4]],
    trial_log_prob=[-2.3, -1.3, -3.6, -0.5, -2.5, -1.9],
    expanded_inputs=[[0, 5, 1, 0]] * 3 + [[0, 8, 7, 0]] * 3,
    initial_index=[1, 2], expanded_initial_index=[1, 1, 1, 2, 2, 2],
    decodes=[[[5, 1, 3, 3], [5, 1, 4, 4], [5, 1, 5, 5]],
             [[8, 7, 3, 3], [8, 7, 4, 4], [8, 7, 5, 5]]],
    scores=[[-3.6, -2.3, -1.3], [-2.5, -1.9, -0.5]])

# :771-804
TOPP_LOG_PROBS = dict(
    logits=np.array([[-1.2, NEG, -2.3, -0.51]], dtype=F),
    kwargs=dict(temperature=1.4, topp=0.7, topk=0),
    seen_logits=[[-0.85714293, NEG, NEG, -0.36428571]])

# Beam search constant-logit cases (beam 2): per batch item logits row.
BEAM_LOGITS_4 = np.array([[NEG, -1e10, -0.1, -0.9], [NEG, -1e10, -0.9, -0.1]],
                         dtype=F)
BEAM_LOGITS_8 = np.array(
    [[NEG, -1e10, -0.1, -0.9, -1e4, -1e4, -1e4, -1e4],
     [NEG, -1e10, -0.9, -0.1, -1e4, -1e4, -1e4, -1e4]], dtype=F)
BEAM_LOGITS_8_EOS = np.array(
    [[NEG, -1e10, -0.1, -0.9, -1e4, -1e4, -1e4, -1e4],
     [NEG, -1.0, -0.9, -0.1, -1e4, -1e4, -1e4, -1e4]], dtype=F)

BEAM_CASES = {
    # :1071-1132
    'force_decode_prefix': dict(
        logits=BEAM_LOGITS_8, inputs=[[0, 7, 0, 0, 0], [0, 4, 5, 0, 0]],
        kwargs=dict(alpha=0),
        expected=[[[7, 3, 2, 2, 2], [7, 2, 2, 2, 2]],
                  [[4, 5, 2, 3, 3], [4, 5, 3, 3, 3]]],
        score_prompt=[[7, 0, 0, 0, 0], [4, 5, 0, 0, 0]]),
    # :1134-1166
    'no_prefix': dict(
        logits=BEAM_LOGITS_4, inputs=[[0, 0, 0, 0, 0], [0, 0, 0, 0, 0]],
        kwargs=dict(),
        expected=[[[3, 2, 2, 2, 2], [2, 2, 2, 2, 2]],
                  [[2, 3, 3, 3, 3], [3, 3, 3, 3, 3]]]),
    # :1325-1362
    'min_log_prob': dict(
        logits=BEAM_LOGITS_4, inputs=[[0, 0, 0, 0, 0], [0, 0, 0, 0, 0]],
        kwargs=dict(min_log_prob=-0.05),
        expected=[[[3, 0, 0, 0, 0], [2, 0, 0, 0, 0]],
                  [[2, 0, 0, 0, 0], [3, 0, 0, 0, 0]]]),
    # :1364-1401
    'max_decode_step': dict(
        logits=BEAM_LOGITS_4, inputs=[[0, 0, 0, 0, 0], [0, 0, 0, 0, 0]],
        kwargs=dict(max_decode_step=2),
        expected=[[[3, 2, 0, 0, 0], [2, 2, 0, 0, 0]],
                  [[2, 3, 0, 0, 0], [3, 3, 0, 0, 0]]]),
    # :1208-1323
    'prefix_initial_index': dict(
        logits=BEAM_LOGITS_8_EOS, inputs=[[0, 7, 0, 0, 0], [0, 4, 5, 0, 0]],
        kwargs=dict(alpha=0, initial_index=np.array([1, 2], np.int32)),
        expected=[[[7, 3, 2, 2, 2], [7, 2, 2, 2, 2]],
                  [[4, 5, 3, 1, 0], [4, 5, 1, 0, 0]]],
        score_prompt=[[7, 0, 0, 0, 0], [4, 5, 0, 0, 0]],
        first_tokens=[[7], [7], [5], [5]], with_cache=True),
    # :1403-1472
    'prefix_initial_index_max_decode_step': dict(
        logits=BEAM_LOGITS_8_EOS, inputs=[[0, 7, 0, 0, 0], [0, 4, 5, 0, 0]],
        kwargs=dict(alpha=0, initial_index=np.array([1, 2], np.int32),
                    max_decode_step=2),
        expected=[[[7, 3, 2, 0, 0], [7, 2, 2, 0, 0]],
                  [[4, 5, 3, 1, 0], [4, 5, 1, 0, 0]]],
        with_cache=True),
}

# :1168-1206
ALIGN = dict(
    prompts=[[0, 0, 0, 0, 0, 0, 0], [1, 2, 3, 4, 5, 6, 7],
             [0, 1, 0, 0, 0, 0, 0], [0, 1, 2, 0, 0, 0, 0],
             [0, 1, 2, 3, 0, 0, 0]],
    right=[[0, 0, 0, 0, 0, 0, 0], [1, 2, 3, 4, 5, 6, 7],
           [0, 0, 0, 0, 0, 0, 1], [0, 0, 0, 0, 0, 1, 2],
           [0, 0, 0, 0, 1, 2, 3]],
    left=[[0, 0, 0, 0, 0, 0, 0], [1, 2, 3, 4, 5, 6, 7],
          [1, 0, 0, 0, 0, 0, 0], [1, 2, 0, 0, 0, 0, 0],
          [1, 2, 3, 0, 0, 0, 0]])


def markov_edge_potentials():
  """The 4-state first-order Markov toy of decoding_test.py:963-1010.

  States: PAD=0, A=1, B=2, START=3, END=4.  Returns (edge_potentials[6,5,5],
  logits0[5]); the best two length-7 paths tie: START-AABBA-END and
  START-BBAAB-END.
  """
  ab = np.asarray([[[1, -1], [-1, 1]], [[-1, 1], [1, -1]],
                   [[1, -1], [-1, 1]], [[-1, 1], [1, -1]]])
  edge = np.ones([6, 5, 5]) * NEG
  edge[1:5, 1:3, 1:3] = ab
  edge[0, 3, 1] = 0
  edge[0, 3, 2] = 0
  edge[5, 1, 4] = 0
  edge[5, 2, 4] = 0
  edge[:, 0, :] = 0
  logits0 = np.asarray([NEG, NEG, NEG, 0, NEG])
  return edge.astype(F), logits0.astype(F)


MARKOV_STATES = ['PAD', 'A', 'B', 'START-', '-END']
MARKOV_EXPECTED = ['START-AABBA-END', 'START-BBAAB-END']
