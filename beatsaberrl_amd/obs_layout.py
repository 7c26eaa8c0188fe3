"""Observation lane contract of the env (obs v49, 630 lanes) as the policy reads it.

Restates the routing tables of the reference (python/policy.py:174-275; source of
truth: python/beat_arena_env/constants.py:461-496): which obs lanes form the two
saber tokens, the torso token and the two leg tokens, where the 24 x 18 entity
block and its slot mask sit, and the lanes inside a saber token that the
note-geometry features read (python/policy.py:319-326)."""

OBS_DIM = 630
N_NOTE_SLOTS = 24
NOTE_FEAT = 18
OFF_NOTES = 102
OFF_NOTE_MASK = OFF_NOTES + N_NOTE_SLOTS * NOTE_FEAT      # 534
OFF_GROUND = OFF_NOTE_MASK + N_NOTE_SLOTS                 # 558: [L_heel, L_toe, R_heel, R_toe]
OFF_BODY_PTS = OFF_GROUND + 4                             # 562: l_elbow r_elbow l_knee r_knee l_foot r_foot (x3)
OFF_BODY_PT_VEL = OFF_BODY_PTS + 18                       # 580
OFF_PREV_L = OFF_BODY_PT_VEL + 18                         # 598
OFF_PREV_R = OFF_PREV_L + 5                               # 603
OFF_TAU = OFF_PREV_R + 5                                  # 608: spine 3, arm 7, leg 6
OFF_TIP_VEL = OFF_TAU + 16                                # 624: [L xyz, R xyz]
OBS_HEAD_Z = 99

SABER_FEAT = 47
TORSO_FEAT = 29
LEG_FEAT = 32
N_LEAD = 5                    # [saber_L, saber_R, torso, leg_L, leg_R]
NOTE_GEO_FEAT = 22
N_ACTION_HEADS = 29
MASK_BIAS = 16384.0           # python/policy.py:428
MASKED_LOGIT = -1e9           # python/policy.py:434


def _span(*pairs):
    lanes = []
    for lo, n in pairs:
        lanes.extend(range(lo, lo + n))
    return tuple(lanes)


# q lanes 15..45 (spine 3, arm_L 8, arm_R 8, leg_L 6, leg_R 6); qd lanes 46..74 (3, 7, 7, 6, 6);
# hand blocks 75..85 / 86..96 (wrist pos 3, wrist vel 3, blade dir 3, meter, post_rem); head 97..99; contacts 100..101
_ARM_TAU = (OFF_TAU + 3, 7)
_LEG_TAU = (OFF_TAU + 10, 6)
SABER_L_IDX = _span((18, 8), (49, 7), (75, 11), (OFF_BODY_PTS, 3), (OFF_BODY_PT_VEL, 3), (OFF_PREV_L, 5), _ARM_TAU,
                    (OFF_TIP_VEL, 3))
SABER_R_IDX = _span((26, 8), (56, 7), (86, 11), (OFF_BODY_PTS + 3, 3), (OFF_BODY_PT_VEL + 3, 3), (OFF_PREV_R, 5),
                    _ARM_TAU, (OFF_TIP_VEL + 3, 3))
TORSO_IDX = _span((0, 18), (46, 3), (97, 5), (OFF_TAU, 3))
LEG_L_IDX = _span((34, 6), (63, 6), (OFF_GROUND, 2), (OFF_BODY_PTS + 6, 3), (OFF_BODY_PTS + 12, 3),
                  (OFF_BODY_PT_VEL + 6, 3), (OFF_BODY_PT_VEL + 12, 3), _LEG_TAU)
LEG_R_IDX = _span((40, 6), (69, 6), (OFF_GROUND + 2, 2), (OFF_BODY_PTS + 9, 3), (OFF_BODY_PTS + 15, 3),
                  (OFF_BODY_PT_VEL + 9, 3), (OFF_BODY_PT_VEL + 15, 3), _LEG_TAU)
BODY3_IDX = TORSO_IDX + LEG_L_IDX + LEG_R_IDX

assert len(SABER_L_IDX) == len(SABER_R_IDX) == SABER_FEAT
assert len(TORSO_IDX) == TORSO_FEAT and len(LEG_L_IDX) == len(LEG_R_IDX) == LEG_FEAT
assert OFF_TIP_VEL + 6 == OBS_DIM

# lanes inside a 47-lane saber token, and the obs normalisers the geometry decodes with
S_WPOS, S_WVEL, S_BLADE, S_TIPV = 15, 18, 21, 44
X_NORM, Y_NORM, Z_SCALE, V_NORM, HANDLE_LEN = 1.0, 0.75, 8.0, 6.0, 0.16
