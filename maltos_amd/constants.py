"""Batch keys and sentinels, identical to the reference's utils/constants.py:1-29."""
IGNORE_INDEX = -100
PAD_SEQUENCE_ID = -1

INPUT_IDS_KEY = "input_ids"
LABELS_KEY = "labels"
POSITION_IDS_KEY = "position_ids"
SEQUENCE_IDS_KEY = "sequence_ids"
POSITION_OFFSET_KEY = "position_offset"
LOSS_WEIGHT_KEY = "loss_weight"
HIDDEN_STATES_KEY = "hidden_states"
