class TensorLayout:
    """Layout of the last three page dimensions (tidal/utils/utils.py:1-5 of the reference)."""

    NHD = 0
    HND = 1

    FORMAT2STR = {0: "NHD", 1: "HND"}
