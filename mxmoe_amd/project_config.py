"""Paths of the run-time artefacts, as in the reference's project_config.py:3-4 (CUR_DIR, CALIB_DIR)."""
import os

CUR_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CALIB_DIR = f"{CUR_DIR}/calib"
