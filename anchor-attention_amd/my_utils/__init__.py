"""Minimal stand-in for the reference's ``my_utils`` package: only the ``Logger`` the operator
calls (``my_utils/my_log/log_performance.py:7-56``).  Messages go to ``log/application.log``
unless ``ANCHOR_ATTN_LOG=0`` is exported."""
import datetime
import os
import time


class Logger:
    log_file_path = "log/application.log"
    enabled = os.environ.get("ANCHOR_ATTN_LOG", "1") != "0"

    @classmethod
    def set_log_file_path(cls, path: str = None):
        cls.log_file_path = os.path.join("log", path or str(time.time()))

    @classmethod
    def log(cls, message: str):
        if not cls.enabled:
            return
        try:
            directory = os.path.dirname(cls.log_file_path)
            if directory:
                os.makedirs(directory, exist_ok=True)
            stamp = datetime.datetime.now().strftime("%Y-%m-%d %H:%M:%S.%f")[:-3]
            with open(cls.log_file_path, "a") as f:
                f.write(f"{stamp} - {message}\n")
        except OSError as e:
            print(f"Unable to write to log file: {e}")

    @classmethod
    def log_error(cls, m: str):
        cls.log(f"ERROR: {m}")

    @classmethod
    def log_warning(cls, m: str):
        cls.log(f"WARNING: {m}")

    @classmethod
    def log_info(cls, m: str):
        cls.log(f"INFO: {m}")
