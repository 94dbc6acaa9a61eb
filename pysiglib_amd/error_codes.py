"""Status code -> message, as the reference does it (pysiglib/error_codes.py:16-54)."""
from ._loader import last_error_message

_MESSAGES = {
    1: "Failed to allocate memory",
    2: "Invalid argument",
    3: "Out of range",
    4: "Filesystem error",
    5: "Could not find prepared cache. Please call the corresponding preparation function with the correct parameters.",
    10: "Runtime error",
    11: "Unknown exception",
}


def err_msg(code):
    if code < 100000:
        text = _MESSAGES.get(code, "Error") + " (" + str(code) + ")"
    else:
        text = "HIP error (" + str(code - 100000) + ")"
    detail = last_error_message()
    return text + (": " + detail if detail else "")
