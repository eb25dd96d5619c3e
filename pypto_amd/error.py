"""Exception types of the operator boundary.

Same names and message convention as the reference's python/pypto/error.py:56-117
(``PyptoError`` carrying ``ErrCode: <hex>, <ExceptionType>: <message>``; ``FeError`` for
everything raised while validating or launching an operator call).
"""

_CODE_UNKNOWN = 0xF00000
_CODES = {TypeError: 0xF00001, ValueError: 0xF00002, RuntimeError: 0xF00003, NotImplementedError: 0xF00005,
          IndexError: 0xF00007}


class PyptoError(Exception):
    def __init__(self, err_code, msg):
        if isinstance(msg, Exception):
            text = str(msg)
            msg = text if "ErrCode" in text else f"ErrCode: {err_code:X}, {type(msg).__name__}: {text}"
        elif "ErrCode" not in msg:
            msg = f"ErrCode: {err_code:X}, {msg}"
        super().__init__(msg)


class PyptoGeneralError(PyptoError):
    def __init__(self, msg):
        code = _CODES.get(type(msg), _CODE_UNKNOWN) if isinstance(msg, Exception) else _CODE_UNKNOWN
        super().__init__(code, msg)
        self.cause_type = type(msg) if isinstance(msg, Exception) else None


class FeError(PyptoGeneralError):
    """Raised for every failure of an operator call (bad operands, launch errors)."""


class PyptoRtError(PyptoGeneralError):
    """Raised when the native library is missing or unusable."""
