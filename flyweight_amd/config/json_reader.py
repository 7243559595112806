"""A small JSON reader of the engine's own, for the three documents it reads: config.json, a
safetensors header, ``model.safetensors.index.json``.

Properties, after the reference's dependency-free parser
(native/include/flyweight_v2_json.hpp:85-272): recursive descent over the bytes of the
document; nesting limited to 64 levels, so a malformed file cannot run the parser off the stack;
integers are read from their literal (Python integers are exact at any size: the 64-bit offsets
of a large checkpoint survive; the reference keeps the literal beside a double for that), and
other numbers keep their literal in ``Number.literal``; errors name the byte offset; anything
but white space behind the document is refused; a key that appears twice is refused (the
reference's map keeps the first silently).
"""

from __future__ import annotations

from typing import Any, Dict, List, Union

MAX_DEPTH = 64
_SPACE = b" \t\n\r"
_ESCAPES = {ord('"'): '"', ord("\\"): "\\", ord("/"): "/", ord("b"): "\b", ord("f"): "\f", ord("n"): "\n",
            ord("r"): "\r", ord("t"): "\t"}


class JsonError(ValueError):
    def __init__(self, what: str, offset: int):
        super().__init__(f"invalid JSON at byte {offset}: {what}")
        self.offset = offset


class Number(float):
    """A number that is not an integer literal: its value, and the text it was written as."""

    def __new__(cls, literal: str):
        self = super().__new__(cls, literal)
        self.literal = literal
        return self


MAX_INTEGER_DIGITS = 64


class _Parser:
    def __init__(self, data: bytes):
        self.data = data
        self.at = 0

    def fail(self, what: str, at: int = None):
        raise JsonError(what, self.at if at is None else at)

    def skip_space(self) -> None:
        data, at, end = self.data, self.at, len(self.data)
        while at < end and data[at] in _SPACE:
            at += 1
        self.at = at

    def peek(self) -> int:
        if self.at >= len(self.data):
            self.fail("the document ends here")
        return self.data[self.at]

    def value(self, depth: int) -> Any:
        if depth > MAX_DEPTH:
            self.fail(f"nested deeper than {MAX_DEPTH} levels")
        self.skip_space()
        c = self.peek()
        if c == ord("{"):
            return self.object(depth)
        if c == ord("["):
            return self.array(depth)
        if c == ord('"'):
            return self.string()
        if c == ord("-") or ord("0") <= c <= ord("9"):
            return self.number()
        for word, result in ((b"true", True), (b"false", False), (b"null", None)):
            if self.data.startswith(word, self.at):
                self.at += len(word)
                return result
        self.fail("expected a value")

    def object(self, depth: int) -> Dict[str, Any]:
        self.at += 1
        result: Dict[str, Any] = {}
        self.skip_space()
        if self.peek() == ord("}"):
            self.at += 1
            return result
        while True:
            self.skip_space()
            if self.peek() != ord('"'):
                self.fail("expected a key in quotes")
            key_at = self.at
            key = self.string()
            if key in result:
                self.fail(f"key '{key}' appears twice", key_at)
            self.skip_space()
            if self.peek() != ord(":"):
                self.fail("expected ':'")
            self.at += 1
            result[key] = self.value(depth + 1)
            self.skip_space()
            c = self.peek()
            self.at += 1
            if c == ord("}"):
                return result
            if c != ord(","):
                self.fail("expected ',' or '}'", self.at - 1)

    def array(self, depth: int) -> List[Any]:
        self.at += 1
        result: List[Any] = []
        self.skip_space()
        if self.peek() == ord("]"):
            self.at += 1
            return result
        while True:
            result.append(self.value(depth + 1))
            self.skip_space()
            c = self.peek()
            self.at += 1
            if c == ord("]"):
                return result
            if c != ord(","):
                self.fail("expected ',' or ']'", self.at - 1)

    def string(self) -> str:
        data = self.data
        start = self.at
        self.at += 1
        pieces: List[str] = []
        run = self.at
        while True:
            if self.at >= len(data):
                self.fail("a string is not closed", start)
            c = data[self.at]
            if c == ord('"'):
                pieces.append(self._text(run, self.at))
                self.at += 1
                return "".join(pieces)
            if c < 0x20:
                self.fail("a control character inside a string")
            if c != ord("\\"):
                self.at += 1
                continue
            pieces.append(self._text(run, self.at))
            if self.at + 1 >= len(data):
                self.fail("a string is not closed", start)
            e = data[self.at + 1]
            if e in _ESCAPES:
                pieces.append(_ESCAPES[e])
                self.at += 2
            elif e == ord("u"):
                escape = self.at
                code = self._hex4(self.at + 2)
                self.at += 6
                if 0xD800 <= code < 0xDC00 and data[self.at:self.at + 2] == b"\\u":     # a surrogate pair
                    low = self._hex4(self.at + 2)
                    if 0xDC00 <= low < 0xE000:
                        code = 0x10000 + ((code - 0xD800) << 10) + (low - 0xDC00)
                        self.at += 6
                if 0xD800 <= code < 0xE000:
                    self.fail("half of a surrogate pair stands alone", escape)      # no character: it could not be written out again
                pieces.append(chr(code))
            else:
                self.fail("unknown escape in a string")
            run = self.at

    def _text(self, begin: int, end: int) -> str:
        try:
            return self.data[begin:end].decode("utf-8")
        except UnicodeDecodeError:
            self.fail("a string is not UTF-8", begin)

    def _hex4(self, at: int) -> int:
        digits = self.data[at:at + 4]
        # (int(..., 16) alone would also take a sign, blanks and underscores)
        if len(digits) != 4 or any(d not in b"0123456789abcdefABCDEF" for d in digits):
            self.fail("\\u needs four hexadecimal digits", at)
        return int(digits, 16)

    def number(self) -> Union[int, Number]:
        data, start = self.data, self.at
        at = start
        if data[at] == ord("-"):
            at += 1
        digits = at
        while at < len(data) and ord("0") <= data[at] <= ord("9"):
            at += 1
        if at == digits or (data[digits] == ord("0") and at - digits > 1):
            self.fail("a number needs digits, and no leading zero", start)
        whole = True
        if at < len(data) and data[at] == ord("."):
            whole = False
            at += 1
            fraction = at
            while at < len(data) and ord("0") <= data[at] <= ord("9"):
                at += 1
            if at == fraction:
                self.fail("a number needs digits behind its point", start)
        if at < len(data) and data[at] in b"eE":
            whole = False
            at += 1
            if at < len(data) and data[at] in b"+-":
                at += 1
            exponent = at
            while at < len(data) and ord("0") <= data[at] <= ord("9"):
                at += 1
            if at == exponent:
                self.fail("a number needs digits in its exponent", start)
        self.at = at
        literal = data[start:at].decode("ascii")
        if not whole:
            return Number(literal)
        # Whole numbers are exact at any size a file can mean (64-bit offsets and beyond); a run of
        # thousands of digits means nothing, and converting it takes time that grows with its square.
        if at - digits > MAX_INTEGER_DIGITS:
            self.fail(f"a whole number of more than {MAX_INTEGER_DIGITS} digits", start)
        return int(literal)


def parse(document: Union[bytes, bytearray, memoryview, str]) -> Any:
    """The value a JSON document holds (objects as dict, arrays as list)."""
    data = document.encode("utf-8") if isinstance(document, str) else bytes(document)
    parser = _Parser(data)
    result = parser.value(1)
    parser.skip_space()
    if parser.at != len(data):
        parser.fail("something follows the document")
    return result


def parse_file(path: str) -> Any:
    with open(path, "rb") as handle:
        return parse(handle.read())
