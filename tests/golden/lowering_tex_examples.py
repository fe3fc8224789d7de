"""Known-answer lowered matrices from docs/lowering/type_1/type_1_lowering_pad_stride.tex.

Letters are replaced by their position in the alphabet (a=1 ... y=25); 0 is zero padding.
Each entry: (n, k, p, s, input as n x n, expected lowered matrix as m*m x k*k); d = b = 1.
"""
import numpy as np

_D4 = np.arange(1, 17, dtype=np.float32).reshape(4, 4)
_D5 = np.arange(1, 26, dtype=np.float32).reshape(5, 5)


def _L(rows):
    tab = {c: i + 1 for i, c in enumerate("abcdefghijklmnopqrstuvwxy")}
    tab["0"] = 0
    return np.array([[tab[t] for t in r.split()] for r in rows], dtype=np.float32)


EXAMPLES = [
    # tex:61-75, p=0 s=1
    (4, 2, 0, 1, _D4, _L(["a b e f", "b c f g", "c d g h", "e f i j", "f g j k", "g h k l",
                          "i j m n", "j k n o", "k l o p"])),
    # tex:88-97, p=0 s=2
    (4, 2, 0, 2, _D4, _L(["a b e f", "c d g h", "i j m n", "k l o p"])),
    # tex:115-130, p=1 s=2
    (4, 2, 1, 2, _D4, _L(["0 0 0 a", "0 0 b c", "0 0 d 0", "0 e 0 i", "f g j k", "h 0 l 0",
                          "0 m 0 0", "n o 0 0", "p 0 0 0"])),
    # tex:132-142, p=1 s=3
    (4, 2, 1, 3, _D4, _L(["0 0 0 a", "0 0 c d", "0 i 0 m", "k l o p"])),
    # tex:144-181, n=5 k=3 p=2 s=2
    (5, 3, 2, 2, _D5, _L([
        "0 0 0 0 0 0 0 0 a", "0 0 0 0 0 0 a b c", "0 0 0 0 0 0 c d e", "0 0 0 0 0 0 e 0 0",
        "0 0 a 0 0 f 0 0 k", "a b c f g h k l m", "c d e h i j m n o", "e 0 0 j 0 0 o 0 0",
        "0 0 k 0 0 p 0 0 u", "k l m p q r u v w", "m n o r s t w x y", "o 0 0 t 0 0 y 0 0",
        "0 0 u 0 0 0 0 0 0", "u v w 0 0 0 0 0 0", "w x y 0 0 0 0 0 0", "y 0 0 0 0 0 0 0 0"])),
]
