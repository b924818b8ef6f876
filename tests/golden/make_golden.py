"""Writes the small known-answer fixtures under tests/golden/.

The reference ships no golden vectors for this path (its scripts only print error norms), so these are
derived by hand from the published formulas: the words below are computed with plain Python integers
(no oracle, no torch), from the pack rule  word = OR_i code[i] << (i*bit)  (quant/pack_unpack.py:40-51)
and from the arange(128) smoke input of quant/pack_unpack.py:382.
"""
import json
from pathlib import Path

HERE = Path(__file__).parent


def pack(codes, bit):
    pf = 32 // bit
    return [sum((c & 0xFFFFFFFF) << (i * bit) for i, c in enumerate(codes[j:j + pf])) & 0xFFFFFFFF
            for j in range(0, len(codes), pf)]


def main():
    cases = [
        dict(name="2bit_0123", bit=2, codes=[0, 1, 2, 3] * 4),
        dict(name="2bit_ramp_two_words", bit=2, codes=[(i * 7) % 4 for i in range(32)]),
        dict(name="4bit_ramp", bit=4, codes=list(range(16))),
        dict(name="8bit_top_bit", bit=8, codes=[255, 0, 128, 1, 2, 3, 4, 200]),
        dict(name="1bit_pattern", bit=1, codes=[1, 0, 0, 1, 1, 1, 0, 0] * 3 + [0, 0, 0, 0, 0, 0, 0, 1]),
    ]
    for c in cases:
        c["words_u32"] = pack(c["codes"], c["bit"])
    (HERE / "pack_vectors.json").write_text(json.dumps({"cases": cases}, indent=1))
    # arange(128) fp16, group 32, 2 bit: scale = fp16(31/3) = 10.3359375, codes = rne(k / 10.3359375)
    codes = [0] * 6 + [1] * 10 + [2] * 10 + [3] * 6
    (HERE / "quant_arange128.json").write_text(json.dumps(
        {"scale": 10.3359375, "zeros": [0, 32, 64, 96], "codes_per_group": codes,
         "words_u32_2bit": pack(codes * 4, 2),
         # 1 bit: scale = 31, codes = rne(k / 31): 15/31 < 0.5 < 16/31
         "scale_1bit": 31.0, "codes_per_group_1bit": [0] * 16 + [1] * 16,
         "words_u32_1bit": pack(([0] * 16 + [1] * 16) * 4, 1)}, indent=1))


if __name__ == "__main__":
    main()
