"""python -m trinity_amd.evaluation.convert_ffn_falcon --n 0 --o 2"""
from .convert_ffn import run

if __name__ == "__main__":
    raise SystemExit(run("falcon"))
