"""Per-computation entry points, tensor-metadata configs and canonical IR
cases (the reference's convert_eval_rms.py / convert_ffn_*.py / run_baseline.py
and evaluation/*.json surface)."""
