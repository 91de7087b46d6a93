"""The Rust binding crates under rust/ cannot be compiled here (no Rust toolchain in the image); what can be
checked is that they are complete and consistent with the C header: the generated sys crate is up to date
and declares every entry point, and every `sys::ft_*` the safe crate calls exists with that many arguments."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SYS = os.path.join(ROOT, "rust", "ferrotensor-hip-sys")
SAFE_DIR = os.path.join(ROOT, "rust", "ferrotensor-backend-hip", "src")
SAFE = [os.path.join(SAFE_DIR, f) for f in ("lib.rs", "step.rs")]


def header_functions():
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "ferrotensor_hip.h")).read(), flags=re.S)
    out = {}
    for name, args in re.findall(r"\n(?:const )?\w+\*?\s+\*?(ft_\w+)\s*\(([^;]*?)\)\s*;", text):
        args = " ".join(args.split())
        out[name] = 0 if args in ("", "void") else len(args.split(","))
    return out


def test_sys_crate_is_generated_from_the_current_header():
    r = subprocess.run([sys.executable, os.path.join(SYS, "gen_bindings.py"), "--check"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr + r.stdout


def test_sys_crate_declares_every_entry_point():
    want = header_functions()
    assert len(want) >= 80
    text = open(os.path.join(SYS, "src", "lib.rs")).read()
    got = {}
    for name, args in re.findall(r"pub fn (ft_\w+)\(([^)]*)\)", text):
        got[name] = 0 if not args.strip() else len(args.split(","))
    assert got == want


def test_safe_crate_calls_existing_entry_points_with_the_right_arity():
    want = header_functions()
    text = "\n".join(open(f).read() for f in SAFE)
    calls = list(re.finditer(r"sys::(ft_\w+)\(", text))
    assert len(calls) >= 70
    for m in calls:
        name = m.group(1)
        assert name in want, name
        depth, i, commas, any_arg = 1, m.end(), 0, False
        while depth:
            ch = text[i]
            if ch in "([{":
                depth += 1
            elif ch in ")]}":
                depth -= 1
            elif ch == "," and depth == 1:
                commas += 1
            elif not ch.isspace():
                any_arg = True
            if ch == "|" :   # closures inside arguments are not used in these calls
                raise AssertionError("unexpected closure in a call of " + name)
            i += 1
        n = commas + 1 if any_arg else 0
        assert n == want[name], (name, n, want[name])


def test_step_driver_wrappers_cover_the_model_and_trainer_entry_points():
    """`Lfm2Model` / `Trainer` of step.rs reach every ft_model_* / ft_trainer_* entry point and the host half
    of train_batch, and carry the reference's method names (ferrotensor-trainer/src/lib.rs:154-213, 228, 371, 426)."""
    text = open(SAFE[1]).read()
    called = set(re.findall(r"sys::(ft_\w+)\(", text))
    want = {n for n in header_functions() if n.startswith(("ft_model_", "ft_trainer_", "ft_train_batch_"))}
    want |= {"ft_pad_chunk", "ft_chunk_padded_len"}
    want -= {"ft_model_set_head_all_rows"}   # a benchmark switch, not part of the reference's surface
    assert want <= called, sorted(want - called)
    for name in ("with_grad_accum_steps", "with_clip_grad_norm", "with_lr_scheduler", "with_length_bucket",
                 "train_step_masked", "train_batch", "train_chunk", "set_optimizer_steps", "optimizer_steps",
                 "forward_batch", "named_params"):
        assert re.search(r"pub fn %s\(" % name, text), name
    fields = re.search(r"pub struct StepStats \{(.*?)\}", text, re.S).group(1)
    for field in ("loss: f32", "tokens: usize", "optimizer_step: bool", "grad_norm: Option<f32>", "lr: Option<f32>"):
        assert field in fields, field
