"""Collects what the parity gates measured, for the summary pytest prints at the end of a run.

Every gate call records the plain figure of the stated tolerance, max|y - y_ref| / rms(y_ref),
and the fraction of elements over 2e-2 * rms, whether or not its test asserts the plain bound;
`pytest -q` drops what tests print, the terminal summary it keeps."""
import json
import os

RECORDS = []          # dicts: name, max_err_over_rms, over_frac, elems, plain_asserted


def record(name: str, worst: float, over_frac: float, elems: int, plain_asserted: bool, floor: float = 0.0) -> None:
    """floor: the same figure for y_ref itself rounded to the output type (what exact arithmetic scores)."""
    RECORDS.append({"name": name, "max_err_over_rms": worst, "over_frac": over_frac, "elems": elems,
                    "plain_asserted": plain_asserted, "rounding_floor": floor})


def summary_lines():
    if not RECORDS:
        return []
    named = [r for r in RECORDS if r["name"].startswith(("c1", "c2", "c3", "c4", "c5"))]
    lines = ["parity vs the oracle's reference-rounded form, max|err| / rms (tolerance 2e-2):"]
    for r in named:
        lines.append(f"  {r['name']}: {r['max_err_over_rms']:.3e}  (over 2e-2*rms: {r['over_frac']:.1e} of {r['elems']}; "
                     f"y_ref rounded to the output type: {r['rounding_floor']:.3e})")
    within = [r for r in RECORDS if r["max_err_over_rms"] <= 2e-2]
    beyond = [r for r in RECORDS if r["max_err_over_rms"] > 2e-2]
    asserted = sum(1 for r in RECORDS if r["plain_asserted"])
    line = (f"  {len(RECORDS)} gate calls: {len(within)} within the plain bound 2e-2*rms ({asserted} of them assert it "
            f"outright, worst {max((r['max_err_over_rms'] for r in within), default=0.0):.3e})")
    if beyond:
        worst = max(beyond, key=lambda r: r["max_err_over_rms"])
        line += (f"; {len(beyond)} beyond it, all within 2e-2*rms + the storage quanta of the 16-bit tensors, every excess "
                 f"element of the one-expert gates and of the full-size calls classified one by one "
                 f"(worst {worst['max_err_over_rms']:.3e}: {worst['name']}, {worst['over_frac']:.1e} of its {worst['elems']} elements)")
    lines.append(line)
    return lines


def dump_if_asked() -> None:
    path = os.environ.get("EK_PARITY_REPORT")
    if path and RECORDS:
        with open(path, "w") as f:
            json.dump(RECORDS, f, indent=0)
