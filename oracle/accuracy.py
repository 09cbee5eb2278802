"""Error accounting for the Black-Scholes configuration against the oracle.

TEST INFRASTRUCTURE, NOT PRODUCT CODE (used by tests/ and by bench.py's parity leg; the
delayrepay_amd package never imports it).

The stated bars for a transcendental expression are <= 2 ulp (float32) and <= 1e-13
relative (float64) of the *result* against the CPU evaluation.  A Black-Scholes price is
a difference of two terms of the size of max(S, K): for options far out of the money the
terms cancel and a last-bit difference in either term is an arbitrarily large relative
difference in the price, in the CPU evaluation as much as on the device.  `bs_report`
therefore measures the result-relative figures on nested subsets |price| >= 2^-k max(S, K)
(k = 0: no cancellation at all) next to the error scaled by max(S, K) over everything,
reports where each maximum occurs, and at those points also measures the oracle's own
error against a 50-digit evaluation (mpmath), so that a large figure can be read as
"cancellation, shared by both" or "the device is off".
"""
import numpy as np

THRESHOLDS = (0, 1, 2, 4, 8, 16)


def ulp_distance(a, b):
    """Distance in units in the last place between same-dtype float arrays (0 where both
    are NaN, infinite where one is)."""
    a = np.asarray(a)
    b = np.asarray(b)
    assert a.dtype == b.dtype and a.dtype.kind == "f"
    itype = np.int32 if a.dtype.itemsize == 4 else np.int64
    ia = a.view(itype).astype(np.int64)
    ib = b.view(itype).astype(np.int64)
    top = np.int64(np.iinfo(itype).min)
    ia = np.where(ia < 0, top - ia, ia)   # map to a monotone integer line
    ib = np.where(ib < 0, top - ib, ib)
    dist = np.abs(ia - ib).astype(np.float64)
    both_nan = np.isnan(a) & np.isnan(b)
    one_nan = np.isnan(a) ^ np.isnan(b)
    dist = np.where(both_nan, 0.0, dist)
    dist = np.where(one_nan, np.inf, dist)
    return dist


def bs_truth(S, K, T, r, sigma, which):
    """Call or put price of one option from its inputs as given (exactly the floating-
    point numbers S, K, T), evaluated with 50 digits."""
    import mpmath as mp
    with mp.workdps(50):
        S, K, T = mp.mpf(float(S)), mp.mpf(float(K)), mp.mpf(float(T))
        r, sigma = mp.mpf(r), mp.mpf(sigma)
        vs = sigma * mp.sqrt(T)
        d1 = (mp.log(S / K) + (r + sigma * sigma / 2) * T) / vs
        d2 = d1 - vs
        N = lambda d: mp.erfc(-d / mp.sqrt(2)) / 2          # no cancellation in either tail
        disc = K * mp.exp(-r * T)
        if which == "call":
            return S * N(d1) - disc * N(d2)
        return disc * N(-d2) - S * N(-d1)


def _at(idx, got, ref, inp, which):
    """Everything worth knowing about one option: inputs, both results, the truth."""
    S, K, T = (inp[k][idx] for k in "SKT")
    truth = bs_truth(S, K, T, inp["r"], inp["sigma"], which)
    dt = got.dtype
    eps_at = float(np.spacing(np.abs(dt.type(float(truth))))) or float(np.finfo(dt).tiny)
    return {"index": int(idx), "S": float(S), "K": float(K), "T": float(T),
            "device": float(got[idx]), "oracle": float(ref[idx]), "truth": float(truth),
            "device_err_ulp_vs_truth": round(abs(float(got[idx]) - float(truth)) / eps_at, 2),
            "oracle_err_ulp_vs_truth": round(abs(float(ref[idx]) - float(truth)) / eps_at, 2)}


def bs_report(got_call, got_put, ref_call, ref_put, inp, detail=True):
    """Error table of device prices against the oracle's.

    Returns {"call": {...}, "put": {...}}; each holds `scaled` (max |d| / max(S, K) in
    units of the dtype's epsilon, with index) and `subsets`: for each k in THRESHOLDS the
    number of options with |oracle price| >= 2^-k max(S, K) and over them the largest ulp
    distance and the largest relative difference, each with the index where it occurs
    (and, with `detail`, the 50-digit truth there)."""
    scale = np.maximum(inp["S"], inp["K"]).astype(np.float64)
    out = {}
    for which, got, ref in (("call", got_call, ref_call), ("put", got_put, ref_put)):
        dt = got.dtype
        eps = float(np.finfo(dt).eps)
        g64, r64 = got.astype(np.float64), ref.astype(np.float64)
        diff = np.abs(g64 - r64)
        scaled = diff / scale
        ulps = ulp_distance(got, ref)
        with np.errstate(divide="ignore", invalid="ignore"):
            rel = np.where(diff == 0, 0.0, diff / np.abs(r64))
        i = int(np.argmax(scaled))
        rep = {"n": int(got.size),
               "scaled": {"max_eps": round(float(scaled[i]) / eps, 3), "index": i},
               "subsets": {}}
        if detail:
            rep["scaled"]["at"] = _at(i, got, ref, inp, which)
        for k in THRESHOLDS:
            mask = np.abs(r64) >= scale * 2.0 ** -k
            count = int(mask.sum())
            entry = {"count": count}
            if count:
                iu = int(np.argmax(np.where(mask, ulps, -1.0)))
                ir = int(np.argmax(np.where(mask, rel, -1.0)))
                entry.update(max_ulp=float(ulps[iu]), max_ulp_index=iu,
                             max_rel=float(rel[ir]), max_rel_index=ir)
                if detail:
                    entry["max_ulp_at"] = _at(iu, got, ref, inp, which)
                    if ir != iu:
                        entry["max_rel_at"] = _at(ir, got, ref, inp, which)
            rep["subsets"][k] = entry
        out[which] = rep
    return out


def format_report(name, report):
    """The table as text (what the GPU test prints and the design notes quote)."""
    lines = [f"Black-Scholes {name}: device vs oracle"]
    for which, rep in report.items():
        s = rep["scaled"]
        lines.append(f"  {which}: n={rep['n']}  max |d|/max(S,K) = {s['max_eps']} eps at index {s['index']}")
        for k, e in rep["subsets"].items():
            if not e["count"]:
                lines.append(f"    |price| >= 2^-{k} max(S,K): none")
                continue
            txt = (f"    |price| >= 2^-{k} max(S,K): {e['count']} options, max {e['max_ulp']:.0f} ulp "
                   f"(index {e['max_ulp_index']}), max rel {e['max_rel']:.3e} (index {e['max_rel_index']})")
            at = e.get("max_ulp_at")
            if at:
                txt += (f"; there the device is {at['device_err_ulp_vs_truth']} ulp and the oracle "
                        f"{at['oracle_err_ulp_vs_truth']} ulp from the 50-digit value")
            lines.append(txt)
    return "\n".join(lines)
