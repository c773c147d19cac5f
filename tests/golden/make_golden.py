"""Writes tests/golden/token_numerics_golden.json: small known-answer vectors for every function
on the path, computed with scalar Python float64 loops from the published definitions (no torch,
no numpy, no import of the reference or of the oracle).

The reference ships no golden vectors for this path, so these are the build's own: an
independent, brute-force evaluation that both the CPU oracle (tests/test_oracle_pins.py) and
the HIP kernels (tests/test_gpu_golden.py) are compared with. Inputs are rounded to fp32 so that
an fp32 kernel sees exactly the stored values.

    python tests/golden/make_golden.py
"""
import json
import math
import os
import random
import struct

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "token_numerics_golden.json")


def f32(x):
    return struct.unpack("f", struct.pack("f", x))[0]


def rand_matrix(rng, rows, cols, scale=1.0, shift=0.0):
    return [[f32(rng.gauss(0.0, 1.0) * scale + shift) for _ in range(cols)] for _ in range(rows)]


def clamp(x, lo, hi):
    return lo if x < lo else (hi if x > hi else x)


# ---------------------------------------------------------------- vocabulary rows
def lse(row):
    m = max(row)
    return m + math.log(sum(math.exp(v - m) for v in row))


def logprob_entropy(logits, labels, temperature):
    lps, ents = [], []
    for row, lab in zip(logits, labels):
        z = [v / temperature for v in row]
        lps.append(z[lab] - lse(z))
        l1 = lse(row)
        ents.append(l1 - sum(math.exp(v - l1) * v for v in row))
    return lps, ents


def logprob_entropy_grad(logits, labels, temperature, g_lp, g_ent):
    out = []
    for row, lab, gl, ge in zip(logits, labels, g_lp, g_ent):
        z = [v / temperature for v in row]
        lz = lse(z)
        l1 = lse(row)
        p = [math.exp(v - l1) for v in row]
        ex = sum(pi * v for pi, v in zip(p, row))
        out.append([
            gl * ((1.0 if j == lab else 0.0) - math.exp(z[j] - lz)) / temperature + ge * p[j] * (ex - row[j])
            for j in range(len(row))
        ])
    return out


# ---------------------------------------------------------------- per-token
def approx_kl(lp, base, est):
    out = []
    for r_lp, r_b in zip(lp, base):
        row = []
        for a, b in zip(r_lp, r_b):
            d = a - b
            v = d if est == "k1" else (d * d / 2.0 if est == "k2" else math.exp(-d) - 1.0 + d)
            row.append(clamp(v, -10.0, 10.0))
        out.append(row)
    return out


def aggregate(loss, mask, token_level, dp_size=1, batch_num_tokens=None, global_batch_size=None):
    if token_level:
        num = sum(l * m for rl, rm in zip(loss, mask) for l, m in zip(rl, rm))
        if batch_num_tokens is None:
            return num / sum(m for rm in mask for m in rm)
        return num / batch_num_tokens * dp_size
    seqs, kept = 0.0, 0
    for rl, rm in zip(loss, mask):
        cnt = sum(rm)
        if cnt > 0:
            seqs += sum(l * m for l, m in zip(rl, rm)) / (cnt + 1e-8)
            kept += 1
    if global_batch_size is None:
        return seqs / kept
    return seqs / global_batch_size * dp_size


def policy_loss(lp, old, adv, mask, rollout, cfg, norm):
    eps_lo, eps_hi = cfg.get("clip_eps_low", 0.2), cfg.get("clip_eps_high", 0.2)
    dual = cfg.get("dual_clip")
    gspo = cfg.get("policy_loss_type", "ppo") == "gspo"
    token_level = cfg.get("token_level_loss", True) and not gspo
    use_is = cfg.get("enable_vllm_is_correction", False)
    is_type = cfg.get("vllm_is_correction_type", "tis")
    lo_hi = cfg.get("vllm_is_truncated_threshold")
    loss, clipped, neg_raw, vk = [], [], [], []
    for b in range(len(lp)):
        cnt = sum(mask[b])
        if gspo:
            ref = rollout[b] if use_is else old[b]
            seq_ratio = math.exp(sum((lp[b][t] - ref[t]) * mask[b][t] for t in range(len(lp[b]))) / max(cnt, 1.0))
        if use_is and not gspo and is_type == "seq-mask-tis":
            if cnt > 0:
                seq_w = math.exp(sum((old[b][t] - rollout[b][t]) * mask[b][t] for t in range(len(lp[b]))) / cnt)
                keep = 1.0 if lo_hi[0] <= seq_w <= lo_hi[1] else 0.0
            else:
                keep = 0.0
        rl, rc, rn, rv = [], [], [], []
        for t in range(len(lp[b])):
            raw = lp[b][t] - old[b][t]
            ratio = seq_ratio * mask[b][t] if gspo else math.exp(clamp(raw, -20.0, 20.0))
            s1 = ratio * adv[b][t]
            s2 = clamp(ratio, 1.0 - eps_lo, 1.0 + eps_hi) * adv[b][t]
            val = min(s1, s2)
            if dual is not None and adv[b][t] < 0:
                val = max(val, dual * adv[b][t])
            tok = -val
            if use_is and not gspo:
                w = math.exp(old[b][t] - rollout[b][t])
                if is_type == "tis":
                    w = clamp(w, lo_hi[0], lo_hi[1])
                elif is_type == "icepop":
                    w = w if lo_hi[0] <= w <= lo_hi[1] else 0.0
                else:
                    w = keep * w
                tok = w * tok
                rv.append(rollout[b][t] - old[b][t])
            rl.append(tok)
            rc.append(1.0 if s2 < s1 else 0.0)
            rn.append(-raw)
        loss.append(rl)
        clipped.append(rc)
        neg_raw.append(rn)
        vk.append(rv)
    total = aggregate(loss, mask, token_level, **norm)
    out = {
        "loss": total,
        "clip_ratio": aggregate(clipped, mask, True),
        "ppo_kl": aggregate(neg_raw, mask, True),
        "vllm_kl": aggregate(vk, mask, True) if (use_is and not gspo) else None,
    }
    return out


def value_loss(values, old, ret, mask, clip_eps, token_level):
    loss = []
    for b in range(len(values)):
        row = []
        for t in range(len(values[b])):
            plain = (values[b][t] - ret[b][t]) ** 2
            if clip_eps is None:
                row.append(plain)
            else:
                vc = old[b][t] + clamp(values[b][t] - old[b][t], -clip_eps, clip_eps)
                row.append(max((vc - ret[b][t]) ** 2, plain))
        loss.append(row)
    return 0.5 * aggregate(loss, mask, token_level)


# ---------------------------------------------------------------- advantages
def compute_reward(r, kl_coef, kl, mask, clip):
    coef = max(kl_coef, 0.0)
    out = []
    for b in range(len(kl)):
        width = len(kl[b])
        last = width - 1
        for t in range(width - 1, -1, -1):
            if mask[b][t] > 0.5:
                last = t
                break
        rb = clamp(r[b], clip[0], clip[1]) if clip else r[b]
        out.append([(rb if t == last else 0.0) - coef * kl[b][t] for t in range(width)])
    return out


def gae(values, rewards, mask, gamma, lambd):
    adv, ret = [], []
    for b in range(len(values)):
        width = len(values[b])
        v = [values[b][t] * mask[b][t] for t in range(width)]
        r = [rewards[b][t] * mask[b][t] for t in range(width)]
        run, row = 0.0, [0.0] * width
        for t in range(width - 1, -1, -1):
            nxt = v[t + 1] if t + 1 < width else 0.0
            run = (r[t] + gamma * nxt - v[t]) + gamma * lambd * run
            row[t] = run
        adv.append(row)
        ret.append([row[t] + v[t] for t in range(width)])
    return adv, ret


def cumulative_returns(rewards, mask, gamma):
    out = []
    for b in range(len(rewards)):
        run, row = 0.0, [0.0] * len(rewards[b])
        for t in range(len(rewards[b]) - 1, -1, -1):
            run = rewards[b][t] * mask[b][t] + gamma * run
            row[t] = run
        out.append(row)
    return out


def group_normalize(rewards, indices, n, estimator):
    total = len(rewards)
    ordered = [0.0] * total
    for i, slot in enumerate(indices):
        ordered[slot] = rewards[i]
    shaped, stds = [0.0] * total, [0.0] * total
    for g0 in range(0, total, n):
        grp = ordered[g0:g0 + n]
        mean = sum(grp) / n
        std = math.sqrt(sum((x - mean) ** 2 for x in grp) / (n - 1))
        for k, x in enumerate(grp):
            if estimator == "rloo":
                y = x - (sum(grp) - x) / (n - 1)
            elif estimator in ("reinforce_baseline", "dr_grpo"):
                y = x - mean
            elif estimator == "group_norm":
                y = (x - mean) / (std + 1e-9)
            else:
                y = x
            shaped[g0 + k] = y
            stds[g0 + k] = std
    return [shaped[s] for s in indices], [stds[s] for s in indices]


def whiten(adv, mask, no_std_norm):
    flat = [(x, m) for ra, rm in zip(adv, mask) for x, m in zip(ra, rm)]
    cnt = sum(m for _, m in flat)
    mean = sum(x * m for x, m in flat) / cnt
    rstd = 1.0
    if not no_std_norm:
        var = sum((x - mean) ** 2 * m for x, m in flat) / cnt
        rstd = 1.0 / math.sqrt(max(var, 1e-8))
    return [[(x - mean) * rstd for x in row] for row in adv]


def sequence_logps(lp, att, prompt_lens, g_sum, g_mean):
    """Scalar restatement of per-sequence sums / means over response tokens and their gradient:
    token t counts when att[b][t+1] != 0 and t+1 >= prompt_lens[b]."""
    sums, means, grads = [], [], []
    for b, row in enumerate(lp):
        m = [1.0 if (att[b][t + 1] != 0 and t + 1 >= prompt_lens[b]) else 0.0 for t in range(len(row))]
        s, c = sum(x * w for x, w in zip(row, m)), sum(m)
        sums.append(s)
        means.append(s / c if c > 0 else None)
        grads.append([w * (g_sum[b] + (g_mean[b] / c if c > 0 else 0.0)) for w in m] if c > 0 else None)
    return sums, means, grads


def log_sigmoid(x):
    return -math.log1p(math.exp(-x)) if x >= 0 else x - math.log1p(math.exp(x))


def sigmoid(x):
    return 1.0 / (1.0 + math.exp(-x)) if x >= 0 else math.exp(x) / (1.0 + math.exp(x))


def pair_loss(kind, chosen, rejected, ref_c, ref_r, beta, smooth):
    """mean loss, d(mean loss)/d(chosen_i) (= -d/d(rejected_i)) and the DPO reward estimates."""
    n = len(chosen)
    losses, grads = [], []
    for i in range(n):
        z = (chosen[i] - rejected[i]) - ((ref_c[i] if ref_c else 0.0) - (ref_r[i] if ref_r else 0.0))
        if kind == "dpo":
            losses.append(-log_sigmoid(beta * z) * (1 - smooth) - log_sigmoid(-beta * z) * smooth)
            grads.append(beta * (-(1 - smooth) * sigmoid(-beta * z) + smooth * sigmoid(beta * z)) / n)
        elif kind == "ipo":
            losses.append((z - 1 / (2 * beta)) ** 2)
            grads.append(2 * (z - 1 / (2 * beta)) / n)
        elif kind == "pairwise":
            losses.append(-log_sigmoid(z))
            grads.append(-sigmoid(-z) / n)
        else:  # logexp: log(1 + exp(-z))
            losses.append(-log_sigmoid(z))
            grads.append(-sigmoid(-z) / n)
    out = {"loss": sum(losses) / n, "g_chosen": grads}
    if kind in ("dpo", "ipo"):
        out["chosen_rewards"] = [beta * (chosen[i] - ref_c[i]) for i in range(n)]
        out["rejected_rewards"] = [beta * (rejected[i] - ref_r[i]) for i in range(n)]
    return out


def masked_normalize(x, mask, eps):
    out = []
    for row, rm in zip(x, mask):
        cnt = max(sum(rm), 1.0)
        mean = sum(v * m for v, m in zip(row, rm)) / cnt
        cen = [(v - mean) * m for v, m in zip(row, rm)]
        var = sum(c * c for c in cen) / cnt
        r = 1.0 / math.sqrt(max(var, eps))
        out.append([c * r for c in cen])
    return out


def kl_rows(lp, base, mask, est):
    kl = approx_kl(lp, base, est)
    means, diffs = [], []
    for b, rm in enumerate(mask):
        c = sum(rm)
        means.append(sum(k * m for k, m in zip(kl[b], rm)) / c if c > 0 else None)
        diffs.append(sum((f32(p) - f32(q)) * m for p, q, m in zip(lp[b], base[b], rm)) / c if c > 0 else None)
    return means, diffs


def main():
    rng = random.Random(20240607)
    gold = {}

    # vocabulary rows: 8 x 257, two temperatures, a spiked row and a wide row
    rows, vocab = 8, 257
    logits = rand_matrix(rng, rows, vocab, scale=2.0)
    logits[2][100] = f32(logits[2][100] + 15.0)
    logits[5] = [f32(v * 6.0) for v in logits[5]]
    labels = [rng.randrange(vocab) for _ in range(rows)]
    labels[2] = 100
    g_lp = [f32(rng.gauss(0, 1)) for _ in range(rows)]
    g_ent = [f32(rng.gauss(0, 1)) for _ in range(rows)]
    cases = []
    for temp in (1.0, 0.7):
        lp, ent = logprob_entropy(logits, labels, temp)
        cases.append({"temperature": temp, "logprob": lp, "entropy": ent,
                      "grad": logprob_entropy_grad(logits, labels, temp, g_lp, g_ent)})
    gold["vocab_rows"] = {"logits": logits, "labels": labels, "g_logprob": g_lp, "g_entropy": g_ent, "cases": cases}

    # per-token tensors 4 x 16 with prompt zeros, a hole, right padding and one empty row
    b, a = 4, 16
    lp = rand_matrix(rng, b, a, scale=0.8, shift=-1.5)
    old = [[f32(v + rng.gauss(0, 0.25)) for v in row] for row in lp]
    old[0][3] = f32(lp[0][3] + 25.0)
    old[0][4] = f32(lp[0][4] - 25.0)
    rollout = [[f32(v + rng.gauss(0, 0.1)) for v in row] for row in old]
    base = [[f32(v + rng.gauss(0, 1.5)) for v in row] for row in lp]
    base[1][2] = f32(lp[1][2] + 14.0)
    base[1][3] = f32(lp[1][3] - 14.0)
    adv = rand_matrix(rng, b, a)
    mask = [[1.0] * a for _ in range(b)]
    for t in (0, 1):
        mask[0][t] = 0.0
    mask[0][7] = 0.0
    for t in range(12, a):
        mask[1][t] = 0.0
    mask[2] = [0.0] * a
    mask[3][0] = 0.0
    gold["tokens"] = {"log_probs": lp, "old_log_probs": old, "rollout_log_probs": rollout, "base_log_probs": base,
                      "advantages": adv, "mask": mask}
    gold["approx_kl"] = {est: approx_kl(lp, base, est) for est in ("k1", "k2", "k3")}
    gold["aggregate"] = {
        "token_mean": aggregate(adv, mask, True),
        "token_mean_global": aggregate(adv, mask, True, dp_size=2, batch_num_tokens=50.0),
        "seq_mean": aggregate(adv, mask, False),
        "seq_mean_global": aggregate(adv, mask, False, dp_size=2, global_batch_size=5.0),
        "row_mean": [(sum(x * m for x, m in zip(ra, rm)) / sum(rm)) if sum(rm) > 0 else None for ra, rm in zip(adv, mask)],
    }
    policy_cfgs = [
        {},
        {"clip_eps_low": 0.1, "clip_eps_high": 0.3},
        {"dual_clip": 3.0},
        {"dual_clip": 3.0, "token_level_loss": False},
        {"enable_vllm_is_correction": True, "vllm_is_truncated_threshold": [0.9, 1.1], "vllm_is_correction_type": "tis"},
        {"enable_vllm_is_correction": True, "vllm_is_truncated_threshold": [0.9, 1.1], "vllm_is_correction_type": "icepop"},
        {"enable_vllm_is_correction": True, "vllm_is_truncated_threshold": [0.97, 1.03], "vllm_is_correction_type": "seq-mask-tis"},
        {"policy_loss_type": "gspo"},
        {"policy_loss_type": "gspo", "enable_vllm_is_correction": True, "vllm_is_truncated_threshold": [0.5, 2.0]},
    ]
    gold["policy_loss"] = []
    for cfg in policy_cfgs:
        for norm in ({}, {"dp_size": 2, "batch_num_tokens": 50.0, "global_batch_size": 5.0}):
            gold["policy_loss"].append({"cfg": cfg, "norm": norm, "out": policy_loss(lp, old, adv, mask, rollout, cfg, norm)})
    values = rand_matrix(rng, b, a)
    old_values = [[f32(v + rng.gauss(0, 0.3)) for v in row] for row in values]
    returns = rand_matrix(rng, b, a)
    gold["value_loss"] = {
        "values": values, "old_values": old_values, "returns": returns,
        "cases": [{"clip_eps": c, "token_level_loss": tl, "out": value_loss(values, old_values, returns, mask, c, tl)}
                  for c in (None, 0.2) for tl in (True, False)],
    }

    # advantages
    kl = rand_matrix(rng, b, a, scale=0.1)
    r = [f32(12.5), f32(-0.5), f32(1.0), f32(-30.0)]
    rewards = compute_reward(r, 0.01, kl, mask, (-10.0, 10.0))
    rewards_f32 = [[f32(x) for x in row] for row in rewards]
    gold["compute_reward"] = {"r": r, "kl": kl, "kl_coef": 0.01, "clip": [-10.0, 10.0], "out": rewards}
    gold["gae"] = []
    for gamma, lambd in ((1.0, 0.95), (0.99, 0.9), (1.0, 1.0), (0.9, 0.0)):
        adv_, ret_ = gae(values, rewards_f32, mask, gamma, lambd)
        gold["gae"].append({"gamma": gamma, "lambd": lambd, "advantages": adv_, "returns": ret_})
    gold["gae_inputs"] = {"values": values, "rewards": rewards_f32}
    gold["cumulative_returns"] = [{"gamma": g_, "out": cumulative_returns(rewards_f32, mask, g_)} for g_ in (1.0, 0.97)]
    n_prompts, n = 3, 4
    scal = [f32(rng.choice([0.0, 1.0])) for _ in range(n_prompts * n)]
    scal[0:4] = [1.0, 1.0, 1.0, 1.0]
    scal[4] = f32(0.37)
    perm = list(range(n_prompts * n))
    rng.shuffle(perm)
    exp_order = [0.0] * len(scal)
    for i, slot in enumerate(perm):
        exp_order[i] = scal[slot]
    gold["group_normalize"] = {"rewards": exp_order, "indices": perm, "n": n, "cases": []}
    for est in ("gae", "rloo", "reinforce_baseline", "dr_grpo", "group_norm"):
        shaped, std = group_normalize(exp_order, perm, n, est)
        gold["group_normalize"]["cases"].append({"estimator": est, "out": shaped, "group_std": std})
    gold["whiten"] = [{"no_std_norm": f, "out": whiten(adv, mask, f)} for f in (False, True)]

    # sequence-level: response sums / means with left padding, right padding, an attention hole and
    # a sequence whose prompt covers everything; pairwise losses with large and tiny logits
    att = [[1] * (a + 1) for _ in range(b)]
    att[0][0] = att[0][1] = 0
    for t in range(13, a + 1):
        att[1][t] = 0
    att[2][9] = 0
    prompt_lens = [5, 3, 7, a + 1]
    g_sum = [f32(rng.gauss(0, 1)) for _ in range(b)]
    g_mean = [f32(rng.gauss(0, 1)) for _ in range(b)]
    sums, means, grads = sequence_logps(lp, att, prompt_lens, g_sum, g_mean)
    gold["sequence_logps"] = {"attention_mask": att, "prompt_id_lens": prompt_lens, "g_sums": g_sum, "g_means": g_mean,
                              "sums": sums, "means": means, "grad": grads}
    n_pairs = 7
    chosen = [f32(rng.gauss(-40, 12)) for _ in range(n_pairs)]
    rejected = [f32(c + rng.gauss(0, 6)) for c in chosen]
    ref_c = [f32(c + rng.gauss(0, 3)) for c in chosen]
    ref_r = [f32(r_ + rng.gauss(0, 3)) for r_ in rejected]
    rejected[0] = f32(chosen[0] - 60.0)
    rejected[1] = f32(chosen[1] + 60.0)
    margin = [f32(rng.uniform(0, 2)) for _ in range(n_pairs)]
    cr = [f32(rng.gauss(0, 2)) for _ in range(n_pairs)]
    rr = [f32(rng.gauss(0, 2)) for _ in range(n_pairs)]
    gold["pair_loss"] = {
        "chosen": chosen, "rejected": rejected, "ref_chosen": ref_c, "ref_rejected": ref_r,
        "chosen_reward": cr, "reject_reward": rr, "margin": margin,
        "dpo": [{"beta": be, "label_smoothing": ls, "ipo": ipo,
                 "out": pair_loss("ipo" if ipo else "dpo", chosen, rejected, ref_c, ref_r, be, ls)}
                for be, ls, ipo in ((0.1, 0.0, False), (0.5, 0.1, False), (0.1, 0.0, True))],
        "pairwise": pair_loss("pairwise", cr, rr, None, None, 1.0, 0.0),
        "pairwise_margin": pair_loss("pairwise", cr, rr, margin, None, 1.0, 0.0),
        "logexp": pair_loss("logexp", cr, rr, None, None, 1.0, 0.0),
    }

    gold["masked_normalize"] = {"eps": 1e-8, "out": masked_normalize(adv, mask, 1e-8)}
    gold["kl_rows"] = {est: dict(zip(("kl_mean", "diff_mean"), kl_rows(lp, base, mask, est))) for est in ("k1", "k3")}
    seq_sums = [sum(x * m for x, m in zip(ra, rm)) for ra, rm in zip(adv, mask)]
    nonempty = [s_ for s_, rm in zip(seq_sums, mask) if sum(rm) > 0]
    gold["aggregate"]["seq_token_sum"] = sum(nonempty) / len(nonempty)
    gold["aggregate"]["seq_token_sum_global"] = sum(nonempty) / 5.0 * 2

    with open(OUT, "w") as fh:
        json.dump(gold, fh)
    print(OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
