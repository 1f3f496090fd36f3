"""Helpers of the GPU tests: model folders, the plain logits, in-process replay."""
import os

import torch

import plain_llama
from tiny_configs import tiny


def make_folder(tmp_path_factory, name, seed=0, store_dtype=torch.float32, std=None):
    from pytriton_llama_amd.weights import write_random_model
    cfg, cstd, norm_std, page = tiny(name)
    folder = str(tmp_path_factory.mktemp(f"tiny_{name}"))
    write_random_model(cfg, folder, seed=seed, dtype=store_dtype, norm_std=norm_std,
                       std=cstd if std is None else std)
    return folder, page


def random_sequences(vocab, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist()
            for i, n in enumerate(lengths)}


def plain_logits(folder, seqs, weights_as=torch.float32):
    """Logits of the plain implementation, in float32 arithmetic, with weights
    rounded to ``weights_as`` first (the values a bfloat16 engine holds)."""
    cfg, w = plain_llama.read_model_folder(folder)
    if weights_as != torch.float32:
        w = {k: (v.to(weights_as).float() if v.dim() == 2 else v) for k, v in w.items()}
    return {rid: plain_llama.forward(cfg, w, toks) for rid, toks in seqs.items()}


def load_runner(folder, dtype, page_size, num_pages, device="cuda:0", max_num_seqs=8):
    import pytriton_llama_amd  # noqa: F401
    from pytriton_llama_amd.config import build_model, read_config_json
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_weights
    model = build_model(read_config_json(folder))
    load_weights(model, folder, dtype, device)
    model.make_decode_copies()                 # as the engine does by default
    return ModelRunner(model, page_size, num_pages, max_num_seqs)


def replay(runner, steps, seqs):
    """Run trace steps in-process; returns {request: float32 [len, vocab]} on the CPU."""
    from pytriton_llama_amd.engine.batch import StepEntry
    V = runner.model.vocab_size
    out = {rid: torch.full((len(t), V), float("nan")) for rid, t in seqs.items()}
    fed = {rid: 0 for rid in seqs}
    for st in steps:
        entries = [StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]]
        logits = runner.step(entries).float().cpu()
        row = 0
        for e in st["entries"]:
            for w in e["want"]:
                out[e["id"]][fed[e["id"]] + w] = logits[row]
                row += 1
            fed[e["id"]] += len(e["tokens"])
        assert row == logits.shape[0]
        for rid in st["end"]:
            runner.end(rid)
        runner.manager.check()
    return out


def first_mismatch(got, want, tol):
    """(request, position, error) of the first place whose logits differ by more
    than tol * (largest |logit| of the plain result), or None."""
    for rid in want:
        scale = float(want[rid].abs().max())
        err = (got[rid] - want[rid]).abs().amax(dim=-1) / scale
        err = torch.where(torch.isnan(err), torch.full_like(err, float("inf")), err)
        bad = torch.nonzero(err > tol)
        if len(bad):
            p = int(bad[0])
            return rid, p, float(err[p])
    return None


# measured on MI355X: float32 stays below 3e-6, bfloat16 below 3e-2 (tests/ tiny and wide models)
TOL = {torch.float32: 2e-5, torch.bfloat16: 4e-2}


def load_graph_runner(folder, dtype, page_size, num_pages, max_model_len, max_num_seqs=8,
                      device="cuda:0", timed_library_products=True):
    """A runner that replays decode steps and single-portion steps as HIP graphs."""
    from pytriton_llama_amd.config import build_model, read_config_json
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_weights
    model = build_model(read_config_json(folder))
    load_weights(model, folder, dtype, device)
    model.make_decode_copies()
    return ModelRunner(model, page_size, num_pages, max_num_seqs, max_model_len=max_model_len,
                       use_graphs=True, timed_library_products=timed_library_products)


def plain_rows(folder, seqs, places, weights_as=torch.float32):
    """{request: float32 [len(places[request]), vocab]}: the plain logits at the given
    positions only (the head is applied to those rows alone, which keeps long sequences and
    large vocabularies cheap)."""
    cfg, w = plain_llama.read_model_folder(folder)
    if weights_as != torch.float32:
        w = {k: (v.to(weights_as).float() if v.dim() == 2 else v) for k, v in w.items()}
    head = w.get("lm_head.weight")
    if head is None or cfg.get("tie_word_embeddings", True):
        head = w["model.embed_tokens.weight"]
    out = {}
    for rid, toks in seqs.items():
        rows = torch.as_tensor(places.get(rid, []), dtype=torch.long)
        if len(rows):
            h = plain_llama.forward(cfg, w, toks, return_hidden=True)
            out[rid] = h[rows] @ head.T
    return out


def replay_wanted(runner, steps, check=True):
    """Run trace steps in-process; {request: float32 [wanted places, vocab]} on the CPU, the
    rows in the order of the positions (steps ask for places in rising order)."""
    from pytriton_llama_amd.engine.batch import StepEntry
    rows = {}
    for st in steps:
        entries = [StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]]
        logits = runner.step(entries).float().cpu()
        row = 0
        for e in st["entries"]:
            n = len(e["want"])
            if n:
                rows.setdefault(e["id"], []).append(logits[row:row + n].clone())
                row += n
        assert row == logits.shape[0]
        for rid in st["end"]:
            runner.end(rid)
        if check:
            runner.manager.check()
    return {rid: torch.cat(r) for rid, r in rows.items()}


def first_wrong_row(got, want, places, tol):
    """(request, position, error) of the first wanted place whose logits differ by more than
    tol * (largest |logit| of the request's plain rows), or None."""
    for rid in want:
        assert got[rid].shape == want[rid].shape, (rid, got[rid].shape, want[rid].shape)
        scale = float(want[rid].abs().max())
        err = (got[rid] - want[rid]).abs().amax(dim=-1) / scale
        err = torch.where(torch.isnan(err), torch.full_like(err, float("inf")), err)
        bad = torch.nonzero(err > tol)
        if len(bad):
            i = int(bad[0])
            return rid, places[rid][i], float(err[i])
    return None
