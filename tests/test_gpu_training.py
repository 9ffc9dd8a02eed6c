"""End-to-end training through the device operator.

Two small callers restate the training gates the reference runs in its device CI
(.github/workflows/cuda-full.yml:68-76): a one-layer token model fitted to a
copy sequence until the loss on recallable targets is at most 0.20
(examples/fit_soft_reference.py:336-417, :459-660), and a shortcut-free
associative recall whose queries start with a wrong sign bit and must learn
the discrete route through the surrogate backward
(examples/associative_recall_gate.py:118-432). Each gate also runs with the
CPU oracle as the operator, from the same initial weights, and the two
trajectories are compared.
"""

import math

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

DEVICE = "cuda:0"


# --------------------------------------------------------------------------
# callers (plain torch modules around an operator with the rosa_soft signature)
# --------------------------------------------------------------------------

class CopyTaskModel(nn.Module):
    """embedding -> norm -> Q/K/V projections -> operator -> output projection -> head."""

    def __init__(self, operator, vocab=8, heads=2, qk_bits=4, value_heads=2, value_bits=4,
                 horizon=8):
        super().__init__()
        self.operator = operator
        self.shape = (heads, qk_bits, value_heads, value_bits)
        self.horizon = horizon
        width = heads * qk_bits
        self.embedding = nn.Embedding(vocab, width)
        self.input_norm = nn.LayerNorm(width)
        self.query = nn.Linear(width, width, bias=False)
        self.key = nn.Linear(width, width, bias=False)
        self.value = nn.Linear(width, value_heads * value_bits, bias=False)
        self.output = nn.Linear(heads * value_bits, width, bias=False)
        self.output_norm = nn.LayerNorm(width)
        self.head = nn.Linear(width, vocab, bias=False)

    def forward(self, tokens, routed_weight=1.0):
        heads, qk_bits, value_heads, value_bits = self.shape
        B, T = tokens.shape
        residual = self.embedding(tokens)
        hidden = self.input_norm(residual)
        routed = self.operator(
            self.query(hidden).view(B, T, heads, qk_bits),
            self.key(hidden).view(B, T, heads, qk_bits),
            self.value(hidden).view(B, T, value_heads, value_bits),
            max_suffix_length=self.horizon,
        )
        hidden = residual + routed_weight * self.output(routed.flatten(2))
        return self.head(self.output_norm(hidden))


def copy_tokens(length=17):
    # token 3 is followed by 1, 5 or 2 depending on what came before it, so the
    # current token alone leaves ln(3)/2 = 0.55 nats on the table
    motif = [3, 1, 3, 5, 3, 2]
    return torch.tensor([(motif * (length // len(motif) + 1))[:length]])


def recallable_targets(tokens, first=6):
    mask = torch.zeros(tokens.size(0), tokens.size(1) - 1, dtype=torch.bool)
    mask[:, first:] = True
    return mask


def masked_loss(logits, tokens, mask):
    prediction = logits[:, :-1].float()[mask]
    return F.cross_entropy(prediction, tokens[:, 1:][mask])


def fit_copy_task(operator, device, steps, seed=0):
    torch.manual_seed(seed)
    model = CopyTaskModel(operator)  # initialised on the host: same weights for every device
    model.to(device)
    tokens = copy_tokens().to(device)
    mask = recallable_targets(tokens).to(device)
    optimizer = torch.optim.AdamW(model.parameters(), lr=0.01, weight_decay=0.01)
    losses = []
    for _ in range(steps):
        optimizer.zero_grad(set_to_none=True)
        loss = masked_loss(model(tokens), tokens, mask)
        loss.backward()
        torch.nn.utils.clip_grad_norm_(model.parameters(), 1.0)
        optimizer.step()
        losses.append(float(loss.detach()))
    with torch.no_grad():
        final = float(masked_loss(model(tokens), tokens, mask))
        blind = float(masked_loss(model(tokens, routed_weight=0.0), tokens, mask))
    return losses, final, blind


# --------------------------------------------------------------------------
# associative recall: the answer exists only as one historical value
# --------------------------------------------------------------------------

def sign_codes(ids, width):
    bits = (torch.tensor(ids).unsqueeze(1) >> torch.arange(width)) & 1
    return bits.to(torch.float32) * 2.0 - 1.0


def recall_task(seed, associations=4, qk_bits=8, value_bits=8):
    """Two episodes with identical inputs at the recall positions and opposite answers.

    Keys 0..A-1 hold distinct cue codes, values 1..A the answers (negated in the second
    episode), every other position a distractor cue and a decoy value. Recall position j
    queries cue j with one sign bit wrong, from small logits that training has to flip.
    """

    generator = torch.Generator().manual_seed(seed)
    cue_ids = torch.randperm(1 << qk_bits, generator=generator)[: associations + 1].tolist()
    # answers: distinct, no answer the complement of another, decoy different from all
    answer_ids = []
    while len(answer_ids) < associations + 1:
        candidate = int(torch.randint(0, 1 << value_bits, (1,), generator=generator))
        complement = candidate ^ ((1 << value_bits) - 1)
        if candidate not in answer_ids and complement not in answer_ids:
            answer_ids.append(candidate)
    cues = sign_codes(cue_ids[:associations], qk_bits)
    distractor = sign_codes(cue_ids[-1:], qk_bits)[0]
    answers = sign_codes(answer_ids[:associations], value_bits)
    decoy = sign_codes(answer_ids[-1:], value_bits)[0]
    length = 2 * associations + 1
    recall = torch.arange(associations + 1, length)
    key = distractor.repeat(2, length, 1, 1)
    key[:, :associations, 0] = cues
    base_query = distractor.repeat(2, length, 1, 1)
    base_query[:, recall, 0] = 0.0
    value = decoy.repeat(2, length, 1, 1)
    targets = torch.stack((answers, -answers))
    value[:, 1: associations + 1, 0] = targets
    start = cues.clone()
    for row in range(associations):
        start[row, int(torch.randint(0, qk_bits, (1,), generator=generator))] *= -1.0
    start = start * (0.05 + 0.1 * torch.rand(associations, qk_bits, generator=generator))
    return dict(base_query=base_query, key=key, value=value, targets=targets, recall=recall,
                start=start, cues=cues)


def run_recall(operator, device, seed, steps=250, learning_rate=0.5):
    task = {name: tensor.to(device) for name, tensor in recall_task(seed).items()}
    logits = nn.Parameter(task["start"].clone())
    optimizer = torch.optim.SGD([logits], lr=learning_rate)
    recall = task["recall"]

    def build_query(rows):
        query = task["base_query"].clone()
        query[:, recall, 0] = query[:, recall, 0] + rows
        return query

    def recalled(rows):
        output = operator(build_query(rows), task["key"], task["value"], max_suffix_length=1)
        return output[:, recall, 0]

    def exact(rows):
        with torch.no_grad():
            return (recalled(rows) == task["targets"]).all(dim=(0, 2))

    report = dict(initial=exact(logits).float().mean().item(),
                  with_true_cues=exact(task["cues"]).float().mean().item(),
                  from_current_value=(task["value"][:, recall, 0] == task["targets"])
                  .all(dim=2).float().mean().item())
    active = torch.ones(len(recall), dtype=torch.bool, device=device)
    first_gradient = None
    solved_at = -1
    for step in range(1, steps + 1):
        optimizer.zero_grad(set_to_none=True)
        per_association = -(recalled(logits) * task["targets"]).mean(dim=(0, 2))
        (per_association * active.float()).sum().backward()
        if first_gradient is None:
            first_gradient = logits.grad.detach().cpu().clone()
        optimizer.step()
        active &= ~exact(logits)
        if not bool(active.any()):
            solved_at = step
            break
    report.update(final=exact(logits).float().mean().item(), solved_at=solved_at,
                  first_gradient=first_gradient)
    return report


# --------------------------------------------------------------------------
# tests
# --------------------------------------------------------------------------

@pytest.fixture(scope="module")
def rosa():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import rosa_soft_amd

    return rosa_soft_amd


@pytest.fixture(scope="module")
def oracle_operator():
    from oracle.rosa_oracle import rosa_soft_oracle

    return rosa_soft_oracle


@pytest.mark.gpu
def test_copy_task_fit_reaches_the_reference_gate(rosa, oracle_operator):
    losses, final, blind = fit_copy_task(rosa.rosa_soft, DEVICE, steps=400)
    assert math.isfinite(final) and final <= 0.20, (final, losses[::50])
    # the routed features carry the fit: without them the same weights are far off
    assert blind > 0.5, blind
    # same weights, same data, oracle as the operator: the first steps coincide
    want, _, _ = fit_copy_task(oracle_operator, "cpu", steps=12)
    torch.testing.assert_close(torch.tensor(losses[:12]), torch.tensor(want), rtol=2e-3, atol=2e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_associative_recall_learns_the_route(rosa, oracle_operator, seed):
    got = run_recall(rosa.rosa_soft, DEVICE, seed)
    assert got["initial"] < 1.0 and got["with_true_cues"] == 1.0
    assert got["from_current_value"] == 0.0
    assert got["final"] == 1.0 and got["solved_at"] > 0, got
    want = run_recall(oracle_operator, "cpu", seed)
    assert want["final"] == 1.0
    torch.testing.assert_close(got["first_gradient"], want["first_gradient"], rtol=1e-4, atol=1e-7)
    assert abs(got["solved_at"] - want["solved_at"]) <= 1, (got["solved_at"], want["solved_at"])


def test_training_gates_pass_with_the_oracle_operator(oracle_operator):
    # the CPU half of the gates above, so that the tasks themselves are known to be
    # solvable by the algorithm and a device failure points at the device
    _, final, blind = fit_copy_task(oracle_operator, "cpu", steps=400)
    assert final <= 0.20 and blind > 0.5, (final, blind)
    for seed in (0, 1, 2):
        report = run_recall(oracle_operator, "cpu", seed)
        assert report["initial"] < 1.0 and report["final"] == 1.0, report
