"""Several AdamW training steps of an engine against its oracle, shared by the Swin-B and GPT-2 tests.

AdamW's first steps are updates of about +-lr per element whatever the size of the gradient (the update is
m / (sqrt(v) + eps), and m^2 ~ v at the start), so the UPDATED WEIGHTS of two correct implementations whose
gradients differ within the stated bound can still differ by 2 lr wherever a gradient is near zero: comparing
free-running weights says little about either implementation.  The steps are therefore checked in three parts,
each well conditioned:

 1. every step's loss and every gradient against the oracle evaluated AT THE ENGINE'S OWN WEIGHTS before that
    step, at the stated bound -- so steps 1 and 2 are held as tightly as step 0.  In bf16 mode the engine's
    matrix products read the bf16 copy of the fp32 master weights (what autocast does with them); `oracle_view`
    turns the master weights into what the engine's kernels read, so that both sides evaluate the same function;
 2. every step's optimizer update against torch.optim.AdamW on the CPU fed the ENGINE'S OWN GRADIENTS (same
    moments carried from step to step): the update w_after - w_before element by element, to 2e-3 of lr plus
    the fp32 rounding of the weight -- this is the optimizer kernel at the model's real size, state carried over
    three steps, decoupled weight decay, bias correction;
 3. the free-running loss of every step against the oracle's own free-running AdamW run (losses are smooth in the
    weights, so this does hold at the stated bound).
"""
import torch


def rel(got, ref):
    return (got.float().cpu() - ref.float()).abs().max().item() / (ref.float().abs().max().item() + 1e-12)


def run_adamw_steps(eng, batches, forward_backward, oracle_loss_and_grads, free_running_losses, lr, weight_decay,
                    tol, grad_tol=None, betas=(0.9, 0.999), eps=1e-8, tag="", oracle_view=None):
    """forward_backward(batch) runs the engine on a batch; oracle_loss_and_grads(state_dict, batch) ->
    (loss, {name: grad}); grad_tol(name, state_dict, batch, grads_ref) -> bound for that tensor (default: tol);
    oracle_view(state_dict) -> the weights the oracle is evaluated at (default: the master weights)."""
    w = {k: v.clone() for k, v in eng.state_dict().items()}
    names = [k for k, v in w.items() if v.is_floating_point()]
    leaf = {k: w[k].clone().requires_grad_(True) for k in names}
    opt = torch.optim.AdamW([leaf[k] for k in names], lr=lr, betas=betas, eps=eps, weight_decay=weight_decay)
    for s, batch in enumerate(batches):
        forward_backward(batch)
        loss = eng.last_loss()
        grads = {k: v.clone() for k, v in eng.grads_dict().items()}
        # 1. oracle at the engine's weights
        w_seen = w if oracle_view is None else oracle_view(w)
        loss_ref, grads_ref = oracle_loss_and_grads(w_seen, batch)
        assert abs(loss - loss_ref.item()) <= tol * abs(loss_ref.item()), (tag, s, loss, loss_ref.item())
        errs = sorted(((rel(grads[k], grads_ref[k]), k) for k in grads_ref), reverse=True)
        print(f"{tag} step {s}: loss {loss:.6f} (oracle at the same weights {loss_ref.item():.6f}, free-running "
              f"{free_running_losses[s]:.6f}); worst gradients {errs[:3]}", flush=True)
        for e, k in errs:
            assert torch.isfinite(grads[k]).all(), (tag, s, k)
            bound = tol if grad_tol is None else grad_tol(k, w_seen, batch, grads_ref)
            assert e <= bound, (tag, s, k, e, bound)
        # 3. free-running loss
        assert abs(loss - free_running_losses[s]) <= tol * abs(free_running_losses[s]), (tag, s, loss, free_running_losses[s])
        # 2. the optimizer, on the engine's own gradients
        for k in names:
            leaf[k].grad = grads[k].float().clone()
        opt.step()
        eng.optimizer_step()
        w_new = {k: v.clone() for k, v in eng.state_dict().items()}
        worst = (0.0, None)
        for k in names:
            d_got = w_new[k].double() - w[k].double()
            d_ref = leaf[k].detach().double() - w[k].double()
            lim = 2e-3 * lr + 2.4e-7 * w[k].double().abs()
            over = ((d_got - d_ref).abs() - lim).max().item()
            if over > worst[0]:
                worst = (over, k)
        print(f"{tag} step {s}: optimizer update within bound" if worst[1] is None else
              f"{tag} step {s}: optimizer update exceeds bound by {worst[0]:.3e} at {worst[1]}", flush=True)
        assert worst[1] is None, (tag, s, worst)
        # the oracle's optimizer goes on from the ENGINE's weights (its moments are its own)
        with torch.no_grad():
            for k in names:
                leaf[k].copy_(w_new[k])
        w = w_new
    return w


def bf16_matrix_view(skip_suffixes=()):
    """oracle_view for an engine in bf16 mode: every parameter with two or more dimensions (projection matrices,
    embeddings, convolution filters) as its bf16 copy; vectors (biases, LayerNorm parameters) and the tensors named
    by `skip_suffixes` stay fp32, as the kernels read them."""
    def view(w):
        return {k: (v.to(torch.bfloat16).float() if v.is_floating_point() and v.dim() >= 2 and not k.endswith(tuple(skip_suffixes))
                    else v) for k, v in w.items()}
    return view
