"""The training-step glue of the reference's example scripts, for models built from the SNN layers:
input encoding, the weight-constraint cost, one Adam/SGD step and the evaluation step
(snntc-mnist.py:55-59, 73-96).  Everything here is stock PyTorch around the gfx950 ops; weights are
saved and restored with ``model.state_dict()`` / ``load_state_dict`` (the reference uses Keras
``save_weights``, snntc-cifar10.py:255-259).
"""
import torch

from .layers import loss_func


def encode_input(images):
    """Pixel intensities in [0,1] -> spike times z = exp(1 - x) >= 1 (snntc-mnist.py:75)."""
    return torch.exp(1.0 - images)


def snn_layers(model):
    return [m for m in model.modules() if hasattr(m, "w_sum_cost") and hasattr(m, "weight")]


def constraint_cost(model, weight_k=100.0, weight_k2=1e-2):
    """K * sum_l mean(max(0, 1 - sum_i w_ij)) + K2 * sum_l mean(w^2)  (snntc-mnist.py:55-59)."""
    layers = snn_layers(model)
    wsc = sum(torch.mean(torch.clamp(1.0 - torch.sum(l.weight, 0), min=0.0)) for l in layers)
    l2 = sum(torch.mean(torch.square(l.weight)) for l in layers)
    return weight_k * wsc + weight_k2 * l2


def predictions_to_classes(predictions):
    """The earliest output spike is the predicted class (snntc-mnist.py:83)."""
    return torch.argmin(predictions, dim=1)


def train_step(model, optimizer, images, labels, num_classes, weight_k=100.0, weight_k2=1e-2):
    """One optimisation step on a batch of images in [0,1]; returns (loss, number of correct samples)."""
    inputs = encode_input(images)
    onehot = torch.nn.functional.one_hot(labels, num_classes).to(inputs.dtype)
    optimizer.zero_grad(set_to_none=True)
    predictions = model(inputs)
    loss = loss_func(logit=predictions, label=onehot) + constraint_cost(model, weight_k, weight_k2)
    loss.backward()
    optimizer.step()
    correct = (predictions_to_classes(predictions.detach()) == labels).sum()
    return loss.detach(), correct


@torch.no_grad()
def test_step(model, images, labels, num_classes, weight_k=100.0, weight_k2=1e-2):
    inputs = encode_input(images)
    onehot = torch.nn.functional.one_hot(labels, num_classes).to(inputs.dtype)
    predictions = model(inputs)
    loss = loss_func(logit=predictions, label=onehot) + constraint_cost(model, weight_k, weight_k2)
    return loss, (predictions_to_classes(predictions) == labels).sum()
