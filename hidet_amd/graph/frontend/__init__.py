from . import torch
