"""What every part is: sizes and constants as constructor arguments, tensors under local names.

A part never learns which model it stands in.  It declares the tensors it needs
(`tensor_specs`), receives them on the device (`bind`), and runs on the rows of a
step (`forward`).  Interfaces:

  Norm         forward(ctx, x, out_dtype) -> rows;  `gain` is the fp32 vector the
               norm multiplies by, so that blocks can fuse a norm into a neighbour.
  Position     `rotary_dim` and `inv_freq(device)`: the rotation table a mixer applies
               to queries and keys before the cache write.
  Mixer        cache_spec() -> TokenSpec | StateSpec | None;
               forward(ctx, x, site) -> rows [M, hidden], x being the normed rows.
  FeedForward  forward(ctx, x) -> rows [M, hidden].
               (A mixer or feed-forward may return what `ops.linear(..., defer=True)` gave it: the block
               hands it to `ops.add_rms_norm`, or turns it into a tensor with `ops.rows`.)
  Block        norm_sites() -> names of its norms;  forward(ctx, stream, site, normed, next_norm)
               -> (stream, normed_next), the residual stream being fp32 [M, hidden].  entry_norm()
               names the norm the block applies to the stream first (or None); the block that ran
               before may already have applied it (`normed`), fused into its last add, and this block
               may do the same for the next one (`next_norm` -> `normed_next`, else None).
  Embedding    forward(ctx, tokens) -> fp32 stream;  Head  forward(ctx, rows) -> fp32 logits.

`ctx` is the step's StepContext: batch geometry on the device, the kernels
(`ctx.ops`), the activation dtype (`ctx.dtype`) and the cache.
"""


class Part:
    def tensor_specs(self):
        """{local tensor name: TensorSpec}."""
        return {}

    def bind(self, tensors, rt):
        """Take the tensors ({local name: device tensor}) and prepare what forward needs."""
        self.rt = rt


class Norm(Part):
    gain = None

    def forward(self, ctx, x, out_dtype=None):
        raise NotImplementedError


class Position(Part):
    rotary_dim = 0
    pairing = "halves"        # which elements of a head a rotation turns together: "halves" (d, d + rotary_dim / 2) or "neighbours" (2d, 2d + 1)

    def inv_freq(self, device):
        raise NotImplementedError


class Mixer(Part):
    def cache_spec(self):
        return None

    def forward(self, ctx, x, site):
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, x):
        raise NotImplementedError


class Block(Part):
    def __init__(self, mixer, feed_forward, make_norm):
        """make_norm(site) builds the norm that stands at one of the block's sites."""
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = {name: make_norm(name) for name in self.norm_sites()}

    @classmethod
    def norm_sites(cls):
        return ()

    def entry_norm(self):
        return None

    def forward(self, ctx, stream, site, normed=None, next_norm=None):
        raise NotImplementedError


class Embedding(Part):
    def forward(self, ctx, tokens):
        raise NotImplementedError


class Head(Part):
    def forward(self, ctx, rows):
        raise NotImplementedError
