"""Write-request kinds an operator finds in `self.req`, one per input or output:
`req.null` (leave it alone), `req.write` / `req.inplace` (overwrite) and `req.add`
(accumulate).  Each constant is its own name as a string, which is what the glue
layers and operator classes compare against (reference: mobula/const.py:1-5)."""

REQUEST_KINDS = ('null', 'write', 'inplace', 'add')

req = type('req', (), {kind: kind for kind in REQUEST_KINDS})
