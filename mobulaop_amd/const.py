"""Write-request kinds passed to operators through `self.req`
(reference: mobula/const.py:1-5)."""


class req:
    null = 'null'
    write = 'write'
    inplace = 'inplace'
    add = 'add'
