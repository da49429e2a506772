from .pages import PagePool, OutOfPages
from .manager import (CacheManager, GroupLayout, RequestCache, NO_PAGE, pages_for_tokens,
                      group_page_need)
from . import layout
